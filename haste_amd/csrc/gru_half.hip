// The half-precision GRU over more than one step (what gru::ForwardPass<__half>::Run and
// BackwardPass<__half>::Run bind to; reference lib/gru_forward_gpu.cu.cc:373,
// lib/gru_backward_gpu.cu.cc:411).
//
// The recurrence is bound by the latency of its per-step exchange and by instruction issue,
// not by the rate of the matrix units or by HBM, so the persistent fp32 kernels are also the
// fastest way to run it on half tensors: what it reads is widened into a staging area at the
// front of the stream's scratch buffer (one launch), it runs on the staged copies, and what the
// caller gets back is rounded to half (one launch).  Between the steps the state stays in fp32:
// the results are those of exact half inputs, rounded once, where the reference rounds every
// step.  The products around the recurrence (x*W; dx, dW, dR) are bound by the matrix units,
// and those run on the half matrix cores (gemm_half_nt.hip: half operands, the gate gradients
// rounded to half as the reference stores them, fp32 accumulation) whenever the operands are
// laid out for it (sizes multiples of 8, 16-byte aligned) and the recurrence is a persistent
// one; otherwise the whole pass runs in fp32 on widened tensors.
#include "common.h"

extern "C" size_t haste_hip_workspace_bytes(int time_steps, int batch_size, int input_size, int hidden_size);

namespace haste_hip {

int gru_forward_impl(hipStream_t stream, int training, int T, int N, int C, int H,
                     const float* W, const float* R, const float* bx, const float* br,
                     const float* x, const float* h, float* h_out, float* v, float* tmp_Wx,
                     float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                     float dc_scale, bool wx_ready, bool half_product);
int gru_backward_impl(hipStream_t stream, int T, int N, int C, int H,
                      const float* W_t, const float* R_t, const float* x_t, const float* h,
                      const float* v, const float* dh_next, float* dx, float* dW, float* dR,
                      float* dbx, float* dbr, float* dh, float* dp, float* dq,
                      const float* zoneout_mask, bool products, bool half_product);
bool gru_forward_resident(int N, int H);
bool gru_backward_resident(int N, int H);
// gemm_half_nt.hip
bool gemm_half_nt_applies(bool a_float, int M, int N, int K, const void* A, int lda, const void* Bt, int ldb);
int gemm_half_nt(hipStream_t stream, bool a_float, int M, int N, int K, const void* A, int lda,
                 const void* Bt, int ldb, float* C, int ldc, bool accumulate, size_t scratch_offset);
int transpose_to_half(hipStream_t stream, bool in_float, int rows, int cols, const void* in, void* out);

namespace {

typedef _Float16 half_t;
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMaxSegments = 16;  // the backward pass stages twelve tensors

// Tensors to convert in one launch: segment s is `count[s]` elements from src[s] to dst[s].
struct ConvertList {
  const void* src[kMaxSegments];
  void* dst[kMaxSegments];
  unsigned long long count[kMaxSegments];
  int n = 0;
  bool overflow = false;
  unsigned long long longest = 0;
  void add(const void* s, void* d, size_t c) {
    if (s == nullptr || d == nullptr || c == 0) return;
    if (n == kMaxSegments) {
      overflow = true;
      return;
    }
    src[n] = s;
    dst[n] = d;
    count[n] = c;
    if (c > longest) longest = c;
    ++n;
  }
};

// blockIdx.y: the segment; a thread converts runs of 8 elements (16-byte accesses on the half
// side when that side is 16-byte aligned; the float side is the staging area, aligned).
template <bool WIDEN>
__global__ __launch_bounds__(256)
void convert_kernel(ConvertList l) {
  const int s = blockIdx.y;
  const unsigned long long n = l.count[s];
  const unsigned long long stride = (unsigned long long)gridDim.x * 256 * 8;
  const half_t* hsrc = static_cast<const half_t*>(l.src[s]);
  half_t* hdst = static_cast<half_t*>(l.dst[s]);
  const float* fsrc = static_cast<const float*>(l.src[s]);
  float* fdst = static_cast<float*>(l.dst[s]);
  const bool aligned = ((WIDEN ? reinterpret_cast<uintptr_t>(hsrc) : reinterpret_cast<uintptr_t>(hdst)) & 15u) == 0;
  for (unsigned long long i = ((unsigned long long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += stride) {
    if (aligned && i + 8 <= n) {
      if constexpr (WIDEN) {
        const half8_t a = *reinterpret_cast<const half8_t*>(hsrc + i);
        float4_t lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] = (float)a[e];
          hi[e] = (float)a[4 + e];
        }
        *reinterpret_cast<float4_t*>(fdst + i) = lo;
        *reinterpret_cast<float4_t*>(fdst + i + 4) = hi;
      } else {
        const float4_t lo = *reinterpret_cast<const float4_t*>(fsrc + i);
        const float4_t hi = *reinterpret_cast<const float4_t*>(fsrc + i + 4);
        half8_t a;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = (half_t)lo[e];
          a[4 + e] = (half_t)hi[e];
        }
        *reinterpret_cast<half8_t*>(hdst + i) = a;
      }
    } else {
      const unsigned long long end = i + 8 < n ? i + 8 : n;
      for (unsigned long long j = i; j < end; ++j) {
        if constexpr (WIDEN) fdst[j] = (float)hsrc[j];
        else hdst[j] = (half_t)fsrc[j];
      }
    }
  }
}

template <bool WIDEN>
int convert(hipStream_t stream, const ConvertList& l) {
  HASTE_HIP_REQUIRE(!l.overflow);
  if (l.n == 0) return HASTE_HIP_OK;
  unsigned long long blocks = (l.longest + 2047) / 2048;
  if (blocks > 4096) blocks = 4096;
  convert_kernel<WIDEN><<<dim3((unsigned)blocks, (unsigned)l.n), dim3(256), 0, stream>>>(l);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

// Lays float tensors out one after the other, each on a 256-byte boundary.
struct Staging {
  size_t floats = 0;
  size_t take(size_t n) {
    const size_t at = floats;
    floats += (n + 63) / 64 * 64;
    return at;
  }
};

// The staging area of `bytes` bytes plus room behind it for everything the fp32 passes ask for.
int staged_workspace(hipStream_t stream, int T, int N, int C, int H, size_t bytes, float** base) {
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, bytes + workspace_scratch_bound(T, N, C, H), &ws));
  *base = ws.scratch;
  return HASTE_HIP_OK;
}

// Where the staged tensors of a forward / backward pass lie (offsets in floats).
struct ForwardStaging {
  size_t W, R, bx, br, x, h, v, Wx, mask, dc, Wt_half, bytes;
  ForwardStaging(int T, int N, int C, int H, bool training, bool has_mask, bool has_dc) {
    const size_t NH = (size_t)N * H, TN = (size_t)T * N;
    Staging st;
    W = st.take((size_t)C * 3 * H); R = st.take((size_t)H * 3 * H);
    bx = st.take(3 * (size_t)H); br = st.take(3 * (size_t)H);
    x = st.take(TN * C); h = st.take((T + 1) * NH);
    v = training ? st.take(TN * 4 * H) : 0;
    Wx = st.take(TN * 3 * H);
    mask = has_mask ? st.take(TN * H) : 0;
    dc = has_dc ? st.take((size_t)H * 3 * H) : 0;
    Wt_half = st.take(((size_t)C * 3 * H + 1) / 2);  // W transposed, in half
    bytes = st.floats * sizeof(float);
  }
};

struct BackwardStaging {
  size_t Wt, Rt, xt, h, v, dhn, mask, dx, dW, dR, dbx, dbr, dh, dp, dq, W_half, dpT_half, dqT_half, hT_half, bytes;
  BackwardStaging(int T, int N, int C, int H, bool has_mask) {
    const size_t NH = (size_t)N * H, TN = (size_t)T * N, H3 = 3 * (size_t)H;
    Staging st;
    Wt = st.take(H3 * C); Rt = st.take(H3 * H); xt = st.take(TN * C);
    h = st.take((T + 1) * NH); v = st.take(TN * 4 * H); dhn = st.take(TN * H);
    mask = has_mask ? st.take(TN * H) : 0;
    dx = st.take(TN * C); dW = st.take(C * H3); dR = st.take(H * H3);
    dbx = st.take(H3); dbr = st.take(H3); dh = st.take(NH);
    dp = st.take(TN * H3); dq = st.take(TN * H3);
    // in half: W (W_t transposed), the gate gradients and h transposed (time contiguous)
    W_half = st.take((C * H3 + 1) / 2);
    dpT_half = st.take((TN * H3 + 1) / 2); dqT_half = st.take((TN * H3 + 1) / 2);
    hT_half = st.take((TN * H + 1) / 2);
    bytes = st.floats * sizeof(float);
  }
};

size_t gru_half_staging_bytes(int T, int N, int C, int H) {
  const size_t f = ForwardStaging(T, N, C, H, true, true, true).bytes;
  const size_t b = BackwardStaging(T, N, C, H, true).bytes;
  return f > b ? f : b;
}

}  // namespace

// h: [(T+1),N,H], the first [N,H] the state before the first step.
int gru_forward_half(hipStream_t stream, int training, int T, int N, int C, int H, const void* W,
                     const void* R, const void* bx, const void* br, const void* x, void* h, void* v,
                     float zoneout_prob, const void* zoneout_mask, const void* dc_mask,
                     float dc_scale) {
  const size_t NH = (size_t)N * H, TN = (size_t)T * N;
  const ForwardStaging at(T, N, C, H, training != 0, zoneout_mask != nullptr, dc_mask != nullptr);
  const size_t oW = at.W, oR = at.R, obx = at.bx, obr = at.br, ox = at.x, oh = at.h, ov = at.v, oWx = at.Wx;
  const size_t om = at.mask, od = at.dc, bytes = at.bytes;
  float* f = nullptr;
  HASTE_HIP_PROPAGATE(staged_workspace(stream, T, N, C, H, bytes, &f));

  // x*W on the half matrix cores, the recurrence alone in fp32
  if (gru_forward_resident(N, H) && (long long)T * N < (1ll << 31) &&
      gemm_half_nt_applies(false, (int)TN, 3 * H, C, x, C, f + at.Wt_half, C)) {
    ConvertList in;
    in.add(R, f + oR, (size_t)H * 3 * H);
    in.add(bx, f + obx, 3 * (size_t)H);
    in.add(br, f + obr, 3 * (size_t)H);
    in.add(h, f + oh, NH);
    if (zoneout_mask) in.add(zoneout_mask, f + om, TN * H);
    if (dc_mask) in.add(dc_mask, f + od, (size_t)H * 3 * H);
    HASTE_HIP_PROPAGATE(convert<true>(stream, in));
    HASTE_HIP_PROPAGATE(transpose_to_half(stream, false, C, 3 * H, W, f + at.Wt_half));
    {
      ScratchPrefix keep(bytes);
      HASTE_HIP_PROPAGATE(gemm_half_nt(stream, false, (int)TN, 3 * H, C, x, C, f + at.Wt_half, C, f + oWx, 3 * H,
                                       false, 0));
      HASTE_HIP_PROPAGATE(gru_forward_impl(stream, training, T, N, C, H, nullptr, f + oR, f + obx, f + obr, nullptr,
                                           f + oh, f + oh + NH, training ? f + ov : nullptr, f + oWx, zoneout_prob,
                                           zoneout_mask ? f + om : nullptr, dc_mask ? f + od : nullptr, dc_scale,
                                           true, true));
    }
    ConvertList out;
    out.add(f + oh + NH, static_cast<half_t*>(h) + NH, TN * H);
    if (training) out.add(f + ov, v, TN * 4 * H);
    return convert<false>(stream, out);
  }

  ConvertList in;
  in.add(W, f + oW, (size_t)C * 3 * H);
  in.add(R, f + oR, (size_t)H * 3 * H);
  in.add(bx, f + obx, 3 * (size_t)H);
  in.add(br, f + obr, 3 * (size_t)H);
  in.add(x, f + ox, TN * C);
  in.add(h, f + oh, NH);
  if (zoneout_mask) in.add(zoneout_mask, f + om, TN * H);
  if (dc_mask) in.add(dc_mask, f + od, (size_t)H * 3 * H);
  HASTE_HIP_PROPAGATE(convert<true>(stream, in));
  {
    ScratchPrefix keep(bytes);
    HASTE_HIP_PROPAGATE(gru_forward_impl(stream, training, T, N, C, H, f + oW, f + oR, f + obx, f + obr,
                                         f + ox, f + oh, f + oh + NH, training ? f + ov : nullptr, f + oWx,
                                         zoneout_prob, zoneout_mask ? f + om : nullptr,
                                         dc_mask ? f + od : nullptr, dc_scale, false, true));
  }
  ConvertList out;
  out.add(f + oh + NH, static_cast<half_t*>(h) + NH, TN * H);
  if (training) out.add(f + ov, v, TN * 4 * H);
  return convert<false>(stream, out);
}

// h: [(T+1),N,H]; dh_next: [T,N,H], the gradients w.r.t. the states after each step.  dW, dR,
// dbx, dbr and dh are added to, as in the fp32 pass (widened, added to in fp32, rounded).  dp and
// dq are work space whose contents the caller is not to use (reference lib/haste/gru.h:164-169):
// the gate gradients live in the staging area and the caller's two buffers are left alone.
int gru_backward_half(hipStream_t stream, int T, int N, int C, int H, const void* W_t,
                      const void* R_t, const void* x_t, const void* h, const void* v,
                      const void* dh_next, void* dx, void* dW, void* dR, void* dbx, void* dbr,
                      void* dh, void* dp, void* dq, const void* zoneout_mask) {
  (void)dp;
  (void)dq;
  const size_t NH = (size_t)N * H, TN = (size_t)T * N, H3 = 3 * (size_t)H;
  const BackwardStaging at(T, N, C, H, zoneout_mask != nullptr);
  const size_t oWt = at.Wt, oRt = at.Rt, oxt = at.xt, oh = at.h, ov = at.v, odn = at.dhn, om = at.mask;
  const size_t odx = at.dx, odW = at.dW, odR = at.dR, odbx = at.dbx, odbr = at.dbr, odh = at.dh;
  const size_t odp = at.dp, odq = at.dq, bytes = at.bytes;
  float* f = nullptr;
  HASTE_HIP_PROPAGATE(staged_workspace(stream, T, N, C, H, bytes, &f));

  // the recurrence alone in fp32; dx = dp * W_t, dW += x_t * dp, dR += h^T * dq on the half
  // matrix cores, every operand with the contraction index contiguous
  const int iTN = (int)TN, iH3 = 3 * H;
  if (gru_backward_resident(N, H) && (long long)T * N < (1ll << 31) &&
      gemm_half_nt_applies(true, iTN, C, iH3, f + odp, iH3, f + at.W_half, iH3) &&
      gemm_half_nt_applies(false, C, iH3, iTN, x_t, iTN, f + at.dpT_half, iTN) &&
      gemm_half_nt_applies(false, H, iH3, iTN, f + at.hT_half, iTN, f + at.dqT_half, iTN)) {
    ConvertList in;
    in.add(R_t, f + oRt, H3 * H);
    in.add(h, f + oh, (T + 1) * NH);
    in.add(v, f + ov, TN * 4 * H);
    in.add(dh_next, f + odn, TN * H);
    if (zoneout_mask) in.add(zoneout_mask, f + om, TN * H);
    in.add(dW, f + odW, C * H3);
    in.add(dR, f + odR, H * H3);
    in.add(dbx, f + odbx, H3);
    in.add(dbr, f + odbr, H3);
    in.add(dh, f + odh, NH);
    HASTE_HIP_PROPAGATE(convert<true>(stream, in));
    HASTE_HIP_PROPAGATE(transpose_to_half(stream, false, iH3, C, W_t, f + at.W_half));
    HASTE_HIP_PROPAGATE(transpose_to_half(stream, false, iTN, H, h, f + at.hT_half));
    {
      ScratchPrefix keep(bytes);
      HASTE_HIP_PROPAGATE(gru_backward_impl(stream, T, N, C, H, nullptr, f + oRt, nullptr, f + oh, f + ov, f + odn,
                                            nullptr, nullptr, nullptr, f + odbx, f + odbr, f + odh, f + odp, f + odq,
                                            zoneout_mask ? f + om : nullptr, false, true));
      HASTE_HIP_PROPAGATE(transpose_to_half(stream, true, iTN, iH3, f + odp, f + at.dpT_half));
      HASTE_HIP_PROPAGATE(transpose_to_half(stream, true, iTN, iH3, f + odq, f + at.dqT_half));
      HASTE_HIP_PROPAGATE(gemm_half_nt(stream, true, iTN, C, iH3, f + odp, iH3, f + at.W_half, iH3, f + odx, C, false, 0));
      HASTE_HIP_PROPAGATE(gemm_half_nt(stream, false, C, iH3, iTN, x_t, iTN, f + at.dpT_half, iTN, f + odW, iH3, true, 0));
      HASTE_HIP_PROPAGATE(gemm_half_nt(stream, false, H, iH3, iTN, f + at.hT_half, iTN, f + at.dqT_half, iTN, f + odR,
                                       iH3, true, 0));
    }
    ConvertList out;
    out.add(f + odx, dx, TN * C);
    out.add(f + odW, dW, C * H3);
    out.add(f + odR, dR, H * H3);
    out.add(f + odbx, dbx, H3);
    out.add(f + odbr, dbr, H3);
    out.add(f + odh, dh, NH);
    return convert<false>(stream, out);
  }

  ConvertList in;
  in.add(W_t, f + oWt, H3 * C);
  in.add(R_t, f + oRt, H3 * H);
  in.add(x_t, f + oxt, TN * C);
  in.add(h, f + oh, (T + 1) * NH);
  in.add(v, f + ov, TN * 4 * H);
  in.add(dh_next, f + odn, TN * H);
  if (zoneout_mask) in.add(zoneout_mask, f + om, TN * H);
  in.add(dW, f + odW, C * H3);
  in.add(dR, f + odR, H * H3);
  in.add(dbx, f + odbx, H3);
  in.add(dbr, f + odbr, H3);
  in.add(dh, f + odh, NH);
  HASTE_HIP_PROPAGATE(convert<true>(stream, in));
  {
    ScratchPrefix keep(bytes);
    HASTE_HIP_PROPAGATE(gru_backward_impl(stream, T, N, C, H, f + oWt, f + oRt, f + oxt, f + oh, f + ov,
                                          f + odn, f + odx, f + odW, f + odR, f + odbx, f + odbr, f + odh,
                                          f + odp, f + odq, zoneout_mask ? f + om : nullptr, true, true));
  }
  ConvertList out;
  out.add(f + odx, dx, TN * C);
  out.add(f + odW, dW, C * H3);
  out.add(f + odR, dR, H * H3);
  out.add(f + odbx, dbx, H3);
  out.add(f + odbr, dbr, H3);
  out.add(f + odh, dh, NH);
  return convert<false>(stream, out);
}

}  // namespace haste_hip

extern "C" size_t haste_hip_gru_half_workspace_bytes(int time_steps, int batch_size, int input_size,
                                                     int hidden_size) {
  if (time_steps < 1 || batch_size < 1 || input_size < 1 || hidden_size < 1) return 0;
  return haste_hip_workspace_bytes(time_steps, batch_size, input_size, hidden_size) +
         haste_hip::gru_half_staging_bytes(time_steps, batch_size, input_size, hidden_size);
}
