// LSTM and GRU for hidden sizes whose recurrent matrix does not fit on chip: the
// recurrent product of every step is an MFMA GEMM that streams R from HBM (268 MB at
// H = 4096: the step is bound by HBM, not by launches), followed by one pointwise kernel
// for the gates, the cell update and zoneout -- the structure of the reference
// (lib/lstm_forward_gpu.cu.cc:210-310, lib/lstm_backward_gpu.cu.cc:246-317,
// lib/gru_forward_gpu.cu.cc:214-312, lib/gru_backward_gpu.cu.cc:252-319), used here only
// where the persistent kernels cannot be: their slices of R must fit a CU's LDS.
//
// Arithmetic as in lstm.hip / gru.hip (reference lib/lstm_forward_gpu.cu.cc:55-86,
// lib/lstm_backward_gpu.cu.cc:47-95, lib/gru_forward_gpu.cu.cc:46-84,
// lib/gru_backward_gpu.cu.cc:45-95).  Bias gradients are column sums of the stored gate
// gradients taken once at the end in row order (deterministic; the reference uses atomics).
#include "recurrent.h"

namespace haste_hip {
namespace {

constexpr int kPointwiseThreads = 256;

inline dim3 pointwise_grid(int N, int H) {
  return dim3((unsigned)(((size_t)N * H + kPointwiseThreads - 1) / kPointwiseThreads));
}

// R_eff = R * mask * scale (DropConnect), materialised once per call.
__global__ __launch_bounds__(256)
void scale_mask_kernel(size_t n, const float* __restrict__ w, const float* __restrict__ mask,
                       float scale, float* __restrict__ out) {
  const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
  if (i < n) out[i] = w[i] * mask[i] * scale;
}

// v_t: in x*W of the step, out (training) the gate activations; rh = h*R of the step.
__global__ __launch_bounds__(kPointwiseThreads)
void lstm_forward_pointwise(int training, int N, int H, const float* __restrict__ rh,
                            const float* __restrict__ b, const float* __restrict__ h,
                            const float* __restrict__ c, float* __restrict__ h_out,
                            float* __restrict__ c_out, float* __restrict__ v_t, float zoneout_prob,
                            const float* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kPointwiseThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 4 * H + j;
  float a[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) a[g] = v_t[g0 + (size_t)g * H] + rh[g0 + (size_t)g * H] + b[g * H + j];
  const float gi = sigmoid_f(a[0]), gg = tanh_f(a[1]), gf = sigmoid_f(a[2]), go = sigmoid_f(a[3]);
  if (training) {
    v_t[g0] = gi;
    v_t[g0 + H] = gg;
    v_t[g0 + 2 * (size_t)H] = gf;
    v_t[g0 + 3 * (size_t)H] = go;
  }
  const float h_old = h[idx];
  const float c_new = gf * c[idx] + gi * gg;
  float h_new = go * tanh_f(c_new);
  if (zoneout_prob != 0.f && mask_t != nullptr) {
    if (training) h_new = (h_new - h_old) * mask_t[idx] + h_old;
    else h_new = zoneout_prob * h_old + (1.0f - zoneout_prob) * h_new;
  }
  c_out[idx] = c_new;
  h_out[idx] = h_new;
}

// v_t: in the gate activations, out the gate gradients; dh, dc carried in place (dh leaves
// holding the part that bypasses the cell; the recurrent product is added to it afterwards).
__global__ __launch_bounds__(kPointwiseThreads)
void lstm_backward_pointwise(int N, int H, const float* __restrict__ c, const float* __restrict__ c_next,
                             const float* __restrict__ dh_next, const float* __restrict__ dc_next,
                             float* __restrict__ dh, float* __restrict__ dc, float* __restrict__ v_t,
                             const float* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kPointwiseThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 4 * H + j;
  const float gi = v_t[g0], gg = v_t[g0 + H], gf = v_t[g0 + 2 * (size_t)H], go = v_t[g0 + 3 * (size_t)H];
  float dc_total = dc_next[idx] + dc[idx];
  float dh_total = dh_next[idx] + dh[idx];
  const float c_tanh = tanh_f(c_next[idx]);
  float dh_keep = 0.f;
  if (mask_t != nullptr) {
    const float m = mask_t[idx];
    dh_keep = (1.0f - m) * dh_total;
    dh_total = m * dh_total;
  }
  const float do_ = c_tanh * dh_total;
  dc_total += d_tanh_f(c_tanh) * (go * dh_total);
  const float df = c[idx] * dc_total;
  const float di = gg * dc_total;
  const float dg = gi * dc_total;
  dc[idx] = gf * dc_total;
  dh[idx] = dh_keep;
  v_t[g0] = d_sigmoid_f(gi) * di;
  v_t[g0 + H] = d_tanh_f(gg) * dg;
  v_t[g0 + 2 * (size_t)H] = d_sigmoid_f(gf) * df;
  v_t[g0 + 3 * (size_t)H] = d_sigmoid_f(go) * do_;
}

__global__ __launch_bounds__(kPointwiseThreads)
void gru_forward_pointwise(int training, int N, int H, const float* __restrict__ wx,
                           const float* __restrict__ rh, const float* __restrict__ bx,
                           const float* __restrict__ br, const float* __restrict__ h,
                           float* __restrict__ h_out, float* __restrict__ v_t, float zoneout_prob,
                           const float* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kPointwiseThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 3 * H + j;
  const float z = sigmoid_f(wx[g0] + rh[g0] + bx[j] + br[j]);
  const float r = sigmoid_f(wx[g0 + H] + rh[g0 + H] + bx[H + j] + br[H + j]);
  const float qg = rh[g0 + 2 * (size_t)H] + br[2 * H + j];
  const float g = tanh_f(wx[g0 + 2 * (size_t)H] + r * qg + bx[2 * H + j]);
  if (training) {
    const size_t v0 = (size_t)n * 4 * H + j;
    v_t[v0] = z;
    v_t[v0 + H] = r;
    v_t[v0 + 2 * (size_t)H] = g;
    v_t[v0 + 3 * (size_t)H] = qg;
  }
  const float h_old = h[idx];
  float h_new = z * h_old + (1.0f - z) * g;
  if (zoneout_prob != 0.f && mask_t != nullptr) {
    if (training) h_new = (h_new - h_old) * mask_t[idx] + h_old;
    else h_new = zoneout_prob * h_old + (1.0f - zoneout_prob) * h_new;
  }
  h_out[idx] = h_new;
}

__global__ __launch_bounds__(kPointwiseThreads)
void gru_backward_pointwise(int N, int H, const float* __restrict__ h, const float* __restrict__ v_t,
                            const float* __restrict__ dh_next, float* __restrict__ dh,
                            float* __restrict__ dp_t, float* __restrict__ dq_t,
                            const float* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kPointwiseThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t v0 = (size_t)n * 4 * H + j, g0 = (size_t)n * 3 * H + j;
  const float z = v_t[v0], r = v_t[v0 + H], g = v_t[v0 + 2 * (size_t)H], qg = v_t[v0 + 3 * (size_t)H];
  float dh_total = dh_next[idx] + dh[idx];
  float dh_keep;
  if (mask_t != nullptr) {
    const float m = mask_t[idx];
    dh_keep = (1.0f - m) * dh_total;
    dh_total = m * dh_total;
    dh_keep += z * dh_total;
  } else {
    dh_keep = z * dh_total;
  }
  const float dg = (1.0f - z) * dh_total;
  const float dz = (h[idx] - g) * dh_total;
  const float dp_g = d_tanh_f(g) * dg;
  const float dq_g = dp_g * r;
  const float dr = dp_g * qg;
  const float dp_r = d_sigmoid_f(r) * dr;
  const float dp_z = d_sigmoid_f(z) * dz;
  dh[idx] = dh_keep;
  dp_t[g0] = dp_z;
  dp_t[g0 + H] = dp_r;
  dp_t[g0 + 2 * (size_t)H] = dp_g;
  dq_t[g0] = dp_z;
  dq_t[g0 + H] = dp_r;
  dq_t[g0 + 2 * (size_t)H] = dq_g;
}

// out[col] += sum over rows of a[rows, cols], rows added in index order by one thread per
// column (consecutive threads read consecutive columns).
__global__ __launch_bounds__(256)
void column_sum_kernel(size_t rows, int cols, const float* __restrict__ a, float* __restrict__ out) {
  const int col = blockIdx.x * 256 + threadIdx.x;
  if (col >= cols) return;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  size_t r = 0;
  for (; r + 4 <= rows; r += 4) {
    s0 += a[r * cols + col];
    s1 += a[(r + 1) * cols + col];
    s2 += a[(r + 2) * cols + col];
    s3 += a[(r + 3) * cols + col];
  }
  for (; r < rows; ++r) s0 += a[r * cols + col];
  out[col] += (s0 + s1) + (s2 + s3);
}

int column_sum(hipStream_t stream, size_t rows, int cols, const float* a, float* out) {
  column_sum_kernel<<<dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, stream>>>(rows, cols, a, out);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

// Scratch of a streamed call: h*R of one step (and R_eff under DropConnect) in front, the
// GEMMs' own scratch behind it.
struct StreamedScratch {
  float* rh = nullptr;
  float* r_eff = nullptr;
  size_t gemm_offset = 0;  // bytes
};

// `gemm_room`: the most scratch any product of the call asks for, so that the buffer does
// not move (and `rh`, `r_eff` with it) once they are in use.
int take_scratch(hipStream_t stream, size_t rh_floats, size_t r_floats, size_t gemm_room,
                 StreamedScratch* out) {
  const size_t rh4 = (rh_floats + 3) / 4 * 4, r4 = (r_floats + 3) / 4 * 4;
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, (rh4 + r4) * sizeof(float) + gemm_room, &ws));
  out->rh = ws.scratch;
  out->r_eff = r_floats ? ws.scratch + rh4 : nullptr;
  out->gemm_offset = (rh4 + r4) * sizeof(float);
  return HASTE_HIP_OK;
}

}  // namespace

int lstm_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                          const float* W, const float* R, const float* b, const float* x,
                          const float* h, const float* c, float* h_out, float* c_out, float* v,
                          float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                          float dc_scale) {
  const size_t NH = (size_t)N * H, N4H = NH * 4;
  StreamedScratch sc;
  size_t room = gemm_f32_scratch_bytes(T * N, 4 * H, C);
  if (gemm_f32_scratch_bytes(N, 4 * H, H) > room) room = gemm_f32_scratch_bytes(N, 4 * H, H);
  HASTE_HIP_PROPAGATE(take_scratch(stream, N4H, dc_mask ? (size_t)H * 4 * H : 0, room, &sc));
  const float* Ruse = R;
  if (dc_mask != nullptr) {
    const size_t n = (size_t)H * 4 * H;
    scale_mask_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(n, R, dc_mask, dc_scale, sc.r_eff);
    HASTE_HIP_TRY(hipGetLastError());
    Ruse = sc.r_eff;
  }
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T * N, 4 * H, C, x, C, W, 4 * H, v, 4 * H, false, sc.gemm_offset));
  ScopedKernelTimer timer("lstm_forward_streamed", stream);
  for (int t = 0; t < T; ++t) {
    const float* h_t = t == 0 ? h : h_out + (size_t)(t - 1) * NH;
    const float* c_t = t == 0 ? c : c_out + (size_t)(t - 1) * NH;
    HASTE_HIP_PROPAGATE(gemm_f32(stream, false, N, 4 * H, H, h_t, H, Ruse, 4 * H, sc.rh, 4 * H, false, sc.gemm_offset));
    lstm_forward_pointwise<<<pointwise_grid(N, H), dim3(kPointwiseThreads), 0, stream>>>(
        training, N, H, sc.rh, b, h_t, c_t, h_out + (size_t)t * NH, c_out + (size_t)t * NH,
        v + (size_t)t * N4H, zoneout_prob, zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

int lstm_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                           const float* W_t, const float* R_t, const float* x_t,
                           const float* h, const float* c, const float* c_next,
                           const float* dh_next, const float* dc_next,
                           float* dx, float* dW, float* dR, float* db, float* dh, float* dc, float* v,
                           const float* zoneout_mask) {
  const size_t NH = (size_t)N * H, N4H = NH * 4;
  StreamedScratch sc;
  HASTE_HIP_PROPAGATE(take_scratch(stream, 0, 0, 0, &sc));
  {
    ScopedKernelTimer timer("lstm_backward_streamed", stream);
    for (int t = T - 1; t >= 0; --t) {
      lstm_backward_pointwise<<<pointwise_grid(N, H), dim3(kPointwiseThreads), 0, stream>>>(
          N, H, c + (size_t)t * NH, c_next + (size_t)t * NH, dh_next + (size_t)t * NH,
          dc_next + (size_t)t * NH, dh, dc, v + (size_t)t * N4H,
          zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
      HASTE_HIP_TRY(hipGetLastError());
      // dh += dv_t * R^T
      HASTE_HIP_PROPAGATE(gemm_f32(stream, false, N, H, 4 * H, v + (size_t)t * N4H, 4 * H, R_t, H, dh, H, true, sc.gemm_offset));
    }
  }
  const int TN = T * N;
  HASTE_HIP_PROPAGATE(column_sum(stream, (size_t)TN, 4 * H, v, db));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, C, 4 * H, TN, x_t, TN, v, 4 * H, dW, 4 * H, true, sc.gemm_offset));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, true, H, 4 * H, TN, h, H, v, 4 * H, dR, 4 * H, true, sc.gemm_offset));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, TN, C, 4 * H, v, 4 * H, W_t, C, dx, C, false, sc.gemm_offset));
  return HASTE_HIP_OK;
}

int gru_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                         const float* W, const float* R, const float* bx, const float* br,
                         const float* x, const float* h, float* h_out, float* v, float* tmp_Wx,
                         float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                         float dc_scale) {
  const size_t NH = (size_t)N * H, N3H = NH * 3, N4H = NH * 4;
  StreamedScratch sc;
  size_t room = gemm_f32_scratch_bytes(T * N, 3 * H, C);
  if (gemm_f32_scratch_bytes(N, 3 * H, H) > room) room = gemm_f32_scratch_bytes(N, 3 * H, H);
  HASTE_HIP_PROPAGATE(take_scratch(stream, N3H, dc_mask ? (size_t)H * 3 * H : 0, room, &sc));
  const float* Ruse = R;
  if (dc_mask != nullptr) {
    const size_t n = (size_t)H * 3 * H;
    scale_mask_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(n, R, dc_mask, dc_scale, sc.r_eff);
    HASTE_HIP_TRY(hipGetLastError());
    Ruse = sc.r_eff;
  }
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T * N, 3 * H, C, x, C, W, 3 * H, tmp_Wx, 3 * H, false, sc.gemm_offset));
  ScopedKernelTimer timer("gru_forward_streamed", stream);
  for (int t = 0; t < T; ++t) {
    const float* h_t = t == 0 ? h : h_out + (size_t)(t - 1) * NH;
    HASTE_HIP_PROPAGATE(gemm_f32(stream, false, N, 3 * H, H, h_t, H, Ruse, 3 * H, sc.rh, 3 * H, false, sc.gemm_offset));
    gru_forward_pointwise<<<pointwise_grid(N, H), dim3(kPointwiseThreads), 0, stream>>>(
        training, N, H, tmp_Wx + (size_t)t * N3H, sc.rh, bx, br, h_t, h_out + (size_t)t * NH,
        v ? v + (size_t)t * N4H : nullptr, zoneout_prob,
        zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

int gru_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                          const float* W_t, const float* R_t, const float* x_t, const float* h,
                          const float* v, const float* dh_next, float* dx, float* dW, float* dR,
                          float* dbx, float* dbr, float* dh, float* dp, float* dq,
                          const float* zoneout_mask) {
  const size_t NH = (size_t)N * H, N3H = NH * 3, N4H = NH * 4;
  StreamedScratch sc;
  HASTE_HIP_PROPAGATE(take_scratch(stream, 0, 0, 0, &sc));
  {
    ScopedKernelTimer timer("gru_backward_streamed", stream);
    for (int t = T - 1; t >= 0; --t) {
      gru_backward_pointwise<<<pointwise_grid(N, H), dim3(kPointwiseThreads), 0, stream>>>(
          N, H, h + (size_t)t * NH, v + (size_t)t * N4H, dh_next + (size_t)t * NH, dh,
          dp + (size_t)t * N3H, dq + (size_t)t * N3H,
          zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
      HASTE_HIP_TRY(hipGetLastError());
      // dh += dq_t * R^T
      HASTE_HIP_PROPAGATE(gemm_f32(stream, false, N, H, 3 * H, dq + (size_t)t * N3H, 3 * H, R_t, H, dh, H, true, sc.gemm_offset));
    }
  }
  const int TN = T * N;
  HASTE_HIP_PROPAGATE(column_sum(stream, (size_t)TN, 3 * H, dp, dbx));
  HASTE_HIP_PROPAGATE(column_sum(stream, (size_t)TN, 3 * H, dq, dbr));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, TN, C, 3 * H, dp, 3 * H, W_t, C, dx, C, false, sc.gemm_offset));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, true, H, 3 * H, TN, h, H, dq, 3 * H, dR, 3 * H, true, sc.gemm_offset));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, C, 3 * H, TN, x_t, TN, dp, 3 * H, dW, 3 * H, true, sc.gemm_offset));
  return HASTE_HIP_OK;
}

}  // namespace haste_hip
