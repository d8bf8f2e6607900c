// Every cell in step-wise form, for `float` and `double`: the recurrent product of each step
// is a GEMM that streams R from HBM, followed by row-wise layer-norm kernels (layer-norm
// cells) and one or two pointwise kernels -- the structure of the reference
// (lib/lstm_forward_gpu.cu.cc:210-310, lib/lstm_backward_gpu.cu.cc:246-317,
// lib/gru_forward_gpu.cu.cc:214-312, lib/gru_backward_gpu.cu.cc:252-319,
// lib/layer_norm_lstm_forward_gpu.cu.cc:276-340, lib/layer_norm_lstm_backward_gpu.cu.cc:255-352,
// lib/layer_norm_gru_forward_gpu.cu.cc:242-305, lib/layer_norm_gru_backward_gpu.cu.cc:219-310,
// lib/indrnn_{forward,backward}_gpu.cu.cc, lib/layer_norm_indrnn_{forward,backward}_gpu.cu.cc).
//
// Used for
//   * float: hidden sizes whose slices of R do not fit a CU's LDS (the persistent kernels
//     of lstm.hip, gru.hip, layer_norm_lstm.hip, layer_norm_gru.hip cannot hold them);
//   * double: every size (the *_f64 entry points at the end of this file; the reference
//     instantiates every class for double as well, e.g. lib/lstm_forward_gpu.cu.cc:368-369).
//
// Arithmetic: reference lib/lstm_forward_gpu.cu.cc:55-86, lib/lstm_backward_gpu.cu.cc:47-95,
// lib/gru_forward_gpu.cu.cc:46-84, lib/gru_backward_gpu.cu.cc:45-95,
// lib/layer_norm_forward_gpu.cu.cc:45-87, lib/layer_norm_backward_gpu.cu.cc:46-92,
// lib/layer_norm_lstm_forward_gpu.cu.cc:50-71,95-108,
// lib/layer_norm_lstm_backward_gpu.cu.cc:44-64,84-117, lib/indrnn_forward_gpu.cu.cc:44-62,
// lib/indrnn_backward_gpu.cu.cc:46-73.  Where the reference adds into bias / gain gradients
// with atomics, column sums are taken here in a fixed order (run-to-run bit equality).
#include "recurrent.h"

namespace haste_hip {

int gemm_f64(hipStream_t stream, bool trans_a, int M, int N, int K, const double* A, int lda,
             const double* B, int ldb, double* C, int ldc, bool accumulate, size_t scratch_offset);
size_t gemm_f64_scratch_bytes(int M, int N, int K);
int gemm_f64_chunks(hipStream_t stream, int M, int N, int K, const double* A, int lda, const double* B,
                    int ldb, size_t scratch_offset, const double** partial, int* chunks);
int gemm_f16(hipStream_t stream, bool trans_a, int M, int N, int K, const void* A, int lda,
             const void* B, int ldb, void* C, int ldc, bool accumulate);
// gru_half.hip: the half GRU over more than one step, on the fp32 kernels.
int gru_forward_half(hipStream_t stream, int training, int T, int N, int C, int H, const void* W,
                     const void* R, const void* bx, const void* br, const void* x, void* h, void* v,
                     float zoneout_prob, const void* zoneout_mask, const void* dc_mask,
                     float dc_scale);
int gru_backward_half(hipStream_t stream, int T, int N, int C, int H, const void* W_t,
                      const void* R_t, const void* x_t, const void* h, const void* v,
                      const void* dh_next, void* dx, void* dW, void* dR, void* dbx, void* dbr,
                      void* dh, void* dp, void* dq, const void* zoneout_mask);

namespace {

constexpr int kThreads = 256;

#define HASTE_LAUNCHED() HASTE_HIP_TRY(hipGetLastError())

inline dim3 blocks_for(size_t n) { return dim3((unsigned)((n + kThreads - 1) / kThreads)); }

// ---- scalar math ------------------------------------------------------------------
// Storage type T, arithmetic type Acc<T>::type: half tensors (GRU only) are computed in float.
typedef _Float16 half_t;
template <typename T> struct Acc { using type = T; };
template <> struct Acc<half_t> { using type = float; };

template <typename T> struct Fn;
template <> struct Fn<float> {
  static __device__ __forceinline__ float sigmoid(float x) { return sigmoid_f(x); }
  static __device__ __forceinline__ float tanh_(float x) { return tanh_f(x); }
  static __device__ __forceinline__ float inv_sqrt(float x) { return 1.0f / sqrtf(x); }
};
template <> struct Fn<double> {
  static __device__ __forceinline__ double sigmoid(double x) { return 1.0 / (1.0 + exp(-x)); }
  static __device__ __forceinline__ double tanh_(double x) { return tanh(x); }
  static __device__ __forceinline__ double inv_sqrt(double x) { return 1.0 / sqrt(x); }
};
template <typename T> __device__ __forceinline__ T d_sigmoid(T y) { return y * (T(1) - y); }
template <typename T> __device__ __forceinline__ T d_tanh(T y) { return T(1) - y * y; }

// ---- products ---------------------------------------------------------------------
inline int gemm(hipStream_t s, bool ta, int M, int N, int K, const float* A, int lda,
                const float* B, int ldb, float* C, int ldc, bool acc, size_t scratch_offset) {
  return gemm_f32(s, ta, M, N, K, A, lda, B, ldb, C, ldc, acc, scratch_offset);
}
inline int gemm(hipStream_t s, bool ta, int M, int N, int K, const double* A, int lda,
                const double* B, int ldb, double* C, int ldc, bool acc, size_t scratch_offset) {
  return gemm_f64(s, ta, M, N, K, A, lda, B, ldb, C, ldc, acc, scratch_offset);
}
inline int gemm(hipStream_t s, bool ta, int M, int N, int K, const half_t* A, int lda,
                const half_t* B, int ldb, half_t* C, int ldc, bool acc, size_t) {
  return gemm_f16(s, ta, M, N, K, A, lda, B, ldb, C, ldc, acc);
}
template <typename T> size_t gemm_room(int M, int N, int K);
template <> size_t gemm_room<float>(int M, int N, int K) { return gemm_f32_scratch_bytes(M, N, K); }
template <> size_t gemm_room<double>(int M, int N, int K) { return gemm_f64_scratch_bytes(M, N, K); }
template <> size_t gemm_room<half_t>(int, int, int) { return 0; }

// A step's product as its consumer reads it: either one finished matrix (chunks == 1,
// stride == 0) or the K chunks of the small-batch streaming kernel, which the consumer adds in
// chunk order itself -- one launch per step less than reducing them first, which is what
// bounds the step at small batch and moderate hidden size.  chunks == 0: nothing pending.
template <typename T>
struct StepProduct {
  const T* base = nullptr;
  int chunks = 0;
  size_t stride = 0;
  // tile_rows != 0: the chunks are the K pieces of the tile kernel (gemm_f32_pieces), element
  // (row, col) of piece k at base[((col / 128 * chunks + k) * tile_rows + row) * 128 + col % 128].
  int tile_rows = 0;
  int row_len = 0;

  __device__ __forceinline__ size_t first(size_t idx) const {
    if (tile_rows == 0) return idx;
    const size_t row = idx / row_len, col = idx % row_len;
    return ((col / 128 * chunks) * tile_rows + row) * 128 + col % 128;
  }
  __device__ __forceinline__ size_t step() const {
    return tile_rows == 0 ? stride : (size_t)tile_rows * 128;
  }
  // out[g] = the product at idx + g * gate_stride, g < G.  Chunks are added in index order;
  // the loads of two chunks and all G gates are issued together.
  template <int G>
  __device__ __forceinline__ void at(size_t idx, size_t gate_stride, typename Acc<T>::type (&out)[G]) const {
    typedef typename Acc<T>::type A;
    size_t at0[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      out[g] = A(0);
      at0[g] = first(idx + g * gate_stride);
    }
    const size_t st = step();
    int k = 0;
    for (; k + 2 <= chunks; k += 2) {
      A v0[G], v1[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        v0[g] = (A)base[at0[g] + k * st];
        v1[g] = (A)base[at0[g] + (k + 1) * st];
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        out[g] += v0[g];
        out[g] += v1[g];
      }
    }
    if (k < chunks) {
#pragma unroll
      for (int g = 0; g < G; ++g) out[g] += (A)base[at0[g] + k * st];
    }
  }
  __device__ __forceinline__ typename Acc<T>::type at(size_t idx) const {
    typename Acc<T>::type out[1];
    at<1>(idx, 0, out);
    return out[0];
  }
};

// C[M,N] = A[M,K] * B[K,N] for one step, for a consumer kernel: into `out` (then the product
// reads as one matrix), or left as chunks.
template <typename T>
int step_product(hipStream_t s, int M, int N, int K, const T* A, const T* B, T* out,
                 size_t scratch_offset, StepProduct<T>* p) {
  HASTE_HIP_PROPAGATE(gemm(s, false, M, N, K, A, K, B, N, out, N, false, scratch_offset));
  p->base = out;
  p->chunks = 1;
  p->stride = 0;
  return HASTE_HIP_OK;
}
template <>
int step_product<double>(hipStream_t s, int M, int N, int K, const double* A, const double* B,
                         double* out, size_t scratch_offset, StepProduct<double>* p) {
  HASTE_HIP_PROPAGATE(gemm_f64_chunks(s, M, N, K, A, K, B, N, scratch_offset, &p->base, &p->chunks));
  if (p->chunks > 0) {
    p->stride = (size_t)M * N;
    return HASTE_HIP_OK;
  }
  HASTE_HIP_PROPAGATE(gemm_f64(s, false, M, N, K, A, K, B, N, out, N, false, scratch_offset));
  p->base = out;
  p->chunks = 1;
  p->stride = 0;
  return HASTE_HIP_OK;
}
template <>
int step_product<float>(hipStream_t s, int M, int N, int K, const float* A, const float* B,
                        float* out, size_t scratch_offset, StepProduct<float>* p) {
  if (gemm_f32_skinny_applies(false, M, N, K, A, K, B, N, out, N)) {
    HASTE_HIP_PROPAGATE(gemm_f32_skinny_chunks(s, M, N, K, A, K, B, N, scratch_offset, &p->base, &p->chunks));
    p->stride = (size_t)M * N;
    return HASTE_HIP_OK;
  }
  int splits = 0, bm = 0;
  HASTE_HIP_PROPAGATE(gemm_f32_pieces(s, M, N, K, A, K, B, N, scratch_offset, &p->base, &splits, &bm));
  if (splits > 0) {
    p->chunks = splits;
    p->tile_rows = bm;
    p->row_len = N;
    return HASTE_HIP_OK;
  }
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, M, N, K, A, K, B, N, out, N, false, scratch_offset));
  p->base = out;
  p->chunks = 1;
  p->stride = 0;
  return HASTE_HIP_OK;
}

// dh += (pending chunks): the recurrent contribution a reverse step leaves for the next
// step's pointwise kernel, added for real after the last step.
template <typename T>
__global__ __launch_bounds__(kThreads)
void add_pending_kernel(size_t n, StepProduct<T> pend, T* __restrict__ dh) {
  const size_t i = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (i < n) dh[i] = T((typename Acc<T>::type)dh[i] + pend.at(i));
}

// The recurrent product of a reverse step, dh += dv_t[M,K] * R_t[K,N]: accumulated into dh
// (nothing pending), or left as chunks for the next consumer of dh.
template <typename T>
int reverse_product(hipStream_t s, int M, int N, int K, const T* A, const T* B, T* dh,
                    size_t scratch_offset, StepProduct<T>* pend) {
  pend->chunks = 0;
  return gemm(s, false, M, N, K, A, K, B, N, dh, N, true, scratch_offset);
}
template <>
int reverse_product<double>(hipStream_t s, int M, int N, int K, const double* A, const double* B,
                            double* dh, size_t scratch_offset, StepProduct<double>* pend) {
  *pend = StepProduct<double>();
  HASTE_HIP_PROPAGATE(gemm_f64_chunks(s, M, N, K, A, K, B, N, scratch_offset, &pend->base, &pend->chunks));
  if (pend->chunks > 0) {
    pend->stride = (size_t)M * N;
    return HASTE_HIP_OK;
  }
  return gemm_f64(s, false, M, N, K, A, K, B, N, dh, N, true, scratch_offset);
}
template <>
int reverse_product<float>(hipStream_t s, int M, int N, int K, const float* A, const float* B,
                           float* dh, size_t scratch_offset, StepProduct<float>* pend) {
  *pend = StepProduct<float>();
  if (gemm_f32_skinny_applies(false, M, N, K, A, K, B, N, dh, N)) {
    HASTE_HIP_PROPAGATE(gemm_f32_skinny_chunks(s, M, N, K, A, K, B, N, scratch_offset, &pend->base, &pend->chunks));
    pend->stride = (size_t)M * N;
    return HASTE_HIP_OK;
  }
  int splits = 0, bm = 0;
  HASTE_HIP_PROPAGATE(gemm_f32_pieces(s, M, N, K, A, K, B, N, scratch_offset, &pend->base, &splits, &bm));
  if (splits > 0) {
    pend->chunks = splits;
    pend->tile_rows = bm;
    pend->row_len = N;
    return HASTE_HIP_OK;
  }
  return gemm_f32(s, false, M, N, K, A, K, B, N, dh, N, true, scratch_offset);
}

template <typename T>
int flush_pending(hipStream_t s, size_t n, const StepProduct<T>& pend, T* dh) {
  if (pend.chunks == 0) return HASTE_HIP_OK;
  add_pending_kernel<T><<<blocks_for(n), dim3(kThreads), 0, s>>>(n, pend, dh);
  HASTE_LAUNCHED();
  return HASTE_HIP_OK;
}

// Scratch of a call: buffers of its own in front, the float GEMM's partial tiles behind
// them.  Everything is sized before the first launch so that the buffer never moves while
// it is in use.
struct Scratch {
  char* base = nullptr;
  size_t used = 0, own = 0;
  template <typename T> T* take(size_t count) {
    T* p = reinterpret_cast<T*>(base + used);
    used += (count * sizeof(T) + 255) / 256 * 256;
    return p;
  }
  size_t gemm_offset() const { return own; }
};
inline size_t padded(size_t bytes) { return (bytes + 255) / 256 * 256; }

int open_scratch(hipStream_t stream, size_t own_bytes, size_t gemm_bytes, Scratch* sc) {
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, own_bytes + gemm_bytes + 256, &ws));
  sc->base = reinterpret_cast<char*>(ws.scratch);
  sc->used = 0;
  sc->own = own_bytes;
  return HASTE_HIP_OK;
}

// ---- small kernels ------------------------------------------------------------------
// R_eff = R * mask * scale (DropConnect), materialised once per call.
template <typename T>
__global__ __launch_bounds__(kThreads)
void scale_mask_kernel(size_t n, const T* __restrict__ w, const T* __restrict__ mask,
                       typename Acc<T>::type scale, T* __restrict__ out) {
  using A = typename Acc<T>::type;
  const size_t i = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (i < n) out[i] = T(A(w[i]) * A(mask[i]) * scale);
}

// Column sums over rows in two deterministic stages.  MODE 0: a[r][col]; MODE 1: the gain
// gradient of a layer norm, (x[r][col] - mean_r) * invstd_r * a[r][col] with (mean, invstd)
// from cache[r].  Stage one: one thread per (column, chunk of rows); stage two adds the
// chunks in index order into out (accumulating).  Sums are kept in the arithmetic type.
template <typename T, int MODE>
__global__ __launch_bounds__(kThreads)
void column_partial_kernel(size_t rows, int cols, size_t rows_per_chunk, const T* __restrict__ a,
                           const T* __restrict__ x, const T* __restrict__ cache,
                           typename Acc<T>::type* __restrict__ partial) {
  using A = typename Acc<T>::type;
  const int col = blockIdx.x * kThreads + threadIdx.x;
  if (col >= cols) return;
  const size_t r0 = blockIdx.y * rows_per_chunk;
  size_t r1 = r0 + rows_per_chunk;
  if (r1 > rows) r1 = rows;
  A s = A(0);
  for (size_t r = r0; r < r1; ++r) {
    const size_t at = r * cols + col;
    if (MODE == 0) s += A(a[at]);
    else s += (A(x[at]) - A(cache[2 * r])) * A(cache[2 * r + 1]) * A(a[at]);
  }
  partial[(size_t)blockIdx.y * cols + col] = s;
}

template <typename T>
__global__ __launch_bounds__(kThreads)
void column_finish_kernel(int chunks, int cols, const typename Acc<T>::type* __restrict__ partial,
                          T* __restrict__ out) {
  using A = typename Acc<T>::type;
  const int col = blockIdx.x * kThreads + threadIdx.x;
  if (col >= cols) return;
  A s = A(0);
  for (int k = 0; k < chunks; ++k) s += partial[(size_t)k * cols + col];
  out[col] = T(A(out[col]) + s);
}

inline int column_chunks(size_t rows, size_t* rows_per_chunk) {
  size_t rpc = (rows + 127) / 128;
  if (rpc < 16) rpc = 16;
  *rows_per_chunk = rpc;
  return (int)((rows + rpc - 1) / rpc);
}
template <typename T>
size_t column_sum_bytes(size_t rows, int cols) {
  size_t rpc;
  return padded((size_t)column_chunks(rows, &rpc) * cols * sizeof(typename Acc<T>::type));
}
// Room for sums over all rows of a call and over the rows of one step.
template <typename T>
size_t column_sum_bytes(size_t all_rows, size_t step_rows, int cols) {
  const size_t a = column_sum_bytes<T>(all_rows, cols), b = column_sum_bytes<T>(step_rows, cols);
  return a > b ? a : b;
}

// out[col] += column sum (MODE 0) or gain gradient (MODE 1); `partial` holds
// column_sum_bytes() bytes.
template <typename T, int MODE>
int column_sum(hipStream_t stream, size_t rows, int cols, const T* a, const T* x, const T* cache,
               void* partial_, T* out) {
  typename Acc<T>::type* partial = static_cast<typename Acc<T>::type*>(partial_);
  size_t rpc;
  const int chunks = column_chunks(rows, &rpc);
  const dim3 grid((unsigned)((cols + kThreads - 1) / kThreads), (unsigned)chunks);
  column_partial_kernel<T, MODE><<<grid, dim3(kThreads), 0, stream>>>(rows, cols, rpc, a, x, cache, partial);
  HASTE_LAUNCHED();
  column_finish_kernel<T><<<dim3(grid.x), dim3(kThreads), 0, stream>>>(chunks, cols, partial, out);
  HASTE_LAUNCHED();
  return HASTE_HIP_OK;
}

// ---- layer norm over rows of any length: one workgroup per row ------------------------
template <typename T>
__device__ __forceinline__ T block_sum(T v, T* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();  // red may still be read from the previous sum
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T>
__device__ __forceinline__ void row_moments(int D, const T* __restrict__ xr, T* red, T* mean, T* invstd) {
  T s = T(0);
  for (int j = threadIdx.x; j < D; j += kThreads) s += xr[j];
  const T m = block_sum(s, red) / T(D);
  T q = T(0);
  for (int j = threadIdx.x; j < D; j += kThreads) {
    const T d = xr[j] - m;
    q += d * d;
  }
  const T var = block_sum(q, red) / T(D);
  *mean = m;
  *invstd = Fn<T>::inv_sqrt(var + T(1e-5));
}

// y = (x - mean) * invstd * gamma (+ beta); cache[row] = (mean, invstd) if cache != null;
// y == null: statistics only.
template <typename T>
__global__ __launch_bounds__(kThreads)
void ln_forward_rows_kernel(int D, const T* __restrict__ gamma, const T* __restrict__ beta,
                            const T* __restrict__ x, T* __restrict__ y, T* __restrict__ cache) {
  __shared__ T red[4];
  const size_t row = blockIdx.x;
  const T* xr = x + row * D;
  T mean, invstd;
  row_moments(D, xr, red, &mean, &invstd);
  if (cache != nullptr && threadIdx.x == 0) {
    cache[2 * row] = mean;
    cache[2 * row + 1] = invstd;
  }
  if (y == nullptr) return;
  T* yr = y + row * D;
  for (int j = threadIdx.x; j < D; j += kThreads) {
    T v = (xr[j] - mean) * invstd * gamma[j];
    if (beta != nullptr) v += beta[j];
    yr[j] = v;
  }
}

// dx of reference lib/layer_norm_backward_gpu.cu.cc:46-92 for one row per workgroup; dx may
// alias dy or x (a thread reads its own elements before it writes them).  cache == null:
// the statistics are recomputed from x.
template <typename T>
__global__ __launch_bounds__(kThreads)
void ln_backward_rows_kernel(int D, const T* __restrict__ gamma, const T* x, const T* dy, T* dx,
                             const T* __restrict__ cache) {
  __shared__ T red[4];
  const size_t row = blockIdx.x;
  const T* xr = x + row * D;
  const T* gr = dy + row * D;
  T mean, invstd;
  if (cache != nullptr) {
    mean = cache[2 * row];
    invstd = cache[2 * row + 1];
  } else {
    row_moments(D, xr, red, &mean, &invstd);
  }
  T s0 = T(0), s1 = T(0), s2 = T(0);
  for (int j = threadIdx.x; j < D; j += kThreads) {
    const T xc = xr[j] - mean, g = gamma[j] * gr[j];
    s0 += xc * g;
    s1 += xc;
    s2 += g;
  }
  s0 = block_sum(s0, red);
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  const T dsigma = T(-0.5) * s0 * invstd * invstd * invstd;
  const T dmu = (T(-2) * s1 * dsigma / T(D)) - (s2 * invstd);
  T* out = dx + row * D;
  for (int j = threadIdx.x; j < D; j += kThreads) {
    const T xc = xr[j] - mean, g = gamma[j] * gr[j];
    out[j] = (T(2) * xc * dsigma / T(D)) + (invstd * g) + (dmu / T(D));
  }
}

template <typename T>
int ln_forward_rows(hipStream_t stream, size_t rows, int D, const T* gamma, const T* beta,
                    const T* x, T* y, T* cache) {
  ln_forward_rows_kernel<T><<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(D, gamma, beta, x, y, cache);
  HASTE_LAUNCHED();
  return HASTE_HIP_OK;
}

// Gain (and shift) gradients, then dx.  `cache` must hold the rows' statistics;
// `partial` as for column_sum.
template <typename T>
int ln_backward_rows(hipStream_t stream, size_t rows, int D, const T* gamma, const T* x,
                     const T* dy, T* dx, T* dgamma, T* dbeta, const T* cache, void* partial) {
  HASTE_HIP_PROPAGATE((column_sum<T, 1>(stream, rows, D, dy, x, cache, partial, dgamma)));
  if (dbeta != nullptr)
    HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, rows, D, dy, nullptr, nullptr, partial, dbeta)));
  ln_backward_rows_kernel<T><<<dim3((unsigned)rows), dim3(kThreads), 0, stream>>>(D, gamma, x, dy, dx, cache);
  HASTE_LAUNCHED();
  return HASTE_HIP_OK;
}

// ---- LSTM pointwise -------------------------------------------------------------------
// v_t: in x*W of the step, out (training) the gate activations; rh = h*R of the step.
template <typename T>
__global__ __launch_bounds__(kThreads)
void lstm_forward_pointwise(int training, int N, int H, StepProduct<T> rh,
                            const T* __restrict__ b, const T* __restrict__ h,
                            const T* __restrict__ c, T* __restrict__ h_out, T* __restrict__ c_out,
                            T* __restrict__ v_t, float zoneout_prob, const T* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 4 * H + j;
  T a[4];
  rh.template at<4>(g0, (size_t)H, a);
#pragma unroll
  for (int g = 0; g < 4; ++g) a[g] = v_t[g0 + (size_t)g * H] + a[g] + b[g * H + j];
  const T gi = Fn<T>::sigmoid(a[0]), gg = Fn<T>::tanh_(a[1]), gf = Fn<T>::sigmoid(a[2]),
          go = Fn<T>::sigmoid(a[3]);
  if (training) {
    v_t[g0] = gi;
    v_t[g0 + H] = gg;
    v_t[g0 + 2 * (size_t)H] = gf;
    v_t[g0 + 3 * (size_t)H] = go;
  }
  const T h_old = h[idx];
  const T c_new = gf * c[idx] + gi * gg;
  T h_new = go * Fn<T>::tanh_(c_new);
  if (zoneout_prob != 0.f && mask_t != nullptr) {
    if (training) h_new = (h_new - h_old) * mask_t[idx] + h_old;
    else h_new = T(zoneout_prob) * h_old + (T(1) - T(zoneout_prob)) * h_new;
  }
  c_out[idx] = c_new;
  h_out[idx] = h_new;
}

// v_t: in the gate activations, out the gate gradients; dh, dc carried in place (dh leaves
// holding the part that bypasses the cell; the recurrent product is added to it afterwards).
template <typename T>
__global__ __launch_bounds__(kThreads)
void lstm_backward_pointwise(int N, int H, const T* __restrict__ c, const T* __restrict__ c_next,
                             const T* __restrict__ dh_next, const T* __restrict__ dc_next,
                             T* __restrict__ dh, StepProduct<T> pend, T* __restrict__ dc,
                             T* __restrict__ v_t, const T* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 4 * H + j;
  const T gi = v_t[g0], gg = v_t[g0 + H], gf = v_t[g0 + 2 * (size_t)H], go = v_t[g0 + 3 * (size_t)H];
  T dc_total = dc_next[idx] + dc[idx];
  T dh_total = dh_next[idx] + (dh[idx] + pend.at(idx));
  const T c_tanh = Fn<T>::tanh_(c_next[idx]);
  T dh_keep = T(0);
  if (mask_t != nullptr) {
    const T m = mask_t[idx];
    dh_keep = (T(1) - m) * dh_total;
    dh_total = m * dh_total;
  }
  const T do_ = c_tanh * dh_total;
  dc_total += d_tanh(c_tanh) * (go * dh_total);
  const T df = c[idx] * dc_total;
  const T di = gg * dc_total;
  const T dg = gi * dc_total;
  dc[idx] = gf * dc_total;
  dh[idx] = dh_keep;
  v_t[g0] = d_sigmoid(gi) * di;
  v_t[g0 + H] = d_tanh(gg) * dg;
  v_t[g0 + 2 * (size_t)H] = d_sigmoid(gf) * df;
  v_t[g0 + 3 * (size_t)H] = d_sigmoid(go) * do_;
}

// ---- GRU pointwise (also the layer-norm GRU: wx, rh are then the normalised products) ----
template <typename T>
__global__ __launch_bounds__(kThreads)
void gru_forward_pointwise(int training, int N, int H, const T* __restrict__ wx,
                           StepProduct<T> rh, const T* __restrict__ bx,
                           const T* __restrict__ br, const T* __restrict__ h,
                           T* __restrict__ h_out, T* __restrict__ v_t, float zoneout_prob,
                           const T* __restrict__ mask_t) {
  using A = typename Acc<T>::type;
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 3 * H + j;
  A q[3];
  rh.template at<3>(g0, (size_t)H, q);
  const A z = Fn<A>::sigmoid(A(wx[g0]) + q[0] + A(bx[j]) + A(br[j]));
  const A r = Fn<A>::sigmoid(A(wx[g0 + H]) + q[1] + A(bx[H + j]) + A(br[H + j]));
  const A qg = q[2] + A(br[2 * H + j]);
  const A g = Fn<A>::tanh_(A(wx[g0 + 2 * (size_t)H]) + r * qg + A(bx[2 * H + j]));
  if (training) {
    const size_t v0 = (size_t)n * 4 * H + j;
    v_t[v0] = T(z);
    v_t[v0 + H] = T(r);
    v_t[v0 + 2 * (size_t)H] = T(g);
    v_t[v0 + 3 * (size_t)H] = T(qg);
  }
  const A h_old = A(h[idx]);
  A h_new = z * h_old + (A(1) - z) * g;
  if (zoneout_prob != 0.f && mask_t != nullptr) {
    if (training) h_new = (h_new - h_old) * A(mask_t[idx]) + h_old;
    else h_new = A(zoneout_prob) * h_old + (A(1) - A(zoneout_prob)) * h_new;
  }
  h_out[idx] = T(h_new);
}

template <typename T>
__global__ __launch_bounds__(kThreads)
void gru_backward_pointwise(int N, int H, const T* __restrict__ h, const T* __restrict__ v_t,
                            const T* __restrict__ dh_next, T* __restrict__ dh,
                            StepProduct<T> pend, T* __restrict__ dp_t, T* __restrict__ dq_t,
                            const T* __restrict__ mask_t) {
  using A = typename Acc<T>::type;
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t v0 = (size_t)n * 4 * H + j, g0 = (size_t)n * 3 * H + j;
  const A z = A(v_t[v0]), r = A(v_t[v0 + H]), g = A(v_t[v0 + 2 * (size_t)H]),
          qg = A(v_t[v0 + 3 * (size_t)H]);
  A dh_total = A(dh_next[idx]) + (A(dh[idx]) + pend.at(idx));
  A dh_keep;
  if (mask_t != nullptr) {
    const A m = A(mask_t[idx]);
    dh_keep = (A(1) - m) * dh_total;
    dh_total = m * dh_total;
    dh_keep += z * dh_total;
  } else {
    dh_keep = z * dh_total;
  }
  const A dg = (A(1) - z) * dh_total;
  const A dz = (A(h[idx]) - g) * dh_total;
  const A dp_g = d_tanh(g) * dg;
  const A dq_g = dp_g * r;
  const A dr = dp_g * qg;
  const A dp_r = d_sigmoid(r) * dr;
  const A dp_z = d_sigmoid(z) * dz;
  dh[idx] = T(dh_keep);
  dp_t[g0] = T(dp_z);
  dp_t[g0 + H] = T(dp_r);
  dp_t[g0 + 2 * (size_t)H] = T(dp_g);
  dq_t[g0] = T(dp_z);
  dq_t[g0 + H] = T(dp_r);
  dq_t[g0 + 2 * (size_t)H] = T(dq_g);
}

// ---- layer-norm LSTM pointwise ------------------------------------------------------------
// Gates and cell state of one step (reference ComputeCellState).  wxn_t: LN(x*W) of the
// step, overwritten with the gate activations when training; rhn: LN(h*R), overwritten with
// the gate activations always (the output kernel reads o from it).
template <typename T>
__global__ __launch_bounds__(kThreads)
void ln_lstm_cell_state(int training, int N, int H, T* __restrict__ wxn_t, T* __restrict__ rhn,
                        const T* __restrict__ b, const T* __restrict__ c, T* __restrict__ c_out) {
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 4 * H + j;
  T a[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) a[g] = wxn_t[g0 + (size_t)g * H] + rhn[g0 + (size_t)g * H] + b[g * H + j];
  const T gi = Fn<T>::sigmoid(a[0]), gg = Fn<T>::tanh_(a[1]), gf = Fn<T>::sigmoid(a[2]),
          go = Fn<T>::sigmoid(a[3]);
  if (training) {
    wxn_t[g0] = gi;
    wxn_t[g0 + H] = gg;
    wxn_t[g0 + 2 * (size_t)H] = gf;
    wxn_t[g0 + 3 * (size_t)H] = go;
  }
  rhn[g0 + 3 * (size_t)H] = go;
  c_out[idx] = gf * c[idx] + gi * gg;
}

// h' = o * tanh(LN(c')) + zoneout (reference ComputeCellOutput).
template <typename T>
__global__ __launch_bounds__(kThreads)
void ln_lstm_cell_output(int training, int N, int H, const T* __restrict__ rhn,
                         const T* __restrict__ c_norm_t, const T* __restrict__ h,
                         T* __restrict__ h_out, float zoneout_prob, const T* __restrict__ mask_t) {
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const T go = rhn[(size_t)n * 4 * H + 3 * (size_t)H + j];
  const T h_old = h[idx];
  T h_new = go * Fn<T>::tanh_(c_norm_t[idx]);
  if (zoneout_prob != 0.f && mask_t != nullptr) {
    if (training) h_new = (h_new - h_old) * mask_t[idx] + h_old;
    else h_new = T(zoneout_prob) * h_old + (T(1) - T(zoneout_prob)) * h_new;
  }
  h_out[idx] = h_new;
}

// Reverse step, first half (reference ComputeOutputGrad): splits dh at the zoneout mask,
// turns o into its gradient and LN(c') into the gradient that enters the cell-state norm.
template <typename T>
__global__ __launch_bounds__(kThreads)
void ln_lstm_output_grad(int N, int H, const T* __restrict__ dh_next, T* __restrict__ dh,
                         StepProduct<T> pend, const T* __restrict__ mask_t, T* __restrict__ c_norm_t, T* __restrict__ v_t) {
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t o_at = (size_t)n * 4 * H + 3 * (size_t)H + j;
  const T go = v_t[o_at];
  T dh_total = dh_next[idx] + (dh[idx] + pend.at(idx));
  T dh_keep = T(0);
  if (mask_t != nullptr) {
    const T m = mask_t[idx];
    dh_keep = (T(1) - m) * dh_total;
    dh_total = m * dh_total;
  }
  const T c_tanh = Fn<T>::tanh_(c_norm_t[idx]);
  v_t[o_at] = d_sigmoid(go) * (c_tanh * dh_total);
  c_norm_t[idx] = d_tanh(c_tanh) * (go * dh_total);
  dh[idx] = dh_keep;
}

// Reverse step, second half: dc_ln is the gradient that came back through the cell-state
// norm; turns i, g, f into their gradients.
template <typename T>
__global__ __launch_bounds__(kThreads)
void ln_lstm_gate_grad(int N, int H, const T* __restrict__ c, const T* __restrict__ dc_next,
                       T* __restrict__ dc, const T* __restrict__ dc_ln, T* __restrict__ v_t) {
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= (size_t)N * H) return;
  const int n = (int)(idx / H), j = (int)(idx % H);
  const size_t g0 = (size_t)n * 4 * H + j;
  const T gi = v_t[g0], gg = v_t[g0 + H], gf = v_t[g0 + 2 * (size_t)H];
  const T dc_total = dc_next[idx] + dc[idx] + dc_ln[idx];
  const T df = c[idx] * dc_total;
  const T di = gg * dc_total;
  const T dg = gi * dc_total;
  dc[idx] = gf * dc_total;
  v_t[g0] = d_sigmoid(gi) * di;
  v_t[g0 + H] = d_tanh(gg) * dg;
  v_t[g0 + 2 * (size_t)H] = d_sigmoid(gf) * df;
}

// ---- IndRNN: one thread per (row, unit) walks the steps ---------------------------------
template <typename T>
__global__ __launch_bounds__(kThreads)
void indrnn_forward_loop(int training, int steps, int N, int H, const T* __restrict__ wx,
                         const T* __restrict__ u, const T* __restrict__ b, T* __restrict__ h,
                         float zoneout_prob, const T* __restrict__ mask) {
  const size_t NH = (size_t)N * H;
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= NH) return;
  const int j = (int)(idx % H);
  const T uj = u[j], bj = b[j];
  T hv = h[idx];
  for (int t = 0; t < steps; ++t) {
    T h_new = Fn<T>::tanh_(wx[t * NH + idx] + uj * hv + bj);
    if (zoneout_prob != 0.f && mask != nullptr) {
      if (training) h_new = (h_new - hv) * mask[t * NH + idx] + hv;
      else h_new = T(zoneout_prob) * hv + (T(1) - T(zoneout_prob)) * h_new;
    }
    h[(t + 1) * NH + idx] = h_new;
    hv = h_new;
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads)
void indrnn_backward_loop(int steps, int N, int H, const T* __restrict__ u, const T* __restrict__ h,
                          const T* __restrict__ dh_new, T* __restrict__ dh, T* __restrict__ dk,
                          const T* __restrict__ mask, T* __restrict__ du_rows, T* __restrict__ db_rows) {
  const size_t NH = (size_t)N * H;
  const size_t idx = blockIdx.x * (size_t)kThreads + threadIdx.x;
  if (idx >= NH) return;
  const T uj = u[idx % H];
  T dhv = dh[idx], du_acc = T(0), db_acc = T(0);
  for (int t = steps - 1; t >= 0; --t) {
    T total = dh_new[(t + 1) * NH + idx] + dhv;
    T keep = T(0);
    if (mask != nullptr) {
      const T m = mask[t * NH + idx];
      keep = (T(1) - m) * total;
      total = m * total;
    }
    const T dkv = d_tanh(h[(t + 1) * NH + idx]) * total;
    dk[t * NH + idx] = dkv;
    dhv = keep + uj * dkv;
    du_acc += h[t * NH + idx] * dkv;
    db_acc += dkv;
  }
  dh[idx] = dhv;
  du_rows[idx] = du_acc;
  db_rows[idx] = db_acc;
}

// ---- the cells --------------------------------------------------------------------------
template <typename T>
int effective_r(hipStream_t stream, size_t n, const T* R, const T* dc_mask, float dc_scale,
                T* r_eff, const T** out) {
  *out = R;
  if (dc_mask == nullptr) return HASTE_HIP_OK;
  scale_mask_kernel<T><<<blocks_for(n), dim3(kThreads), 0, stream>>>(n, R, dc_mask, typename Acc<T>::type(dc_scale), r_eff);
  HASTE_LAUNCHED();
  *out = r_eff;
  return HASTE_HIP_OK;
}

inline size_t max2(size_t a, size_t b) { return a > b ? a : b; }

template <typename T>
int lstm_forward_steps(hipStream_t stream, int training, int steps, int N, int C, int H,
                       const T* W, const T* R, const T* b, const T* x, const T* h, const T* c,
                       T* h_out, T* c_out, T* v, float zoneout_prob, const T* zoneout_mask,
                       const T* dc_mask, float dc_scale) {
  const size_t NH = (size_t)N * H, N4H = NH * 4, r_count = (size_t)H * 4 * H;
  const size_t own = padded(N4H * sizeof(T)) + (dc_mask ? padded(r_count * sizeof(T)) : 0);
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, max2(gemm_room<T>(steps * N, 4 * H, C), gemm_room<T>(N, 4 * H, H)), &sc));
  T* rh = sc.take<T>(N4H);
  const T* Ruse;
  HASTE_HIP_PROPAGATE(effective_r(stream, r_count, R, dc_mask, dc_scale, dc_mask ? sc.take<T>(r_count) : nullptr, &Ruse));
  HASTE_HIP_PROPAGATE(gemm(stream, false, steps * N, 4 * H, C, x, C, W, 4 * H, v, 4 * H, false, sc.gemm_offset()));
  ScopedKernelTimer timer("lstm_forward_steps", stream);
  for (int t = 0; t < steps; ++t) {
    const T* h_t = t == 0 ? h : h_out + (size_t)(t - 1) * NH;
    const T* c_t = t == 0 ? c : c_out + (size_t)(t - 1) * NH;
    StepProduct<T> prod;
    HASTE_HIP_PROPAGATE(step_product<T>(stream, N, 4 * H, H, h_t, Ruse, rh, sc.gemm_offset(), &prod));
    lstm_forward_pointwise<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
        training, N, H, prod, b, h_t, c_t, h_out + (size_t)t * NH, c_out + (size_t)t * NH,
        v + (size_t)t * N4H, zoneout_prob, zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
    HASTE_LAUNCHED();
  }
  return HASTE_HIP_OK;
}

template <typename T>
int lstm_backward_steps(hipStream_t stream, int steps, int N, int C, int H, const T* W_t,
                        const T* R_t, const T* x_t, const T* h, const T* c, const T* c_next,
                        const T* dh_next, const T* dc_next, T* dx, T* dW, T* dR, T* db, T* dh,
                        T* dc, T* v, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H, N4H = NH * 4;
  const int TN = steps * N;
  const size_t own = column_sum_bytes<T>((size_t)TN, 4 * H);
  size_t room = max2(gemm_room<T>(N, H, 4 * H), gemm_room<T>(C, 4 * H, TN));
  room = max2(room, max2(gemm_room<T>(H, 4 * H, TN), gemm_room<T>(TN, C, 4 * H)));
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, room, &sc));
  void* partial = sc.take<char>(own);
  {
    ScopedKernelTimer timer("lstm_backward_steps", stream);
    StepProduct<T> pend;
    for (int t = steps - 1; t >= 0; --t) {
      lstm_backward_pointwise<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
          N, H, c + (size_t)t * NH, c_next + (size_t)t * NH, dh_next + (size_t)t * NH,
          dc_next + (size_t)t * NH, dh, pend, dc, v + (size_t)t * N4H,
          zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
      HASTE_LAUNCHED();
      // dh += dv_t * R^T
      HASTE_HIP_PROPAGATE(reverse_product<T>(stream, N, H, 4 * H, v + (size_t)t * N4H, R_t, dh, sc.gemm_offset(), &pend));
    }
    HASTE_HIP_PROPAGATE(flush_pending<T>(stream, NH, pend, dh));
  }
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)TN, 4 * H, v, nullptr, nullptr, partial, db)));
  HASTE_HIP_PROPAGATE(gemm(stream, false, C, 4 * H, TN, x_t, TN, v, 4 * H, dW, 4 * H, true, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, true, H, 4 * H, TN, h, H, v, 4 * H, dR, 4 * H, true, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, C, 4 * H, v, 4 * H, W_t, C, dx, C, false, sc.gemm_offset()));
  return HASTE_HIP_OK;
}

template <typename T>
int gru_forward_steps(hipStream_t stream, int training, int steps, int N, int C, int H, const T* W,
                      const T* R, const T* bx, const T* br, const T* x, const T* h, T* h_out, T* v,
                      T* tmp_Wx, float zoneout_prob, const T* zoneout_mask, const T* dc_mask,
                      float dc_scale) {
  const size_t NH = (size_t)N * H, N3H = NH * 3, N4H = NH * 4, r_count = (size_t)H * 3 * H;
  const size_t own = padded(N3H * sizeof(T)) + (dc_mask ? padded(r_count * sizeof(T)) : 0);
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, max2(gemm_room<T>(steps * N, 3 * H, C), gemm_room<T>(N, 3 * H, H)), &sc));
  T* rh = sc.take<T>(N3H);
  const T* Ruse;
  HASTE_HIP_PROPAGATE(effective_r(stream, r_count, R, dc_mask, dc_scale, dc_mask ? sc.take<T>(r_count) : nullptr, &Ruse));
  HASTE_HIP_PROPAGATE(gemm(stream, false, steps * N, 3 * H, C, x, C, W, 3 * H, tmp_Wx, 3 * H, false, sc.gemm_offset()));
  ScopedKernelTimer timer("gru_forward_steps", stream);
  for (int t = 0; t < steps; ++t) {
    const T* h_t = t == 0 ? h : h_out + (size_t)(t - 1) * NH;
    StepProduct<T> prod;
    HASTE_HIP_PROPAGATE(step_product<T>(stream, N, 3 * H, H, h_t, Ruse, rh, sc.gemm_offset(), &prod));
    gru_forward_pointwise<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
        training, N, H, tmp_Wx + (size_t)t * N3H, prod, bx, br, h_t, h_out + (size_t)t * NH,
        v ? v + (size_t)t * N4H : nullptr, zoneout_prob,
        zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
    HASTE_LAUNCHED();
  }
  return HASTE_HIP_OK;
}

template <typename T>
int gru_backward_steps(hipStream_t stream, int steps, int N, int C, int H, const T* W_t,
                       const T* R_t, const T* x_t, const T* h, const T* v, const T* dh_next, T* dx,
                       T* dW, T* dR, T* dbx, T* dbr, T* dh, T* dp, T* dq, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H, N3H = NH * 3, N4H = NH * 4;
  const int TN = steps * N;
  const size_t own = column_sum_bytes<T>((size_t)TN, 3 * H);
  size_t room = max2(gemm_room<T>(N, H, 3 * H), gemm_room<T>(C, 3 * H, TN));
  room = max2(room, max2(gemm_room<T>(H, 3 * H, TN), gemm_room<T>(TN, C, 3 * H)));
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, room, &sc));
  void* partial = sc.take<char>(own);
  {
    ScopedKernelTimer timer("gru_backward_steps", stream);
    StepProduct<T> pend;
    for (int t = steps - 1; t >= 0; --t) {
      gru_backward_pointwise<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
          N, H, h + (size_t)t * NH, v + (size_t)t * N4H, dh_next + (size_t)t * NH, dh, pend,
          dp + (size_t)t * N3H, dq + (size_t)t * N3H,
          zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
      HASTE_LAUNCHED();
      // dh += dq_t * R^T
      HASTE_HIP_PROPAGATE(reverse_product<T>(stream, N, H, 3 * H, dq + (size_t)t * N3H, R_t, dh, sc.gemm_offset(), &pend));
    }
    HASTE_HIP_PROPAGATE(flush_pending<T>(stream, NH, pend, dh));
  }
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)TN, 3 * H, dp, nullptr, nullptr, partial, dbx)));
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)TN, 3 * H, dq, nullptr, nullptr, partial, dbr)));
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, C, 3 * H, dp, 3 * H, W_t, C, dx, C, false, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, true, H, 3 * H, TN, h, H, dq, 3 * H, dR, 3 * H, true, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, false, C, 3 * H, TN, x_t, TN, dp, 3 * H, dW, 3 * H, true, sc.gemm_offset()));
  return HASTE_HIP_OK;
}

template <typename T>
int ln_lstm_forward_steps(hipStream_t stream, int training, int steps, int N, int C, int H,
                          const T* W, const T* R, const T* b, const T* x, T* h, T* c, T* act_Wx,
                          const T* gamma1, T* cache1, T* act_Wx_norm, T* act_Rh, const T* gamma2,
                          T* cache2, const T* gamma_h, const T* beta_h, T* cache3, T* act_c_norm,
                          float zoneout_prob, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H, N4H = NH * 4;
  const int TN = steps * N;
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, padded(N4H * sizeof(T)), max2(gemm_room<T>(TN, 4 * H, C), gemm_room<T>(N, 4 * H, H)), &sc));
  T* rhn = sc.take<T>(N4H);
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, 4 * H, C, x, C, W, 4 * H, act_Wx, 4 * H, false, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)TN, 4 * H, gamma1, nullptr, act_Wx, act_Wx_norm, cache1));
  ScopedKernelTimer timer("layer_norm_lstm_forward_steps", stream);
  for (int t = 0; t < steps; ++t) {
    const T* h_t = h + (size_t)t * NH;
    T* rh_t = act_Rh + (size_t)t * N4H;
    HASTE_HIP_PROPAGATE(gemm(stream, false, N, 4 * H, H, h_t, H, R, 4 * H, rh_t, 4 * H, false, sc.gemm_offset()));
    HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)N, 4 * H, gamma2, nullptr, rh_t, rhn,
                                           cache2 ? cache2 + (size_t)t * N * 2 : nullptr));
    ln_lstm_cell_state<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
        training, N, H, act_Wx_norm + (size_t)t * N4H, rhn, b, c + (size_t)t * NH, c + (size_t)(t + 1) * NH);
    HASTE_LAUNCHED();
    HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)N, H, gamma_h, beta_h, c + (size_t)(t + 1) * NH,
                                           act_c_norm + (size_t)t * NH,
                                           cache3 ? cache3 + (size_t)t * N * 2 : nullptr));
    ln_lstm_cell_output<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
        training, N, H, rhn, act_c_norm + (size_t)t * NH, h_t, h + (size_t)(t + 1) * NH, zoneout_prob,
        zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
    HASTE_LAUNCHED();
  }
  return HASTE_HIP_OK;
}

template <typename T>
int ln_lstm_backward_steps(hipStream_t stream, int steps, int N, int C, int H, const T* W_t,
                           const T* R_t, const T* x_t, const T* h, const T* c, const T* dh_new,
                           const T* dc_new, T* dx, T* dW, T* dR, T* db, T* dh, T* dc, T* act_Wx,
                           const T* gamma1, T* dgamma1, T* v, T* act_Rh, const T* gamma2,
                           T* dgamma2, const T* cache2, const T* gamma_h, T* dgamma_h, T* dbeta_h,
                           const T* cache3, T* act_c_norm, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H, N4H = NH * 4;
  const int TN = steps * N;
  const size_t part_bytes = column_sum_bytes<T>((size_t)TN, (size_t)N, 4 * H);
  const size_t own = part_bytes + padded((size_t)TN * 2 * sizeof(T));
  size_t room = max2(gemm_room<T>(N, H, 4 * H), gemm_room<T>(C, 4 * H, TN));
  room = max2(room, max2(gemm_room<T>(H, 4 * H, TN), gemm_room<T>(TN, C, 4 * H)));
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, room, &sc));
  void* partial = sc.take<char>(part_bytes);
  T* stats1 = sc.take<T>((size_t)TN * 2);
  {
    ScopedKernelTimer timer("layer_norm_lstm_backward_steps", stream);
    StepProduct<T> pend;
    for (int t = steps - 1; t >= 0; --t) {
      T* v_t = v + (size_t)t * N4H;
      T* cn_t = act_c_norm + (size_t)t * NH;
      T* rh_t = act_Rh + (size_t)t * N4H;
      const T* mask_t = zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr;
      ln_lstm_output_grad<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
          N, H, dh_new + (size_t)(t + 1) * NH, dh, pend, mask_t, cn_t, v_t);
      HASTE_LAUNCHED();
      // through the norm of the cell state, in place over act_c_norm[t]
      HASTE_HIP_PROPAGATE(ln_backward_rows<T>(stream, (size_t)N, H, gamma_h, c + (size_t)(t + 1) * NH, cn_t, cn_t,
                                              dgamma_h, dbeta_h, cache3 + (size_t)t * N * 2, partial));
      ln_lstm_gate_grad<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
          N, H, c + (size_t)t * NH, dc_new + (size_t)(t + 1) * NH, dc, cn_t, v_t);
      HASTE_LAUNCHED();
      // through the norm of h*R, in place over act_Rh[t]
      HASTE_HIP_PROPAGATE(ln_backward_rows<T>(stream, (size_t)N, 4 * H, gamma2, rh_t, v_t, rh_t, dgamma2,
                                              nullptr, cache2 + (size_t)t * N * 2, partial));
      HASTE_HIP_PROPAGATE(reverse_product<T>(stream, N, H, 4 * H, rh_t, R_t, dh, sc.gemm_offset(), &pend));
    }
    HASTE_HIP_PROPAGATE(flush_pending<T>(stream, NH, pend, dh));
  }
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)TN, 4 * H, v, nullptr, nullptr, partial, db)));
  // through the norm of x*W, in place over act_Wx
  HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)TN, 4 * H, gamma1, nullptr, act_Wx, nullptr, stats1));
  HASTE_HIP_PROPAGATE(ln_backward_rows<T>(stream, (size_t)TN, 4 * H, gamma1, act_Wx, v, act_Wx, dgamma1, nullptr, stats1, partial));
  HASTE_HIP_PROPAGATE(gemm(stream, false, C, 4 * H, TN, x_t, TN, act_Wx, 4 * H, dW, 4 * H, true, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, true, H, 4 * H, TN, h, H, act_Rh, 4 * H, dR, 4 * H, true, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, C, 4 * H, act_Wx, 4 * H, W_t, C, dx, C, false, sc.gemm_offset()));
  return HASTE_HIP_OK;
}

template <typename T>
int ln_gru_forward_steps(hipStream_t stream, int training, int steps, int N, int C, int H,
                         const T* W, const T* R, const T* bx, const T* br, const T* x, T* h, T* v,
                         T* act_Wx, const T* gamma1, T* cache1, T* tmp_Wx_norm, T* act_Rh,
                         const T* gamma2, T* cache2, float zoneout_prob, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H, N3H = NH * 3, N4H = NH * 4;
  const int TN = steps * N;
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, padded(N3H * sizeof(T)), max2(gemm_room<T>(TN, 3 * H, C), gemm_room<T>(N, 3 * H, H)), &sc));
  T* rhn = sc.take<T>(N3H);
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, 3 * H, C, x, C, W, 3 * H, act_Wx, 3 * H, false, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)TN, 3 * H, gamma1, nullptr, act_Wx, tmp_Wx_norm, cache1));
  ScopedKernelTimer timer("layer_norm_gru_forward_steps", stream);
  for (int t = 0; t < steps; ++t) {
    const T* h_t = h + (size_t)t * NH;
    T* rh_t = act_Rh + (size_t)t * N3H;
    HASTE_HIP_PROPAGATE(gemm(stream, false, N, 3 * H, H, h_t, H, R, 3 * H, rh_t, 3 * H, false, sc.gemm_offset()));
    HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)N, 3 * H, gamma2, nullptr, rh_t, rhn,
                                           cache2 ? cache2 + (size_t)t * N * 2 : nullptr));
    StepProduct<T> normed;
    normed.base = rhn;
    normed.chunks = 1;
    gru_forward_pointwise<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
        training, N, H, tmp_Wx_norm + (size_t)t * N3H, normed, bx, br, h_t, h + (size_t)(t + 1) * NH,
        v ? v + (size_t)t * N4H : nullptr, zoneout_prob,
        zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
    HASTE_LAUNCHED();
  }
  return HASTE_HIP_OK;
}

template <typename T>
int ln_gru_backward_steps(hipStream_t stream, int steps, int N, int C, int H, const T* W_t,
                          const T* R_t, const T* x_t, const T* h, const T* v, const T* dh_new,
                          T* dx, T* dW, T* dR, T* dbx, T* dbr, T* dh, T* dp, T* dq,
                          const T* act_Wx, const T* gamma1, T* dgamma1, const T* act_Rh,
                          const T* gamma2, T* dgamma2, const T* cache2, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H, N3H = NH * 3, N4H = NH * 4;
  const int TN = steps * N;
  const size_t part_bytes = column_sum_bytes<T>((size_t)TN, (size_t)N, 3 * H);
  const size_t own = part_bytes + padded((size_t)TN * 2 * sizeof(T));
  size_t room = max2(gemm_room<T>(N, H, 3 * H), gemm_room<T>(C, 3 * H, TN));
  room = max2(room, max2(gemm_room<T>(H, 3 * H, TN), gemm_room<T>(TN, C, 3 * H)));
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, room, &sc));
  void* partial = sc.take<char>(part_bytes);
  T* stats1 = sc.take<T>((size_t)TN * 2);
  {
    ScopedKernelTimer timer("layer_norm_gru_backward_steps", stream);
    StepProduct<T> pend;
    for (int t = steps - 1; t >= 0; --t) {
      T* dq_t = dq + (size_t)t * N3H;
      gru_backward_pointwise<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
          N, H, h + (size_t)t * NH, v + (size_t)t * N4H, dh_new + (size_t)(t + 1) * NH, dh, pend,
          dp + (size_t)t * N3H, dq_t, zoneout_mask ? zoneout_mask + (size_t)t * NH : nullptr);
      HASTE_LAUNCHED();
      // the recurrent bias sees dq before the norm; then through the norm of h*R, in place
      HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)N, 3 * H, dq_t, nullptr, nullptr, partial, dbr)));
      HASTE_HIP_PROPAGATE(ln_backward_rows<T>(stream, (size_t)N, 3 * H, gamma2, act_Rh + (size_t)t * N3H, dq_t, dq_t,
                                              dgamma2, nullptr, cache2 + (size_t)t * N * 2, partial));
      HASTE_HIP_PROPAGATE(reverse_product<T>(stream, N, H, 3 * H, dq_t, R_t, dh, sc.gemm_offset(), &pend));
    }
    HASTE_HIP_PROPAGATE(flush_pending<T>(stream, NH, pend, dh));
  }
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)TN, 3 * H, dp, nullptr, nullptr, partial, dbx)));
  HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)TN, 3 * H, gamma1, nullptr, act_Wx, nullptr, stats1));
  HASTE_HIP_PROPAGATE(ln_backward_rows<T>(stream, (size_t)TN, 3 * H, gamma1, act_Wx, dp, dp, dgamma1, nullptr, stats1, partial));
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, C, 3 * H, dp, 3 * H, W_t, C, dx, C, false, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, true, H, 3 * H, TN, h, H, dq, 3 * H, dR, 3 * H, true, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, false, C, 3 * H, TN, x_t, TN, dp, 3 * H, dW, 3 * H, true, sc.gemm_offset()));
  return HASTE_HIP_OK;
}

// IndRNN, with gamma1 != null the layer-norm IndRNN (act_Wx then holds x*W, workspace its norm).
template <typename T>
int indrnn_forward_steps(hipStream_t stream, int training, int steps, int N, int C, int H,
                         const T* W, const T* u, const T* b, const T* x, T* h, T* workspace,
                         T* act_Wx, const T* gamma1, T* cache1, float zoneout_prob,
                         const T* zoneout_mask) {
  const int TN = steps * N;
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, 0, gemm_room<T>(TN, H, C), &sc));
  T* wx = gamma1 ? act_Wx : workspace;
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, H, C, x, C, W, H, wx, H, false, sc.gemm_offset()));
  if (gamma1) HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)TN, H, gamma1, nullptr, act_Wx, workspace, cache1));
  ScopedKernelTimer timer("indrnn_forward_steps", stream);
  indrnn_forward_loop<T><<<blocks_for((size_t)N * H), dim3(kThreads), 0, stream>>>(
      training, steps, N, H, workspace, u, b, h, zoneout_prob, zoneout_mask);
  HASTE_LAUNCHED();
  return HASTE_HIP_OK;
}

template <typename T>
int indrnn_backward_steps(hipStream_t stream, int steps, int N, int C, int H, const T* W_t,
                          const T* u, const T* x_t, const T* h, const T* dh_new, T* dx, T* dW,
                          T* du, T* db, T* dh, T* workspace, const T* act_Wx, const T* gamma1,
                          T* dgamma1, const T* zoneout_mask) {
  const size_t NH = (size_t)N * H;
  const int TN = steps * N;
  const size_t part_bytes = column_sum_bytes<T>((size_t)TN, (size_t)N, H);
  const size_t own = part_bytes + 2 * padded(NH * sizeof(T)) + padded((size_t)TN * 2 * sizeof(T));
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, own, max2(gemm_room<T>(C, H, TN), gemm_room<T>(TN, C, H)), &sc));
  void* partial = sc.take<char>(part_bytes);
  T* du_rows = sc.take<T>(NH);
  T* db_rows = sc.take<T>(NH);
  T* stats1 = sc.take<T>((size_t)TN * 2);
  {
    ScopedKernelTimer timer("indrnn_backward_steps", stream);
    indrnn_backward_loop<T><<<blocks_for(NH), dim3(kThreads), 0, stream>>>(
        steps, N, H, u, h, dh_new, dh, workspace, zoneout_mask, du_rows, db_rows);
    HASTE_LAUNCHED();
  }
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)N, H, du_rows, nullptr, nullptr, partial, du)));
  HASTE_HIP_PROPAGATE((column_sum<T, 0>(stream, (size_t)N, H, db_rows, nullptr, nullptr, partial, db)));
  if (gamma1) {
    HASTE_HIP_PROPAGATE(ln_forward_rows<T>(stream, (size_t)TN, H, gamma1, nullptr, act_Wx, nullptr, stats1));
    HASTE_HIP_PROPAGATE(ln_backward_rows<T>(stream, (size_t)TN, H, gamma1, act_Wx, workspace, workspace, dgamma1,
                                            nullptr, stats1, partial));
  }
  HASTE_HIP_PROPAGATE(gemm(stream, false, C, H, TN, x_t, TN, workspace, H, dW, H, false, sc.gemm_offset()));
  HASTE_HIP_PROPAGATE(gemm(stream, false, TN, C, H, workspace, H, W_t, C, dx, C, false, sc.gemm_offset()));
  return HASTE_HIP_OK;
}

}  // namespace

// ---- float: what the persistent implementations fall back to -------------------------------
int lstm_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                          const float* W, const float* R, const float* b, const float* x,
                          const float* h, const float* c, float* h_out, float* c_out, float* v,
                          float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                          float dc_scale) {
  return lstm_forward_steps<float>(stream, training, T, N, C, H, W, R, b, x, h, c, h_out, c_out, v,
                                   zoneout_prob, zoneout_mask, dc_mask, dc_scale);
}
int lstm_backward_streamed(hipStream_t stream, int T, int N, int C, int H, const float* W_t,
                           const float* R_t, const float* x_t, const float* h, const float* c,
                           const float* c_next, const float* dh_next, const float* dc_next,
                           float* dx, float* dW, float* dR, float* db, float* dh, float* dc, float* v,
                           const float* zoneout_mask) {
  return lstm_backward_steps<float>(stream, T, N, C, H, W_t, R_t, x_t, h, c, c_next, dh_next, dc_next,
                                    dx, dW, dR, db, dh, dc, v, zoneout_mask);
}
int gru_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                         const float* W, const float* R, const float* bx, const float* br,
                         const float* x, const float* h, float* h_out, float* v, float* tmp_Wx,
                         float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                         float dc_scale) {
  return gru_forward_steps<float>(stream, training, T, N, C, H, W, R, bx, br, x, h, h_out, v, tmp_Wx,
                                  zoneout_prob, zoneout_mask, dc_mask, dc_scale);
}
int gru_backward_streamed(hipStream_t stream, int T, int N, int C, int H, const float* W_t,
                          const float* R_t, const float* x_t, const float* h, const float* v,
                          const float* dh_next, float* dx, float* dW, float* dR, float* dbx,
                          float* dbr, float* dh, float* dp, float* dq, const float* zoneout_mask) {
  return gru_backward_steps<float>(stream, T, N, C, H, W_t, R_t, x_t, h, v, dh_next, dx, dW, dR, dbx,
                                   dbr, dh, dp, dq, zoneout_mask);
}
// Row-wise layer norm of any width (one workgroup per row): what layer_norm.hip hands rows
// to that do not fit a wavefront's registers.
int layer_norm_forward_wide(hipStream_t stream, int rows, int dim, const float* gamma,
                            const float* beta, const float* x, float* y, float* cache) {
  return ln_forward_rows<float>(stream, (size_t)rows, dim, gamma, beta, x, y, cache);
}
int layer_norm_backward_wide(hipStream_t stream, int rows, int dim, const float* gamma,
                             const float* x, const float* dy, float* dx, float* dgamma,
                             float* dbeta) {
  const size_t part_bytes = column_sum_bytes<float>((size_t)rows, dim);
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, part_bytes + padded((size_t)rows * 2 * sizeof(float)), 0, &sc));
  void* partial = sc.take<char>(part_bytes);
  float* stats = sc.take<float>((size_t)rows * 2);
  HASTE_HIP_PROPAGATE(ln_forward_rows<float>(stream, (size_t)rows, dim, gamma, nullptr, x, nullptr, stats));
  return ln_backward_rows<float>(stream, (size_t)rows, dim, gamma, x, dy, dx, dgamma, dbeta, stats, partial);
}

int layer_norm_lstm_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                                     const float* W, const float* R, const float* b, const float* x,
                                     float* h, float* c, float* act_Wx, const float* gamma1,
                                     float* cache1, float* act_Wx_norm, float* act_Rh,
                                     const float* gamma2, float* cache2, const float* gamma_h,
                                     const float* beta_h, float* cache3, float* act_c_norm,
                                     float zoneout_prob, const float* zoneout_mask) {
  return ln_lstm_forward_steps<float>(stream, training, T, N, C, H, W, R, b, x, h, c, act_Wx, gamma1,
                                      cache1, act_Wx_norm, act_Rh, gamma2, cache2, gamma_h, beta_h,
                                      cache3, act_c_norm, zoneout_prob, zoneout_mask);
}
int layer_norm_lstm_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                                      const float* W_t, const float* R_t, const float* x_t,
                                      const float* h, const float* c, const float* dh_new,
                                      const float* dc_new, float* dx, float* dW, float* dR, float* db,
                                      float* dh, float* dc, float* act_Wx, const float* gamma1,
                                      float* dgamma1, float* act_Wx_norm, float* act_Rh,
                                      const float* gamma2, float* dgamma2, const float* cache2,
                                      const float* gamma_h, float* dgamma_h, float* dbeta_h,
                                      const float* cache3, float* act_c_norm,
                                      const float* zoneout_mask) {
  return ln_lstm_backward_steps<float>(stream, T, N, C, H, W_t, R_t, x_t, h, c, dh_new, dc_new, dx, dW,
                                       dR, db, dh, dc, act_Wx, gamma1, dgamma1, act_Wx_norm, act_Rh,
                                       gamma2, dgamma2, cache2, gamma_h, dgamma_h, dbeta_h, cache3,
                                       act_c_norm, zoneout_mask);
}
int layer_norm_gru_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                                    const float* W, const float* R, const float* bx, const float* br,
                                    const float* x, float* h, float* v, float* act_Wx,
                                    const float* gamma1, float* cache1, float* tmp_Wx_norm,
                                    float* act_Rh, const float* gamma2, float* cache2,
                                    float zoneout_prob, const float* zoneout_mask) {
  return ln_gru_forward_steps<float>(stream, training, T, N, C, H, W, R, bx, br, x, h, v, act_Wx, gamma1,
                                     cache1, tmp_Wx_norm, act_Rh, gamma2, cache2, zoneout_prob,
                                     zoneout_mask);
}
int layer_norm_gru_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                                     const float* W_t, const float* R_t, const float* x_t,
                                     const float* h, const float* v, const float* dh_new, float* dx,
                                     float* dW, float* dR, float* dbx, float* dbr, float* dh,
                                     float* dp, float* dq, const float* act_Wx, const float* gamma1,
                                     float* dgamma1, const float* act_Rh, const float* gamma2,
                                     float* dgamma2, const float* cache2,
                                     const float* zoneout_mask) {
  return ln_gru_backward_steps<float>(stream, T, N, C, H, W_t, R_t, x_t, h, v, dh_new, dx, dW, dR, dbx,
                                      dbr, dh, dp, dq, act_Wx, gamma1, dgamma1, act_Rh, gamma2,
                                      dgamma2, cache2, zoneout_mask);
}

}  // namespace haste_hip

// ---- double: the C ABI ------------------------------------------------------------------------
using namespace haste_hip;

extern "C" {

int haste_hip_lstm_forward_f64(int training, int steps, int batch_size, int input_size,
                               int hidden_size, const double* W, const double* R, const double* b,
                               const double* x, double* h, double* c, double* v, double* tmp_Rh,
                               float zoneout_prob, const double* zoneout_mask, void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && b && x && h && c && v);
  const size_t NH = (size_t)batch_size * hidden_size;
  return lstm_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                    hidden_size, W, R, b, x, h, c, h + NH, c + NH, v, zoneout_prob,
                                    zoneout_mask, nullptr, 1.f);
}

int haste_hip_lstm_forward_dropconnect_f64(int training, int steps, int batch_size, int input_size,
                                           int hidden_size, const double* W, const double* R,
                                           const double* b, const double* x, double* h, double* c,
                                           double* v, float zoneout_prob, const double* zoneout_mask,
                                           const double* dropconnect_mask, float dropconnect_scale,
                                           void* stream) {
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && b && x && h && c && v);
  const size_t NH = (size_t)batch_size * hidden_size;
  return lstm_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                    hidden_size, W, R, b, x, h, c, h + NH, c + NH, v, zoneout_prob,
                                    zoneout_mask, dropconnect_mask, dropconnect_scale);
}

int haste_hip_lstm_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                                const double* W_t, const double* R_t, const double* b,
                                const double* x_t, const double* h, const double* c,
                                const double* dh_new, const double* dc_new, double* dx, double* dW,
                                double* dR, double* db, double* dh, double* dc, double* v,
                                const double* zoneout_mask, void* stream) {
  (void)b;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && c && dh_new && dc_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && db && dh && dc && v);
  const size_t NH = (size_t)batch_size * hidden_size;
  return lstm_backward_steps<double>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                     W_t, R_t, x_t, h, c, c + NH, dh_new + NH, dc_new + NH, dx, dW, dR,
                                     db, dh, dc, v, zoneout_mask);
}

int haste_hip_lstm_forward_iterate_f64(int training, int batch_size, int input_size,
                                       int hidden_size, const double* W, const double* R,
                                       const double* b, const double* x, const double* h,
                                       const double* c, double* h_out, double* c_out, double* v,
                                       double* tmp_Rh, float zoneout_prob,
                                       const double* zoneout_mask, void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && b && x && h && c && h_out && c_out && v);
  return lstm_forward_steps<double>(as_stream(stream), training, 1, batch_size, input_size,
                                    hidden_size, W, R, b, x, h, c, h_out, c_out, v, zoneout_prob,
                                    zoneout_mask, nullptr, 1.f);
}

int haste_hip_lstm_backward_iterate_f64(int batch_size, int input_size, int hidden_size,
                                        const double* W_t, const double* R_t, const double* b,
                                        const double* x_t, const double* h, const double* c,
                                        const double* c_new, const double* dh_new,
                                        const double* dc_new, double* dx, double* dW, double* dR,
                                        double* db, double* dh, double* dc, double* v,
                                        const double* zoneout_mask, void* stream) {
  (void)b;
  HASTE_HIP_REQUIRE(batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && c && c_new && dh_new && dc_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && db && dh && dc && v);
  return lstm_backward_steps<double>(as_stream(stream), 1, batch_size, input_size, hidden_size, W_t,
                                     R_t, x_t, h, c, c_new, dh_new, dc_new, dx, dW, dR, db, dh, dc, v,
                                     zoneout_mask);
}

int haste_hip_gru_forward_f64(int training, int steps, int batch_size, int input_size,
                              int hidden_size, const double* W, const double* R, const double* bx,
                              const double* br, const double* x, double* h, double* v,
                              double* tmp_Wx, double* tmp_Rh, float zoneout_prob,
                              const double* zoneout_mask, void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && tmp_Wx && (v || !training));
  const size_t NH = (size_t)batch_size * hidden_size;
  return gru_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                   hidden_size, W, R, bx, br, x, h, h + NH, v, tmp_Wx, zoneout_prob,
                                   zoneout_mask, nullptr, 1.f);
}

int haste_hip_gru_forward_dropconnect_f64(int training, int steps, int batch_size, int input_size,
                                          int hidden_size, const double* W, const double* R,
                                          const double* bx, const double* br, const double* x,
                                          double* h, double* v, double* tmp_Wx, float zoneout_prob,
                                          const double* zoneout_mask, const double* dropconnect_mask,
                                          float dropconnect_scale, void* stream) {
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && tmp_Wx && (v || !training));
  const size_t NH = (size_t)batch_size * hidden_size;
  return gru_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                   hidden_size, W, R, bx, br, x, h, h + NH, v, tmp_Wx, zoneout_prob,
                                   zoneout_mask, dropconnect_mask, dropconnect_scale);
}

int haste_hip_gru_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                               const double* W_t, const double* R_t, const double* bx,
                               const double* br, const double* x_t, const double* h, const double* v,
                               const double* dh_new, double* dx, double* dW, double* dR, double* dbx,
                               double* dbr, double* dh, double* dp, double* dq,
                               const double* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && v && dh_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && dbx && dbr && dh && dp && dq);
  const size_t NH = (size_t)batch_size * hidden_size;
  return gru_backward_steps<double>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                    W_t, R_t, x_t, h, v, dh_new + NH, dx, dW, dR, dbx, dbr, dh, dp, dq,
                                    zoneout_mask);
}

int haste_hip_gru_forward_iterate_f64(int training, int batch_size, int input_size, int hidden_size,
                                      const double* W, const double* R, const double* bx,
                                      const double* br, const double* x, const double* h,
                                      double* h_out, double* v, double* tmp_Wx, double* tmp_Rh,
                                      float zoneout_prob, const double* zoneout_mask, void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && h_out && tmp_Wx && (v || !training));
  return gru_forward_steps<double>(as_stream(stream), training, 1, batch_size, input_size,
                                   hidden_size, W, R, bx, br, x, h, h_out, v, tmp_Wx, zoneout_prob,
                                   zoneout_mask, nullptr, 1.f);
}

int haste_hip_gru_backward_iterate_f64(int batch_size, int input_size, int hidden_size,
                                       const double* W_t, const double* R_t, const double* bx,
                                       const double* br, const double* x_t, const double* h,
                                       const double* v, const double* dh_new, double* dx, double* dW,
                                       double* dR, double* dbx, double* dbr, double* dh, double* dp,
                                       double* dq, const double* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  HASTE_HIP_REQUIRE(batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && v && dh_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && dbx && dbr && dh && dp && dq);
  return gru_backward_steps<double>(as_stream(stream), 1, batch_size, input_size, hidden_size, W_t,
                                    R_t, x_t, h, v, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq,
                                    zoneout_mask);
}

int haste_hip_layer_norm_forward_f64(int rows, int dim, const double* gamma, const double* beta,
                                     const double* x, double* y, double* cache, void* stream) {
  HASTE_HIP_REQUIRE(rows > 0 && dim > 0 && gamma && x && y);
  ScopedKernelTimer timer("layer_norm_forward_f64", as_stream(stream));
  return ln_forward_rows<double>(as_stream(stream), (size_t)rows, dim, gamma, beta, x, y, cache);
}

int haste_hip_layer_norm_backward_f64(int rows, int dim, const double* gamma, const double* x,
                                      const double* dy, double* dx, double* dgamma, double* dbeta,
                                      const double* cache, void* stream_) {
  (void)cache;
  HASTE_HIP_REQUIRE(rows > 0 && dim > 0 && gamma && x && dy && dx && dgamma);
  hipStream_t stream = as_stream(stream_);
  const size_t part_bytes = column_sum_bytes<double>((size_t)rows, dim);
  Scratch sc;
  HASTE_HIP_PROPAGATE(open_scratch(stream, part_bytes + padded((size_t)rows * 2 * sizeof(double)), 0, &sc));
  void* partial = sc.take<char>(part_bytes);
  double* stats = sc.take<double>((size_t)rows * 2);
  ScopedKernelTimer timer("layer_norm_backward_f64", stream);
  HASTE_HIP_PROPAGATE(ln_forward_rows<double>(stream, (size_t)rows, dim, gamma, nullptr, x, nullptr, stats));
  return ln_backward_rows<double>(stream, (size_t)rows, dim, gamma, x, dy, dx, dgamma, dbeta, stats, partial);
}

int haste_hip_layer_norm_lstm_forward_f64(int training, int steps, int batch_size, int input_size,
                                          int hidden_size, const double* W, const double* R,
                                          const double* b, const double* x, double* h, double* c,
                                          double* act_Wx, double* tmp_Rh, const double* gamma1,
                                          double* cache1, double* act_Wx_norm, double* act_Rh,
                                          const double* gamma2, double* cache2, const double* gamma_h,
                                          const double* beta_h, double* cache3, double* act_c_norm,
                                          float zoneout_prob, const double* zoneout_mask,
                                          void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && b && x && h && c && act_Wx && gamma1 && act_Wx_norm && act_Rh);
  HASTE_HIP_REQUIRE(gamma2 && gamma_h && beta_h && act_c_norm);
  return ln_lstm_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                       hidden_size, W, R, b, x, h, c, act_Wx, gamma1, cache1,
                                       act_Wx_norm, act_Rh, gamma2, cache2, gamma_h, beta_h, cache3,
                                       act_c_norm, zoneout_prob, zoneout_mask);
}

int haste_hip_layer_norm_lstm_backward_f64(int steps, int batch_size, int input_size,
                                           int hidden_size, const double* W_t, const double* R_t,
                                           const double* b, const double* x_t, const double* h,
                                           const double* c, const double* dh_new,
                                           const double* dc_new, double* dx, double* dW, double* dR,
                                           double* db, double* dh, double* dc, double* act_Wx,
                                           const double* gamma1, double* dgamma1, double* act_Wx_norm,
                                           double* act_Rh, const double* gamma2, double* dgamma2,
                                           const double* cache2, const double* gamma_h,
                                           const double* beta_h, double* dgamma_h, double* dbeta_h,
                                           const double* cache3, double* act_c_norm,
                                           const double* zoneout_mask, void* stream) {
  (void)b;
  (void)beta_h;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && c && dh_new && dc_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && db && dh && dc && act_Wx && gamma1 && dgamma1);
  HASTE_HIP_REQUIRE(act_Wx_norm && act_Rh && gamma2 && dgamma2 && cache2 && gamma_h);
  HASTE_HIP_REQUIRE(dgamma_h && dbeta_h && cache3 && act_c_norm);
  return ln_lstm_backward_steps<double>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                        W_t, R_t, x_t, h, c, dh_new, dc_new, dx, dW, dR, db, dh, dc,
                                        act_Wx, gamma1, dgamma1, act_Wx_norm, act_Rh, gamma2, dgamma2,
                                        cache2, gamma_h, dgamma_h, dbeta_h, cache3, act_c_norm,
                                        zoneout_mask);
}

int haste_hip_layer_norm_gru_forward_f64(int training, int steps, int batch_size, int input_size,
                                         int hidden_size, const double* W, const double* R,
                                         const double* bx, const double* br, const double* x,
                                         double* h, double* v, double* act_Wx, const double* gamma1,
                                         double* cache1, double* tmp_Wx_norm, double* act_Rh,
                                         const double* gamma2, double* cache2, double* tmp_Rh_norm,
                                         float zoneout_prob, const double* zoneout_mask,
                                         void* stream) {
  (void)tmp_Rh_norm;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && act_Wx && gamma1 && tmp_Wx_norm && act_Rh && gamma2);
  HASTE_HIP_REQUIRE(v || !training);
  return ln_gru_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                      hidden_size, W, R, bx, br, x, h, v, act_Wx, gamma1, cache1,
                                      tmp_Wx_norm, act_Rh, gamma2, cache2, zoneout_prob, zoneout_mask);
}

int haste_hip_layer_norm_gru_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                                          const double* W_t, const double* R_t, const double* bx,
                                          const double* br, const double* x_t, const double* h,
                                          const double* v, const double* dh_new, double* dx,
                                          double* dW, double* dR, double* dbx, double* dbr, double* dh,
                                          double* dp, double* dq, const double* act_Wx,
                                          const double* gamma1, double* dgamma1, const double* act_Rh,
                                          const double* gamma2, double* dgamma2, const double* cache2,
                                          const double* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && v && dh_new && dx && dW && dR && dbx && dbr && dh);
  HASTE_HIP_REQUIRE(dp && dq && act_Wx && gamma1 && dgamma1 && act_Rh && gamma2 && dgamma2 && cache2);
  return ln_gru_backward_steps<double>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                       W_t, R_t, x_t, h, v, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq,
                                       act_Wx, gamma1, dgamma1, act_Rh, gamma2, dgamma2, cache2,
                                       zoneout_mask);
}

int haste_hip_indrnn_forward_f64(int training, int steps, int batch_size, int input_size,
                                 int hidden_size, const double* W, const double* u, const double* b,
                                 const double* x, double* h, double* workspace, float zoneout_prob,
                                 const double* zoneout_mask, void* stream) {
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && u && b && x && h && workspace);
  return indrnn_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                      hidden_size, W, u, b, x, h, workspace, nullptr, nullptr, nullptr,
                                      zoneout_prob, zoneout_mask);
}

int haste_hip_indrnn_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                                  const double* W_t, const double* u, const double* b,
                                  const double* x_t, const double* h, const double* dh_new,
                                  double* dx, double* dW, double* du, double* db, double* dh,
                                  double* workspace, const double* zoneout_mask, void* stream) {
  (void)b;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && u && x_t && h && dh_new && dx && dW && du && db && dh && workspace);
  return indrnn_backward_steps<double>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                       W_t, u, x_t, h, dh_new, dx, dW, du, db, dh, workspace, nullptr,
                                       nullptr, nullptr, zoneout_mask);
}

int haste_hip_layer_norm_indrnn_forward_f64(int training, int steps, int batch_size, int input_size,
                                            int hidden_size, const double* W, const double* u,
                                            const double* b, const double* x, double* h,
                                            double* workspace, double* act_Wx, const double* gamma1,
                                            double* cache1, float zoneout_prob,
                                            const double* zoneout_mask, void* stream) {
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && u && b && x && h && workspace && act_Wx && gamma1);
  return indrnn_forward_steps<double>(as_stream(stream), training, steps, batch_size, input_size,
                                      hidden_size, W, u, b, x, h, workspace, act_Wx, gamma1, cache1,
                                      zoneout_prob, zoneout_mask);
}

int haste_hip_layer_norm_indrnn_backward_f64(int steps, int batch_size, int input_size,
                                             int hidden_size, const double* W_t, const double* u,
                                             const double* b, const double* x_t, const double* h,
                                             const double* dh_new, double* dx, double* dW, double* du,
                                             double* db, double* dh, double* workspace,
                                             const double* act_Wx, const double* gamma1,
                                             double* dgamma1, const double* zoneout_mask,
                                             void* stream) {
  (void)b;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && u && x_t && h && dh_new && dx && dW && du && db && dh && workspace);
  HASTE_HIP_REQUIRE(act_Wx && gamma1 && dgamma1);
  return indrnn_backward_steps<double>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                       W_t, u, x_t, h, dh_new, dx, dW, du, db, dh, workspace, act_Wx,
                                       gamma1, dgamma1, zoneout_mask);
}

// ---- half (GRU only, as in the reference: lib/gru_forward_gpu.cu.cc:373,
// lib/gru_backward_gpu.cu.cc:411).  Tensors are IEEE binary16 passed as void*; products are
// accumulated and the pointwise math is done in float, results rounded to half.  Passes over
// more than one step run on the persistent fp32 kernels (gru_half.hip); a single step
// (Iterate) of at most 8 rows is one kernel (single_step.hip), of more rows it runs here, one
// product and one pointwise launch per side.
static inline const half_t* hp(const void* p) { return static_cast<const half_t*>(p); }
static inline half_t* hp(void* p) { return static_cast<half_t*>(p); }

int haste_hip_gru_forward_f16(int training, int steps, int batch_size, int input_size,
                              int hidden_size, const void* W, const void* R, const void* bx,
                              const void* br, const void* x, void* h, void* v, void* tmp_Wx,
                              void* tmp_Rh, float zoneout_prob, const void* zoneout_mask,
                              void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && tmp_Wx && (v || !training));
  const size_t NH = (size_t)batch_size * hidden_size;
  if (steps > 1)
    return gru_forward_half(as_stream(stream), training, steps, batch_size, input_size, hidden_size, W, R,
                            bx, br, x, h, v, zoneout_prob, zoneout_mask, nullptr, 1.f);
  if (single_step_applies(batch_size, input_size, hidden_size))
    return gru_forward_single_step_half(as_stream(stream), training, batch_size, input_size, hidden_size,
                                        W, R, bx, br, x, h, hp(h) + NH, v, zoneout_prob, zoneout_mask,
                                        nullptr, 1.f);
  return gru_forward_steps<half_t>(as_stream(stream), training, steps, batch_size, input_size,
                                   hidden_size, hp(W), hp(R), hp(bx), hp(br), hp(x), hp(h),
                                   hp(h) + NH, hp(v), hp(tmp_Wx), zoneout_prob, hp(zoneout_mask),
                                   nullptr, 1.f);
}

int haste_hip_gru_forward_dropconnect_f16(int training, int steps, int batch_size, int input_size,
                                          int hidden_size, const void* W, const void* R,
                                          const void* bx, const void* br, const void* x, void* h,
                                          void* v, void* tmp_Wx, float zoneout_prob,
                                          const void* zoneout_mask, const void* dropconnect_mask,
                                          float dropconnect_scale, void* stream) {
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && tmp_Wx && (v || !training));
  const size_t NH = (size_t)batch_size * hidden_size;
  if (steps > 1)
    return gru_forward_half(as_stream(stream), training, steps, batch_size, input_size, hidden_size, W, R,
                            bx, br, x, h, v, zoneout_prob, zoneout_mask, dropconnect_mask,
                            dropconnect_scale);
  if (single_step_applies(batch_size, input_size, hidden_size))
    return gru_forward_single_step_half(as_stream(stream), training, batch_size, input_size, hidden_size,
                                        W, R, bx, br, x, h, hp(h) + NH, v, zoneout_prob, zoneout_mask,
                                        dropconnect_mask, dropconnect_scale);
  return gru_forward_steps<half_t>(as_stream(stream), training, steps, batch_size, input_size,
                                   hidden_size, hp(W), hp(R), hp(bx), hp(br), hp(x), hp(h),
                                   hp(h) + NH, hp(v), hp(tmp_Wx), zoneout_prob, hp(zoneout_mask),
                                   hp(dropconnect_mask), dropconnect_scale);
}

int haste_hip_gru_backward_f16(int steps, int batch_size, int input_size, int hidden_size,
                               const void* W_t, const void* R_t, const void* bx, const void* br,
                               const void* x_t, const void* h, const void* v, const void* dh_new,
                               void* dx, void* dW, void* dR, void* dbx, void* dbr, void* dh, void* dp,
                               void* dq, const void* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  HASTE_HIP_REQUIRE(steps > 0 && batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && v && dh_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && dbx && dbr && dh && dp && dq);
  const size_t NH = (size_t)batch_size * hidden_size;
  if (steps > 1)
    return gru_backward_half(as_stream(stream), steps, batch_size, input_size, hidden_size, W_t, R_t, x_t,
                             h, v, hp(dh_new) + NH, dx, dW, dR, dbx, dbr, dh, dp, dq, zoneout_mask);
  return gru_backward_steps<half_t>(as_stream(stream), steps, batch_size, input_size, hidden_size,
                                    hp(W_t), hp(R_t), hp(x_t), hp(h), hp(v), hp(dh_new) + NH, hp(dx),
                                    hp(dW), hp(dR), hp(dbx), hp(dbr), hp(dh), hp(dp), hp(dq),
                                    hp(zoneout_mask));
}

int haste_hip_gru_forward_iterate_f16(int training, int batch_size, int input_size, int hidden_size,
                                      const void* W, const void* R, const void* bx, const void* br,
                                      const void* x, const void* h, void* h_out, void* v,
                                      void* tmp_Wx, void* tmp_Rh, float zoneout_prob,
                                      const void* zoneout_mask, void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && h_out && tmp_Wx && (v || !training));
  if (single_step_applies(batch_size, input_size, hidden_size))
    return gru_forward_single_step_half(as_stream(stream), training, batch_size, input_size, hidden_size,
                                        W, R, bx, br, x, h, h_out, v, zoneout_prob, zoneout_mask, nullptr,
                                        1.f);
  return gru_forward_steps<half_t>(as_stream(stream), training, 1, batch_size, input_size,
                                   hidden_size, hp(W), hp(R), hp(bx), hp(br), hp(x), hp(h), hp(h_out),
                                   hp(v), hp(tmp_Wx), zoneout_prob, hp(zoneout_mask), nullptr, 1.f);
}

int haste_hip_gru_backward_iterate_f16(int batch_size, int input_size, int hidden_size,
                                       const void* W_t, const void* R_t, const void* bx,
                                       const void* br, const void* x_t, const void* h, const void* v,
                                       const void* dh_new, void* dx, void* dW, void* dR, void* dbx,
                                       void* dbr, void* dh, void* dp, void* dq,
                                       const void* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  HASTE_HIP_REQUIRE(batch_size > 0 && input_size > 0 && hidden_size > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && v && dh_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && dbx && dbr && dh && dp && dq);
  return gru_backward_steps<half_t>(as_stream(stream), 1, batch_size, input_size, hidden_size,
                                    hp(W_t), hp(R_t), hp(x_t), hp(h), hp(v), hp(dh_new), hp(dx),
                                    hp(dW), hp(dR), hp(dbx), hp(dbr), hp(dh), hp(dp), hp(dq),
                                    hp(zoneout_mask));
}

}  // extern "C"
