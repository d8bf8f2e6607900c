// IndRNN and LayerNormIndRNN forward and backward passes.
//
// The recurrence h_{t+1} = tanh((xW)_t + u*h_t + b) is elementwise, so there is no
// exchange between threads: one thread owns one (batch row, hidden unit) pair and
// walks all T steps.  Each thread keeps a block of U future steps' operands in flight
// while it computes the current block; what remains is the dependent chain of the steps.  Consecutive lanes own consecutive hidden units (coalesced 256-byte rows).
//
// Arithmetic follows reference lib/indrnn_forward_gpu.cu.cc:44-62 and
// lib/indrnn_backward_gpu.cu.cc:46-73; orchestration replaces :114-210 and :122-207
// (and lib/layer_norm_indrnn_{forward,backward}_gpu.cu.cc:114-213 / 122-209).
#include "recurrent.h"

namespace haste_hip {
namespace {

// Steps of operands kept in flight per thread (twice that while the next batch is requested).
// 16 is 5-14 % faster than 8 (N*H = 8192 .. 131072 chains); 32 no better, nor are two or three
// batches in flight beyond the current one: the time is the dependent chain of a step, not the
// loads.  Whole batches run without a bounds check per step (17 % faster: the check is a scalar
// compare and a branch in every step of the chain); requests beyond the sequence read its last
// step again and are never used.
constexpr int U = 16;

template <bool TRAINING, bool ZONEOUT>
__global__ __launch_bounds__(256)
void indrnn_forward_kernel(int T, int N, int H, const float* __restrict__ Wx,
                           const float* __restrict__ u, const float* __restrict__ b,
                           float* __restrict__ h, float zoneout_prob,
                           const float* __restrict__ mask) {
  const int j = blockIdx.x * 64 + (threadIdx.x & 63);
  const int n = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (j >= H || n >= N) return;
  const size_t NH = (size_t)N * H;
  const size_t idx = (size_t)n * H + j;
  const float uj = u[j], bj = b[j];
  float hv = h[idx];

  float wx_cur[U], mk_cur[U], wx_nxt[U], mk_nxt[U];
  auto fetch = [&](int t0, float (&wx)[U], float (&mk)[U]) {
#pragma unroll
    for (int i = 0; i < U; ++i) {
      const int t = t0 + i < T ? t0 + i : T - 1;
      wx[i] = Wx[(size_t)t * NH + idx];
      mk[i] = (ZONEOUT && TRAINING) ? mask[(size_t)t * NH + idx] : 1.f;
    }
  };
  auto step = [&](int t, float wx, float mk) {
    float hn = tanh_f(wx + uj * hv + bj);
    if (ZONEOUT) {
      if (TRAINING) hn = (hn - hv) * mk + hv;
      else hn = zoneout_prob * hv + (1.0f - zoneout_prob) * hn;
    }
    h[(size_t)(t + 1) * NH + idx] = hn;
    hv = hn;
  };
  fetch(0, wx_cur, mk_cur);
  int t0 = 0;
  for (; t0 + U <= T; t0 += U) {
    fetch(t0 + U, wx_nxt, mk_nxt);
#pragma unroll
    for (int i = 0; i < U; ++i) step(t0 + i, wx_cur[i], mk_cur[i]);
#pragma unroll
    for (int i = 0; i < U; ++i) { wx_cur[i] = wx_nxt[i]; mk_cur[i] = mk_nxt[i]; }
  }
  // the last, partial batch
#pragma unroll
  for (int i = 0; i < U; ++i)
    if (t0 + i < T) step(t0 + i, wx_cur[i], mk_cur[i]);
}

// Walks the steps backwards; h[t+1] of a step is h[t] of the step before it in the walk, so
// every state is loaded once.
template <bool ZONEOUT>
__global__ __launch_bounds__(256)
void indrnn_backward_kernel(int T, int N, int H, const float* __restrict__ u,
                            const float* __restrict__ h, const float* __restrict__ dh_new,
                            float* __restrict__ dh, float* __restrict__ dk,
                            const float* __restrict__ mask, float* __restrict__ partial) {
  __shared__ float red[2][4][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int j = blockIdx.x * 64 + lane;
  const int n = blockIdx.y * 4 + w;
  const bool live = j < H && n < N;
  const size_t NH = (size_t)N * H;
  const size_t idx = live ? (size_t)n * H + j : 0;
  float du_sum = 0.f, db_sum = 0.f;

  if (live) {
    const float uj = u[j];
    float dh_io = dh[idx];
    float hn = h[(size_t)T * NH + idx];

    struct In { float hp, d, m; };
    In cur[U], nxt[U];
    auto fetch = [&](int t_hi, In (&s)[U]) {
#pragma unroll
      for (int i = 0; i < U; ++i) {
        const int t = t_hi - i > 0 ? t_hi - i : 0;
        s[i].hp = h[(size_t)t * NH + idx];
        s[i].d = dh_new[(size_t)(t + 1) * NH + idx];
        s[i].m = ZONEOUT ? mask[(size_t)t * NH + idx] : 1.f;
      }
    };
    auto step = [&](int t, const In& in) {
      float dh_total = in.d + dh_io;
      float keep = 0.f;
      if (ZONEOUT) {
        keep = (1.0f - in.m) * dh_total;
        dh_total = in.m * dh_total;
      }
      const float k = d_tanh_f(hn) * dh_total;
      dk[(size_t)t * NH + idx] = k;
      dh_io = keep + uj * k;
      du_sum += in.hp * k;
      db_sum += k;
      hn = in.hp;
    };
    fetch(T - 1, cur);
    int t_hi = T - 1;
    for (; t_hi - U + 1 >= 0; t_hi -= U) {
      fetch(t_hi - U, nxt);
#pragma unroll
      for (int i = 0; i < U; ++i) step(t_hi - i, cur[i]);
#pragma unroll
      for (int i = 0; i < U; ++i) cur[i] = nxt[i];
    }
    // the last, partial batch
#pragma unroll
    for (int i = 0; i < U; ++i)
      if (t_hi - i >= 0) step(t_hi - i, cur[i]);
    dh[idx] = dh_io;
  }

  // Column sums over the batch: 4 rows per workgroup in LDS, then workgroups in order.
  red[0][w][lane] = du_sum;
  red[1][w][lane] = db_sum;
  __syncthreads();
  if (threadIdx.x < 128) {
    const int which = threadIdx.x >> 6;
    const float s = (red[which][0][lane] + red[which][1][lane]) + (red[which][2][lane] + red[which][3][lane]);
    if (j < H) partial[((size_t)blockIdx.y * 2 + which) * H + j] = s;
  }
}

int run_forward_recurrence(hipStream_t stream, int training, int T, int N, int H, const float* Wx,
                           const float* u, const float* b, float* h, float zoneout_prob,
                           const float* mask) {
  const bool zoneout = zoneout_prob != 0.f && mask != nullptr;
  dim3 grid((H + 63) / 64, (N + 3) / 4), block(256);
  ScopedKernelTimer timer("indrnn_forward_recurrence", stream);
  if (training && zoneout)
    indrnn_forward_kernel<true, true><<<grid, block, 0, stream>>>(T, N, H, Wx, u, b, h, zoneout_prob, mask);
  else if (training)
    indrnn_forward_kernel<true, false><<<grid, block, 0, stream>>>(T, N, H, Wx, u, b, h, 0.f, nullptr);
  else if (zoneout)
    indrnn_forward_kernel<false, true><<<grid, block, 0, stream>>>(T, N, H, Wx, u, b, h, zoneout_prob, mask);
  else
    indrnn_forward_kernel<false, false><<<grid, block, 0, stream>>>(T, N, H, Wx, u, b, h, 0.f, nullptr);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

int run_backward_recurrence(hipStream_t stream, int T, int N, int H, const float* u, const float* h,
                            const float* dh_new, float* du, float* db, float* dh, float* dk,
                            const float* mask) {
  dim3 grid((H + 63) / 64, (N + 3) / 4), block(256);
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, (size_t)grid.y * 2 * H * sizeof(float), &ws));
  ScopedKernelTimer timer("indrnn_backward_recurrence", stream);
  if (mask != nullptr)
    indrnn_backward_kernel<true><<<grid, block, 0, stream>>>(T, N, H, u, h, dh_new, dh, dk, mask, ws.scratch);
  else
    indrnn_backward_kernel<false><<<grid, block, 0, stream>>>(T, N, H, u, h, dh_new, dh, dk, nullptr, ws.scratch);
  HASTE_HIP_TRY(hipGetLastError());
  // du, db += the workgroups' column sums, in workgroup order
  HASTE_HIP_PROPAGATE(add_column_partials(stream, (int)grid.y, H, ws.scratch, du, db));
  return HASTE_HIP_OK;
}

}  // namespace
}  // namespace haste_hip

extern "C" {

using namespace haste_hip;

int haste_hip_indrnn_forward_f32(int training, int steps, int batch_size, int input_size,
                                 int hidden_size,
                                 const float* W, const float* u, const float* b, const float* x,
                                 float* h, float* workspace,
                                 float zoneout_prob, const float* zoneout_mask, void* stream) {
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W && u && b && x && h && workspace);
  hipStream_t s = as_stream(stream);
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, T * N, H, C, x, C, W, H, workspace, H, false));
  return run_forward_recurrence(s, training, T, N, H, workspace, u, b, h, zoneout_prob, zoneout_mask);
}

int haste_hip_indrnn_backward_f32(int steps, int batch_size, int input_size, int hidden_size,
                                  const float* W_t, const float* u, const float* b,
                                  const float* x_t, const float* h, const float* dh_new,
                                  float* dx, float* dW, float* du, float* db, float* dh,
                                  float* workspace, const float* zoneout_mask, void* stream) {
  (void)b;
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W_t && u && x_t && h && dh_new && dx && dW && du && db && dh && workspace);
  hipStream_t s = as_stream(stream);
  HASTE_HIP_PROPAGATE(run_backward_recurrence(s, T, N, H, u, h, dh_new, du, db, dh, workspace,
                                              zoneout_mask));
  // dW = x^T dk (assigned, as in the reference); dx = dk W^T.
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, C, H, T * N, x_t, T * N, workspace, H, dW, H, false));
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, T * N, C, H, workspace, H, W_t, C, dx, C, false));
  return HASTE_HIP_OK;
}

int haste_hip_layer_norm_indrnn_forward_f32(int training, int steps, int batch_size,
                                            int input_size, int hidden_size,
                                            const float* W, const float* u, const float* b,
                                            const float* x, float* h, float* workspace,
                                            float* act_Wx, const float* gamma1, float* cache1,
                                            float zoneout_prob, const float* zoneout_mask,
                                            void* stream) {
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W && u && b && x && h && workspace && act_Wx && gamma1);
  hipStream_t s = as_stream(stream);
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, T * N, H, C, x, C, W, H, act_Wx, H, false));
  HASTE_HIP_PROPAGATE(layer_norm_forward(s, T * N, H, gamma1, nullptr, act_Wx, workspace, cache1));
  return run_forward_recurrence(s, training, T, N, H, workspace, u, b, h, zoneout_prob, zoneout_mask);
}

int haste_hip_layer_norm_indrnn_backward_f32(int steps, int batch_size, int input_size,
                                             int hidden_size,
                                             const float* W_t, const float* u, const float* b,
                                             const float* x_t, const float* h,
                                             const float* dh_new,
                                             float* dx, float* dW, float* du, float* db, float* dh,
                                             float* workspace,
                                             const float* act_Wx, const float* gamma1,
                                             float* dgamma1,
                                             const float* zoneout_mask, void* stream) {
  (void)b;
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W_t && u && x_t && h && dh_new && dx && dW && du && db && dh && workspace);
  HASTE_HIP_REQUIRE(act_Wx && gamma1 && dgamma1);
  hipStream_t s = as_stream(stream);
  HASTE_HIP_PROPAGATE(run_backward_recurrence(s, T, N, H, u, h, dh_new, du, db, dh, workspace,
                                              zoneout_mask));
  HASTE_HIP_PROPAGATE(layer_norm_backward(s, T * N, H, gamma1, act_Wx, workspace, workspace,
                                          dgamma1, nullptr));
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, C, H, T * N, x_t, T * N, workspace, H, dW, H, false));
  HASTE_HIP_PROPAGATE(gemm_f32(s, false, T * N, C, H, workspace, H, W_t, C, dx, C, false));
  return HASTE_HIP_OK;
}

}  // extern "C"
