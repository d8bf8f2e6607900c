// One time step of an LSTM or GRU forward pass for a small batch, as one kernel: what
// ForwardPass::Iterate (reference lib/haste/lstm.h:73-86, lib/haste/gru.h:72-84) is called for
// in autoregressive decoding.  The all-steps kernels keep a slice of R on chip for a whole
// sequence; for a single step there is nothing to keep -- every weight is used once -- and
// their set-up (roles, exchange tiles, the slice, a group barrier) and the separate x * W
// launch cost more than the step.  Here [x_t | h] (length C + H) is multiplied with the stacked
// [W; R] straight from memory: a workgroup takes 16 hidden units (all their gate columns) and
// a run of the contraction, parks its partial sums, and the last workgroup of a column block
// to finish adds the runs in index order and does the pointwise step (gates, cell update,
// zoneout) -- one launch, no float atomics, results independent of timing.  The GRU's half
// entry points use the same kernel on half tensors (sums and pointwise step in float).
//
// Arithmetic: reference lib/lstm_forward_gpu.cu.cc:55-86, lib/gru_forward_gpu.cu.cc:46-84.
#include "recurrent.h"

namespace haste_hip {
namespace {

constexpr int kStepUnits = 16;      // hidden units per workgroup
constexpr int kStepMaxRun = 512;    // contraction indices per workgroup and side

typedef _Float16 half_t;

// T: the caller's tensors (float, or half with the sums and the pointwise step in float).
template <typename T>
struct StepParams {
  int training, N, C, H;
  const T* W;            // [C, G*H]
  const T* R;            // [H, G*H]
  const T* b;            // LSTM: [4H]; GRU: bx [3H]
  const T* br;           // GRU: [3H]
  const T* x;            // [N, C]
  const T* h;            // [N, H]
  const T* c;            // LSTM: [N, H]
  T* h_out;              // [N, H]
  T* c_out;              // LSTM: [N, H]
  T* v;                  // [N, 4H] (training; GRU: always when non-null)
  float zoneout_prob;
  const T* zoneout_mask;      // [N, H] or null
  const T* dc_mask;           // DropConnect mask of R or null
  float dc_scale;
  float* h_stage;        // [N, H] when h_out overlaps h (state updated in place), else null
  float* partial;        // [runs][2 sides][NB][column blocks * 64]; unused with one run
  ControlBlock* cb;
};

// Unit j = 16 cw + u of row n: its pre-activations from x * W (wx) and h * R (rh), then the
// pointwise step.
template <int GATES, typename T>
__device__ __forceinline__ void finish_unit(const StepParams<T>& p, int n, int j, const float (&wx)[GATES],
                                            const float (&rh)[GATES]) {
  const int H = p.H;
  const size_t e = (size_t)n * H + j;
  const float h_old = (float)p.h[e];
  const bool zoneout = p.zoneout_prob != 0.f && p.zoneout_mask != nullptr;
  float h_new;
  if constexpr (GATES == 4) {
    float a[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) a[g] = wx[g] + rh[g] + (float)p.b[g * H + j];
    const float gi = sigmoid_f(a[0]), gg = tanh_f(a[1]), gf = sigmoid_f(a[2]), go = sigmoid_f(a[3]);
    const float c_new = gf * (float)p.c[e] + gi * gg;
    h_new = go * tanh_f(c_new);
    p.c_out[e] = (T)c_new;
    if (p.training) {
      T* vt = p.v + (size_t)n * 4 * H + j;
      vt[0] = (T)gi; vt[H] = (T)gg; vt[2 * H] = (T)gf; vt[3 * H] = (T)go;
    }
  } else {
    const float z = sigmoid_f(wx[0] + rh[0] + (float)p.b[j] + (float)p.br[j]);
    const float r = sigmoid_f(wx[1] + rh[1] + (float)p.b[H + j] + (float)p.br[H + j]);
    const float qg = rh[2] + (float)p.br[2 * H + j];
    const float g = tanh_f(wx[2] + r * qg + (float)p.b[2 * H + j]);
    h_new = z * h_old + (1.0f - z) * g;
    if (p.training && p.v != nullptr) {
      T* vt = p.v + (size_t)n * 4 * H + j;
      vt[0] = (T)z; vt[H] = (T)r; vt[2 * H] = (T)g; vt[3 * H] = (T)qg;
    }
  }
  if (zoneout) {
    if (p.training) h_new = (h_new - h_old) * (float)p.zoneout_mask[e] + h_old;
    else h_new = p.zoneout_prob * h_old + (1.0f - p.zoneout_prob) * h_new;
  }
  if (p.h_stage == nullptr) p.h_out[e] = (T)h_new;
  else store_agent(&p.h_stage[e], h_new);
}

// h_out overlaps h: other workgroups may still be reading h when a column block is finished,
// so the new state is parked and copied out by the last column block to finish, when every
// run of every block has been read.  Called by the finishing workgroups, all threads.
template <typename T>
__device__ __forceinline__ void copy_staged_state(const StepParams<T>& p, unsigned int* flag) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned int old = __hip_atomic_fetch_add(&p.cb->grid_exit_counter[0], 1u, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
    const bool last = old == gridDim.x - 1;
    if (last)
      __hip_atomic_store(&p.cb->grid_exit_counter[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last ? 1u : 0u;
  }
  __syncthreads();
  if (*flag == 0u) return;
  const int count = p.N * p.H;
  for (int i = threadIdx.x; i < count; i += 256) p.h_out[i] = (T)load_exchanged(&p.h_stage[i]);
}

// GATES = 4: LSTM (i, g, f, o); GATES = 3: GRU (z, r, g).  NB: batch rows (N <= NB).
// Workgroup (cw, run): columns of units 16 cw .. 16 cw + 15, run `run` of gridDim.y of the rows
// of W and of the rows of R.  With a single run the workgroup finishes its units itself,
// straight from LDS.
template <int GATES, int NB, typename T>
__global__ __launch_bounds__(256)
void forward_step_kernel(StepParams<T> p) {
  constexpr int COLS = 64;  // 16 units x up to 4 gates (a GRU leaves the last 16 idle)
  extern __shared__ float s_dyn[];
  __shared__ float s_red[2][4][NB][COLS];
  __shared__ unsigned int s_flag;
  const int tid = threadIdx.x, col = tid & 63, q = tid >> 6;
  const int cw = blockIdx.x, run = blockIdx.y, runs = gridDim.y;
  const int N = p.N, H = p.H, GH = GATES * H;
  const int gate = col / kStepUnits, unit = cw * kStepUnits + col % kStepUnits;
  const bool col_ok = gate < GATES && unit < H;
  const size_t col_off = (size_t)gate * H + unit;

  const int len[2] = {p.C, H};
  int per_run[2], kb[2], ke[2];
#pragma unroll
  for (int side = 0; side < 2; ++side) {
    per_run[side] = ((len[side] + runs - 1) / runs + 3) / 4 * 4;
    kb[side] = run * per_run[side];
    ke[side] = kb[side] + per_run[side] < len[side] ? kb[side] + per_run[side] : len[side];
  }
  float* s_in[2] = {s_dyn, s_dyn + NB * per_run[0]};

  // Row k of side `side` (0: W, 1: R under DropConnect), this thread's column; rows beyond the
  // run read row kb and are not used.
  auto weight = [&](int side, int k) {
    const T* M = side == 0 ? p.W : p.R;
    const bool any = kb[side] < ke[side] && col_ok;
    const size_t at = (size_t)(k < ke[side] ? k : kb[side]) * GH + col_off;
    float w = any ? (float)M[at] : 0.f;
    if (side == 1 && p.dc_mask != nullptr && any) w = w * (float)p.dc_mask[at] * p.dc_scale;
    return w;
  };
  // The first eight rows of each side are requested before anything waits for the inputs.
  float w0[2][8];
#pragma unroll
  for (int side = 0; side < 2; ++side)
#pragma unroll
    for (int u = 0; u < 8; ++u) w0[side][u] = weight(side, kb[side] + q + 4 * u);

#pragma unroll
  for (int side = 0; side < 2; ++side) {
    const T* in = side == 0 ? p.x : p.h;
    for (int i = tid; i < NB * per_run[side]; i += 256) {
      const int n = i / per_run[side], k = kb[side] + i % per_run[side];
      s_in[side][i] = (n < N && k < ke[side]) ? (float)in[(size_t)n * len[side] + k] : 0.f;
    }
  }
  __syncthreads();

#pragma unroll
  for (int side = 0; side < 2; ++side) {
    float acc[NB];
#pragma unroll
    for (int n = 0; n < NB; ++n) acc[n] = 0.f;
    const float* sin = s_in[side];
    const int pr = per_run[side], b0 = kb[side], e0 = ke[side];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int k = b0 + q + 4 * u;
      if (k < e0) {  // the same for a whole wavefront
#pragma unroll
        for (int n = 0; n < NB; ++n) acc[n] = fmaf(w0[side][u], sin[n * pr + k - b0], acc[n]);
      }
    }
    // the rest of the run, eight rows in flight per thread
    for (int k0 = b0 + q + 32; k0 < e0; k0 += 32) {
      float w[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) w[u] = weight(side, k0 + 4 * u);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int k = k0 + 4 * u;
        if (k < e0) {
#pragma unroll
          for (int n = 0; n < NB; ++n) acc[n] = fmaf(w[u], sin[n * pr + k - b0], acc[n]);
        }
      }
    }
#pragma unroll
    for (int n = 0; n < NB; ++n) s_red[side][q][n][col] = acc[n];
  }
  __syncthreads();
  auto quarter_sum = [&](int side, int n, int cc) {
    return (s_red[side][0][n][cc] + s_red[side][1][n][cc]) + (s_red[side][2][n][cc] + s_red[side][3][n][cc]);
  };
  const int n = tid / kStepUnits, u = tid % kStepUnits;
  const int j = cw * kStepUnits + u;
  const bool mine = n < N && j < H;  // thread (n, u) finishes unit u of row n
  float wx[GATES], rh[GATES];

  if (runs == 1) {
    if (mine) {
#pragma unroll
      for (int g = 0; g < GATES; ++g) {
        wx[g] = quarter_sum(0, n, g * kStepUnits + u);
        rh[g] = quarter_sum(1, n, g * kStepUnits + u);
      }
      finish_unit<GATES, T>(p, n, j, wx, rh);
    }
    if (p.h_stage != nullptr) copy_staged_state(p, &s_flag);
    return;
  }

  // Several runs: park this one's sums; the last workgroup of the column block to arrive adds
  // the runs in index order (eight runs and all gates in flight per round trip).
  const int slots = gridDim.x * COLS;
  for (int i = tid; i < 2 * NB * COLS; i += 256) {
    const int side = i / (NB * COLS), nn = (i / COLS) % NB, cc = i % COLS;
    store_agent(&p.partial[(((size_t)run * 2 + side) * NB + nn) * slots + cw * COLS + cc], quarter_sum(side, nn, cc));
  }
  if (!column_last_arrival(p.cb, cw, runs, &s_flag)) return;
  if (mine) {
#pragma unroll
    for (int g = 0; g < GATES; ++g) wx[g] = rh[g] = 0.f;
    const size_t side_stride = (size_t)NB * slots, run_stride = 2 * side_stride;
    const float* first = p.partial + (size_t)n * slots + cw * COLS + u;
    for (int r0 = 0; r0 < runs; r0 += 8) {
      float part[2][GATES][8];
#pragma unroll
      for (int side = 0; side < 2; ++side)
#pragma unroll
        for (int g = 0; g < GATES; ++g)
#pragma unroll
          for (int i = 0; i < 8; ++i)
            part[side][g][i] = r0 + i < runs ? load_exchanged(first + (size_t)(r0 + i) * run_stride +
                                                              side * side_stride + g * kStepUnits)
                                             : 0.f;
#pragma unroll
      for (int g = 0; g < GATES; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          wx[g] += part[0][g][i];
          rh[g] += part[1][g][i];
        }
    }
    finish_unit<GATES, T>(p, n, j, wx, rh);
  }
  if (p.h_stage != nullptr) copy_staged_state(p, &s_flag);
}

template <int GATES, typename T>
int launch_step(hipStream_t stream, StepParams<T>& p, const char* name) {
  const int gx = (p.H + kStepUnits - 1) / kStepUnits;
  // Runs of the contraction: enough workgroups for about two per CU, at most 64 runs, a run
  // keeping at least 32 rows of the longer side.  The step is bound by memory latency, not
  // bandwidth -- a thread has 8 to 16 loads of 4 bytes in flight -- so many small workgroups
  // beat few large ones although their sums then meet in memory: at N = 1, C = H = 512 one run
  // (32 workgroups streaming 256 KiB each, no second phase) takes 22 us, 16 runs 7 us.
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const int longest = p.C > p.H ? p.C : p.H;
  int runs = (2 * cus + gx - 1) / gx;
  if (runs > 64) runs = 64;
  const int most = (longest + 31) / 32;
  if (runs > most) runs = most;
  if (runs < 1) runs = 1;
  const int least = (longest + kStepMaxRun - 1) / kStepMaxRun;
  if (runs < least) runs = least;
  const int nb = p.N <= 1 ? 1 : (p.N <= 2 ? 2 : (p.N <= 4 ? 4 : 8));
  const size_t partial_bytes = runs > 1 ? (size_t)runs * 2 * nb * gx * 64 * sizeof(float) : 0;
  const size_t state_floats = (size_t)p.N * p.H;
  const bool in_place = p.h_out < p.h + state_floats && p.h < p.h_out + state_floats;
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, partial_bytes + (in_place ? state_floats * sizeof(float) : 0) + 256, &ws));
  p.partial = ws.scratch;
  p.h_stage = in_place ? ws.scratch + partial_bytes / sizeof(float) : nullptr;
  p.cb = ws.control;
  const dim3 grid((unsigned)gx, (unsigned)runs);
  auto padded_run = [&](int len) { return ((len + runs - 1) / runs + 3) / 4 * 4; };
  const size_t lds = (size_t)nb * (padded_run(p.C) + padded_run(p.H)) * sizeof(float);
  ScopedKernelTimer timer(name, stream);
  if (nb == 1) forward_step_kernel<GATES, 1, T><<<grid, dim3(256), lds, stream>>>(p);
  else if (nb == 2) forward_step_kernel<GATES, 2, T><<<grid, dim3(256), lds, stream>>>(p);
  else if (nb == 4) forward_step_kernel<GATES, 4, T><<<grid, dim3(256), lds, stream>>>(p);
  else forward_step_kernel<GATES, 8, T><<<grid, dim3(256), lds, stream>>>(p);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

}  // namespace

bool single_step_applies(int N, int C, int H) {
  // per-run staging in LDS and the tile counters of the control block bound the sizes
  // the tile counters of the control block and the 64 runs of at most kStepMaxRun bound the sizes
  return N <= 8 && (H + kStepUnits - 1) / kStepUnits <= 4096 && C <= 64 * kStepMaxRun && H <= 64 * kStepMaxRun;
}

int lstm_forward_single_step(hipStream_t stream, int training, int N, int C, int H, const float* W,
                             const float* R, const float* b, const float* x, const float* h,
                             const float* c, float* h_out, float* c_out, float* v,
                             float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                             float dc_scale) {
  StepParams<float> p = {};
  p.training = training; p.N = N; p.C = C; p.H = H;
  p.W = W; p.R = R; p.b = b; p.x = x; p.h = h; p.c = c;
  p.h_out = h_out; p.c_out = c_out; p.v = v;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.dc_mask = dc_mask; p.dc_scale = dc_scale;
  return launch_step<4>(stream, p, "lstm_forward_step");
}

int gru_forward_single_step(hipStream_t stream, int training, int N, int C, int H, const float* W,
                            const float* R, const float* bx, const float* br, const float* x,
                            const float* h, float* h_out, float* v, float zoneout_prob,
                            const float* zoneout_mask, const float* dc_mask, float dc_scale) {
  StepParams<float> p = {};
  p.training = training; p.N = N; p.C = C; p.H = H;
  p.W = W; p.R = R; p.b = bx; p.br = br; p.x = x; p.h = h;
  p.h_out = h_out; p.v = v;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.dc_mask = dc_mask; p.dc_scale = dc_scale;
  return launch_step<3>(stream, p, "gru_forward_step");
}

int gru_forward_single_step_half(hipStream_t stream, int training, int N, int C, int H, const void* W,
                                 const void* R, const void* bx, const void* br, const void* x,
                                 const void* h, void* h_out, void* v, float zoneout_prob,
                                 const void* zoneout_mask, const void* dc_mask, float dc_scale) {
  auto in = [](const void* q) { return static_cast<const half_t*>(q); };
  StepParams<half_t> p = {};
  p.training = training; p.N = N; p.C = C; p.H = H;
  p.W = in(W); p.R = in(R); p.b = in(bx); p.br = in(br); p.x = in(x); p.h = in(h);
  p.h_out = static_cast<half_t*>(h_out); p.v = static_cast<half_t*>(v);
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = in(zoneout_mask);
  p.dc_mask = in(dc_mask); p.dc_scale = dc_scale;
  return launch_step<3>(stream, p, "gru_forward_step_half");
}

}  // namespace haste_hip
