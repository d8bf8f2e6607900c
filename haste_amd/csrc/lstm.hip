// LSTM forward and backward passes: one MFMA GEMM for the time-fused input
// projection, one persistent kernel for the T-step recurrence (gate nonlinearities,
// cell update, zoneout and optional DropConnect fused in), and for the backward pass
// one persistent reverse-time kernel followed by the three batched GEMMs.
//
// Arithmetic follows reference lib/lstm_forward_gpu.cu.cc:55-86 and
// lib/lstm_backward_gpu.cu.cc:47-95; orchestration replaces :313-366 and :319-405.
#include "scatter_backward.h"

namespace haste_hip {
namespace {

struct LstmFwdParams {
  int training, T, N, H;
  const float* R;       // [H,4H]
  const float* b;       // [4H]
  const float* h;       // [N,H] state before the first step
  const float* c;       // [N,H]
  float* h_out;         // [T,N,H] states after each step (may start at h + N*H)
  float* c_out;         // [T,N,H]
  float* v;             // [T,N,4H] in: x*W, out (training): activations
  float zoneout_prob;
  const float* zoneout_mask;   // [T,N,H] or null
  const float* dc_mask;        // DropConnect mask [H,4H] or null
  float dc_scale;
  float* xh;                   // polled exchange tiles of h: [batch tiles][4][Kpad/4][NB][4]
  // kernels that compute the input projection themselves (XSG > 0): v does not hold x*W
  const float* x;              // [T,N,C]
  const float* W;              // [C,4H]
  int C;
  LaunchShape ls;
};

// HS hidden units per workgroup = 4*CT (their 4 gate columns fill CT MFMA column tiles).
// SETS sets of 256 threads, each with a batch tile of NB rows of its own.  Two sets share
// the resident slice but nothing else: while one waits for its exchange the other computes,
// which a single tile of 2*NB rows cannot do.
// XSG > 0 (4-row tiles): the kernel also computes the input projection x[t] * W, on the matrix
// units while its wavefronts wait for h[t] (InputProjection in recurrent.h; a wavefront takes
// XSG super-groups of 64 input features), instead of reading it from v.
// REG > 0 (tiles of 16 rows and more): the slice exceeds LDS; every wavefront keeps the first REG
// k-groups of its share of the contraction in registers (tall_tile_product).
template <int NB, int CT, int SETS, int XSG = 0, int REG = 0>
__global__ __launch_bounds__(256 * SETS, 1)
void lstm_forward_kernel(LstmFwdParams p) {
  static_assert(SETS == 1 || (SETS == 2 && NB < 16), "two sets: short tiles only");
  static_assert(XSG == 0 || NB == 4, "fused input projection: 4-row tiles only");
  static_assert(REG == 0 || (NB >= 16 && SETS == 1), "register-resident slice rows: tall tiles only");
  constexpr bool kFusedInput = XSG > 0;
  constexpr int HS = 4 * CT;
  constexpr int NCOLS = 16 * CT;
  constexpr int PP = (NB * HS + 255) / 256;
  constexpr int RED = ProductTile<NB, CT>::kRedFloats;
  constexpr bool kPolledPartials = SETS == 2;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int H = p.H, N = p.N, T = p.T;
  const int Kpad = round_up(H, 64);
  const int set = set_index<SETS>();
  float* w_lds = lds;
  // one set: one area of partial tiles behind workgroup barriers; two sets: two polled
  // areas each, alternating by step
  float* red = lds + (Kpad - 64 * REG) * NCOLS + (SETS == 1 ? 0 : set * 2 * RED);
  // The role is handed round through a word of the partial-tile area, which nothing else
  // uses before the first step: the kernel has no static LDS, so that a slice and its
  // partial tiles may fill the workgroup's 160 KiB exactly (N = 128, H = 1024).
  const Role role = take_role(p.ls, reinterpret_cast<unsigned int*>(lds + (Kpad - 64 * REG) * NCOLS));
  if (!role.active) return;

  const int tid = set_thread<SETS>();
  const int j0 = role.cw * HS;
  const int n0 = (role.bt * SETS + set) * NB;
  const int rows_here = (N - n0) < NB ? (N - n0) : NB;  // <= 0: a set without rows
  const size_t NH = (size_t)N * H;

  const int tile_floats = Kpad * NB;
  float* xh = p.xh + (size_t)(role.bt * SETS + set) * kPolledTiles * tile_floats;

  const TileBuffer xhb = make_tile_buffer(xh, kPolledTiles * tile_floats);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);

  // Own k range of the exchange tiles (the last workgroup also owns the padding): rows and
  // k beyond the problem stay zero for the whole launch.
  zero_tile_share<SETS>(gs, xh, tile_floats, NB, j0 / 4,
                        (role.cw == p.ls.gx - 1 ? Kpad - j0 : HS) / 4, kPolledTiles);

  // The wavefront's share of W, in registers (requested before the slice, whose loads then
  // overlap with these).
  using Projection = std::conditional_t<kFusedInput, InputProjection<CT, kFusedInput ? XSG : 1>, NoSideWork>;
  Projection proj;
  if constexpr (kFusedInput) {
    proj.setup(p.W, p.x, p.C, N, 4 * H, set_wave<SETS>(), n0 < N ? n0 : N - 1, [=](int col) {
      const int gate = col / HS, j = j0 + col % HS;
      return j < H ? (long long)gate * H + j : -1ll;
    });
    proj.request();
    proj.settle();
  }

  // Resident slice: column c of the slice is gate c/HS, hidden unit j0 + c%HS.
  float4_t breg[REG > 0 ? REG : 1][CT];
  {
    const bool fast = H % 4 == 0 && ((reinterpret_cast<uintptr_t>(p.R) |
                                      reinterpret_cast<uintptr_t>(p.dc_mask)) & 15u) == 0;
    auto offset = [=](int k, int col) {
      const int gate = col / HS, j = j0 + col % HS;
      return (k < H && j < H) ? (long long)k * 4 * H + gate * H + j : -1ll;
    };
    if constexpr (REG > 0) {
      const int groups = Kpad >> 6;
      fill_slice<NCOLS>(w_lds, Kpad - 64 * REG, p.R, p.dc_mask, p.dc_scale, fast, [=](int k, int col) {
        return offset(resident_split_k(k, groups, REG), col);
      });
      load_resident_rows<REG, CT>(breg, groups, p.R, p.dc_mask, p.dc_scale, offset);
    } else {
      fill_slice<NCOLS>(w_lds, Kpad, p.R, p.dc_mask, p.dc_scale, fast, offset);
    }
  }

  // Pointwise ownership: thread slot pp handles batch row n, hidden unit j.
  int pn[PP], pj[PP], pl[PP], pc[PP];
  bool act[PP];
  float c_prev[PP], h_prev[PP], bias[PP][4];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    pl[pp] = idx / HS;           // local batch row
    pc[pp] = idx % HS;           // local hidden unit
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    act[pp] = idx < NB * HS && pl[pp] < rows_here && pj[pp] < H;
    c_prev[pp] = 0.f;
    h_prev[pp] = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) bias[pp][g] = 0.f;
    if (act[pp]) {
      c_prev[pp] = p.c[(size_t)pn[pp] * H + pj[pp]];
      h_prev[pp] = p.h[(size_t)pn[pp] * H + pj[pp]];
#pragma unroll
      for (int g = 0; g < 4; ++g) bias[pp][g] = p.b[g * H + pj[pp]];
    }
  }
  const bool zoneout = p.zoneout_prob != 0.f && p.zoneout_mask != nullptr;
  // Tile 0 receives h[0]; the elements of the other tiles that steps will publish start out
  // unwritten.  One real barrier: nobody polls a tile before all of its owners have set it up.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (act[pp]) {
      float* e = &xh[xchg_index(pj[pp], pl[pp], NB)];
      store_exchanged(gs, e, publishable(h_prev[pp]));
      for (int b = 1; b < kPolledTiles; ++b) store_exchanged(gs, e + (size_t)b * tile_floats, unwritten_value());
    }
  if constexpr (SETS == 2) reset_partials<NB, CT>(red, live_partials<CT>(Kpad));
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);
  if (SETS == 2 && rows_here <= 0) return;  // no workgroup barrier from here on

  // Inputs of a step that do not depend on the recurrence (x*W, the zoneout mask) are
  // fetched one step ahead, while the matrix units work on the step before.
  // Every thread loads (threads without an element, and the request after the last step, some
  // valid address: their values are never used) and nothing but the loads writes these
  // registers inside the loop: a default written there first would have to wait for loads a
  // thread skipped waiting for and, the counter being in order, for the step's stores with them.
  float wx_next[PP][4], mk_next[PP];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    mk_next[pp] = 1.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) wx_next[pp][g] = 0.f;
  }
  auto fetch = [&](int t) {
    const int tt = t < T ? t : T - 1;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      if constexpr (!kFusedInput) {
        const float* vt = p.v + ((size_t)tt * N + row) * 4 * H + unit;
#pragma unroll
        for (int g = 0; g < 4; ++g) wx_next[pp][g] = vt[g * H];
      }
      if (zoneout && p.training) mk_next[pp] = p.zoneout_mask[(size_t)tt * NH + row * H + unit];
    }
  };
  fetch(0);

  for (int t = 0; t < T; ++t) {
    float wx[PP][4], mk[PP];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      mk[pp] = mk_next[pp];
#pragma unroll
      for (int g = 0; g < 4; ++g) wx[pp][g] = wx_next[pp][g];
    }
    // The operand loads wait for h[t] themselves (polled tile t % 4).
    float* red_t = !kPolledPartials ? red : red + (t & 1) * RED;
    if constexpr (kFusedInput) {
      tile_product<NB, CT, false, true, kPolledPartials, Projection>(xhb, (t & 3) * tile_floats, Kpad,
                                                                      w_lds, red_t, &gs, &proj);
      if (t + 1 < T) proj.request();  // x[t+1]: a whole step to arrive
    } else if constexpr (REG > 0) {
      tile_product<NB, CT, false, true, false, NoSideWork, REG, float4_t[REG][CT]>(
          xhb, (t & 3) * tile_floats, Kpad, w_lds, red_t, &gs, nullptr, &breg);
    } else {
      tile_product<NB, CT, false, true, kPolledPartials>(xhb, (t & 3) * tile_floats, Kpad, w_lds, red_t, &gs);
    }
    if constexpr (!kPolledPartials) __syncthreads();

    float gate[PP][4], h_pub[PP];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      float rh[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (kPolledPartials) {
        // whole wavefronts: the wait is a wavefront-wide vote
        if (((tid + 256 * pp) & ~63) < NB * HS)
          take_product<NB, CT, 4>(gs, red_t, pl[pp], pc[pp], HS, tid + 256 * pp < NB * HS,
                                  live_partials<CT>(Kpad), rh);
      } else if (act[pp]) {
#pragma unroll
        for (int g = 0; g < 4; ++g) rh[g] = sum_product<NB, CT>(red, pl[pp], g * HS + pc[pp]);
      }
      if (act[pp]) {
        float a[4];
#pragma unroll
        for (int g = 0; g < 4; ++g)
          a[g] = kFusedInput ? rh[g] + bias[pp][g] : wx[pp][g] + rh[g] + bias[pp][g];
        gate[pp][0] = sigmoid_f(a[0]);
        gate[pp][1] = tanh_f(a[1]);
        gate[pp][2] = sigmoid_f(a[2]);
        gate[pp][3] = sigmoid_f(a[3]);
        const float c_new = gate[pp][2] * c_prev[pp] + gate[pp][0] * gate[pp][1];
        float h_new = gate[pp][3] * tanh_f(c_new);
        if (zoneout) {
          if (p.training) h_new = (h_new - h_prev[pp]) * mk[pp] + h_prev[pp];
          else h_new = p.zoneout_prob * h_prev[pp] + (1.0f - p.zoneout_prob) * h_new;
        }
        c_prev[pp] = c_new;
        h_prev[pp] = h_new;
      }
      h_pub[pp] = publishable(h_prev[pp]);
    }
    // Everything this wavefront stored during the previous step (its resets among it) has
    // landed before h[t+1] becomes visible.
    // (x[t+1] arrives with the same wait.)
    if constexpr (kFusedInput) proj.settle();
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (t + 1 < T) {
      float* xh_next = xh + ((t + 1) & 3) * tile_floats;
      float* xh_done = xh + ((t + 3) & 3) * tile_floats;  // read at step t-1: nobody needs it any more
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        if (act[pp]) {
          const int e = xchg_index(pj[pp], pl[pp], NB);
          store_exchanged(gs, &xh_next[e], h_pub[pp]);
          if (t + 3 < T) store_exchanged(gs, &xh_done[e], unwritten_value());
        }
    }
    fetch(t + 1);
    if constexpr (!kPolledPartials) __syncthreads();  // `red` may be overwritten by the next step's product
    // The caller's copies are written last: nobody in the launch waits for them.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if (act[pp]) {
        if (p.training) {
          float* vt = p.v + ((size_t)t * N + pn[pp]) * 4 * H + pj[pp];
#pragma unroll
          for (int g = 0; g < 4; ++g) vt[g * H] = gate[pp][g];
        }
        const size_t o = (size_t)t * NH + (size_t)pn[pp] * H + pj[pp];
        p.c_out[o] = c_prev[pp];
        p.h_out[o] = h_prev[pp];
      }
    }
  }
}

// The forward pass of a single batch row (see "one batch row" in recurrent.h): 16 hidden units
// x 4 gates per workgroup, the recurrent weights in registers.
// A fifth wavefront (kSingleRowThreads = 320) takes no part in the product: it requests the inputs
// of the step after the next one (x*W of the 64 columns, the zoneout mask) and parks them in LDS
// for the sixteen threads that own the hidden units.  Those inputs come from memory that is cold
// in this launch, and a wavefront's loads return in order: requested by the owners they stood
// before the polls of the next product (1.43 -> 1.34 us per step with warm inputs).
template <int KW_MAX>
__global__ __launch_bounds__(kSingleRowThreads, 1)
void lstm_forward_single_row_kernel(LstmFwdParams p) {
  constexpr int HS = kSingleRowUnits, NCOLS = kSingleRowCols;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float (*h_lds)[KW_MAX] = reinterpret_cast<float (*)[KW_MAX]>(lds);
  float (*red)[4][NCOLS] = reinterpret_cast<float (*)[4][NCOLS]>(lds + 4 * KW_MAX);
  float (*park)[5][HS] = reinterpret_cast<float (*)[5][HS]>(lds + 4 * KW_MAX + 2 * 4 * NCOLS + 4);
  const int H = p.H, T = p.T;
  const int Kpad = round_up(H, 64);
  const int KW = Kpad / 4;  // multiple of 16
  const Role role = take_role(p.ls, reinterpret_cast<unsigned int*>(lds + 4 * KW_MAX + 2 * 4 * NCOLS));
  if (!role.active) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j0 = role.cw * HS;
  float* xh = p.xh;  // one batch tile: [4 polled tiles][Kpad]
  const TileBuffer xhb = make_tile_buffer(xh, kPolledTiles * Kpad);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);
  // Own k range of the exchange tiles (the last workgroup also owns the padding).
  zero_tile_share(gs, xh, Kpad, 1, j0 / 4, (role.cw == p.ls.gx - 1 ? Kpad - j0 : HS) / 4, kPolledTiles);

  float w[KW_MAX];
  single_row_weights<KW_MAX>(w, p.R, p.dc_mask, p.dc_scale, KW, H, 4 * H, (lane / HS) * H + j0 + lane % HS,
                             j0 + lane % HS < H);
  for (int i = tid; i < 4 * KW_MAX; i += kSingleRowThreads) (&h_lds[0][0])[i] = 0.f;  // ordered by group_arrive's barrier

  // Pointwise ownership: thread u < 16 handles hidden unit j0 + u.
  const int pj = j0 + tid;
  const bool act = tid < HS && pj < H;
  float c_prev = 0.f, h_prev = 0.f, bias[4] = {0.f, 0.f, 0.f, 0.f};
  if (act) {
    c_prev = p.c[pj];
    h_prev = p.h[pj];
#pragma unroll
    for (int g = 0; g < 4; ++g) bias[g] = p.b[g * H + pj];
  }
  const bool zoneout = p.zoneout_prob != 0.f && p.zoneout_mask != nullptr;
  // Tile 0 receives h[0]; the elements of the other tiles that steps will publish start out
  // unwritten.  One real barrier: nobody polls a tile before all of its owners have set it up.
  if (act) {
    store_exchanged(gs, &xh[pj], publishable(h_prev));
    for (int b = 1; b < kPolledTiles; ++b) store_exchanged(gs, &xh[b * Kpad + pj], unwritten_value());
  }

  // The helper's requests: lane l = 16 g + u asks for x*W of gate g, unit j0 + u; the first
  // sixteen lanes also for the mask.  Every lane loads (some valid address where its element
  // does not exist, and the last step again after the end).
  const bool helper = wave == 4;
  float in_v = 0.f, in_m = 1.f;
  auto request = [&](int t) {
    const int tt = t < T ? t : T - 1;
    const int unit = j0 + lane % HS < H ? j0 + lane % HS : 0;
    in_v = p.v[(size_t)tt * 4 * H + (size_t)(lane / HS) * H + unit];
    if (zoneout && p.training) in_m = p.zoneout_mask[(size_t)tt * H + unit];
  };
  auto park_inputs = [&](int t) {
    park[t & 1][lane / HS][lane % HS] = in_v;
    if (lane < HS) park[t & 1][4][lane] = in_m;
  };
  if (helper) {
    request(0);
    park_inputs(0);
    request(1);
    park_inputs(1);
  }
  group_arrive(gs);
  group_wait(gs);

  for (int t = 0; t < T; ++t) {
    // parked two steps ago (the first two: before the barrier above)
    float wx[4] = {0.f, 0.f, 0.f, 0.f}, mk = 1.f;
    if (act) {
#pragma unroll
      for (int g = 0; g < 4; ++g) wx[g] = park[t & 1][g][tid];
      mk = park[t & 1][4][tid];
    }

    if (helper) {
      request(t + 2);
    } else {
      // The wavefront's share of h[t] (polled tile t % 4) against the thread's weights.
      red[t & 1][wave][lane] =
          single_row_product<KW_MAX>(gs, xhb, (t & 3) * Kpad + wave * KW, KW, h_lds[wave], w);
    }
    __syncthreads();
    // The owners have read this parity's inputs before the barrier.
    if (helper) park_inputs(t + 2);

    float gate[4] = {0.f, 0.f, 0.f, 0.f};
    if (act) {
      float a[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float* r = &red[t & 1][0][g * HS + tid];
        a[g] = wx[g] + ((r[0] + r[NCOLS]) + (r[2 * NCOLS] + r[3 * NCOLS])) + bias[g];
      }
      gate[0] = sigmoid_f(a[0]);
      gate[1] = tanh_f(a[1]);
      gate[2] = sigmoid_f(a[2]);
      gate[3] = sigmoid_f(a[3]);
      const float c_new = gate[2] * c_prev + gate[0] * gate[1];
      float h_new = gate[3] * tanh_f(c_new);
      if (zoneout) {
        if (p.training) h_new = (h_new - h_prev) * mk + h_prev;
        else h_new = p.zoneout_prob * h_prev + (1.0f - p.zoneout_prob) * h_new;
      }
      c_prev = c_new;
      h_prev = h_new;
    }
    // Everything this wavefront stored during the previous step (its resets among it) has
    // landed before h[t+1] becomes visible.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (act && t + 1 < T) {
      store_exchanged(gs, &xh[((t + 1) & 3) * Kpad + pj], publishable(h_prev));
      // the tile read at step t-1: nobody needs it any more
      if (t + 3 < T) store_exchanged(gs, &xh[((t + 3) & 3) * Kpad + pj], unwritten_value());
    }
    // The caller's copies are written last: nobody in the launch waits for them.
    if (act) {
      if (p.training) {
        float* vt = p.v + (size_t)t * 4 * H + pj;
#pragma unroll
        for (int g = 0; g < 4; ++g) vt[g * H] = gate[g];
      }
      p.c_out[(size_t)t * H + pj] = c_prev;
      p.h_out[(size_t)t * H + pj] = h_prev;
    }
  }
}

struct LstmBwdParams {
  int T, N, H;
  const float* R_t;     // [4H,H]
  const float* c;       // [T,N,H] cell state before each step
  const float* c_next;  // [T,N,H] cell state after each step (may be c + N*H)
  const float* dh_next; // [T,N,H] upstream gradient of the h each step produced
  const float* dc_next; // [T,N,H] same for c
  float* db;            // [4H] accumulated
  float* dh;            // [N,H] in/out
  float* dc;            // [N,H] in/out
  float* v;             // [T,N,4H] in: activations, out: gate gradients
  const float* zoneout_mask;
  float* db_partial;    // [batch tiles, 4H] scratch
  float* xdv;           // polled exchange tiles of the gate gradients: [batch tiles][4][Kpad/4][NB][4]
                        // (scattered form: the pieces of partial sums, see the kernel)
  LaunchShape ls;
};

// A workgroup owns 16 hidden units (HSB) for NB batch rows; its slice of R_t is
// [4H x 16]: dh[:, its units] = dv_t[:, all 4H] * R_t[:, its units].  Inside the launch
// the contraction index runs unit-major (k = 4*unit + gate), so a thread publishes the
// four gate gradients of its (row, unit) with one 16-byte store.  SETS sets of 256 threads,
// each with a batch tile of NB rows of its own (see lstm_forward_kernel).
// REG > 0: the slice exceeds LDS; every wavefront keeps the first REG k-groups of its share
// of the contraction in registers (tall_tile_product).
template <int NB, int SETS, int REG = 0>
__global__ __launch_bounds__(256 * SETS, 1)
void lstm_backward_kernel(LstmBwdParams p) {
  static_assert(SETS == 1 || (SETS == 2 && NB < 16), "two sets: short tiles only");
  static_assert(REG == 0 || NB >= 16, "register-resident slice rows: tall tiles only");
  constexpr int HSB = 16;
  constexpr int NCOLS = 16;
  constexpr int PP = (NB * HSB + 255) / 256;
  constexpr int RED = ProductTile<NB, 1>::kRedFloats;
  constexpr bool kPolledPartials = SETS == 2;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ unsigned int s_role;
  const Role role = take_role(p.ls, &s_role);
  if (!role.active) return;
  __shared__ unsigned int s_flag;

  const int H = p.H, N = p.N, T = p.T;
  const int Kpad = 64 * p.ls.gx;  // 4 gates of the 16 units of every workgroup
  const int set = set_index<SETS>();
  float* w_lds = lds;
  // the partial tiles (two sets: two polled areas each, alternating by step), reused for
  // the db reduction
  float* red = lds + (Kpad - 64 * REG) * NCOLS + (SETS == 1 ? 0 : set * 2 * RED);

  const int tid = set_thread<SETS>();
  const int j0 = role.cw * HSB;
  const int bt = role.bt * SETS + set;  // this set's batch tile
  const int n0 = bt * NB;
  const int rows_here = (N - n0) < NB ? (N - n0) : NB;  // <= 0: a set without rows
  const size_t NH = (size_t)N * H;

  GroupSync gs;
  group_sync_init(gs, p.ls, role);

  const int tile_floats = Kpad * NB;
  float* xdv = p.xdv + (size_t)bt * kPolledTiles * tile_floats;
  const TileBuffer xdvb = make_tile_buffer(xdv, kPolledTiles * tile_floats);

  float4_t breg[REG > 0 ? REG : 1][1];
  {
    const bool fast = H % 4 == 0 && (reinterpret_cast<uintptr_t>(p.R_t) & 15u) == 0;
    auto offset = [=](int k, int col) {
      const int unit = k >> 2, gate = k & 3;
      return (unit < H && j0 + col < H) ? ((long long)gate * H + unit) * H + j0 + col : -1ll;
    };
    if constexpr (REG > 0) {
      const int groups = Kpad >> 6;
      fill_slice<NCOLS>(w_lds, Kpad - 64 * REG, p.R_t, nullptr, 1.0f, fast, [=](int k, int col) {
        return offset(resident_split_k(k, groups, REG), col);
      });
      load_resident_rows<REG, 1>(breg, groups, p.R_t, nullptr, 1.0f, offset);
    } else {
      fill_slice<NCOLS>(w_lds, Kpad, p.R_t, nullptr, 1.0f, fast, offset);
    }
  }

  int pn[PP], pj[PP], pl[PP], pc[PP];
  bool act[PP];
  float dh[PP], dc[PP], dbacc[PP][4];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    pl[pp] = idx / HSB;
    pc[pp] = idx % HSB;
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    act[pp] = idx < NB * HSB && pl[pp] < rows_here && pj[pp] < H;
    dh[pp] = act[pp] ? p.dh[(size_t)pn[pp] * H + pj[pp]] : 0.f;
    dc[pp] = act[pp] ? p.dc[(size_t)pn[pp] * H + pj[pp]] : 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) dbacc[pp][g] = 0.f;
  }
  const bool zoneout = p.zoneout_mask != nullptr;
  // Every element of the polled tiles belongs to the thread that publishes it (rows and
  // units beyond the problem are published as zeros); all start out unwritten.  One real
  // barrier: nobody polls a tile before all of its owners have set it up.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (tid + 256 * pp < NB * HSB) {
      const float u = unwritten_value();
      for (int b = 0; b < kPolledTiles; ++b)
        store_exchanged4(gs, xdv + (size_t)b * tile_floats + ((size_t)pj[pp] * NB + pl[pp]) * 4, u, u, u, u);
    }
  if constexpr (SETS == 2) reset_partials<NB, 1>(red, live_partials<1>(Kpad));
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);

  // Step inputs that do not depend on the recurrence, fetched one step ahead.
  struct StepIn { float vt[4], c0, c1, dhn, dcn, m; };
  StepIn nxt[PP];
  // Every thread loads (threads without an element, and the request after the last step, some
  // valid address: their values are never used) and nothing but the loads writes `nxt`.  A
  // default written here first would have to wait for whatever loads of these registers a
  // thread skipped waiting for -- and with them, the counter being in order, for this step's
  // stores: the round trip of the publication, on the critical path of the step.
  StepIn nxt_init = {{0.f, 0.f, 0.f, 0.f}, 0.f, 0.f, 0.f, 0.f, 1.f};
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) nxt[pp] = nxt_init;
  // (Two sets per workgroup: measured 1.5 % slower per step that way, 0.2887 -> 0.2931 ms at
  // N = 64, T = 100, H = 512; there only the threads with an element load.)
  // Tiles of 32 and 64 rows (one set per workgroup, the whole slice in LDS): requested two steps
  // ahead, right after a product (`later`).  These inputs come from memory that is cold in this
  // launch, and a wavefront's loads return in order -- requested just before a product they keep
  // its polls waiting.  Placed there, the next loads the wavefront issues are the polls of the
  // following product, a pointwise phase and a publication later.  Backward pass, T = 100:
  // N = 256, H = 256 0.914 -> 0.856 ms, N = 512, H = 128 0.989 -> 0.921; 16-row tiles do not
  // change (N = 128, H = 512), 4-row tiles lose 2 %, tiles with slice rows in registers up to
  // 10 % (N = 32, H = 1024: the second set of inputs costs them registers), two sets per
  // workgroup 1 %: those keep the request before the product.
  constexpr bool kRequestAfterProduct = SETS == 1 && REG == 0 && NB >= 32;
  StepIn later[PP];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) later[pp] = nxt_init;
  auto fetch = [&](StepIn (&dst)[PP], int t) {
    const int tt = t >= 0 ? t : 0;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if (SETS == 2 && !(act[pp] && t >= 0)) {
        dst[pp] = nxt_init;
        continue;
      }
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      const size_t e = (size_t)tt * NH + row * H + unit;
      const float* vt = p.v + ((size_t)tt * N + row) * 4 * H + unit;
#pragma unroll
      for (int g = 0; g < 4; ++g) dst[pp].vt[g] = vt[g * H];
      dst[pp].c0 = p.c[e];
      dst[pp].c1 = p.c_next[e];
      dst[pp].dhn = p.dh_next[e];
      dst[pp].dcn = p.dc_next[e];
      if (zoneout) dst[pp].m = p.zoneout_mask[e];
    }
  };
  fetch(nxt, T - 1);
  if constexpr (kRequestAfterProduct) fetch(later, T - 2);

  // A set without rows skips the steps (two sets: no workgroup barrier inside them).
  for (int t = (SETS == 2 && rows_here <= 0) ? -1 : T - 1; t >= 0; --t) {
    float dh_keep[PP], dv[PP][4];
    const int done = T - 1 - t;  // steps done so far; this step uses polled tile done % 4
    float* xdv_t = xdv + (done & 3) * tile_floats;
    float* xdv_done = xdv + ((done + 2) & 3) * tile_floats;  // read two steps ago
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      dh_keep[pp] = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) dv[pp][g] = 0.f;
      if (act[pp]) {
        const StepIn s = nxt[pp];
        const float gi = s.vt[0], gg = s.vt[1], gf = s.vt[2], go = s.vt[3];
        float dc_total = s.dcn + dc[pp];
        float dh_total = s.dhn + dh[pp];
        const float c_tanh = tanh_f(s.c1);
        if (zoneout) {
          dh_keep[pp] = (1.0f - s.m) * dh_total;
          dh_total = s.m * dh_total;
        }
        const float do_ = c_tanh * dh_total;
        const float dc_tanh = go * dh_total;
        dc_total += d_tanh_f(c_tanh) * dc_tanh;
        const float df = s.c0 * dc_total;
        dc[pp] = gf * dc_total;
        const float di = gg * dc_total;
        const float dg = gi * dc_total;
        const float dv_i = d_sigmoid_f(gi) * di;
        const float dv_g = d_tanh_f(gg) * dg;
        const float dv_f = d_sigmoid_f(gf) * df;
        const float dv_o = d_sigmoid_f(go) * do_;
        dv[pp][0] = dv_i;
        dv[pp][1] = dv_g;
        dv[pp][2] = dv_f;
        dv[pp][3] = dv_o;
#pragma unroll
        for (int g = 0; g < 4; ++g) dbacc[pp][g] += dv[pp][g];
      }
    }
    // What this wavefront stored during the previous step (its resets among it) has landed
    // before the gate gradients of this step become visible.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      // rows and units beyond the problem are published as zeros
      if (tid + 256 * pp < NB * HSB) {
        const size_t e = ((size_t)pj[pp] * NB + pl[pp]) * 4;
        store_exchanged4(gs, xdv_t + e, publishable(dv[pp][0]), publishable(dv[pp][1]),
                         publishable(dv[pp][2]), publishable(dv[pp][3]));
        if (done + 2 < T) {
          const float u = unwritten_value();
          store_exchanged4(gs, xdv_done + e, u, u, u, u);
        }
      }
    }
    // The caller's copy: nobody in the launch waits for it.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if (act[pp]) {
        float* vt = p.v + ((size_t)t * N + pn[pp]) * 4 * H + pj[pp];
#pragma unroll
        for (int g = 0; g < 4; ++g) vt[g * H] = dv[pp][g];
      }
    }
    // The operand loads of the product wait for dv_t of every unit themselves.
    if constexpr (!kRequestAfterProduct) fetch(nxt, t - 1);
    float* red_t = !kPolledPartials ? red : red + (done & 1) * RED;
    if constexpr (REG > 0)
      tile_product<NB, 1, true, true, false, NoSideWork, REG, float4_t[REG][1]>(
          xdvb, (done & 3) * tile_floats, Kpad, w_lds, red_t, &gs, nullptr, &breg);
    else
      tile_product<NB, 1, true, true, kPolledPartials>(xdvb, (done & 3) * tile_floats, Kpad, w_lds, red_t, &gs);
    // What was requested a step ago becomes the next step's inputs; the step after that is
    // requested now.
    if constexpr (kRequestAfterProduct) {
#pragma unroll
      for (int pp = 0; pp < PP; ++pp) nxt[pp] = later[pp];
      fetch(later, t - 2);
    }
    if constexpr (kPolledPartials) {
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        if (((tid + 256 * pp) & ~63) < NB * HSB) {  // whole wavefronts: the wait is a vote
          float rdv[1];
          take_product<NB, 1, 1>(gs, red_t, pl[pp], pc[pp], 0, tid + 256 * pp < NB * HSB,
                                 live_partials<1>(Kpad), rdv);
          if (tid + 256 * pp < NB * HSB) dh[pp] = dh_keep[pp] + rdv[0];
        }
    } else {
      __syncthreads();
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        if (tid + 256 * pp < NB * HSB) dh[pp] = dh_keep[pp] + sum_product<NB, 1>(red, pl[pp], pc[pp]);
      __syncthreads();  // `red` may be overwritten by the next step's product
    }
  }

#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    if (act[pp]) {
      p.dh[(size_t)pn[pp] * H + pj[pp]] = dh[pp];
      p.dc[(size_t)pn[pp] * H + pj[pp]] = dc[pp];
    }
  }

  // Bias gradient: sum over this tile's rows in LDS (fixed order), park per tile,
  // and let the last workgroup of the launch add the tiles in order.
  __syncthreads();
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (tid + 256 * pp < NB * HSB) {
#pragma unroll
      for (int g = 0; g < 4; ++g) red[(pl[pp] * 4 + g) * HSB + pc[pp]] = act[pp] ? dbacc[pp][g] : 0.f;
    }
  __syncthreads();
  if (tid < 4 * HSB) {
    const int g = tid / HSB, jj = tid % HSB;
    float s = 0.f;
    for (int r = 0; r < NB; ++r) s += red[(r * 4 + g) * HSB + jj];
    if (j0 + jj < H) store_agent(&p.db_partial[(size_t)bt * 4 * H + g * H + j0 + jj], s);
  }
  if (column_last_arrival(p.ls.cb, role.cw, (unsigned)p.ls.gy, &s_flag)) {
    if (set == 0 && tid < 4 * HSB && j0 + tid % HSB < H) {
      const int col = (tid / HSB) * H + j0 + tid % HSB;
      p.db[col] += sum_over_tiles(p.db_partial + col, (size_t)4 * H, p.ls.gy * SETS);
    }
  }
}

// The LSTM's pointwise backward step for the scattered form of the recurrence
// (scatter_backward.h): arithmetic as in lstm_backward_kernel.
struct LstmScatterCell {
  using Params = LstmBwdParams;
  static constexpr int kGates = 4;
  static constexpr int kInputs = 9;  // v (4 gates), c before and after, dh_next, dc_next, mask
  static constexpr int kSums = 4;
  float dh, dc, dh_keep;
  float gi, gg, gf, go, c0, dhn, m, c_tanh, k_c, k_i, k_g, k_f, k_o, dc_total;

  __device__ __forceinline__ static float* pieces(const Params& p) { return p.xdv; }
  __device__ __forceinline__ static void request(const Params& p, float (&in)[kInputs], size_t e, size_t ve,
                                                 bool zoneout) {
    const float* vt = p.v + ve;
#pragma unroll
    for (int g = 0; g < 4; ++g) in[g] = vt[g * (size_t)p.H];
    in[4] = p.c[e];
    in[5] = p.c_next[e];
    in[6] = p.dh_next[e];
    in[7] = p.dc_next[e];
    if (zoneout) in[8] = p.zoneout_mask[e];
  }
  __device__ __forceinline__ void load_state(const Params& p, size_t e, bool mine) {
    dh = mine ? p.dh[e] : 0.f;
    dc = mine ? p.dc[e] : 0.f;
    dh_keep = 0.f;
  }
  __device__ __forceinline__ void store_state(const Params& p, size_t e) const {
    p.dh[e] = dh;
    p.dc[e] = dc;
  }
  __device__ __forceinline__ void prepare(const float (&sv)[kInputs]) {
    gi = sv[0]; gg = sv[1]; gf = sv[2]; go = sv[3];
    c0 = sv[4]; dhn = sv[6]; m = sv[8];
    c_tanh = tanh_f(sv[5]);
    k_c = d_tanh_f(c_tanh);
    k_i = d_sigmoid_f(gi);
    k_g = d_tanh_f(gg);
    k_f = d_sigmoid_f(gf);
    k_o = d_sigmoid_f(go);
    dc_total = sv[7] + dc;
  }
  __device__ __forceinline__ void add_gathered(float sum) { dh = dh_keep + sum; }
  __device__ __forceinline__ float4_t step(bool act, bool zoneout, float (&sums)[kSums]) {
    float4_t dv = {0.f, 0.f, 0.f, 0.f};
    dh_keep = 0.f;
    if (act) {
      float dh_total = dhn + dh;
      if (zoneout) {
        dh_keep = (1.0f - m) * dh_total;
        dh_total = m * dh_total;
      }
      const float do_ = c_tanh * dh_total;
      const float dc_tanh = go * dh_total;
      dc_total += k_c * dc_tanh;
      const float df = c0 * dc_total;
      dc = gf * dc_total;
      const float di = gg * dc_total;
      const float dg = gi * dc_total;
      dv = float4_t{k_i * di, k_g * dg, k_f * df, k_o * do_};
#pragma unroll
      for (int g = 0; g < 4; ++g) sums[g] += dv[g];
    }
    return dv;
  }
  __device__ __forceinline__ static void store_copy(const Params& p, int t, size_t n, size_t j, const float4_t& a) {
    float* vt = p.v + ((size_t)t * p.N + n) * 4 * p.H + j;
#pragma unroll
    for (int g = 0; g < 4; ++g) vt[g * (size_t)p.H] = a[g];
  }
  __device__ __forceinline__ static void add_sums(const Params& p, int col, float s) { p.db[col] += s; }
};

}  // namespace

// The forward pass of a single batch row with H <= 512: the recurrent weights live in the
// registers of the 16-unit workgroups of one XCD (lstm_forward_single_row_kernel).
int lstm_forward_single_row(hipStream_t stream, int training, int T, int C, int H,
                            const float* W, const float* R, const float* b, const float* x,
                            const float* h, const float* c, float* h_out, float* c_out, float* v,
                            float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                            float dc_scale) {
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T, 4 * H, C, x, C, W, 4 * H, v, 4 * H, false));
  const int Kpad = (H + 63) / 64 * 64;
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, (size_t)kPolledTiles * Kpad * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));
  LstmFwdParams p;
  p.training = training; p.T = T; p.N = 1; p.H = H;
  p.R = R; p.b = b; p.h = h; p.c = c; p.h_out = h_out; p.c_out = c_out; p.v = v;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.dc_mask = dc_mask; p.dc_scale = dc_scale;
  p.xh = ws.scratch;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, (H + 15) / 16, 1, 1,
                                  single_row_lds_bytes(single_row_kw_max(Kpad)) + kSingleRowParkBytes,
                                  (unsigned)T + 1, &plan));
  plan.threads = kSingleRowThreads;
  p.ls = plan.shape;
  const char* name = "lstm_forward_recurrence";
  if (Kpad <= 128) return launch_persistent(name, lstm_forward_single_row_kernel<32>, plan, p, stream);
  if (Kpad <= 256) return launch_persistent(name, lstm_forward_single_row_kernel<64>, plan, p, stream);
  return launch_persistent(name, lstm_forward_single_row_kernel<128>, plan, p, stream);
}

// h, c: [N,H] state before the first step; h_out, c_out: [T,N,H] states after each step.
int lstm_forward_impl(hipStream_t stream, int training, int T, int N, int C, int H,
                      const float* W, const float* R, const float* b, const float* x,
                      const float* h, const float* c, float* h_out, float* c_out, float* v,
                      float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                      float dc_scale) {
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W && R && b && x && h && c && h_out && c_out && v);
  // A single step of a small batch (Iterate): one kernel, nothing kept on chip.
  if (T == 1 && single_step_applies(N, C, H))
    return lstm_forward_single_step(stream, training, N, C, H, W, R, b, x, h, c, h_out, c_out, v,
                                    zoneout_prob, zoneout_mask, dc_mask, dc_scale);
  if (N == 1 && H <= 512 && xcd_local_fits((H + 15) / 16, 1))
    return lstm_forward_single_row(stream, training, T, C, H, W, R, b, x, h, c, h_out, c_out, v,
                                   zoneout_prob, zoneout_mask, dc_mask, dc_scale);
  const ForwardTile tile = pick_forward_tile(4, N, H, 0, kWorkgroupLdsBytes, false, 2);
  // No slice of R fits a CU: stream R from HBM every step instead.
  if (!tile.ok)
    return lstm_forward_streamed(stream, training, T, N, C, H, W, R, b, x, h, c, h_out, c_out, v,
                                 zoneout_prob, zoneout_mask, dc_mask, dc_scale);
  // An 8-row tile is run as two sets of 4 rows when the partial tiles of both fit beside the
  // slice (exchange tiles: one per set, together as large as the tile's).  Measured at
  // H = 512: 6 % faster per step; two sets of 8 rows instead of a 16-row tile: 6 % slower.
  const size_t paired_lds = paired_lds_bytes((H + 63) / 64 * 64, tile.ct);
  const bool paired = tile.nb == 8 && paired_lds <= kWorkgroupLdsBytes &&
                      tile.reg_groups == 0;

  // With 4-row tiles the recurrence computes x * W itself, beside its waits (every wavefront of
  // a set must have a share of the recurrent product, H > 192, to keep in step with the readers
  // of its partial tiles; the projection's weights must fit the registers, C <= 512).
  // Otherwise: v = x * W for all steps at once.
  const int xsg = (C + 255) / 256;  // super-groups of 64 input features per wavefront
  const bool fused = (paired || tile.nb == 4) && H > 192 && C <= 512 && C % 4 == 0 &&
                     (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && fused_input_enabled();
  if (!fused)
    HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T * N, 4 * H, C, x, C, W, 4 * H, v, 4 * H, false));

  // Taken after the GEMM, which may replace the stream's scratch buffer with a larger one.
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(
      stream, exchange_floats(H, tile.nb, tile.gy, kPolledTiles) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  LstmFwdParams p;
  p.training = training; p.T = T; p.N = N; p.H = H;
  p.R = R; p.b = b; p.h = h; p.c = c; p.h_out = h_out; p.c_out = c_out; p.v = v;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.dc_mask = dc_mask; p.dc_scale = dc_scale;
  p.xh = ws.scratch;
  p.x = x; p.W = W; p.C = C;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, tile.gx, tile.gy, tile.nb,
                                  paired ? paired_lds : tile.lds_bytes, (unsigned)T + 1, &plan));
  p.ls = plan.shape;
  if (paired) plan.threads = 512;
#define HASTE_LAUNCH_FWD_RESIDENT(NB_, REG_)                                                     \
  if (tile.reg_groups == REG_ && tile.nb == NB_ && tile.ct == 2)                                 \
    return launch_persistent("lstm_forward_recurrence", lstm_forward_kernel<NB_, 2, 1, 0, REG_>, \
                             plan, p, stream);
  HASTE_LAUNCH_FWD_RESIDENT(16, 8) HASTE_LAUNCH_FWD_RESIDENT(32, 8) HASTE_LAUNCH_FWD_RESIDENT(64, 8)
  HASTE_LAUNCH_FWD_RESIDENT(16, 16) HASTE_LAUNCH_FWD_RESIDENT(32, 16) HASTE_LAUNCH_FWD_RESIDENT(64, 16)
#undef HASTE_LAUNCH_FWD_RESIDENT
  if (tile.reg_groups > 0) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
#define HASTE_LAUNCH_FWD_FUSED(CT_, XSG_)                                                       \
  if (fused && tile.ct == CT_ && xsg == XSG_) {                                                  \
    if (paired)                                                                                  \
      return launch_persistent("lstm_forward_recurrence", lstm_forward_kernel<4, CT_, 2, XSG_>,  \
                               plan, p, stream);                                                 \
    return launch_persistent("lstm_forward_recurrence", lstm_forward_kernel<4, CT_, 1, XSG_>,    \
                             plan, p, stream);                                                   \
  }
  HASTE_LAUNCH_FWD_FUSED(1, 1) HASTE_LAUNCH_FWD_FUSED(2, 1) HASTE_LAUNCH_FWD_FUSED(4, 1)
  HASTE_LAUNCH_FWD_FUSED(1, 2) HASTE_LAUNCH_FWD_FUSED(2, 2) HASTE_LAUNCH_FWD_FUSED(4, 2)
#undef HASTE_LAUNCH_FWD_FUSED
#define HASTE_LAUNCH_FWD_PAIRED(CT_)                                                       \
  if (paired && tile.ct == CT_)                                                            \
    return launch_persistent("lstm_forward_recurrence", lstm_forward_kernel<4, CT_, 2>, plan, p, \
                             stream);
  HASTE_LAUNCH_FWD_PAIRED(1) HASTE_LAUNCH_FWD_PAIRED(2) HASTE_LAUNCH_FWD_PAIRED(4)
#undef HASTE_LAUNCH_FWD_PAIRED
#define HASTE_LAUNCH_FWD(NB_, CT_)                                                         \
  if (tile.nb == NB_ && tile.ct == CT_)                                                    \
    return launch_persistent("lstm_forward_recurrence", lstm_forward_kernel<NB_, CT_, 1>, plan, p, \
                             stream);
  HASTE_LAUNCH_FWD(4, 1) HASTE_LAUNCH_FWD(4, 2) HASTE_LAUNCH_FWD(4, 4)
  HASTE_LAUNCH_FWD(8, 1) HASTE_LAUNCH_FWD(8, 2) HASTE_LAUNCH_FWD(8, 4)
  HASTE_LAUNCH_FWD(16, 1) HASTE_LAUNCH_FWD(16, 2) HASTE_LAUNCH_FWD(16, 4)
  HASTE_LAUNCH_FWD(32, 1) HASTE_LAUNCH_FWD(32, 2) HASTE_LAUNCH_FWD(32, 4)
  HASTE_LAUNCH_FWD(64, 1) HASTE_LAUNCH_FWD(64, 2) HASTE_LAUNCH_FWD(64, 4)
#undef HASTE_LAUNCH_FWD
  return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
}

// h, c: [T,N,H] states before each step; c_next: [T,N,H] cell states after each step;
// dh_next, dc_next: [T,N,H] upstream gradients of the states each step produced.
int lstm_backward_impl(hipStream_t stream, int T, int N, int C, int H,
                       const float* W_t, const float* R_t, const float* x_t,
                       const float* h, const float* c, const float* c_next,
                       const float* dh_next, const float* dc_next,
                       float* dx, float* dW, float* dR, float* db, float* dh, float* dc, float* v,
                       const float* zoneout_mask) {
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && c && c_next && dh_next && dc_next);
  HASTE_HIP_REQUIRE(dx && dW && dR && db && dh && dc && v);
  const BackwardTile tile = pick_backward_tile(4 * H, N, H, 4 * 16, 0, true);
  if (!tile.ok)
    return lstm_backward_streamed(stream, T, N, C, H, W_t, R_t, x_t, h, c, c_next, dh_next, dc_next,
                                  dx, dW, dR, db, dh, dc, v, zoneout_mask);

  // An 8-row tile is run as two sets of 4 rows (see lstm_forward_impl): four polled areas of
  // partial tiles beside the slice.
  const size_t paired_lds = paired_lds_bytes(64 * tile.gx, 1);
  // 4-row tiles (8 rows: two sets of 4) with H <= 512 take the scattered form: partial sums of
  // dh go to their owners instead of the gate gradients to everybody.
  // (Measured over H = 64 ... 512, T = 100: with two sets per workgroup it is 5-15 % faster
  // at every H, with one set from H = 384 on; below, one set is 5-20 % faster the other way.)
  const bool scatter = tile.reg_groups == 0 && H <= 512 &&
                       (tile.nb == 8 || (tile.nb == 4 && H > 320));
  const bool paired = scatter ? tile.nb == 8
                              : tile.nb == 8 && paired_lds <= kMaxLdsBytes;
  const int sets = paired ? 2 : 1;
  const int ctn = H <= 256 ? 1 : 2;  // column tiles of 64 per wavefront

  Workspace ws;
  const size_t db_floats = (size_t)tile.gy * sets * 4 * H;
  const size_t xdv_floats = scatter ? (size_t)tile.gy * sets * kScatterTiles * scatter_tile_floats(tile.gx, ctn)
                                    : exchange_floats(64 * tile.gx, tile.nb, tile.gy, kPolledTiles);
  HASTE_HIP_PROPAGATE(get_workspace(stream, ((db_floats + 3) / 4 * 4 + xdv_floats) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  LstmBwdParams p;
  p.T = T; p.N = N; p.H = H;
  p.R_t = R_t; p.c = c; p.c_next = c_next; p.dh_next = dh_next; p.dc_next = dc_next;
  p.db = db; p.dh = dh; p.dc = dc; p.v = v; p.zoneout_mask = zoneout_mask;
  p.db_partial = ws.scratch;
  p.xdv = ws.scratch + (db_floats + 3) / 4 * 4;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, tile.gx, tile.gy, tile.nb,
                                  scatter ? sets * kScatterSetFloats * sizeof(float) : (paired ? paired_lds : tile.lds_bytes), (unsigned)T + 1, &plan));
  p.ls = plan.shape;
  if (paired) plan.threads = 512;
  int rc = HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  const char* name = "lstm_backward_recurrence";
  if (scatter) {
    rc = launch_scatter_backward<LstmScatterCell>(name, H, sets, plan, p, stream);
  } else
#define HASTE_LAUNCH_BWD_RESIDENT(NB_)                                                            \
  (tile.reg_groups == 8    ? launch_persistent(name, lstm_backward_kernel<NB_, 1, 8>, plan, p, stream)  \
   : tile.reg_groups == 16 ? launch_persistent(name, lstm_backward_kernel<NB_, 1, 16>, plan, p, stream) \
   : tile.reg_groups == 24 ? launch_persistent(name, lstm_backward_kernel<NB_, 1, 24>, plan, p, stream) \
                           : launch_persistent(name, lstm_backward_kernel<NB_, 1, 32>, plan, p, stream))
  if (tile.reg_groups > 0) {
    if (tile.nb == 16) rc = HASTE_LAUNCH_BWD_RESIDENT(16);
    else if (tile.nb == 32) rc = HASTE_LAUNCH_BWD_RESIDENT(32);
    else if (tile.nb == 64) rc = HASTE_LAUNCH_BWD_RESIDENT(64);
  }
#undef HASTE_LAUNCH_BWD_RESIDENT
  else if (paired) rc = launch_persistent(name, lstm_backward_kernel<4, 2>, plan, p, stream);
  else if (tile.nb == 4) rc = launch_persistent(name, lstm_backward_kernel<4, 1>, plan, p, stream);
  else if (tile.nb == 8) rc = launch_persistent(name, lstm_backward_kernel<8, 1>, plan, p, stream);
  else if (tile.nb == 16) rc = launch_persistent(name, lstm_backward_kernel<16, 1>, plan, p, stream);
  else if (tile.nb == 32) rc = launch_persistent(name, lstm_backward_kernel<32, 1>, plan, p, stream);
  else if (tile.nb == 64) rc = launch_persistent(name, lstm_backward_kernel<64, 1>, plan, p, stream);
  HASTE_HIP_PROPAGATE(rc);

  // dW += x^T dv ; dR += h[0:T]^T dv ; dx = dv W^T  (dv now lives in v).
  const int TN = T * N;
  // dW += x^T dv and dR += h^T dv: one launch when that halves their K pieces
  HASTE_HIP_PROPAGATE(gemm_f32_pair(stream, C, H, 4 * H, TN, x_t, TN, v, 4 * H, dW, 4 * H,
                                    h, H, v, 4 * H, dR, 4 * H, true));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, TN, C, 4 * H, v, 4 * H, W_t, C, dx, C, false));
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" {

int haste_hip_lstm_forward_f32(int training, int steps, int batch_size, int input_size,
                               int hidden_size,
                               const float* W, const float* R, const float* b, const float* x,
                               float* h, float* c, float* v, float* tmp_Rh,
                               float zoneout_prob, const float* zoneout_mask, void* stream) {
  (void)tmp_Rh;  // the recurrent product never leaves the chip
  HASTE_HIP_REQUIRE(h && c && batch_size > 0 && hidden_size > 0);
  const size_t NH = (size_t)batch_size * hidden_size;
  return haste_hip::lstm_forward_impl(haste_hip::as_stream(stream), training, steps, batch_size,
                                      input_size, hidden_size, W, R, b, x, h, c, h + NH, c + NH, v,
                                      zoneout_prob, zoneout_mask, nullptr, 1.0f);
}

int haste_hip_lstm_forward_dropconnect_f32(int training, int steps, int batch_size,
                                           int input_size, int hidden_size,
                                           const float* W, const float* R, const float* b,
                                           const float* x, float* h, float* c, float* v,
                                           float zoneout_prob, const float* zoneout_mask,
                                           const float* dropconnect_mask, float dropconnect_scale,
                                           void* stream) {
  HASTE_HIP_REQUIRE(h && c && batch_size > 0 && hidden_size > 0);
  const size_t NH = (size_t)batch_size * hidden_size;
  return haste_hip::lstm_forward_impl(haste_hip::as_stream(stream), training, steps, batch_size,
                                      input_size, hidden_size, W, R, b, x, h, c, h + NH, c + NH, v,
                                      zoneout_prob, zoneout_mask, dropconnect_mask,
                                      dropconnect_scale);
}

int haste_hip_lstm_backward_f32(int steps, int batch_size, int input_size, int hidden_size,
                                const float* W_t, const float* R_t, const float* b,
                                const float* x_t, const float* h, const float* c,
                                const float* dh_new, const float* dc_new,
                                float* dx, float* dW, float* dR, float* db,
                                float* dh, float* dc, float* v,
                                const float* zoneout_mask, void* stream) {
  (void)b;  // unused by the reference as well (lib/lstm_backward_gpu.cu.cc:319-405)
  HASTE_HIP_REQUIRE(c && dh_new && dc_new && batch_size > 0 && hidden_size > 0);
  const size_t NH = (size_t)batch_size * hidden_size;
  return haste_hip::lstm_backward_impl(haste_hip::as_stream(stream), steps, batch_size, input_size,
                                       hidden_size, W_t, R_t, x_t, h, c, c + NH, dh_new + NH,
                                       dc_new + NH, dx, dW, dR, db, dh, dc, v, zoneout_mask);
}

int haste_hip_lstm_forward_iterate_f32(int training, int batch_size, int input_size,
                                       int hidden_size,
                                       const float* W, const float* R, const float* b,
                                       const float* x, const float* h, const float* c,
                                       float* h_out, float* c_out, float* v, float* tmp_Rh,
                                       float zoneout_prob, const float* zoneout_mask,
                                       void* stream) {
  (void)tmp_Rh;
  return haste_hip::lstm_forward_impl(haste_hip::as_stream(stream), training, 1, batch_size,
                                      input_size, hidden_size, W, R, b, x, h, c, h_out, c_out, v,
                                      zoneout_prob, zoneout_mask, nullptr, 1.0f);
}

int haste_hip_lstm_backward_iterate_f32(int batch_size, int input_size, int hidden_size,
                                        const float* W_t, const float* R_t, const float* b,
                                        const float* x_t, const float* h, const float* c,
                                        const float* c_new, const float* dh_new,
                                        const float* dc_new, float* dx, float* dW, float* dR,
                                        float* db, float* dh, float* dc, float* v,
                                        const float* zoneout_mask, void* stream) {
  (void)b;
  return haste_hip::lstm_backward_impl(haste_hip::as_stream(stream), 1, batch_size, input_size,
                                       hidden_size, W_t, R_t, x_t, h, c, c_new, dh_new, dc_new, dx,
                                       dW, dR, db, dh, dc, v, zoneout_mask);
}

}  // extern "C"
