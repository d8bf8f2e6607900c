// GRU forward and backward passes (gate order z, r, g; "reset-after" variant):
// one MFMA GEMM for x*W over all steps, one persistent kernel for the recurrence with
// the gate math, zoneout and optional DropConnect fused in; backward is a persistent
// reverse-time kernel followed by three batched GEMMs.
//
// Arithmetic follows reference lib/gru_forward_gpu.cu.cc:46-84 and
// lib/gru_backward_gpu.cu.cc:45-95; orchestration replaces :314-371 and :321-409.
#include "scatter_backward.h"

namespace haste_hip {
namespace {

struct GruFwdParams {
  int training, T, N, H;
  const float* R;        // [H,3H]
  const float* bx;       // [3H]
  const float* br;       // [3H]
  const float* h;        // [N,H] state before the first step
  float* h_out;          // [T,N,H] states after each step (may start at h + N*H)
  float* v;              // [T,N,4H] (training) or null
  const float* Wx;       // [T,N,3H] = x*W (kernels that compute the input projection themselves: unused)
  const float* W;        // [C,3H] and
  const float* x;        // [T,N,C], for those kernels
  int C;
  float zoneout_prob;
  const float* zoneout_mask;
  const float* dc_mask;  // DropConnect mask [H,3H] or null
  float dc_scale;
  float* xh;             // polled exchange tiles of h: [batch tiles][4][Kpad/4][NB][4]
  LaunchShape ls;
};

// HS hidden units per workgroup; their 3 gate columns occupy 3*HS of the 16*CT slice
// columns (the rest are zero padding).
// SETS sets of 256 threads, each with a batch tile of NB rows of its own.  Two sets share
// the resident slice but nothing else: while one waits for its exchange the other computes,
// which a single tile of 2*NB rows cannot do.
// REG > 0 (tiles of 16 rows and more): the slice exceeds LDS; every wavefront keeps the first REG
// k-groups of its share of the contraction in registers (tall_tile_product).
// HALF (4-row tiles): the step's product on the half matrix cores, for widened half tensors.
// XSG > 0 (4-row tiles, 16 units per workgroup): the kernel also computes the input projection
// x[t] * W beside its waits (see InputProjection): the z and r columns into the accumulators of
// the recurrent product, the candidate gate's -- which needs x*W and h*R apart -- into a tile of
// its own, which rides behind the slice's three in the partial tiles (rows of 64 columns).
template <int NB, int CT, int HS, int SETS, int REG = 0, bool HALF = false, int XSG = 0>
__global__ __launch_bounds__(256 * SETS, 1)
void gru_forward_kernel(GruFwdParams p) {
  static_assert(!HALF || (NB == 4 && REG == 0), "half product: 4-row tiles");
  constexpr bool kFusedInput = XSG > 0;
  static_assert(!kFusedInput || (NB == 4 && CT == 3 && HS == 16 && REG == 0 && !HALF), "fused input projection");
  constexpr int RCT = kFusedInput ? 4 : CT;  // column tiles of a partial tile's rows
  constexpr int NG = kFusedInput ? 4 : 3;    // sums per element: z, r, h*R of g (, x*W of g)
  static_assert(3 * HS <= 16 * CT, "slice too narrow");
  static_assert(SETS == 1 || (SETS == 2 && NB < 16), "two sets: short tiles only");
  static_assert(REG == 0 || (NB >= 16 && SETS == 1), "register-resident slice rows: tall tiles only");
  constexpr int NCOLS = 16 * CT;
  constexpr int PP = (NB * HS + 255) / 256;
  constexpr int RED = ProductTile<NB, RCT>::kRedFloats;
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
  using Projection = std::conditional_t<kFusedInput, InputProjection<CT, kFusedInput ? XSG : 1, true>, NoSideWork>;
  Projection proj;
  if constexpr (kFusedInput) {
    proj.setup(p.W, p.x, p.C, N, 3 * H, set_wave<SETS>(), n0 < N ? n0 : N - 1, [=](int col) {
      const int gate = col / HS, j = j0 + col % HS;
      return j < H ? (long long)gate * H + j : -1ll;
    });
    proj.request();
    proj.settle();
  }

  float4_t breg[REG > 0 ? REG : 1][CT];
  {
    const bool fast = H % 4 == 0 && ((reinterpret_cast<uintptr_t>(p.R) |
                                      reinterpret_cast<uintptr_t>(p.dc_mask)) & 15u) == 0;
    auto offset = [=](int k, int col) {
      const int gate = col / HS, j = j0 + col % HS;
      return (k < H && gate < 3 && j < H) ? (long long)k * 3 * H + gate * H + j : -1ll;
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

  int pn[PP], pj[PP], pl[PP], pc[PP];
  bool act[PP];
  float h_prev[PP], bxv[PP][3], brv[PP][3];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    pl[pp] = idx / HS;
    pc[pp] = idx % HS;
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    act[pp] = idx < NB * HS && pl[pp] < rows_here && pj[pp] < H;
    h_prev[pp] = 0.f;
#pragma unroll
    for (int g = 0; g < 3; ++g) bxv[pp][g] = brv[pp][g] = 0.f;
    if (act[pp]) {
      h_prev[pp] = p.h[(size_t)pn[pp] * H + pj[pp]];
#pragma unroll
      for (int g = 0; g < 3; ++g) {
        bxv[pp][g] = p.bx[g * H + pj[pp]];
        brv[pp][g] = p.br[g * H + pj[pp]];
      }
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
  if constexpr (SETS == 2) reset_partials<NB, RCT>(red, live_partials<CT>(Kpad));
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);
  if (SETS == 2 && rows_here <= 0) return;  // no workgroup barrier from here on

  // Inputs of a step that do not depend on the recurrence (x*W, the zoneout mask) are
  // fetched one step ahead.
  float wx_next[PP][3], mk_next[PP];
  // Every thread loads (threads without an element, and the request after the last step, some
  // valid address: their values are never used) and nothing but the loads writes these
  // registers inside the loop (see lstm_forward_kernel).
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    mk_next[pp] = 1.f;
#pragma unroll
    for (int g = 0; g < 3; ++g) wx_next[pp][g] = 0.f;
  }
  auto fetch = [&](int t) {
    const int tt = t < T ? t : T - 1;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      if constexpr (!kFusedInput) {
        const float* wt = p.Wx + ((size_t)tt * N + row) * 3 * H + unit;
#pragma unroll
        for (int g = 0; g < 3; ++g) wx_next[pp][g] = wt[g * H];
      }
      if (zoneout && p.training) mk_next[pp] = p.zoneout_mask[(size_t)tt * NH + row * H + unit];
    }
  };
  fetch(0);

  for (int t = 0; t < T; ++t) {
    float wx[PP][3], mk[PP];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      mk[pp] = mk_next[pp];
#pragma unroll
      for (int g = 0; g < 3; ++g) wx[pp][g] = wx_next[pp][g];
    }
    // The operand loads wait for h[t] themselves (polled tile t % 4).
    float* red_t = !kPolledPartials ? red : red + (t & 1) * RED;
    if constexpr (kFusedInput) {
      tile_product<NB, CT, false, true, kPolledPartials, Projection, 0, NoResidentRows, false, RCT>(
          xhb, (t & 3) * tile_floats, Kpad, w_lds, red_t, &gs, &proj);
      if (t + 1 < T) proj.request();  // x[t+1]: a whole step to arrive
    } else if constexpr (REG > 0) {
      tile_product<NB, CT, false, true, false, NoSideWork, REG, float4_t[REG][CT]>(
          xhb, (t & 3) * tile_floats, Kpad, w_lds, red_t, &gs, nullptr, &breg);
    } else {
      tile_product<NB, CT, false, true, kPolledPartials, NoSideWork, 0, NoResidentRows, HALF>(
          xhb, (t & 3) * tile_floats, Kpad, w_lds, red_t, &gs);
    }
    if constexpr (!kPolledPartials) __syncthreads();

    float saved[PP][4];  // z, r, g, q of the step for the caller's cache
    float h_pub[PP];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      // z and r: h*R (with x*W when the projection runs here); h*R of g; x*W of g
      float rh[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) rh[g] = 0.f;
      if constexpr (kPolledPartials) {
        // whole wavefronts: the wait is a wavefront-wide vote
        if (((tid + 256 * pp) & ~63) < NB * HS)
          take_product<NB, RCT, NG>(gs, red_t, pl[pp], pc[pp], HS, tid + 256 * pp < NB * HS,
                                    live_partials<CT>(Kpad), rh);
      } else if (act[pp]) {
#pragma unroll
        for (int g = 0; g < NG; ++g) rh[g] = sum_product<NB, RCT>(red, pl[pp], g * HS + pc[pp]);
      }
      if (act[pp]) {
        const float wz = kFusedInput ? 0.f : wx[pp][0], wr = kFusedInput ? 0.f : wx[pp][1];
        const float wg = kFusedInput ? rh[NG - 1] : wx[pp][2];
        const float z = sigmoid_f(wz + rh[0] + bxv[pp][0] + brv[pp][0]);
        const float r = sigmoid_f(wr + rh[1] + bxv[pp][1] + brv[pp][1]);
        const float qg = rh[2] + brv[pp][2];
        const float g = tanh_f(wg + r * qg + bxv[pp][2]);
        saved[pp][0] = z;
        saved[pp][1] = r;
        saved[pp][2] = g;
        saved[pp][3] = qg;
        float h_new = z * h_prev[pp] + (1.0f - z) * g;
        if (zoneout) {
          if (p.training) h_new = (h_new - h_prev[pp]) * mk[pp] + h_prev[pp];
          else h_new = p.zoneout_prob * h_prev[pp] + (1.0f - p.zoneout_prob) * h_new;
        }
        h_prev[pp] = h_new;
      }
      h_pub[pp] = publishable(h_prev[pp]);
    }
    // Everything this wavefront stored during the previous step (its resets among it) has
    // landed before h[t+1] becomes visible.  (x[t+1] arrives with the same wait.)
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
          for (int g = 0; g < 4; ++g) vt[g * H] = saved[pp][g];
        }
        p.h_out[(size_t)t * NH + (size_t)pn[pp] * H + pj[pp]] = h_prev[pp];
      }
    }
  }
}

// The forward pass of a single batch row (see "one batch row" in recurrent.h): 16 hidden units
// x 3 gates per workgroup (the fourth 16 columns of the 64 are idle), the recurrent weights in
// registers.
template <int KW_MAX>
__global__ __launch_bounds__(kSingleRowThreads, 1)
void gru_forward_single_row_kernel(GruFwdParams p) {
  constexpr int HS = kSingleRowUnits, NCOLS = kSingleRowCols;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float (*h_lds)[KW_MAX] = reinterpret_cast<float (*)[KW_MAX]>(lds);
  float (*red)[4][NCOLS] = reinterpret_cast<float (*)[4][NCOLS]>(lds + 4 * KW_MAX);
  // inputs of a step (x*W of the three gates, the mask), parked by the fifth wavefront as in
  // lstm_forward_single_row_kernel
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
  single_row_weights<KW_MAX>(w, p.R, p.dc_mask, p.dc_scale, KW, H, 3 * H, (lane / HS) * H + j0 + lane % HS,
                             lane / HS < 3 && j0 + lane % HS < H);
  for (int i = tid; i < 4 * KW_MAX; i += kSingleRowThreads) (&h_lds[0][0])[i] = 0.f;  // ordered by group_arrive's barrier

  // Pointwise ownership: thread u < 16 handles hidden unit j0 + u.
  const int pj = j0 + tid;
  const bool act = tid < HS && pj < H;
  float h_prev = 0.f, bxv[3] = {0.f, 0.f, 0.f}, brv[3] = {0.f, 0.f, 0.f};
  if (act) {
    h_prev = p.h[pj];
#pragma unroll
    for (int g = 0; g < 3; ++g) {
      bxv[g] = p.bx[g * H + pj];
      brv[g] = p.br[g * H + pj];
    }
  }
  const bool zoneout = p.zoneout_prob != 0.f && p.zoneout_mask != nullptr;
  // Tile 0 receives h[0]; the elements of the other tiles that steps will publish start out
  // unwritten.  One real barrier: nobody polls a tile before all of its owners have set it up.
  if (act) {
    store_exchanged(gs, &xh[pj], publishable(h_prev));
    for (int b = 1; b < kPolledTiles; ++b) store_exchanged(gs, &xh[b * Kpad + pj], unwritten_value());
  }
  // The helper's requests: lane l = 16 g + u asks for x*W of gate g < 3, unit j0 + u; the first
  // sixteen lanes also for the mask.  Every lane loads (some valid address where its element
  // does not exist, and the last step again after the end).
  const bool helper = wave == 4;
  float in_v = 0.f, in_m = 1.f;
  auto request = [&](int t) {
    const int tt = t < T ? t : T - 1;
    const int unit = j0 + lane % HS < H ? j0 + lane % HS : 0;
    const int gate = lane / HS < 3 ? lane / HS : 0;
    in_v = p.Wx[(size_t)tt * 3 * H + (size_t)gate * H + unit];
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
    float wx[3] = {0.f, 0.f, 0.f}, mk = 1.f;
    if (act) {
#pragma unroll
      for (int g = 0; g < 3; ++g) wx[g] = park[t & 1][g][tid];
      mk = park[t & 1][4][tid];
    }

    // The wavefront's share of h[t] (polled tile t % 4) against the thread's weights.
    if (helper) {
      request(t + 2);
    } else {
      red[t & 1][wave][lane] =
          single_row_product<KW_MAX>(gs, xhb, (t & 3) * Kpad + wave * KW, KW, h_lds[wave], w);
    }
    __syncthreads();
    // The owners have read this parity's inputs before the barrier.
    if (helper) park_inputs(t + 2);

    float saved[4] = {0.f, 0.f, 0.f, 0.f};  // z, r, g, q of the step for the caller's cache
    if (act) {
      float rh[3];
#pragma unroll
      for (int g = 0; g < 3; ++g) {
        const float* r = &red[t & 1][0][g * HS + tid];
        rh[g] = (r[0] + r[NCOLS]) + (r[2 * NCOLS] + r[3 * NCOLS]);
      }
      const float z = sigmoid_f(wx[0] + rh[0] + bxv[0] + brv[0]);
      const float r = sigmoid_f(wx[1] + rh[1] + bxv[1] + brv[1]);
      const float qg = rh[2] + brv[2];
      const float g = tanh_f(wx[2] + r * qg + bxv[2]);
      saved[0] = z;
      saved[1] = r;
      saved[2] = g;
      saved[3] = qg;
      float h_new = z * h_prev + (1.0f - z) * g;
      if (zoneout) {
        if (p.training) h_new = (h_new - h_prev) * mk + h_prev;
        else h_new = p.zoneout_prob * h_prev + (1.0f - p.zoneout_prob) * h_new;
      }
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
        for (int g = 0; g < 4; ++g) vt[g * H] = saved[g];
      }
      p.h_out[(size_t)t * H + pj] = h_prev;
    }
  }
}

struct GruBwdParams {
  int T, N, H;
  const float* R_t;     // [3H,H]
  const float* h;       // [T,N,H] states before each step
  const float* v;       // [T,N,4H]
  const float* dh_next; // [T,N,H] upstream gradient of the h each step produced
  float* dbx;           // [3H] accumulated
  float* dbr;           // [3H] accumulated
  float* dh;            // [N,H] in/out
  float* dp;            // [T,N,3H]
  float* dq;            // [T,N,3H]
  const float* zoneout_mask;
  float* db_partial;    // [batch tiles, 6H] scratch
  float* xdq;           // exchange tiles of dq: [batch tiles][2][Kpad/4][NB][4]
                        // (scattered form: the pieces of partial sums, scatter_backward.h)
  LaunchShape ls;
};

// Contraction length of the backward recurrence inside the launch: k = 3*unit + gate over
// the 16 units of every column workgroup, padded to the MFMA granularity.
inline int gru_backward_k(int H) { return 48 * ((H + 15) / 16); }


// A workgroup owns 16 hidden units for NB batch rows; its slice of R_t is [3H x 16].
// Inside the launch the contraction index runs unit-major (k = 3*unit + gate), so every
// workgroup publishes one contiguous k range of the exchange tile.  SETS sets of 256 threads,
// each with a batch tile of NB rows of its own (see gru_forward_kernel).
// REG > 0: the slice exceeds LDS; every wavefront keeps the first REG k-groups of its share
// of the contraction in registers (tall_tile_product).
template <int NB, int SETS, int REG = 0>
__global__ __launch_bounds__(256 * SETS, 1)
void gru_backward_kernel(GruBwdParams p) {
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
  const int Kpad = round_up(48 * p.ls.gx, 64);
  const int set = set_index<SETS>();
  float* w_lds = lds;
  // the partial tiles or NB*6*16 floats, whichever is more (two sets: two polled areas of
  // partial tiles each, alternating by step)
  float* red = lds + (Kpad - 64 * REG) * NCOLS + (SETS == 1 ? 0 : set * 2 * RED);

  const int tid = set_thread<SETS>();
  const int j0 = role.cw * HSB;
  const int bt = role.bt * SETS + set;  // this set's batch tile
  const int n0 = bt * NB;
  const int rows_here = (N - n0) < NB ? (N - n0) : NB;  // <= 0: a set without rows
  const size_t NH = (size_t)N * H;

  const int tile_floats = Kpad * NB;
  float* xdq = p.xdq + (size_t)bt * kPolledTiles * tile_floats;
  const TileBuffer xdqb = make_tile_buffer(xdq, kPolledTiles * tile_floats);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);

  // Own k range of the exchange tiles (the last workgroup also owns the padding); only
  // rows and units of the problem are written afterwards.
  zero_tile_share<SETS>(gs, xdq, tile_floats, NB, 12 * role.cw,
                        (role.cw == p.ls.gx - 1 ? Kpad - 48 * role.cw : 48) / 4, kPolledTiles);

  float4_t breg[REG > 0 ? REG : 1][1];
  {
    const bool fast = H % 4 == 0 && (reinterpret_cast<uintptr_t>(p.R_t) & 15u) == 0;
    auto offset = [=](int k, int col) {
      const int unit = k / 3, gate = k % 3;
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
  float dh[PP], dbacc[PP][6];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    pl[pp] = idx / HSB;
    pc[pp] = idx % HSB;
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    act[pp] = idx < NB * HSB && pl[pp] < rows_here && pj[pp] < H;
    dh[pp] = act[pp] ? p.dh[(size_t)pn[pp] * H + pj[pp]] : 0.f;
#pragma unroll
    for (int g = 0; g < 6; ++g) dbacc[pp][g] = 0.f;
  }
  const bool zoneout = p.zoneout_mask != nullptr;
  // The elements that steps will publish start out unwritten (rows and units beyond the
  // problem stay zero).  One real barrier: nobody polls a tile before its owners have set
  // it up.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (act[pp])
      for (int b = 0; b < kPolledTiles; ++b)
        for (int g = 0; g < 3; ++g)
          store_exchanged(gs, xdq + (size_t)b * tile_floats + xchg_index(3 * pj[pp] + g, pl[pp], NB),
                          unwritten_value());
  if constexpr (SETS == 2) reset_partials<NB, 1>(red, live_partials<1>(Kpad));
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);

  struct StepIn { float vt[4], h0, dhn, m; };
  StepIn nxt[PP];
  // Every thread loads (threads without an element, and the request after the last step, some
  // valid address: their values are never used) and nothing but the loads writes `nxt` inside
  // the loop (see lstm_backward_kernel).
  {
    const StepIn nxt_init = {{0.f, 0.f, 0.f, 0.f}, 0.f, 0.f, 1.f};
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) nxt[pp] = nxt_init;
  }
  auto fetch = [&](int t) {
    const int tt = t >= 0 ? t : 0;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      const size_t e = (size_t)tt * NH + row * H + unit;
      const float* vt = p.v + ((size_t)tt * N + row) * 4 * H + unit;
#pragma unroll
      for (int g = 0; g < 4; ++g) nxt[pp].vt[g] = vt[g * H];
      nxt[pp].h0 = p.h[e];
      nxt[pp].dhn = p.dh_next[e];
      if (zoneout) nxt[pp].m = p.zoneout_mask[e];
    }
  };
  fetch(T - 1);

  // A set without rows skips the steps (two sets: no workgroup barrier inside them).
  for (int t = (SETS == 2 && rows_here <= 0) ? -1 : T - 1; t >= 0; --t) {
    float dh_keep[PP], dpv[PP][3], dqv[PP];
    const int done = T - 1 - t;  // steps done so far; this step uses polled tile done % 4
    float* xdq_t = xdq + (done & 3) * tile_floats;
    float* xdq_done = xdq + ((done + 2) & 3) * tile_floats;  // read two steps ago
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      dh_keep[pp] = 0.f;
      if (act[pp]) {
        const StepIn s = nxt[pp];
        const float z = s.vt[0], r = s.vt[1], g = s.vt[2], qg = s.vt[3];
        float dh_total = s.dhn + dh[pp];
        if (zoneout) {
          dh_keep[pp] = (1.0f - s.m) * dh_total;
          dh_total = s.m * dh_total;
          dh_keep[pp] += z * dh_total;
        } else {
          dh_keep[pp] = z * dh_total;
        }
        const float dg = (1.0f - z) * dh_total;
        const float dz = (s.h0 - g) * dh_total;
        const float dp_g = d_tanh_f(g) * dg;
        const float dq_g = dp_g * r;
        const float dr = dp_g * qg;
        const float dp_r = d_sigmoid_f(r) * dr;
        const float dp_z = d_sigmoid_f(z) * dz;
        dpv[pp][0] = dp_z;
        dpv[pp][1] = dp_r;
        dpv[pp][2] = dp_g;
        dqv[pp] = dq_g;
        dbacc[pp][0] += dp_z;
        dbacc[pp][1] += dp_r;
        dbacc[pp][2] += dp_g;
        dbacc[pp][3] += dp_z;
        dbacc[pp][4] += dp_r;
        dbacc[pp][5] += dq_g;
      }
    }
    // What this wavefront stored during the previous step (its resets among it) has landed
    // before the gate gradients of this step become visible.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
      if (act[pp]) {
        const float q[3] = {dpv[pp][0], dpv[pp][1], dqv[pp]};
#pragma unroll
        for (int g = 0; g < 3; ++g) {
          const int e = xchg_index(3 * pj[pp] + g, pl[pp], NB);
          store_exchanged(gs, xdq_t + e, publishable(q[g]));
          if (done + 2 < T) store_exchanged(gs, xdq_done + e, unwritten_value());
        }
      }
    // The caller's copies: nobody in the launch waits for them.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if (act[pp]) {
        const size_t o3 = ((size_t)t * N + pn[pp]) * 3 * H + pj[pp];
        p.dp[o3] = dpv[pp][0];
        p.dp[o3 + H] = dpv[pp][1];
        p.dp[o3 + 2 * H] = dpv[pp][2];
        p.dq[o3] = dpv[pp][0];
        p.dq[o3 + H] = dpv[pp][1];
        p.dq[o3 + 2 * H] = dqv[pp];
      }
    }
    fetch(t - 1);
    // The operand loads wait for dq_t of every unit themselves.
    float* red_t = !kPolledPartials ? red : red + (done & 1) * RED;
    if constexpr (REG > 0)
      tile_product<NB, 1, true, true, false, NoSideWork, REG, float4_t[REG][1]>(
          xdqb, (done & 3) * tile_floats, Kpad, w_lds, red_t, &gs, nullptr, &breg);
    else
      tile_product<NB, 1, true, true, kPolledPartials>(xdqb, (done & 3) * tile_floats, Kpad, w_lds, red_t, &gs);
    if constexpr (kPolledPartials) {
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        if (((tid + 256 * pp) & ~63) < NB * HSB) {  // whole wavefronts: the wait is a vote
          float rdq[1];
          take_product<NB, 1, 1>(gs, red_t, pl[pp], pc[pp], 0, tid + 256 * pp < NB * HSB,
                                 live_partials<1>(Kpad), rdq);
          if (tid + 256 * pp < NB * HSB) dh[pp] = dh_keep[pp] + rdq[0];
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
  for (int pp = 0; pp < PP; ++pp)
    if (act[pp]) p.dh[(size_t)pn[pp] * H + pj[pp]] = dh[pp];

  __syncthreads();
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (tid + 256 * pp < NB * HSB) {
#pragma unroll
      for (int g = 0; g < 6; ++g) red[(pl[pp] * 6 + g) * HSB + pc[pp]] = act[pp] ? dbacc[pp][g] : 0.f;
    }
  __syncthreads();
  if (tid < 6 * HSB) {
    const int g = tid / HSB, jj = tid % HSB;
    float s = 0.f;
    for (int r = 0; r < NB; ++r) s += red[(r * 6 + g) * HSB + jj];
    if (j0 + jj < H) store_agent(&p.db_partial[(size_t)bt * 6 * H + g * H + j0 + jj], s);
  }
  if (column_last_arrival(p.ls.cb, role.cw, (unsigned)p.ls.gy, &s_flag)) {
    if (set == 0 && tid < 6 * HSB && j0 + tid % HSB < H) {
      const int col = (tid / HSB) * H + j0 + tid % HSB;
      const float s = sum_over_tiles(p.db_partial + col, (size_t)6 * H, p.ls.gy * SETS);
      if (col < 3 * H) p.dbx[col] += s;
      else p.dbr[col - 3 * H] += s;
    }
  }
}

// The GRU's pointwise backward step for the scattered form of the recurrence
// (scatter_backward.h): arithmetic as in gru_backward_kernel.  dh contracts over
// dq = (dp_z, dp_r, dq_g); the operand's fourth component carries dp_g for the caller's copy.
struct GruScatterCell {
  using Params = GruBwdParams;
  static constexpr int kGates = 3;
  static constexpr int kInputs = 7;  // v (z, r, g, q_g), h before the step, dh_next, mask
  static constexpr int kSums = 6;    // dbx (3), dbr (3)
  float dh, dh_keep;
  float z, r, g, qg, h0, dhn, m, k_g, k_r, k_z;

  __device__ __forceinline__ static float* pieces(const Params& p) { return p.xdq; }
  __device__ __forceinline__ static void request(const Params& p, float (&in)[kInputs], size_t e, size_t ve,
                                                 bool zoneout) {
    const float* vt = p.v + ve;
#pragma unroll
    for (int i = 0; i < 4; ++i) in[i] = vt[i * (size_t)p.H];
    in[4] = p.h[e];
    in[5] = p.dh_next[e];
    if (zoneout) in[6] = p.zoneout_mask[e];
  }
  __device__ __forceinline__ void load_state(const Params& p, size_t e, bool mine) {
    dh = mine ? p.dh[e] : 0.f;
    dh_keep = 0.f;
  }
  __device__ __forceinline__ void store_state(const Params& p, size_t e) const { p.dh[e] = dh; }
  __device__ __forceinline__ void prepare(const float (&sv)[kInputs]) {
    z = sv[0]; r = sv[1]; g = sv[2]; qg = sv[3];
    h0 = sv[4]; dhn = sv[5]; m = sv[6];
    k_g = d_tanh_f(g);
    k_r = d_sigmoid_f(r);
    k_z = d_sigmoid_f(z);
  }
  __device__ __forceinline__ void add_gathered(float sum) { dh = dh_keep + sum; }
  __device__ __forceinline__ float4_t step(bool act, bool zoneout, float (&sums)[kSums]) {
    float4_t a = {0.f, 0.f, 0.f, 0.f};
    dh_keep = 0.f;
    if (act) {
      float dh_total = dhn + dh;
      if (zoneout) {
        dh_keep = (1.0f - m) * dh_total;
        dh_total = m * dh_total;
        dh_keep += z * dh_total;
      } else {
        dh_keep = z * dh_total;
      }
      const float dg = (1.0f - z) * dh_total;
      const float dz = (h0 - g) * dh_total;
      const float dp_g = k_g * dg;
      const float dq_g = dp_g * r;
      const float dr = dp_g * qg;
      const float dp_r = k_r * dr;
      const float dp_z = k_z * dz;
      a = float4_t{dp_z, dp_r, dq_g, dp_g};
      sums[0] += dp_z;
      sums[1] += dp_r;
      sums[2] += dp_g;
      sums[3] += dp_z;
      sums[4] += dp_r;
      sums[5] += dq_g;
    }
    return a;
  }
  __device__ __forceinline__ static void store_copy(const Params& p, int t, size_t n, size_t j, const float4_t& a) {
    const size_t H = p.H;
    const size_t o3 = ((size_t)t * p.N + n) * 3 * H + j;
    p.dp[o3] = a[0];
    p.dp[o3 + H] = a[1];
    p.dp[o3 + 2 * H] = a[3];
    p.dq[o3] = a[0];
    p.dq[o3 + H] = a[1];
    p.dq[o3 + 2 * H] = a[2];
  }
  __device__ __forceinline__ static void add_sums(const Params& p, int col, float s) {
    if (col < 3 * p.H) p.dbx[col] += s;
    else p.dbr[col - 3 * p.H] += s;
  }
};

}  // namespace

// The forward pass of a single batch row with H <= 512: the recurrent weights live in the
// registers of the 16-unit workgroups of one XCD (gru_forward_single_row_kernel).
int gru_forward_single_row(hipStream_t stream, int training, int T, int C, int H, const float* W,
                           const float* R, const float* bx, const float* br, const float* x,
                           const float* h, float* h_out, float* v, float* tmp_Wx, float zoneout_prob,
                           const float* zoneout_mask, const float* dc_mask, float dc_scale, bool wx_ready) {
  if (!wx_ready)
    HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T, 3 * H, C, x, C, W, 3 * H, tmp_Wx, 3 * H, false));
  const int Kpad = (H + 63) / 64 * 64;
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, (size_t)kPolledTiles * Kpad * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));
  GruFwdParams p;
  p.training = training; p.T = T; p.N = 1; p.H = H;
  p.R = R; p.bx = bx; p.br = br; p.h = h; p.h_out = h_out; p.v = v; p.Wx = tmp_Wx;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.dc_mask = dc_mask; p.dc_scale = dc_scale;
  p.xh = ws.scratch;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, (H + 15) / 16, 1, 1,
                                  single_row_lds_bytes(single_row_kw_max(Kpad)) + kSingleRowParkBytes,
                                  (unsigned)T + 1, &plan));
  plan.threads = kSingleRowThreads;
  p.ls = plan.shape;
  const char* name = "gru_forward_recurrence";
  if (Kpad <= 128) return launch_persistent(name, gru_forward_single_row_kernel<32>, plan, p, stream);
  if (Kpad <= 256) return launch_persistent(name, gru_forward_single_row_kernel<64>, plan, p, stream);
  return launch_persistent(name, gru_forward_single_row_kernel<128>, plan, p, stream);
}

// True when a pass over more than one step keeps the recurrent weights on chip (the persistent
// kernels) instead of streaming them every step: then the recurrence can be run by itself, on
// products computed elsewhere (wx_ready / products below).
bool gru_forward_resident(int N, int H) {
  if (N == 1 && H <= 512 && xcd_local_fits((H + 15) / 16, 1)) return true;
  return pick_forward_tile(3, N, H, 0, kWorkgroupLdsBytes, false, 3).ok;
}
bool gru_backward_resident(int N, int H) {
  return pick_backward_tile(gru_backward_k(H), N, H, 6 * 16, 0, true).ok;
}

// h: [N,H] state before the first step; h_out: [T,N,H] states after each step.
// wx_ready (T > 1, gru_forward_resident): tmp_Wx already holds x*W, and W and x are not looked at.
// half_product: the tensors are widened half tensors (gru_half.hip); with 4-row tiles the step's
// product h * R goes to the half matrix cores (h rounded to half there, as such a cell stores it).
int gru_forward_impl(hipStream_t stream, int training, int T, int N, int C, int H,
                     const float* W, const float* R, const float* bx, const float* br,
                     const float* x, const float* h, float* h_out, float* v, float* tmp_Wx,
                     float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                     float dc_scale, bool wx_ready, bool half_product) {
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(R && bx && br && h && h_out && tmp_Wx && (wx_ready || (W && x)));
  HASTE_HIP_REQUIRE(!training || v != nullptr);
  HASTE_HIP_REQUIRE(!wx_ready || (T > 1 && gru_forward_resident(N, H)));
  // A single step of a small batch (Iterate): one kernel, nothing kept on chip (tmp_Wx is
  // scratch of the other paths and is left alone).
  if (T == 1 && single_step_applies(N, C, H))
    return gru_forward_single_step(stream, training, N, C, H, W, R, bx, br, x, h, h_out, v,
                                   zoneout_prob, zoneout_mask, dc_mask, dc_scale);
  if (N == 1 && H <= 512 && xcd_local_fits((H + 15) / 16, 1))
    return gru_forward_single_row(stream, training, T, C, H, W, R, bx, br, x, h, h_out, v, tmp_Wx,
                                  zoneout_prob, zoneout_mask, dc_mask, dc_scale, wx_ready);
  const ForwardTile tile = pick_forward_tile(3, N, H, 0, kWorkgroupLdsBytes, false, 3);
  // No slice of R fits a CU: stream R from HBM every step instead.
  if (!tile.ok)
    return gru_forward_streamed(stream, training, T, N, C, H, W, R, bx, br, x, h, h_out, v, tmp_Wx,
                                zoneout_prob, zoneout_mask, dc_mask, dc_scale);
  // An 8-row tile is run as two sets of 4 rows when the partial tiles of both fit beside the
  // slice (exchange tiles: one per set, together as large as the tile's).
  const int Kpad = (H + 63) / 64 * 64;
  size_t paired_lds = paired_lds_bytes(Kpad, tile.ct);
  const bool paired = tile.nb == 8 && paired_lds <= kWorkgroupLdsBytes &&
                      tile.reg_groups == 0;
  // 4-row tiles of 16-unit workgroups compute x*W themselves, beside their waits, when a
  // wavefront's share of W (C/4 x 48 columns) fits its registers (the step's x*W GEMM, its split
  // reduce and the round trip of tmp_Wx through memory go away).  The partial tiles then have
  // rows of 64 columns: the slice's 48 and the candidate gate's x*W.
  const bool fused = !wx_ready && !half_product && (paired || tile.nb == 4) && tile.hs == 16 &&
                     tile.reg_groups == 0 && C <= 512 && C % 4 == 0 &&
                     (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && fused_input_enabled();
  const int xsg = C <= 256 ? 1 : 2;
  size_t lds_bytes = paired ? paired_lds : tile.lds_bytes;
  if (fused)
    lds_bytes = ((size_t)Kpad * 48 + (paired ? 4 : 1) * (size_t)ProductTile<4, 4>::kRedFloats) * sizeof(float);
  if (!wx_ready && !fused)
    HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T * N, 3 * H, C, x, C, W, 3 * H, tmp_Wx, 3 * H, false));

  // Taken after the GEMM, which may replace the stream's scratch buffer with a larger one.
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(
      stream, exchange_floats(H, tile.nb, tile.gy, kPolledTiles) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  GruFwdParams p;
  p.training = training; p.T = T; p.N = N; p.H = H;
  p.R = R; p.bx = bx; p.br = br; p.h = h; p.h_out = h_out; p.v = v; p.Wx = tmp_Wx;
  p.W = W; p.x = x; p.C = C;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.dc_mask = dc_mask; p.dc_scale = dc_scale;
  p.xh = ws.scratch;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, tile.gx, tile.gy, tile.nb, lds_bytes, (unsigned)T + 1, &plan));
  p.ls = plan.shape;
  if (paired) plan.threads = 512;
#define HASTE_LAUNCH_FWD_FUSED(XSG_)                                                                       \
  if (fused && xsg == XSG_) {                                                                              \
    if (paired)                                                                                            \
      return launch_persistent("gru_forward_recurrence", gru_forward_kernel<4, 3, 16, 2, 0, false, XSG_>,  \
                               plan, p, stream);                                                           \
    return launch_persistent("gru_forward_recurrence", gru_forward_kernel<4, 3, 16, 1, 0, false, XSG_>,    \
                             plan, p, stream);                                                             \
  }
  HASTE_LAUNCH_FWD_FUSED(1) HASTE_LAUNCH_FWD_FUSED(2)
#undef HASTE_LAUNCH_FWD_FUSED
#define HASTE_LAUNCH_FWD_RESIDENT(NB_, CT_, HS_, REG_)                                              \
  if (tile.reg_groups == REG_ && tile.nb == NB_ && tile.hs == HS_)                                 \
    return launch_persistent("gru_forward_recurrence", gru_forward_kernel<NB_, CT_, HS_, 1, REG_>, \
                             plan, p, stream);
  HASTE_LAUNCH_FWD_RESIDENT(16, 2, 8, 8) HASTE_LAUNCH_FWD_RESIDENT(32, 2, 8, 8) HASTE_LAUNCH_FWD_RESIDENT(64, 2, 8, 8)
  HASTE_LAUNCH_FWD_RESIDENT(16, 2, 8, 16) HASTE_LAUNCH_FWD_RESIDENT(32, 2, 8, 16) HASTE_LAUNCH_FWD_RESIDENT(64, 2, 8, 16)
  HASTE_LAUNCH_FWD_RESIDENT(16, 3, 16, 8) HASTE_LAUNCH_FWD_RESIDENT(32, 3, 16, 8) HASTE_LAUNCH_FWD_RESIDENT(64, 3, 16, 8)
#undef HASTE_LAUNCH_FWD_RESIDENT
  if (tile.reg_groups > 0) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
#define HASTE_LAUNCH_FWD_PAIRED(CT_, HS_)                                                     \
  if (paired && tile.hs == HS_ && half_product)                                               \
    return launch_persistent("gru_forward_recurrence", gru_forward_kernel<4, CT_, HS_, 2, 0, true>, \
                             plan, p, stream);                                                \
  if (paired && tile.hs == HS_)                                                               \
    return launch_persistent("gru_forward_recurrence", gru_forward_kernel<4, CT_, HS_, 2>,    \
                             plan, p, stream);
  HASTE_LAUNCH_FWD_PAIRED(1, 4) HASTE_LAUNCH_FWD_PAIRED(2, 8) HASTE_LAUNCH_FWD_PAIRED(3, 16)
#undef HASTE_LAUNCH_FWD_PAIRED
#define HASTE_LAUNCH_FWD(NB_, CT_, HS_)                                                       \
  if (tile.nb == NB_ && tile.hs == HS_)                                                       \
    return launch_persistent("gru_forward_recurrence", gru_forward_kernel<NB_, CT_, HS_, 1>,  \
                             plan, p, stream);
#define HASTE_LAUNCH_FWD_HALF(CT_, HS_)                                                             \
  if (half_product && tile.nb == 4 && tile.hs == HS_)                                               \
    return launch_persistent("gru_forward_recurrence", gru_forward_kernel<4, CT_, HS_, 1, 0, true>, \
                             plan, p, stream);
  HASTE_LAUNCH_FWD_HALF(1, 4) HASTE_LAUNCH_FWD_HALF(2, 8) HASTE_LAUNCH_FWD_HALF(3, 16)
#undef HASTE_LAUNCH_FWD_HALF
  HASTE_LAUNCH_FWD(4, 1, 4) HASTE_LAUNCH_FWD(4, 2, 8) HASTE_LAUNCH_FWD(4, 3, 16)
  HASTE_LAUNCH_FWD(8, 1, 4) HASTE_LAUNCH_FWD(8, 2, 8) HASTE_LAUNCH_FWD(8, 3, 16)
  HASTE_LAUNCH_FWD(16, 1, 4) HASTE_LAUNCH_FWD(16, 2, 8) HASTE_LAUNCH_FWD(16, 3, 16)
  HASTE_LAUNCH_FWD(32, 1, 4) HASTE_LAUNCH_FWD(32, 2, 8) HASTE_LAUNCH_FWD(32, 3, 16)
  HASTE_LAUNCH_FWD(64, 1, 4) HASTE_LAUNCH_FWD(64, 2, 8) HASTE_LAUNCH_FWD(64, 3, 16)
#undef HASTE_LAUNCH_FWD
  return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
}

// products == false (gru_backward_resident): the recurrence only -- dp, dq, dbx, dbr, dh; the
// caller computes dx, dW and dR from dp and dq itself, and W_t, x_t, dx, dW, dR are not looked at.
// half_product: the tensors are widened half tensors (gru_half.hip); where the scattered form
// runs, its product dh = (gate gradients) * R_t goes to the half matrix cores.
int gru_backward_impl(hipStream_t stream, int T, int N, int C, int H,
                      const float* W_t, const float* R_t, const float* x_t, const float* h,
                      const float* v, const float* dh_next, float* dx, float* dW, float* dR,
                      float* dbx, float* dbr, float* dh, float* dp, float* dq,
                      const float* zoneout_mask, bool products, bool half_product) {
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(R_t && h && v && dh_next && (!products || (W_t && x_t)));
  HASTE_HIP_REQUIRE(dbx && dbr && dh && dp && dq && (!products || (dx && dW && dR)));
  HASTE_HIP_REQUIRE(products || gru_backward_resident(N, H));
  // per row: the partial tiles or the 6 bias-gradient columns of 16 floats
  const BackwardTile tile = pick_backward_tile(gru_backward_k(H), N, H, 6 * 16, 0, true);
  if (!tile.ok)
    return gru_backward_streamed(stream, T, N, C, H, W_t, R_t, x_t, h, v, dh_next, dx, dW, dR, dbx,
                                 dbr, dh, dp, dq, zoneout_mask);

  // An 8-row tile is run as two sets of 4 rows (see gru_forward_impl).
  const size_t paired_lds = paired_lds_bytes((gru_backward_k(H) + 63) / 64 * 64, 1);
  // 4-row tiles (8 rows: two sets of 4) with H <= 512 take the scattered form: partial sums of
  // dh go to their owners instead of the gate gradients to everybody.
  // (Measured over H = 64 ... 512, T = 100: with two sets per workgroup it is 5-15 % faster
  // at every H, with one set from H = 384 on; below, one set is 5-20 % faster the other way.)
  const bool scatter = tile.reg_groups == 0 && H <= 512 &&
                       (tile.nb == 8 || (tile.nb == 4 && H > 320));
  const bool paired = scatter ? tile.nb == 8
                              : tile.nb == 8 && paired_lds <= kMaxLdsBytes;
  const int sets = paired ? 2 : 1;

  Workspace ws;
  const size_t db_floats = ((size_t)tile.gy * sets * 6 * H + 3) / 4 * 4;
  const size_t xdq_floats =
      scatter ? (size_t)tile.gy * sets * kScatterTiles * scatter_tile_floats(tile.gx, H <= 256 ? 1 : 2)
              : exchange_floats(gru_backward_k(H), tile.nb, tile.gy, kPolledTiles);
  HASTE_HIP_PROPAGATE(get_workspace(stream, (db_floats + xdq_floats) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  GruBwdParams p;
  p.T = T; p.N = N; p.H = H;
  p.R_t = R_t; p.h = h; p.v = v; p.dh_next = dh_next;
  p.dbx = dbx; p.dbr = dbr; p.dh = dh; p.dp = dp; p.dq = dq; p.zoneout_mask = zoneout_mask;
  p.db_partial = ws.scratch;
  p.xdq = ws.scratch + db_floats;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, tile.gx, tile.gy, tile.nb,
                                  scatter ? sets * kScatterSetFloats * sizeof(float)
                                          : (paired ? paired_lds : tile.lds_bytes),
                                  (unsigned)T + 1, &plan));
  p.ls = plan.shape;
  if (paired) plan.threads = 512;
  int rc = HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  const char* name = "gru_backward_recurrence";
  if (scatter && half_product) rc = launch_scatter_backward<GruScatterCell, true>(name, H, sets, plan, p, stream);
  else if (scatter) rc = launch_scatter_backward<GruScatterCell>(name, H, sets, plan, p, stream);
  else
#define HASTE_LAUNCH_BWD_RESIDENT(NB_)                                                           \
  (tile.reg_groups == 8    ? launch_persistent(name, gru_backward_kernel<NB_, 1, 8>, plan, p, stream)  \
   : tile.reg_groups == 16 ? launch_persistent(name, gru_backward_kernel<NB_, 1, 16>, plan, p, stream) \
   : tile.reg_groups == 24 ? launch_persistent(name, gru_backward_kernel<NB_, 1, 24>, plan, p, stream) \
                           : launch_persistent(name, gru_backward_kernel<NB_, 1, 32>, plan, p, stream))
  if (tile.reg_groups > 0) {
    if (tile.nb == 16) rc = HASTE_LAUNCH_BWD_RESIDENT(16);
    else if (tile.nb == 32) rc = HASTE_LAUNCH_BWD_RESIDENT(32);
    else if (tile.nb == 64) rc = HASTE_LAUNCH_BWD_RESIDENT(64);
  }
#undef HASTE_LAUNCH_BWD_RESIDENT
  else if (paired) rc = launch_persistent(name, gru_backward_kernel<4, 2>, plan, p, stream);
  else if (tile.nb == 4) rc = launch_persistent(name, gru_backward_kernel<4, 1>, plan, p, stream);
  else if (tile.nb == 8) rc = launch_persistent(name, gru_backward_kernel<8, 1>, plan, p, stream);
  else if (tile.nb == 16) rc = launch_persistent(name, gru_backward_kernel<16, 1>, plan, p, stream);
  else if (tile.nb == 32) rc = launch_persistent(name, gru_backward_kernel<32, 1>, plan, p, stream);
  else if (tile.nb == 64) rc = launch_persistent(name, gru_backward_kernel<64, 1>, plan, p, stream);
  HASTE_HIP_PROPAGATE(rc);
  if (!products) return HASTE_HIP_OK;

  const int TN = T * N;
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, TN, C, 3 * H, dp, 3 * H, W_t, C, dx, C, false));
  // dW += x^T dp and dR += h^T dq: one launch when that halves their K pieces
  HASTE_HIP_PROPAGATE(gemm_f32_pair(stream, C, H, 3 * H, TN, x_t, TN, dp, 3 * H, dW, 3 * H,
                                    h, H, dq, 3 * H, dR, 3 * H, true));
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" {

int haste_hip_gru_forward_f32(int training, int steps, int batch_size, int input_size,
                              int hidden_size,
                              const float* W, const float* R, const float* bx, const float* br,
                              const float* x, float* h, float* v, float* tmp_Wx, float* tmp_Rh,
                              float zoneout_prob, const float* zoneout_mask, void* stream) {
  (void)tmp_Rh;
  HASTE_HIP_REQUIRE(h && batch_size > 0 && hidden_size > 0);
  return haste_hip::gru_forward_impl(haste_hip::as_stream(stream), training, steps, batch_size,
                                     input_size, hidden_size, W, R, bx, br, x, h,
                                     h + (size_t)batch_size * hidden_size, v, tmp_Wx,
                                     zoneout_prob, zoneout_mask, nullptr, 1.0f, false, false);
}

int haste_hip_gru_forward_dropconnect_f32(int training, int steps, int batch_size,
                                          int input_size, int hidden_size,
                                          const float* W, const float* R, const float* bx,
                                          const float* br, const float* x, float* h, float* v,
                                          float* tmp_Wx, float zoneout_prob,
                                          const float* zoneout_mask,
                                          const float* dropconnect_mask, float dropconnect_scale,
                                          void* stream) {
  HASTE_HIP_REQUIRE(h && batch_size > 0 && hidden_size > 0);
  return haste_hip::gru_forward_impl(haste_hip::as_stream(stream), training, steps, batch_size,
                                     input_size, hidden_size, W, R, bx, br, x, h,
                                     h + (size_t)batch_size * hidden_size, v, tmp_Wx,
                                     zoneout_prob, zoneout_mask, dropconnect_mask,
                                     dropconnect_scale, false, false);
}

int haste_hip_gru_backward_f32(int steps, int batch_size, int input_size, int hidden_size,
                               const float* W_t, const float* R_t, const float* bx,
                               const float* br, const float* x_t, const float* h, const float* v,
                               const float* dh_new, float* dx, float* dW, float* dR,
                               float* dbx, float* dbr, float* dh, float* dp, float* dq,
                               const float* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  HASTE_HIP_REQUIRE(dh_new && batch_size > 0 && hidden_size > 0);
  return haste_hip::gru_backward_impl(haste_hip::as_stream(stream), steps, batch_size, input_size,
                                      hidden_size, W_t, R_t, x_t, h, v,
                                      dh_new + (size_t)batch_size * hidden_size, dx, dW, dR, dbx,
                                      dbr, dh, dp, dq, zoneout_mask, true, false);
}

int haste_hip_gru_forward_iterate_f32(int training, int batch_size, int input_size,
                                      int hidden_size,
                                      const float* W, const float* R, const float* bx,
                                      const float* br, const float* x, const float* h,
                                      float* h_out, float* v, float* tmp_Wx, float* tmp_Rh,
                                      float zoneout_prob, const float* zoneout_mask,
                                      void* stream) {
  (void)tmp_Rh;
  return haste_hip::gru_forward_impl(haste_hip::as_stream(stream), training, 1, batch_size,
                                     input_size, hidden_size, W, R, bx, br, x, h, h_out, v, tmp_Wx,
                                     zoneout_prob, zoneout_mask, nullptr, 1.0f, false, false);
}

int haste_hip_gru_backward_iterate_f32(int batch_size, int input_size, int hidden_size,
                                       const float* W_t, const float* R_t, const float* bx,
                                       const float* br, const float* x_t, const float* h,
                                       const float* v, const float* dh_new, float* dx, float* dW,
                                       float* dR, float* dbx, float* dbr, float* dh, float* dp,
                                       float* dq, const float* zoneout_mask, void* stream) {
  (void)bx;
  (void)br;
  return haste_hip::gru_backward_impl(haste_hip::as_stream(stream), 1, batch_size, input_size,
                                      hidden_size, W_t, R_t, x_t, h, v, dh_new, dx, dW, dR, dbx,
                                      dbr, dh, dp, dq, zoneout_mask, true, false);
}

}  // extern "C"
