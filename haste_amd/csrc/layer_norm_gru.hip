// LayerNormGRU forward and backward passes.
//
// Forward: GEMM x*W, stand-alone layer norm over all T*N rows, then one persistent
// kernel in which the per-step layer norm of h*R (3H columns) is computed inside the
// step through a per-row moment exchange (two group barriers per step).  Backward
// mirrors it in reverse time, then a stand-alone layer-norm backward and three GEMMs.
//
// Arithmetic follows reference lib/layer_norm_gru_forward_gpu.cu.cc:25-83 and
// lib/layer_norm_gru_backward_gpu.cu.cc:25-95; orchestration replaces :242-305 and :219-310.
#include "ln_exchange.h"

namespace haste_hip {
namespace {

struct LnGruFwdParams {
  int training, T, N, H;
  const float* R;        // [H,3H]
  const float* bx;       // [3H]
  const float* br;       // [3H]
  float* h;              // [T+1,N,H]
  float* v;              // [T,N,4H] or null
  const float* Wxn;      // [T,N,3H] LN1(x*W)
  float* act_Rh;         // [T,N,3H] out
  const float* gamma2;   // [3H]
  float* cache2;         // [T*N,2] or null
  float zoneout_prob;
  const float* zoneout_mask;
  unsigned long long* part2;  // tagged row exchange [groups][2][gx][NB] slots: moments of h*R
  float* xh;             // exchange tiles of h: [batch tiles][2][Kpad/4][NB][4]
  LaunchShape ls;
};

// NB batch rows per workgroup.  REG > 0 (tiles of 16 rows and more): the slice exceeds LDS; every
// wavefront keeps the first REG k-groups of its share of the contraction in registers
// (tall_tile_product).
template <int NB, int CT, int HS, int REG = 0>
__global__ __launch_bounds__(256, 1)
void ln_gru_forward_kernel(LnGruFwdParams p) {
  static_assert(3 * HS <= 16 * CT, "slice too narrow");
  static_assert(REG == 0 || NB >= 16, "register-resident slice rows: tall tiles only");
  constexpr int NCOLS = 16 * CT;
  constexpr int PP = (NB * HS + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ unsigned int s_role;
  const Role role = take_role(p.ls, &s_role);
  if (!role.active) return;

  const int H = p.H, N = p.N, T = p.T;
  const int Kpad = round_up(H, 64);
  float* w_lds = lds;
  float* red = lds + (Kpad - 64 * REG) * NCOLS;
  float* stat = red + ProductTile<NB, CT>::kRedFloats;  // [NB][2] row statistics (long rows only)

  const int tid = threadIdx.x;
  const int gx = p.ls.gx;
  const bool in_wavefront = row_gather_in_wavefront<HS, NB>(gx);
  const int j0 = role.cw * HS;
  const int n0 = role.bt * p.ls.tile_rows;
  const int rows_here = (N - n0) < p.ls.tile_rows ? (N - n0) : p.ls.tile_rows;
  const size_t NH = (size_t)N * H;
  const int own_units = (H - j0) < HS ? (H - j0) : HS;
  const float inv_own_columns = 1.0f / (3.0f * (float)own_units);
  const int last_units = H - (gx - 1) * HS;
  const size_t row_words = tagged_row_words(gx, NB, 2);
  unsigned long long* part2 = p.part2 + (size_t)role.bt * 2 * row_words;

  const int tile_floats = Kpad * NB;
  float* xh = p.xh + (size_t)role.bt * kPolledTiles * tile_floats;
  const TileBuffer xhb = make_tile_buffer(xh, kPolledTiles * tile_floats);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);

  // Own k range of the exchange tiles (the last workgroup also owns the padding): rows and
  // k beyond the problem stay zero for the whole launch.
  zero_tile_share(gs, xh, tile_floats, NB, j0 / 4, (role.cw == gx - 1 ? Kpad - j0 : HS) / 4,
                  kPolledTiles);
  clear_row_words(gs, part2, gx, role.cw, NB, 2);

  float4_t breg[REG > 0 ? REG : 1][CT];
  {
    const bool fast = H % 4 == 0 && (reinterpret_cast<uintptr_t>(p.R) & 15u) == 0;
    auto offset = [=](int k, int col) {
      const int gate = col / HS, j = j0 + col % HS;
      return (k < H && gate < 3 && j < H) ? (long long)k * 3 * H + gate * H + j : -1ll;
    };
    if constexpr (REG > 0) {
      const int groups = Kpad >> 6;
      fill_slice<NCOLS>(w_lds, Kpad - 64 * REG, p.R, nullptr, 1.0f, fast, [=](int k, int col) {
        return offset(resident_split_k(k, groups, REG), col);
      });
      load_resident_rows<REG, CT>(breg, groups, p.R, nullptr, 1.0f, offset);
    } else {
      fill_slice<NCOLS>(w_lds, Kpad, p.R, nullptr, 1.0f, fast, offset);
    }
  }

  int pn[PP], pj[PP], pl[PP], pc[PP];
  bool act[PP], colok[PP];
  float h_prev[PP], bxv[PP][3], brv[PP][3], g2[PP][3];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    pl[pp] = idx < NB * HS ? idx / HS : 0;  // surplus threads shadow row 0, never store
    pc[pp] = idx % HS;
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    colok[pp] = idx < NB * HS && pj[pp] < H;
    act[pp] = colok[pp] && pl[pp] < rows_here;
    h_prev[pp] = act[pp] ? p.h[(size_t)pn[pp] * H + pj[pp]] : 0.f;
#pragma unroll
    for (int g = 0; g < 3; ++g) {
      bxv[pp][g] = colok[pp] ? p.bx[g * H + pj[pp]] : 0.f;
      brv[pp][g] = colok[pp] ? p.br[g * H + pj[pp]] : 0.f;
      g2[pp][g] = colok[pp] ? p.gamma2[g * H + pj[pp]] : 0.f;
    }
  }
  const bool zoneout = p.zoneout_prob != 0.f && p.zoneout_mask != nullptr;
  // Tile 0 receives h[0]; the elements of the other tiles that steps will publish start out
  // unwritten.  One real barrier: nobody polls before every owner has set its share up.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (act[pp]) {
      float* e = &xh[xchg_index(pj[pp], pl[pp], NB)];
      store_exchanged(gs, e, publishable(h_prev[pp]));
      for (int b = 1; b < kPolledTiles; ++b) store_exchanged(gs, e + (size_t)b * tile_floats, unwritten_value());
    }
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);

  // Inputs of a step that do not depend on the recurrence, fetched one step ahead.
  float wx_next[PP][3], mk_next[PP];
  // Every thread loads (threads without an element, and the request after the last step, some
  // valid address: their values are never used) and nothing but the loads writes these
  // registers inside the loop (see ln_lstm_forward_kernel).
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
      const float* wt = p.Wxn + ((size_t)tt * N + row) * 3 * H + unit;
#pragma unroll
      for (int g = 0; g < 3; ++g) wx_next[pp][g] = wt[g * H];
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
    const unsigned int tag = gs.epoch + 2u + (unsigned int)t;  // names this step's row exchange
    unsigned long long* ex2 = part2 + (size_t)(t & 1) * row_words;

    // The operand loads wait for h[t] themselves (polled tile t % 4).
    if constexpr (REG > 0)
      tile_product<NB, CT, false, true, false, NoSideWork, REG, float4_t[REG][CT]>(
          xhb, (t & 3) * tile_floats, Kpad, w_lds, red, &gs, nullptr, &breg);
    else
      tile_product<NB, CT, false, true>(xhb, (t & 3) * tile_floats, Kpad, w_lds, red, &gs);
    __syncthreads();

    float rh[PP][3];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      float s = 0.f;
#pragma unroll
      for (int g = 0; g < 3; ++g) {
        // every thread reads (the address is valid for all of them): a read per branch would
        // wait out the LDS latency once per gate
        const float sum = sum_product<NB, CT>(red, pl[pp], g * HS + pc[pp]);
        rh[pp][g] = colok[pp] ? sum : 0.f;
        s += rh[pp][g];
      }
      const float mean = segment_sum<HS>(s) * inv_own_columns;
      float q = 0.f;
#pragma unroll
      for (int g = 0; g < 3; ++g) {
        const float d = rh[pp][g] - mean;
        q += colok[pp] ? d * d : 0.f;
      }
      q = segment_sum<HS>(q);
      if (pc[pp] == 0 && tid + 256 * pp < NB * HS) {
        const float mq[2] = {mean, q};
        publish_row<2>(gs, ex2, NB, role.cw, pl[pp], mq, tag);
      }
    }
    float saved[PP][4], mu2[PP], is2[PP], h_pub[PP];
    if (in_wavefront) {
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        gather_row_moments<HS>(gs, ex2, NB, gx, tag, 3.0f * HS, 3.0f * last_units, 3.0f * H, pl[pp],
                               tid + 256 * pp < NB * HS, mu2[pp], is2[pp]);
    } else {
      merge_row_moments_polled<NB>(gs, ex2, gx, tag, 3.0f * HS, 3.0f * last_units, 3.0f * H, stat);
      __syncthreads();
#pragma unroll
      for (int pp = 0; pp < PP; ++pp) {
        mu2[pp] = stat[pl[pp] * 2];
        is2[pp] = stat[pl[pp] * 2 + 1];
      }
    }
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
#pragma unroll
      for (int g = 0; g < 4; ++g) saved[pp][g] = 0.f;
      if (act[pp]) {
        float rn[3];
#pragma unroll
        for (int g = 0; g < 3; ++g) rn[g] = (rh[pp][g] - mu2[pp]) * is2[pp] * g2[pp][g];
        const float z = sigmoid_f(wx[pp][0] + rn[0] + bxv[pp][0] + brv[pp][0]);
        const float r = sigmoid_f(wx[pp][1] + rn[1] + bxv[pp][1] + brv[pp][1]);
        const float qg = rn[2] + brv[pp][2];
        const float g = tanh_f(wx[pp][2] + r * qg + bxv[pp][2]);
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
    // landed before h[t+1] becomes visible.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
    __syncthreads();  // red and stat may be overwritten by the next step
    // The caller's copies are written last: nobody in the launch waits for them.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if (act[pp]) {
        float* ar = p.act_Rh + ((size_t)t * N + pn[pp]) * 3 * H + pj[pp];
#pragma unroll
        for (int g = 0; g < 3; ++g) ar[g * H] = rh[pp][g];
        if (p.training) {
          float* vt = p.v + ((size_t)t * N + pn[pp]) * 4 * H + pj[pp];
#pragma unroll
          for (int g = 0; g < 4; ++g) vt[g * H] = saved[pp][g];
        }
        p.h[(size_t)(t + 1) * NH + (size_t)pn[pp] * H + pj[pp]] = h_prev[pp];
        if (role.cw == 0 && pc[pp] == 0 && p.cache2 != nullptr) {
          p.cache2[((size_t)t * N + pn[pp]) * 2 + 0] = mu2[pp];
          p.cache2[((size_t)t * N + pn[pp]) * 2 + 1] = is2[pp];
        }
      }
    }
  }
}

struct LnGruBwdParams {
  int T, N, H;
  const float* R_t;      // [3H,H]
  const float* h;        // [T+1,N,H]
  const float* v;        // [T,N,4H]
  const float* dh_new;   // [T+1,N,H]
  float* dbx;            // [3H]
  float* dbr;            // [3H]
  float* dh;             // [N,H]
  float* dp;             // [T,N,3H]
  float* dq;             // [T,N,3H] out: gradient w.r.t. h*R before its norm
  const float* act_Rh;   // [T,N,3H]
  const float* gamma2;   // [3H]
  float* dgamma2;        // [3H]
  const float* cache2;   // [T*N,2]
  const float* zoneout_mask;
  unsigned long long* part;  // tagged row exchange [groups][2][gx][NB] slots: h*R norm sums
  float* col_partial;    // [batch tiles][9][H]
  float* xdq;            // polled exchange tiles of dq: [batch tiles][4][Kpad/4][NB][4]
  LaunchShape ls;
};

// Contraction length of the backward recurrence inside the launch: k = 3*unit + gate over
// the 16 units of every column workgroup.
inline int ln_gru_backward_k(int H) { return 48 * ((H + 15) / 16); }


// REG > 0: the slice exceeds LDS; every wavefront keeps the first REG k-groups of its share
// of the contraction in registers (tall_tile_product).
// PARK (tiles of 4 rows): the idle last wavefront requests the inputs of the following step
// and parks them in LDS for the owners of the elements, see ln_lstm_backward_kernel.
constexpr int kLnGruBwdInputs = 12;  // floats per element and step, see StepIn
template <int NB, int REG = 0, bool PARK = false>
__global__ __launch_bounds__(256, 1)
void ln_gru_backward_kernel(LnGruBwdParams p) {
  static_assert(!PARK || (NB == 4 && REG == 0), "parked inputs: 4-row tiles");
  constexpr int HSB = 16;
  constexpr int NCOLS = 16;
  constexpr int PP = (NB * HSB + 255) / 256;
  constexpr int NACC = 9;  // dbx x3, dbr x3, dgamma2 x3
  constexpr int RED = NB * NACC * HSB > ProductTile<NB, 1>::kRedFloats
                          ? NB * NACC * HSB : ProductTile<NB, 1>::kRedFloats;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ unsigned int s_role;
  const Role role = take_role(p.ls, &s_role);
  if (!role.active) return;
  __shared__ unsigned int s_flag;

  const int H = p.H, N = p.N, T = p.T;
  const int Kpad = round_up(48 * p.ls.gx, 64);
  float* w_lds = lds;
  float* red = lds + (Kpad - 64 * REG) * NCOLS;  // the partial tiles, reused for the column sums
  float* sums = red + RED;           // [NB][4] row sums of the norm (long rows only)
  float* park = sums + 4 * NB;       // PARK: [2][12][NB * 16] inputs of a step, by step parity

  const int tid = threadIdx.x;
  const int gx = p.ls.gx;
  const int j0 = role.cw * HSB;
  const int n0 = role.bt * p.ls.tile_rows;
  const int rows_here = (N - n0) < p.ls.tile_rows ? (N - n0) : p.ls.tile_rows;
  const size_t NH = (size_t)N * H;
  const bool in_wavefront = row_sums_gather_in_wavefront<HSB>(gx, NB);
  const size_t row_words = tagged_row_words(gx, NB, 3);
  unsigned long long* part = p.part + (size_t)role.bt * 2 * row_words;

  const int tile_floats = Kpad * NB;
  float* xdq = p.xdq + (size_t)role.bt * kPolledTiles * tile_floats;
  const TileBuffer xdqb = make_tile_buffer(xdq, kPolledTiles * tile_floats);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);

  // Own k range of the exchange tiles (the last workgroup also owns the padding); only
  // rows and units of the problem are written afterwards, the rest stays zero.
  zero_tile_share(gs, xdq, tile_floats, NB, 12 * role.cw,
                  (role.cw == gx - 1 ? Kpad - 48 * role.cw : 48) / 4, kPolledTiles);
  clear_row_words(gs, part, gx, role.cw, NB, 3);

  static_assert(REG == 0 || NB >= 16, "register-resident slice rows: tall tiles only");
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
  bool act[PP], own[PP];
  float dh[PP], accs[PP][NACC], g2[PP][3];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    own[pp] = idx < NB * HSB;  // surplus threads of a short tile shadow row 0, never store
    pl[pp] = own[pp] ? idx / HSB : 0;
    pc[pp] = idx % HSB;
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    act[pp] = own[pp] && pl[pp] < rows_here && pj[pp] < H;
    dh[pp] = act[pp] ? p.dh[(size_t)pn[pp] * H + pj[pp]] : 0.f;
#pragma unroll
    for (int g = 0; g < 3; ++g) g2[pp][g] = pj[pp] < H ? p.gamma2[g * H + pj[pp]] : 0.f;
#pragma unroll
    for (int a = 0; a < NACC; ++a) accs[pp][a] = 0.f;
  }
  const bool zoneout = p.zoneout_mask != nullptr;
  // The elements that steps will publish start out unwritten.  One real barrier: nobody
  // polls before every owner has set its share up.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (act[pp])
      for (int b = 0; b < kPolledTiles; ++b)
        for (int k = 0; k < 3; ++k)
          store_exchanged(gs, xdq + (size_t)b * tile_floats + xchg_index(3 * pj[pp] + k, pl[pp], NB),
                          unwritten_value());
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);

  struct StepIn { float vt[4], rh[3], h0, dhn, m, mu2, is2; };
  StepIn nxt[PP];
  // Every thread loads and nothing but the loads writes `nxt` inside the loop (see
  // ln_lstm_forward_kernel).
  {
    const StepIn nxt_init = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}, 0.f, 0.f, 1.f, 0.f, 0.f};
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) nxt[pp] = nxt_init;
  }
  // PARK: the helper wavefront's side.  Lane l requests the inputs of the elements l, l + 64, ...
  // of the tile for step t and parks them in the buffer of t's parity.
  constexpr int kElements = NB * HSB;
  const bool helper = PARK && (tid >> 6) == 3;
  auto park_inputs = [&](int t) {
    float* dst = park + (size_t)(t & 1) * kLnGruBwdInputs * kElements;
#pragma unroll
    for (int q = 0; q < (kElements + 63) / 64; ++q) {
      const int idx = (tid & 63) + 64 * q;
      const int r_ = idx / HSB, u_ = idx % HSB;
      const bool exists = idx < kElements && r_ < rows_here && j0 + u_ < H;
      const size_t row = exists ? (size_t)(n0 + r_) : 0, unit = exists ? (size_t)(j0 + u_) : 0;
      const size_t e = row * H + unit;
      const float* vt = p.v + ((size_t)t * N + row) * 4 * H + unit;
      const float* ar = p.act_Rh + ((size_t)t * N + row) * 3 * H + unit;
      float in[kLnGruBwdInputs];
#pragma unroll
      for (int g = 0; g < 4; ++g) in[g] = vt[(size_t)g * H];
#pragma unroll
      for (int g = 0; g < 3; ++g) in[4 + g] = ar[(size_t)g * H];
      in[7] = p.h[(size_t)t * NH + e];
      in[8] = p.dh_new[(size_t)(t + 1) * NH + e];
      in[9] = zoneout ? p.zoneout_mask[(size_t)t * NH + e] : 1.f;
      in[10] = p.cache2[((size_t)t * N + row) * 2];
      in[11] = p.cache2[((size_t)t * N + row) * 2 + 1];
      if (idx < kElements) {
#pragma unroll
        for (int i = 0; i < kLnGruBwdInputs; ++i) dst[i * kElements + idx] = in[i];
      }
    }
  };
  // ... and the owners' side: the inputs of step t from the buffer of its parity.
  auto take_parked = [&](int t, StepIn (&s)[PP]) {
    const float* src = park + (size_t)(t & 1) * kLnGruBwdInputs * kElements;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const int idx = own[pp] ? tid + 256 * pp : 0;
      float in[kLnGruBwdInputs];
#pragma unroll
      for (int i = 0; i < kLnGruBwdInputs; ++i) in[i] = src[i * kElements + idx];
#pragma unroll
      for (int g = 0; g < 4; ++g) s[pp].vt[g] = in[g];
#pragma unroll
      for (int g = 0; g < 3; ++g) s[pp].rh[g] = in[4 + g];
      s[pp].h0 = in[7]; s[pp].dhn = in[8]; s[pp].m = in[9]; s[pp].mu2 = in[10]; s[pp].is2 = in[11];
    }
  };
  auto fetch = [&](int t) {
    if constexpr (PARK) return;
    const int tt = t >= 0 ? t : 0;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      const size_t e = row * H + unit;
      const float* vt = p.v + ((size_t)tt * N + row) * 4 * H + unit;
      const float* ar = p.act_Rh + ((size_t)tt * N + row) * 3 * H + unit;
#pragma unroll
      for (int g = 0; g < 4; ++g) nxt[pp].vt[g] = vt[(size_t)g * H];
#pragma unroll
      for (int g = 0; g < 3; ++g) nxt[pp].rh[g] = ar[(size_t)g * H];
      nxt[pp].h0 = p.h[(size_t)tt * NH + e];
      nxt[pp].dhn = p.dh_new[(size_t)(tt + 1) * NH + e];
      if (zoneout) nxt[pp].m = p.zoneout_mask[(size_t)tt * NH + e];
      nxt[pp].mu2 = p.cache2[((size_t)tt * N + row) * 2];
      nxt[pp].is2 = p.cache2[((size_t)tt * N + row) * 2 + 1];
    }
  };
  fetch(T - 1);
  if constexpr (PARK) {
    if (helper) park_inputs(T - 1);
    __syncthreads();
  }

  const float inv3H = 1.0f / (float)(3 * H);
  for (int t = T - 1; t >= 0; --t) {
    StepIn s[PP];
    if constexpr (PARK) {
      // Parked during the previous step, before its product's barrier; the buffer this step's
      // helper fills was last read a step ago.
      take_parked(t, s);
      if (helper && t > 0) park_inputs(t - 1);
    }
    float dh_keep[PP], xc[PP][3], gd[PP][3], dps[PP][3], dqs[PP][3];
    const int done = T - 1 - t;  // steps done so far
    const unsigned int tag = gs.epoch + 2u + (unsigned int)done;  // names this step's row exchange
    unsigned long long* ex = part + (size_t)(done & 1) * row_words;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if constexpr (!PARK) s[pp] = nxt[pp];
      dh_keep[pp] = 0.f;
#pragma unroll
      for (int k = 0; k < 3; ++k) dps[pp][k] = dqs[pp][k] = 0.f;
      float t0 = 0.f, t1 = 0.f, t2 = 0.f;
#pragma unroll
      for (int g = 0; g < 3; ++g) xc[pp][g] = gd[pp][g] = 0.f;
      if (act[pp]) {
        const float z = s[pp].vt[0], r = s[pp].vt[1], g = s[pp].vt[2], qg = s[pp].vt[3];
        float dh_total = s[pp].dhn + dh[pp];
        if (zoneout) {
          dh_keep[pp] = (1.0f - s[pp].m) * dh_total;
          dh_total = s[pp].m * dh_total;
          dh_keep[pp] += z * dh_total;
        } else {
          dh_keep[pp] = z * dh_total;
        }
        const float dg = (1.0f - z) * dh_total;
        const float dz = (s[pp].h0 - g) * dh_total;
        const float dp_g = d_tanh_f(g) * dg;
        const float dq_g = dp_g * r;
        const float dr = dp_g * qg;
        const float dp_r = d_sigmoid_f(r) * dr;
        const float dp_z = d_sigmoid_f(z) * dz;
        dps[pp][0] = dp_z;
        dps[pp][1] = dp_r;
        dps[pp][2] = dp_g;
        const float dqv[3] = {dp_z, dp_r, dq_g};
        accs[pp][0] += dp_z;
        accs[pp][1] += dp_r;
        accs[pp][2] += dp_g;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
          accs[pp][3 + k] += dqv[k];
          xc[pp][k] = s[pp].rh[k] - s[pp].mu2;
          gd[pp][k] = g2[pp][k] * dqv[k];
          accs[pp][6 + k] += xc[pp][k] * s[pp].is2 * dqv[k];
          t0 += xc[pp][k] * gd[pp][k];
          t1 += xc[pp][k];
          t2 += gd[pp][k];
        }
      }
      t0 = segment_sum<HSB>(t0);
      t1 = segment_sum<HSB>(t1);
      t2 = segment_sum<HSB>(t2);
      if (pc[pp] == 0 && own[pp]) {
        const float v3[3] = {t0, t1, t2};
        publish_row<3>(gs, ex, NB, role.cw, pl[pp], v3, tag);
      }
    }
    if (!in_wavefront) {
      sum_row_partials_polled<NB>(gs, ex, gx, tag, sums);
      __syncthreads();
    }
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      float rs[3];
      if (in_wavefront) {
        gather_row_sums<HSB, 3>(gs, ex, NB, gx, tag, pl[pp], own[pp], rs);
      } else {
#pragma unroll
        for (int i = 0; i < 3; ++i) rs[i] = sums[pl[pp] * 4 + i];
      }
      if (act[pp]) {
        const float is2 = s[pp].is2;
        const float dsigma = -0.5f * rs[0] * is2 * is2 * is2;
        const float dmu = (-2.0f * rs[1] * dsigma * inv3H) - (rs[2] * is2);
#pragma unroll
        for (int k = 0; k < 3; ++k)
          dqs[pp][k] = (2.0f * xc[pp][k] * dsigma * inv3H) + (is2 * gd[pp][k]) + (dmu * inv3H);
      }
    }
    // What this wavefront stored during the previous step (its resets among it) has landed
    // before the gradients of this step become visible.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    {
      float* xdq_t = xdq + (done & 3) * tile_floats;
      float* xdq_done = xdq + ((done + 2) & 3) * tile_floats;  // read two steps ago
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        if (act[pp]) {
#pragma unroll
          for (int k = 0; k < 3; ++k) {
            const int e = xchg_index(3 * pj[pp] + k, pl[pp], NB);
            store_exchanged(gs, xdq_t + e, publishable(dqs[pp][k]));
            if (done + 2 < T) store_exchanged(gs, xdq_done + e, unwritten_value());
          }
        }
    }
    // The caller's copies: nobody in the launch waits for them.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
      if (act[pp]) {
        const size_t o3 = ((size_t)t * N + pn[pp]) * 3 * H + pj[pp];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
          p.dp[o3 + (size_t)k * H] = dps[pp][k];
          p.dq[o3 + (size_t)k * H] = dqs[pp][k];
        }
      }
    fetch(t - 1);
    // The operand loads wait for dq_t of every unit themselves.
    if constexpr (REG > 0)
      tile_product<NB, 1, true, true, false, NoSideWork, REG, float4_t[REG][1]>(
          xdqb, (done & 3) * tile_floats, Kpad, w_lds, red, &gs, nullptr, &breg);
    else
      tile_product<NB, 1, true, true>(xdqb, (done & 3) * tile_floats, Kpad, w_lds, red, &gs);
    __syncthreads();
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
      dh[pp] = dh_keep[pp] + sum_product<NB, 1>(red, pl[pp], pc[pp]);
    __syncthreads();  // red may be overwritten by the next step
  }

#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (act[pp]) p.dh[(size_t)pn[pp] * H + pj[pp]] = dh[pp];

  __syncthreads();
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
#pragma unroll
    for (int a = 0; a < NACC; ++a)
      if (own[pp]) red[(pl[pp] * NACC + a) * HSB + pc[pp]] = act[pp] ? accs[pp][a] : 0.f;
  __syncthreads();
  if (tid < NACC * HSB) {
    const int a = tid / HSB, jj = tid % HSB;
    float sum = 0.f;
    for (int r = 0; r < NB; ++r) sum += red[(r * NACC + a) * HSB + jj];
    if (j0 + jj < H) store_agent(&p.col_partial[((size_t)role.bt * NACC + a) * H + j0 + jj], sum);
  }
  if (column_last_arrival(p.ls.cb, role.cw, (unsigned)p.ls.gy, &s_flag)) {
    if (tid < NACC * HSB && j0 + tid % HSB < H) {
      const int a = tid / HSB, col = j0 + tid % HSB;
      const float sum = sum_over_tiles(p.col_partial + (size_t)a * H + col, (size_t)NACC * H, p.ls.gy);
      if (a < 3) p.dbx[a * H + col] += sum;
      else if (a < 6) p.dbr[(a - 3) * H + col] += sum;
      else p.dgamma2[(a - 6) * H + col] += sum;
    }
  }
}

}  // namespace
}  // namespace haste_hip

extern "C" {

using namespace haste_hip;

int haste_hip_layer_norm_gru_forward_f32(int training, int steps, int batch_size,
                                         int input_size, int hidden_size,
                                         const float* W, const float* R, const float* bx,
                                         const float* br, const float* x, float* h, float* v,
                                         float* act_Wx, const float* gamma1, float* cache1,
                                         float* tmp_Wx_norm, float* act_Rh,
                                         const float* gamma2, float* cache2, float* tmp_Rh_norm,
                                         float zoneout_prob, const float* zoneout_mask,
                                         void* stream_) {
  (void)tmp_Rh_norm;
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W && R && bx && br && x && h && act_Wx && gamma1 && tmp_Wx_norm && act_Rh && gamma2);
  HASTE_HIP_REQUIRE(!training || v != nullptr);
  hipStream_t stream = as_stream(stream_);
  const ForwardTile tile = pick_forward_tile(3, N, H, 2 * sizeof(float), kMaxLdsBytes, true,
                                             3);
  if (!tile.ok)
    return layer_norm_gru_forward_streamed(stream, training, T, N, C, H, W, R, bx, br, x, h, v, act_Wx,
                                           gamma1, cache1, tmp_Wx_norm, act_Rh, gamma2, cache2,
                                           zoneout_prob, zoneout_mask);
  const int gx = tile.gx, gy = tile.gy;
  const int NB = tile.nb;
  // the tagged row exchange: [groups][2] buffers of 8-byte words, counted in floats
  const size_t part_floats = (size_t)gy * 2 * tagged_row_words(gx, NB, 2) * 2;

  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T * N, 3 * H, C, x, C, W, 3 * H, act_Wx, 3 * H, false));
  HASTE_HIP_PROPAGATE(layer_norm_forward(stream, T * N, 3 * H, gamma1, nullptr, act_Wx, tmp_Wx_norm, cache1));

  // Taken after the GEMM, which may replace the stream's scratch buffer with a larger one.
  Workspace ws;
  const size_t xh_floats = exchange_floats(H, NB, gy, kPolledTiles);
  HASTE_HIP_PROPAGATE(get_workspace(stream, (part_floats + xh_floats) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  LnGruFwdParams p;
  p.training = training; p.T = T; p.N = N; p.H = H;
  p.R = R; p.bx = bx; p.br = br; p.h = h; p.v = v; p.Wxn = tmp_Wx_norm; p.act_Rh = act_Rh;
  p.gamma2 = gamma2; p.cache2 = cache2;
  p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.part2 = reinterpret_cast<unsigned long long*>(ws.scratch);
  p.xh = ws.scratch + part_floats;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, gx, gy, tile.nb, tile.lds_bytes, 2u * (unsigned)T + 1, &plan));
  p.ls = plan.shape;
#define HASTE_LAUNCH_RESIDENT(NB_, CT_, HS_, REG_)                                            \
  if (tile.reg_groups == REG_ && tile.nb == NB_ && tile.hs == HS_)                           \
    return launch_persistent("layer_norm_gru_forward_recurrence",                            \
                             ln_gru_forward_kernel<NB_, CT_, HS_, REG_>, plan, p, stream);
  HASTE_LAUNCH_RESIDENT(16, 2, 8, 8) HASTE_LAUNCH_RESIDENT(32, 2, 8, 8) HASTE_LAUNCH_RESIDENT(64, 2, 8, 8)
  HASTE_LAUNCH_RESIDENT(16, 2, 8, 16) HASTE_LAUNCH_RESIDENT(32, 2, 8, 16) HASTE_LAUNCH_RESIDENT(64, 2, 8, 16)
  HASTE_LAUNCH_RESIDENT(16, 3, 16, 8) HASTE_LAUNCH_RESIDENT(32, 3, 16, 8) HASTE_LAUNCH_RESIDENT(64, 3, 16, 8)
#undef HASTE_LAUNCH_RESIDENT
  if (tile.reg_groups > 0) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
#define HASTE_LAUNCH(NB_, CT_, HS_)                                                          \
  if (tile.nb == NB_ && tile.hs == HS_)                                                      \
    return launch_persistent("layer_norm_gru_forward_recurrence",                            \
                             ln_gru_forward_kernel<NB_, CT_, HS_>, plan, p, stream);
  HASTE_LAUNCH(4, 1, 4) HASTE_LAUNCH(4, 2, 8) HASTE_LAUNCH(4, 3, 16)
  HASTE_LAUNCH(8, 1, 4) HASTE_LAUNCH(8, 2, 8) HASTE_LAUNCH(8, 3, 16)
  HASTE_LAUNCH(16, 1, 4) HASTE_LAUNCH(16, 2, 8) HASTE_LAUNCH(16, 3, 16)
  HASTE_LAUNCH(32, 1, 4) HASTE_LAUNCH(32, 2, 8) HASTE_LAUNCH(32, 3, 16)
  HASTE_LAUNCH(64, 1, 4) HASTE_LAUNCH(64, 2, 8) HASTE_LAUNCH(64, 3, 16)
#undef HASTE_LAUNCH
  return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
}

int haste_hip_layer_norm_gru_backward_f32(int steps, int batch_size, int input_size,
                                          int hidden_size,
                                          const float* W_t, const float* R_t, const float* bx,
                                          const float* br, const float* x_t, const float* h,
                                          const float* v, const float* dh_new,
                                          float* dx, float* dW, float* dR, float* dbx, float* dbr,
                                          float* dh, float* dp, float* dq,
                                          const float* act_Wx, const float* gamma1, float* dgamma1,
                                          const float* act_Rh, const float* gamma2, float* dgamma2,
                                          const float* cache2,
                                          const float* zoneout_mask, void* stream_) {
  (void)bx;
  (void)br;
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && v && dh_new && dx && dW && dR && dbx && dbr && dh);
  HASTE_HIP_REQUIRE(dp && dq && act_Wx && gamma1 && dgamma1 && act_Rh && gamma2 && dgamma2 && cache2);
  hipStream_t stream = as_stream(stream_);
  // per row: 9 column-sum accumulators of 16 floats (or the partial tiles, whichever is more) + 4 sums
  const BackwardTile tile = pick_backward_tile(ln_gru_backward_k(H), N, H, 9 * 16, 4, true);
  if (!tile.ok)
    return layer_norm_gru_backward_streamed(stream, T, N, C, H, W_t, R_t, x_t, h, v, dh_new, dx, dW, dR,
                                            dbx, dbr, dh, dp, dq, act_Wx, gamma1, dgamma1, act_Rh,
                                            gamma2, dgamma2, cache2, zoneout_mask);
  const int gx = tile.gx, gy = tile.gy;
  const int NB = tile.nb;
  // the tagged row exchange: [groups][2] buffers of 8-byte words, counted in floats
  const size_t part_floats = (size_t)gy * 2 * tagged_row_words(gx, NB, 3) * 2;
  const size_t col_floats = ((size_t)gy * 9 * H + 3) / 4 * 4;
  const size_t xdq_floats = exchange_floats(ln_gru_backward_k(H), NB, gy, kPolledTiles);

  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, (part_floats + col_floats + xdq_floats) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  LnGruBwdParams p;
  p.T = T; p.N = N; p.H = H;
  p.R_t = R_t; p.h = h; p.v = v; p.dh_new = dh_new;
  p.dbx = dbx; p.dbr = dbr; p.dh = dh; p.dp = dp; p.dq = dq;
  p.act_Rh = act_Rh; p.gamma2 = gamma2; p.dgamma2 = dgamma2; p.cache2 = cache2;
  p.zoneout_mask = zoneout_mask;
  p.part = reinterpret_cast<unsigned long long*>(ws.scratch);
  p.col_partial = ws.scratch + part_floats;
  p.xdq = ws.scratch + part_floats + col_floats;
  // 4-row tiles park the inputs of a step in LDS when there is room: [2][12][NB * 16] floats
  // (8-row tiles measured 2.6 % slower with it at N = 64, H = 512).
  const size_t park_bytes = (size_t)2 * kLnGruBwdInputs * NB * 16 * sizeof(float);
  const bool parked = NB <= 4 && tile.reg_groups == 0 && tile.lds_bytes + park_bytes <= kMaxLdsBytes;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, gx, gy, tile.nb, tile.lds_bytes + (parked ? park_bytes : 0),
                                  2u * (unsigned)T + 1, &plan));
  p.ls = plan.shape;
  int rc = HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  const char* name = "layer_norm_gru_backward_recurrence";
#define HASTE_LAUNCH_BWD_RESIDENT(NB_)                                                          \
  (tile.reg_groups == 8    ? launch_persistent(name, ln_gru_backward_kernel<NB_, 8>, plan, p, stream)  \
   : tile.reg_groups == 16 ? launch_persistent(name, ln_gru_backward_kernel<NB_, 16>, plan, p, stream) \
   : tile.reg_groups == 24 ? launch_persistent(name, ln_gru_backward_kernel<NB_, 24>, plan, p, stream) \
                           : launch_persistent(name, ln_gru_backward_kernel<NB_, 32>, plan, p, stream))
  if (tile.reg_groups > 0) {
    if (NB == 16) rc = HASTE_LAUNCH_BWD_RESIDENT(16);
    else if (NB == 32) rc = HASTE_LAUNCH_BWD_RESIDENT(32);
    else if (NB == 64) rc = HASTE_LAUNCH_BWD_RESIDENT(64);
  }
#undef HASTE_LAUNCH_BWD_RESIDENT
  else if (NB == 4 && parked) rc = launch_persistent(name, ln_gru_backward_kernel<4, 0, true>, plan, p, stream);
  else if (NB == 4) rc = launch_persistent(name, ln_gru_backward_kernel<4>, plan, p, stream);
  else if (NB == 8) rc = launch_persistent(name, ln_gru_backward_kernel<8>, plan, p, stream);
  else if (NB == 16) rc = launch_persistent(name, ln_gru_backward_kernel<16>, plan, p, stream);
  else if (NB == 32) rc = launch_persistent(name, ln_gru_backward_kernel<32>, plan, p, stream);
  else if (NB == 64) rc = launch_persistent(name, ln_gru_backward_kernel<64>, plan, p, stream);
  HASTE_HIP_PROPAGATE(rc);

  const int TN = T * N;
  HASTE_HIP_PROPAGATE(layer_norm_backward(stream, TN, 3 * H, gamma1, act_Wx, dp, dp, dgamma1, nullptr));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, TN, C, 3 * H, dp, 3 * H, W_t, C, dx, C, false));
  // dW += x^T dp and dR += h^T dq: one launch when that halves their K pieces
  HASTE_HIP_PROPAGATE(gemm_f32_pair(stream, C, H, 3 * H, TN, x_t, TN, dp, 3 * H, dW, 3 * H,
                                    h, H, dq, 3 * H, dR, 3 * H, true));
  return HASTE_HIP_OK;
}

}  // extern "C"
