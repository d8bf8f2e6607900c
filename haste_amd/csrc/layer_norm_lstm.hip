// LayerNormLSTM forward and backward passes.
//
// Forward: GEMM x*W, one stand-alone layer norm over all T*N rows, then one persistent
// kernel for the recurrence in which the two per-step layer norms (on h*R over 4H
// columns and on the new cell state over H columns) are computed inside the step:
// each workgroup reduces its own columns, the group exchanges per-row moments, and a
// step therefore has three group barriers (h_t ready, norm of h*R, norm of c).
// Backward mirrors it in reverse time with two waits per step: the row sums of both norms
// travel in one exchange (those of the h*R norm as coefficients, see the step), then the
// gradient w.r.t. h*R.  One stand-alone layer-norm backward over all rows and the three
// batched GEMMs follow.
//
// Arithmetic follows reference lib/layer_norm_lstm_forward_gpu.cu.cc:50-71,95-108 and
// lib/layer_norm_lstm_backward_gpu.cu.cc:44-64,84-117; orchestration replaces
// :276-340 and :255-352.
#include "ln_exchange.h"

namespace haste_hip {
namespace {

struct LnLstmFwdParams {
  int training, T, N, H;
  const float* R;         // [H,4H]
  const float* b;         // [4H]
  float* h;               // [T+1,N,H]
  float* c;               // [T+1,N,H]
  float* v;               // act_Wx_norm [T,N,4H]: in LN1(x*W), out (training) gate activations
  float* act_Rh;          // [T,N,4H] out: h*R before its norm
  const float* gamma2;    // [4H]
  float* cache2;          // [T*N,2] or null
  const float* gamma_h;   // [H]
  const float* beta_h;    // [H]
  float* cache3;          // [T*N,2] or null
  float* act_c_norm;      // [T,N,H] out
  float zoneout_prob;
  const float* zoneout_mask;
  unsigned long long* part2;  // tagged row exchange [groups][2][gx][NB][2] words: moments of h*R
  unsigned long long* part3;  // tagged row exchange [groups][2][gx][NB][2] words: moments of c
  float* xh;              // polled exchange tiles of h: [batch tiles][4][Kpad/4][NB][4]
  LaunchShape ls;
};

// NB batch rows per workgroup.  PARK (the tile's elements leave the last wavefront idle): that
// wavefront requests the next step's inputs and parks them in LDS for the owners of the elements,
// see ln_lstm_backward_kernel.
constexpr int kLnLstmFwdInputs = 5;  // floats per element and step: LN(x*W) of the four gates, the mask
// REG > 0 (tiles of 16 rows and more): the slice exceeds LDS; every wavefront keeps the first REG
// k-groups of its share of the contraction in registers (tall_tile_product).
template <int NB, int CT, bool PARK = false, int REG = 0>
__global__ __launch_bounds__(256, 1)
void ln_lstm_forward_kernel(LnLstmFwdParams p) {
  static_assert(!PARK || NB * 4 * CT <= 64, "parked inputs: one element per lane of the idle last wavefront");
  static_assert(REG == 0 || (NB >= 16 && !PARK), "register-resident slice rows: tall tiles only");
  constexpr int HS = 4 * CT;
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
  float* stat = red + ProductTile<NB, CT>::kRedFloats;  // [2][NB][2] row statistics (long rows only)
  float* park = stat + 4 * NB;  // PARK: [2][5][NB * HS] inputs of a step, by step parity

  const int tid = threadIdx.x;
  const int gx = p.ls.gx;
  const bool in_wavefront = row_gather_in_wavefront<HS, NB>(gx);
  const int j0 = role.cw * HS;
  const int n0 = role.bt * p.ls.tile_rows;
  const int rows_here = (N - n0) < p.ls.tile_rows ? (N - n0) : p.ls.tile_rows;
  const size_t NH = (size_t)N * H;
  const int own_units = (H - j0) < HS ? (H - j0) : HS;     // valid hidden units here
  const float inv_own_units = 1.0f / (float)own_units, inv_own_columns = 1.0f / (4.0f * (float)own_units);
  const int last_units = H - (gx - 1) * HS;                 // ... in the last workgroup
  const size_t row_words = tagged_row_words(gx, NB, 2);
  unsigned long long* part2 = p.part2 + (size_t)role.bt * 2 * row_words;
  unsigned long long* part3 = p.part3 + (size_t)role.bt * 2 * row_words;

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
  clear_row_words(gs, part3, gx, role.cw, NB, 2);

  float4_t breg[REG > 0 ? REG : 1][CT];
  {
    const bool fast = H % 4 == 0 && (reinterpret_cast<uintptr_t>(p.R) & 15u) == 0;
    auto offset = [=](int k, int col) {
      const int gate = col / HS, j = j0 + col % HS;
      return (k < H && j < H) ? (long long)k * 4 * H + gate * H + j : -1ll;
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
  float c_prev[PP], h_prev[PP], bias[PP][4], g2[PP][4], gh[PP], bh[PP];
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    const int idx = tid + 256 * pp;
    pl[pp] = idx < NB * HS ? idx / HS : 0;  // surplus threads shadow row 0, never store
    pc[pp] = idx % HS;
    pn[pp] = n0 + pl[pp];
    pj[pp] = j0 + pc[pp];
    colok[pp] = idx < NB * HS && pj[pp] < H;
    act[pp] = colok[pp] && pl[pp] < rows_here;
    c_prev[pp] = h_prev[pp] = gh[pp] = bh[pp] = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) bias[pp][g] = g2[pp][g] = 0.f;
    if (colok[pp]) {
      gh[pp] = p.gamma_h[pj[pp]];
      bh[pp] = p.beta_h[pj[pp]];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        bias[pp][g] = p.b[g * H + pj[pp]];
        g2[pp][g] = p.gamma2[g * H + pj[pp]];
      }
    }
    if (act[pp]) {
      c_prev[pp] = p.c[(size_t)pn[pp] * H + pj[pp]];
      h_prev[pp] = p.h[(size_t)pn[pp] * H + pj[pp]];
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
  float wx_next[PP][4], mk_next[PP];
  // Every thread loads (threads without an element, and the request after the last step, some
  // valid address: their values are never used) and nothing but the loads writes these
  // registers inside the loop: a default written there first would have to wait for loads a
  // thread skipped waiting for and, the counter being in order, for the step's stores with them.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    mk_next[pp] = 1.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) wx_next[pp][g] = 0.f;
  }
  auto fetch = [&](int t) {
    if constexpr (PARK) return;
    const int tt = t < T ? t : T - 1;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      const float* vt = p.v + ((size_t)tt * N + row) * 4 * H + unit;
#pragma unroll
      for (int g = 0; g < 4; ++g) wx_next[pp][g] = vt[g * H];
      if (zoneout && p.training) mk_next[pp] = p.zoneout_mask[(size_t)tt * NH + row * H + unit];
    }
  };
  fetch(0);
  // PARK: lane l of the helper wavefront requests the inputs of the elements l, l + 64, ... of
  // the tile for step t and parks them in the buffer of t's parity.
  constexpr int kElements = NB * HS;
  const bool helper = PARK && (tid >> 6) == 3;
  auto park_inputs = [&](int t) {
    float* dst = park + (size_t)(t & 1) * kLnLstmFwdInputs * kElements;
#pragma unroll
    for (int q = 0; q < (kElements + 63) / 64; ++q) {
      const int idx = (tid & 63) + 64 * q;
      const int r_ = idx / HS, u_ = idx % HS;
      const bool exists = idx < kElements && r_ < rows_here && j0 + u_ < H;
      const size_t row = exists ? (size_t)(n0 + r_) : 0, unit = exists ? (size_t)(j0 + u_) : 0;
      const float* vt = p.v + ((size_t)t * N + row) * 4 * H + unit;
      float in[kLnLstmFwdInputs];
#pragma unroll
      for (int g = 0; g < 4; ++g) in[g] = vt[g * H];
      in[4] = zoneout && p.training ? p.zoneout_mask[(size_t)t * NH + row * H + unit] : 1.f;
      if (idx < kElements) {
#pragma unroll
        for (int i = 0; i < kLnLstmFwdInputs; ++i) dst[i * kElements + idx] = in[i];
      }
    }
  };
  if constexpr (PARK) {
    if (helper) park_inputs(0);
    __syncthreads();
  }

  for (int t = 0; t < T; ++t) {
    float wx[PP][4], mk[PP];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if constexpr (PARK) {
        // parked during the previous step, before its closing barrier
        const float* src = park + (size_t)(t & 1) * kLnLstmFwdInputs * kElements;
        const int idx = tid + 256 * pp < kElements ? tid + 256 * pp : 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) wx[pp][g] = src[g * kElements + idx];
        mk[pp] = src[4 * kElements + idx];
      } else {
        mk[pp] = mk_next[pp];
#pragma unroll
        for (int g = 0; g < 4; ++g) wx[pp][g] = wx_next[pp][g];
      }
    }
    const unsigned int tag = gs.epoch + 2u + (unsigned int)t;  // names this step's row exchanges
    unsigned long long* ex2 = part2 + (size_t)(t & 1) * row_words;
    unsigned long long* ex3 = part3 + (size_t)(t & 1) * row_words;

    // The operand loads wait for h[t] themselves (polled tile t % 4).
    if constexpr (REG > 0)
      tile_product<NB, CT, false, true, false, NoSideWork, REG, float4_t[REG][CT]>(
          xhb, (t & 3) * tile_floats, Kpad, w_lds, red, &gs, nullptr, &breg);
    else
      tile_product<NB, CT, false, true>(xhb, (t & 3) * tile_floats, Kpad, w_lds, red, &gs);
    __syncthreads();
    // After its share of the product the helper has nothing to do until the step's closing
    // barrier: time enough for loads from memory nobody has touched.
    if constexpr (PARK) {
      if (helper && t + 1 < T) park_inputs(t + 1);
    }

    // h*R of the owned columns; moments of those columns per row, published.
    float rh[PP][4];
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      float s = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // every thread reads (the address is valid for all of them): a read per branch would
        // wait out the LDS latency once per gate
        const float sum = sum_product<NB, CT>(red, pl[pp], g * HS + pc[pp]);
        rh[pp][g] = colok[pp] ? sum : 0.f;
        s += rh[pp][g];
      }
      const float mean = segment_sum<HS>(s) * inv_own_columns;
      float q = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float d = rh[pp][g] - mean;
        q += colok[pp] ? d * d : 0.f;
      }
      q = segment_sum<HS>(q);
      if (pc[pp] == 0 && tid + 256 * pp < NB * HS) {
        const float mq[2] = {mean, q};
        publish_row<2>(gs, ex2, NB, role.cw, pl[pp], mq, tag);
      }
    }
    float gate[PP][4], c_new[PP], mu2[PP], is2[PP];
    if (in_wavefront) {
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        gather_row_moments<HS>(gs, ex2, NB, gx, tag, 4.0f * HS, 4.0f * last_units, 4.0f * H, pl[pp],
                               tid + 256 * pp < NB * HS, mu2[pp], is2[pp]);
    } else {
      merge_row_moments_polled<NB>(gs, ex2, gx, tag, 4.0f * HS, 4.0f * last_units, 4.0f * H, stat);
      __syncthreads();
#pragma unroll
      for (int pp = 0; pp < PP; ++pp) {
        mu2[pp] = stat[pl[pp] * 2];
        is2[pp] = stat[pl[pp] * 2 + 1];
      }
    }
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      c_new[pp] = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) gate[pp][g] = 0.f;
      if (act[pp]) {
        float a[4];
#pragma unroll
        for (int g = 0; g < 4; ++g)
          a[g] = wx[pp][g] + (rh[pp][g] - mu2[pp]) * is2[pp] * g2[pp][g] + bias[pp][g];
        gate[pp][0] = sigmoid_f(a[0]);
        gate[pp][1] = tanh_f(a[1]);
        gate[pp][2] = sigmoid_f(a[2]);
        gate[pp][3] = sigmoid_f(a[3]);
        c_new[pp] = gate[pp][2] * c_prev[pp] + gate[pp][0] * gate[pp][1];
        c_prev[pp] = c_new[pp];
      }
      // moments of the new cell state over the owned hidden units
      const float cv = colok[pp] ? c_new[pp] : 0.f;
      const float mean = segment_sum<HS>(cv) * inv_own_units;
      const float d = cv - mean;
      const float q = segment_sum<HS>(colok[pp] ? d * d : 0.f);
      if (pc[pp] == 0 && tid + 256 * pp < NB * HS) {
        const float mq[2] = {mean, q};
        publish_row<2>(gs, ex3, NB, role.cw, pl[pp], mq, tag);
      }
    }
    float cn[PP], mu3[PP], is3[PP], h_pub[PP];
    if (in_wavefront) {
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        gather_row_moments<HS>(gs, ex3, NB, gx, tag, (float)HS, (float)last_units, (float)H, pl[pp],
                               tid + 256 * pp < NB * HS, mu3[pp], is3[pp]);
    } else {
      // the second half of `stat`: a fast wavefront may be here while a slow one still reads the first
      merge_row_moments_polled<NB>(gs, ex3, gx, tag, (float)HS, (float)last_units, (float)H, stat + 2 * NB);
      __syncthreads();
#pragma unroll
      for (int pp = 0; pp < PP; ++pp) {
        mu3[pp] = stat[2 * NB + pl[pp] * 2];
        is3[pp] = stat[2 * NB + pl[pp] * 2 + 1];
      }
    }
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      cn[pp] = 0.f;
      if (act[pp]) {
        cn[pp] = (c_new[pp] - mu3[pp]) * is3[pp] * gh[pp] + bh[pp];
        float h_new = gate[pp][3] * tanh_f(cn[pp]);
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
        const size_t e4 = ((size_t)t * N + pn[pp]) * 4 * H + pj[pp];
        const size_t e = (size_t)pn[pp] * H + pj[pp];
#pragma unroll
        for (int g = 0; g < 4; ++g) p.act_Rh[e4 + (size_t)g * H] = rh[pp][g];
        if (p.training) {
#pragma unroll
          for (int g = 0; g < 4; ++g) p.v[e4 + (size_t)g * H] = gate[pp][g];
        }
        p.c[(size_t)(t + 1) * NH + e] = c_new[pp];
        p.act_c_norm[(size_t)t * NH + e] = cn[pp];
        p.h[(size_t)(t + 1) * NH + e] = h_prev[pp];
        if (role.cw == 0 && pc[pp] == 0) {
          const size_t r = ((size_t)t * N + pn[pp]) * 2;
          if (p.cache2 != nullptr) {
            p.cache2[r] = mu2[pp];
            p.cache2[r + 1] = is2[pp];
          }
          if (p.cache3 != nullptr) {
            p.cache3[r] = mu3[pp];
            p.cache3[r + 1] = is3[pp];
          }
        }
      }
    }
  }
}

struct LnLstmBwdParams {
  int T, N, H;
  const float* R_t;        // [4H,H]
  const float* c;          // [T+1,N,H]
  const float* dh_new;     // [T+1,N,H]
  const float* dc_new;     // [T+1,N,H]
  float* db;               // [4H]
  float* dh;               // [N,H]
  float* dc;               // [N,H]
  float* v;                // act_Wx_norm: in gate activations, out gate gradients
  float* act_Rh;           // in h*R before its norm, out gradient w.r.t. it
  const float* gamma2;     // [4H]
  float* dgamma2;          // [4H]
  const float* cache2;     // [T*N,2]
  const float* gamma_h;    // [H]
  float* dgamma_h;         // [H]
  float* dbeta_h;          // [H]
  const float* cache3;     // [T*N,2]
  const float* act_c_norm; // [T,N,H]
  const float* zoneout_mask;
  unsigned long long* part;    // tagged row exchange [groups][2][gx][NB][10] words: the sums of both norms
  float* col_partial;      // [batch tiles][10][H]
  float* xd;               // polled exchange tiles of the gradient w.r.t. h*R: [batch tiles][4][Kpad/4][NB][4]
  LaunchShape ls;
};

// REG > 0: the slice exceeds LDS; every wavefront keeps the first REG k-groups of its share
// of the contraction in registers (tall_tile_product).
// PARK (tiles of 4 or 8 rows, whose elements keep at most two wavefronts busy): the last
// wavefront, idle between two products, requests the inputs of the following step and parks
// them in LDS for the threads that own the elements.  Those inputs come from memory nobody has
// touched in this launch, and a wavefront's loads return in order: requested by the owners
// themselves they stand before the polls of the product that follows (0.2 ms of 1.9 at N = 32,
// T = 500, H = 256).
constexpr int kLnLstmBwdInputs = 18;  // floats per element and step, see StepIn
template <int NB, int REG = 0, bool PARK = false>
__global__ __launch_bounds__(256, 1)
void ln_lstm_backward_kernel(LnLstmBwdParams p) {
  static_assert(!PARK || (NB <= 8 && REG == 0), "parked inputs: short tiles");
  constexpr int HSB = 16;
  constexpr int NCOLS = 16;
  constexpr int PP = (NB * HSB + 255) / 256;
  constexpr int NACC = 10;  // db x4, dgamma2 x4, dgamma_h, dbeta_h
  constexpr int kRowValues = 10;  // floats per row and workgroup in the step's row exchange
  constexpr int RED = NB * NACC * HSB > ProductTile<NB, 1>::kRedFloats
                          ? NB * NACC * HSB : ProductTile<NB, 1>::kRedFloats;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ unsigned int s_role;
  const Role role = take_role(p.ls, &s_role);
  if (!role.active) return;
  __shared__ unsigned int s_flag;

  const int H = p.H, N = p.N, T = p.T;
  const int Kpad = 64 * p.ls.gx;  // k = 4*unit + gate over the 16 units of every workgroup
  float* w_lds = lds;
  float* red = lds + (Kpad - 64 * REG) * NCOLS;  // the partial tiles, reused for the column sums
  float* sums = red + RED;           // [NB][10] row sums of the two norms (long rows only)
  float* park = sums + 10 * NB;      // PARK: [2][18][NB * 16] inputs of a step, by step parity

  const int tid = threadIdx.x;
  const int gx = p.ls.gx;
  const int j0 = role.cw * HSB;
  const int n0 = role.bt * p.ls.tile_rows;
  const int rows_here = (N - n0) < p.ls.tile_rows ? (N - n0) : p.ls.tile_rows;
  const size_t NH = (size_t)N * H;
  const bool in_wavefront = row_sums_gather_in_wavefront<HSB>(gx, NB);
  const size_t row_words = tagged_row_words(gx, NB, kRowValues);
  unsigned long long* part = p.part + (size_t)role.bt * 2 * row_words;

  const int tile_floats = Kpad * NB;
  float* xd = p.xd + (size_t)role.bt * kPolledTiles * tile_floats;
  const TileBuffer xdb = make_tile_buffer(xd, kPolledTiles * tile_floats);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);
  clear_row_words(gs, part, gx, role.cw, NB, kRowValues);

  static_assert(REG == 0 || NB >= 16, "register-resident slice rows: tall tiles only");
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
  bool act[PP], own[PP];
  float dh[PP], dc[PP], accs[PP][NACC], g2[PP][4], gh[PP];
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
    dc[pp] = act[pp] ? p.dc[(size_t)pn[pp] * H + pj[pp]] : 0.f;
    gh[pp] = pj[pp] < H ? p.gamma_h[pj[pp]] : 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) g2[pp][g] = pj[pp] < H ? p.gamma2[g * H + pj[pp]] : 0.f;
#pragma unroll
    for (int a = 0; a < NACC; ++a) accs[pp][a] = 0.f;
  }
  const bool zoneout = p.zoneout_mask != nullptr;
  // Every element of the polled tiles belongs to the thread that publishes it (rows and
  // units beyond the problem are published as zeros); all start out unwritten.  One real
  // barrier: nobody polls before every owner has set its share up.
#pragma unroll
  for (int pp = 0; pp < PP; ++pp)
    if (own[pp]) {
      const float u = unwritten_value();
      for (int b = 0; b < kPolledTiles; ++b)
        store_exchanged4(gs, xd + (size_t)b * tile_floats + ((size_t)pj[pp] * NB + pl[pp]) * 4, u, u, u, u);
    }
  group_arrive(gs);  // also: the slice is complete in LDS
  group_wait(gs);

  struct StepIn { float vt[4], rh[4], c0, c1, dhn, dcn, m, cn, mu2, is2, mu3, is3; };
  StepIn nxt[PP];
  // Every thread loads and nothing but the loads writes `nxt` inside the loop (see the
  // forward kernel).
  {
    const StepIn nxt_init = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, 0.f, 0.f, 0.f, 0.f, 1.f, 0.f,
                             0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) nxt[pp] = nxt_init;
  }
  // PARK: the helper wavefront's side.  Lane l requests the inputs of the elements l, l + 64, ...
  // of the tile for step t and parks them in the buffer of t's parity.
  constexpr int kElements = NB * HSB;
  const bool helper = PARK && (tid >> 6) == 3;
  auto park_inputs = [&](int t) {
    float* dst = park + (size_t)(t & 1) * kLnLstmBwdInputs * kElements;
#pragma unroll
    for (int q = 0; q < (kElements + 63) / 64; ++q) {
      const int idx = (tid & 63) + 64 * q;
      const int r_ = idx / HSB, u_ = idx % HSB;
      const bool exists = idx < kElements && r_ < rows_here && j0 + u_ < H;
      const size_t row = exists ? (size_t)(n0 + r_) : 0, unit = exists ? (size_t)(j0 + u_) : 0;
      const size_t e = row * H + unit;
      const size_t e4 = ((size_t)t * N + row) * 4 * H + unit;
      const size_t r = ((size_t)t * N + row) * 2;
      float in[kLnLstmBwdInputs];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        in[g] = p.v[e4 + (size_t)g * H];
        in[4 + g] = p.act_Rh[e4 + (size_t)g * H];
      }
      in[8] = p.c[(size_t)t * NH + e];
      in[9] = p.c[(size_t)(t + 1) * NH + e];
      in[10] = p.dh_new[(size_t)(t + 1) * NH + e];
      in[11] = p.dc_new[(size_t)(t + 1) * NH + e];
      in[12] = zoneout ? p.zoneout_mask[(size_t)t * NH + e] : 1.f;
      in[13] = p.act_c_norm[(size_t)t * NH + e];
      in[14] = p.cache2[r];
      in[15] = p.cache2[r + 1];
      in[16] = p.cache3[r];
      in[17] = p.cache3[r + 1];
      if (idx < kElements) {
#pragma unroll
        for (int i = 0; i < kLnLstmBwdInputs; ++i) dst[i * kElements + idx] = in[i];
      }
    }
  };
  // ... and the owners' side: the inputs of step t from the buffer of its parity.
  auto take_parked = [&](int t, StepIn (&s)[PP]) {
    const float* src = park + (size_t)(t & 1) * kLnLstmBwdInputs * kElements;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const int idx = own[pp] ? tid + 256 * pp : 0;
      float in[kLnLstmBwdInputs];
#pragma unroll
      for (int i = 0; i < kLnLstmBwdInputs; ++i) in[i] = src[i * kElements + idx];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        s[pp].vt[g] = in[g];
        s[pp].rh[g] = in[4 + g];
      }
      s[pp].c0 = in[8]; s[pp].c1 = in[9]; s[pp].dhn = in[10]; s[pp].dcn = in[11];
      s[pp].m = in[12]; s[pp].cn = in[13];
      s[pp].mu2 = in[14]; s[pp].is2 = in[15]; s[pp].mu3 = in[16]; s[pp].is3 = in[17];
    }
  };
  auto fetch = [&](int t) {
    if constexpr (PARK) return;
    const int tt = t >= 0 ? t : 0;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      const size_t row = act[pp] ? (size_t)pn[pp] : 0, unit = act[pp] ? (size_t)pj[pp] : 0;
      const size_t e = row * H + unit;
      const size_t e4 = ((size_t)tt * N + row) * 4 * H + unit;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        nxt[pp].vt[g] = p.v[e4 + (size_t)g * H];
        nxt[pp].rh[g] = p.act_Rh[e4 + (size_t)g * H];
      }
      nxt[pp].c0 = p.c[(size_t)tt * NH + e];
      nxt[pp].c1 = p.c[(size_t)(tt + 1) * NH + e];
      nxt[pp].dhn = p.dh_new[(size_t)(tt + 1) * NH + e];
      nxt[pp].dcn = p.dc_new[(size_t)(tt + 1) * NH + e];
      nxt[pp].cn = p.act_c_norm[(size_t)tt * NH + e];
      if (zoneout) nxt[pp].m = p.zoneout_mask[(size_t)tt * NH + e];
      const size_t r = ((size_t)tt * N + row) * 2;
      nxt[pp].mu2 = p.cache2[r];
      nxt[pp].is2 = p.cache2[r + 1];
      nxt[pp].mu3 = p.cache3[r];
      nxt[pp].is3 = p.cache3[r + 1];
    }
  };
  fetch(T - 1);
  if constexpr (PARK) {
    if (helper) park_inputs(T - 1);
    __syncthreads();
  }

  const float invH = 1.0f / (float)H;
  const float inv4H = 1.0f / (float)(4 * H);
  for (int t = T - 1; t >= 0; --t) {
    StepIn s[PP];
    if constexpr (PARK) {
      // Parked during the previous step, before its product's barrier; the buffer this step's
      // helper fills was last read a step ago.
      take_parked(t, s);
      if (helper && t > 0) park_inputs(t - 1);
    }
    float dh_keep[PP], dv_o[PP], xc3[PP], gd3[PP], xc2[PP][4];
    const int done = T - 1 - t;  // steps done so far
    const unsigned int tag = gs.epoch + 2u + (unsigned int)done;  // names this step's row exchange
    unsigned long long* ex = part + (size_t)(done & 1) * row_words;
    // One row exchange serves both norms.  The sums of the h*R norm are taken over the gate
    // gradients dv, and those depend on the row sums of the cell-state norm (through dsigma and
    // dmu below) -- but linearly: dc_total = base + X * dsigma + dmu / H per unit, dv = k *
    // dc_total for the gates i, g, f.  So every workgroup publishes, beside its parts of the
    // cell-state sums, its parts of the h*R sums as coefficients of (1, dsigma, dmu / H), and
    // every reader puts the totals together once it knows dsigma and dmu.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if constexpr (!PARK) s[pp] = nxt[pp];
      dh_keep[pp] = dv_o[pp] = xc3[pp] = gd3[pp] = 0.f;
      float part_sum[kRowValues];
#pragma unroll
      for (int i = 0; i < kRowValues; ++i) part_sum[i] = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) xc2[pp][g] = 0.f;
      if (act[pp]) {
        float dh_total = s[pp].dhn + dh[pp];
        if (zoneout) {
          dh_keep[pp] = (1.0f - s[pp].m) * dh_total;
          dh_total = s[pp].m * dh_total;
        }
        const float go = s[pp].vt[3];
        const float c_tanh = tanh_f(s[pp].cn);
        const float do_ = c_tanh * dh_total;
        const float dln3 = d_tanh_f(c_tanh) * (go * dh_total);
        dv_o[pp] = d_sigmoid_f(go) * do_;
        xc3[pp] = s[pp].c1 - s[pp].mu3;
        gd3[pp] = gh[pp] * dln3;
        accs[pp][8] += xc3[pp] * s[pp].is3 * dln3;
        accs[pp][9] += dln3;

        const float gi = s[pp].vt[0], gg = s[pp].vt[1], gf = s[pp].vt[2];
        const float base = s[pp].dcn + dc[pp] + s[pp].is3 * gd3[pp];
        const float X = 2.0f * xc3[pp] * invH;
        const float k[3] = {d_sigmoid_f(gi) * gg, d_tanh_f(gg) * gi, d_sigmoid_f(gf) * s[pp].c0};
        float F = 0.f, G = 0.f, x2 = 0.f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          xc2[pp][g] = s[pp].rh[g] - s[pp].mu2;
          x2 += xc2[pp][g];
        }
#pragma unroll
        for (int g = 0; g < 3; ++g) {
          F += xc2[pp][g] * g2[pp][g] * k[g];
          G += g2[pp][g] * k[g];
        }
        const float e2 = g2[pp][3] * dv_o[pp];
        part_sum[0] = xc3[pp] * gd3[pp];
        part_sum[1] = xc3[pp];
        part_sum[2] = gd3[pp];
        part_sum[3] = xc2[pp][3] * e2 + F * base;
        part_sum[4] = F * X;
        part_sum[5] = F;
        part_sum[6] = x2;
        part_sum[7] = e2 + G * base;
        part_sum[8] = G * X;
        part_sum[9] = G;
      }
#pragma unroll
      for (int i = 0; i < kRowValues; ++i) part_sum[i] = segment_sum<HSB>(part_sum[i]);
      if (pc[pp] == 0 && own[pp]) publish_row<kRowValues>(gs, ex, NB, role.cw, pl[pp], part_sum, tag);
    }
    float gd2[PP][4], dvs[PP][4], dr[PP][4];
    if (!in_wavefront) {
      sum_row_values_polled<NB, kRowValues>(gs, ex, gx, tag, sums);
      __syncthreads();
    }
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      float rs[kRowValues];
      if (in_wavefront) {
        gather_row_sums<HSB, kRowValues>(gs, ex, NB, gx, tag, pl[pp], own[pp], rs);
      } else {
#pragma unroll
        for (int i = 0; i < kRowValues; ++i) rs[i] = sums[pl[pp] * RowSlot<kRowValues>::kWords + i];
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) gd2[pp][g] = dvs[pp][g] = dr[pp][g] = 0.f;
      if (act[pp]) {
        const float is3 = s[pp].is3;
        const float dsigma = -0.5f * rs[0] * is3 * is3 * is3;
        const float dmu = (-2.0f * rs[1] * dsigma * invH) - (rs[2] * is3);
        const float dc_ln = (2.0f * xc3[pp] * dsigma * invH) + (is3 * gd3[pp]) + (dmu * invH);
        const float gi = s[pp].vt[0], gg = s[pp].vt[1], gf = s[pp].vt[2];
        const float dc_total = s[pp].dcn + dc[pp] + dc_ln;
        const float df = s[pp].c0 * dc_total;
        dc[pp] = gf * dc_total;
        const float di = gg * dc_total;
        const float dg = gi * dc_total;
        float dv[4];
        dv[0] = d_sigmoid_f(gi) * di;
        dv[1] = d_tanh_f(gg) * dg;
        dv[2] = d_sigmoid_f(gf) * df;
        dv[3] = dv_o[pp];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          dvs[pp][g] = dv[g];
          accs[pp][g] += dv[g];
          gd2[pp][g] = g2[pp][g] * dv[g];
          accs[pp][4 + g] += xc2[pp][g] * s[pp].is2 * dv[g];
        }
        // the row sums of the h*R norm from their coefficients
        const float dmuH = dmu * invH;
        const float t0 = rs[3] + dsigma * rs[4] + dmuH * rs[5];
        const float t1 = rs[6];
        const float t2 = rs[7] + dsigma * rs[8] + dmuH * rs[9];
        const float is2 = s[pp].is2;
        const float dsigma2 = -0.5f * t0 * is2 * is2 * is2;
        const float dmu2 = (-2.0f * t1 * dsigma2 * inv4H) - (t2 * is2);
#pragma unroll
        for (int g = 0; g < 4; ++g)
          dr[pp][g] = (2.0f * xc2[pp][g] * dsigma2 * inv4H) + (is2 * gd2[pp][g]) + (dmu2 * inv4H);
      }
    }
    // What this wavefront stored during the previous step (its resets among it) has landed
    // before the gradients of this step become visible.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    {
      float* xd_t = xd + (done & 3) * tile_floats;
      float* xd_done = xd + ((done + 2) & 3) * tile_floats;  // read two steps ago
#pragma unroll
      for (int pp = 0; pp < PP; ++pp)
        // rows and units beyond the problem are published as zeros
        if (own[pp]) {
          const size_t e = ((size_t)pj[pp] * NB + pl[pp]) * 4;
          store_exchanged4(gs, xd_t + e, publishable(dr[pp][0]), publishable(dr[pp][1]),
                           publishable(dr[pp][2]), publishable(dr[pp][3]));
          if (done + 2 < T) {
            const float u = unwritten_value();
            store_exchanged4(gs, xd_done + e, u, u, u, u);
          }
        }
    }
    // The caller's copies: nobody in the launch waits for them.
#pragma unroll
    for (int pp = 0; pp < PP; ++pp) {
      if (act[pp]) {
        const size_t e4 = ((size_t)t * N + pn[pp]) * 4 * H + pj[pp];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          p.v[e4 + (size_t)g * H] = dvs[pp][g];
          p.act_Rh[e4 + (size_t)g * H] = dr[pp][g];
        }
      }
    }
    fetch(t - 1);
    // The operand loads wait for the gradient w.r.t. h*R of every unit themselves.
    if constexpr (REG > 0)
      tile_product<NB, 1, true, true, false, NoSideWork, REG, float4_t[REG][1]>(
          xdb, (done & 3) * tile_floats, Kpad, w_lds, red, &gs, nullptr, &breg);
    else
      tile_product<NB, 1, true, true>(xdb, (done & 3) * tile_floats, Kpad, w_lds, red, &gs);
    __syncthreads();
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
      dh[pp] = dh_keep[pp] + sum_product<NB, 1>(red, pl[pp], pc[pp]);
    __syncthreads();  // red may be overwritten by the next step
  }

#pragma unroll
  for (int pp = 0; pp < PP; ++pp) {
    if (act[pp]) {
      p.dh[(size_t)pn[pp] * H + pj[pp]] = dh[pp];
      p.dc[(size_t)pn[pp] * H + pj[pp]] = dc[pp];
    }
  }

  // Column sums (bias and norm-scale gradients): rows of this tile in LDS, then tiles in order.
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
      if (a < 4) p.db[a * H + col] += sum;
      else if (a < 8) p.dgamma2[(a - 4) * H + col] += sum;
      else if (a == 8) p.dgamma_h[col] += sum;
      else p.dbeta_h[col] += sum;
    }
  }
}

}  // namespace
}  // namespace haste_hip

extern "C" {

using namespace haste_hip;

int haste_hip_layer_norm_lstm_forward_f32(int training, int steps, int batch_size,
                                          int input_size, int hidden_size,
                                          const float* W, const float* R, const float* b,
                                          const float* x, float* h, float* c,
                                          float* act_Wx, float* tmp_Rh,
                                          const float* gamma1, float* cache1,
                                          float* act_Wx_norm, float* act_Rh,
                                          const float* gamma2, float* cache2,
                                          const float* gamma_h, const float* beta_h, float* cache3,
                                          float* act_c_norm,
                                          float zoneout_prob, const float* zoneout_mask,
                                          void* stream_) {
  (void)tmp_Rh;
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W && R && b && x && h && c && act_Wx && gamma1 && act_Wx_norm && act_Rh);
  HASTE_HIP_REQUIRE(gamma2 && gamma_h && beta_h && act_c_norm);
  hipStream_t stream = as_stream(stream_);
  const ForwardTile tile = pick_forward_tile(4, N, H, 4 * sizeof(float), kMaxLdsBytes, true,
                                             2);
  if (!tile.ok)
    return layer_norm_lstm_forward_streamed(stream, training, T, N, C, H, W, R, b, x, h, c, act_Wx,
                                            gamma1, cache1, act_Wx_norm, act_Rh, gamma2, cache2,
                                            gamma_h, beta_h, cache3, act_c_norm, zoneout_prob,
                                            zoneout_mask);
  const int gx = tile.gx, gy = tile.gy;
  const int NB = tile.nb;
  // one tagged row exchange: [groups][2] buffers of 8-byte words, counted in floats
  const size_t part_floats = (size_t)gy * 2 * tagged_row_words(gx, NB, 2) * 2;

  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, T * N, 4 * H, C, x, C, W, 4 * H, act_Wx, 4 * H, false));
  HASTE_HIP_PROPAGATE(layer_norm_forward(stream, T * N, 4 * H, gamma1, nullptr, act_Wx, act_Wx_norm, cache1));

  // Taken after the GEMM, which may replace the stream's scratch buffer with a larger one.
  Workspace ws;
  const size_t xh_floats = exchange_floats(H, NB, gy, kPolledTiles);
  HASTE_HIP_PROPAGATE(get_workspace(stream, (2 * part_floats + xh_floats) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  LnLstmFwdParams p;
  p.training = training; p.T = T; p.N = N; p.H = H;
  p.R = R; p.b = b; p.h = h; p.c = c; p.v = act_Wx_norm; p.act_Rh = act_Rh;
  p.gamma2 = gamma2; p.cache2 = cache2; p.gamma_h = gamma_h; p.beta_h = beta_h; p.cache3 = cache3;
  p.act_c_norm = act_c_norm; p.zoneout_prob = zoneout_prob; p.zoneout_mask = zoneout_mask;
  p.part2 = reinterpret_cast<unsigned long long*>(ws.scratch);
  p.part3 = reinterpret_cast<unsigned long long*>(ws.scratch + part_floats);
  p.xh = ws.scratch + 2 * part_floats;
  // Tiles of at most 64 elements (one per lane of the idle last wavefront) park the inputs of a
  // step in LDS when there is room: [2][5][NB * HS] floats.  Measured forward, T = 200-500:
  // N = 32, H = 256 -3.5 %, N = 8, H = 128 -3.5 %, N = 4, H = 512 -5 %; with two elements per
  // lane +1.3 % (N = 64, H = 512), and with rows too long for the gathers inside a wavefront
  // +2.5 % (N = 16, H = 1024), so those keep their own requests.
  const size_t park_bytes = (size_t)2 * kLnLstmFwdInputs * NB * tile.hs * sizeof(float);
  const bool parked = tile.reg_groups == 0 && NB * tile.hs <= 64 && gx <= 4 * tile.hs &&
                      tile.lds_bytes + park_bytes <= kMaxLdsBytes;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, gx, gy, tile.nb, tile.lds_bytes + (parked ? park_bytes : 0),
                                  3u * (unsigned)T + 1, &plan));
  p.ls = plan.shape;
#define HASTE_LAUNCH_RESIDENT(NB_, REG_)                                                      \
  if (tile.reg_groups == REG_ && tile.nb == NB_ && tile.ct == 2)                             \
    return launch_persistent("layer_norm_lstm_forward_recurrence",                           \
                             ln_lstm_forward_kernel<NB_, 2, false, REG_>, plan, p, stream);
  HASTE_LAUNCH_RESIDENT(16, 8) HASTE_LAUNCH_RESIDENT(32, 8) HASTE_LAUNCH_RESIDENT(64, 8)
  HASTE_LAUNCH_RESIDENT(16, 16) HASTE_LAUNCH_RESIDENT(32, 16) HASTE_LAUNCH_RESIDENT(64, 16)
#undef HASTE_LAUNCH_RESIDENT
  if (tile.reg_groups > 0) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
#define HASTE_LAUNCH_PARKED(NB_, CT_)                                                        \
  if (parked && tile.nb == NB_ && tile.ct == CT_)                                            \
    return launch_persistent("layer_norm_lstm_forward_recurrence",                           \
                             ln_lstm_forward_kernel<NB_, CT_, true>, plan, p, stream);
  HASTE_LAUNCH_PARKED(4, 1) HASTE_LAUNCH_PARKED(4, 2) HASTE_LAUNCH_PARKED(4, 4)
  HASTE_LAUNCH_PARKED(8, 1) HASTE_LAUNCH_PARKED(8, 2) HASTE_LAUNCH_PARKED(16, 1)
#undef HASTE_LAUNCH_PARKED
#define HASTE_LAUNCH(NB_, CT_)                                                               \
  if (tile.nb == NB_ && tile.ct == CT_)                                                      \
    return launch_persistent("layer_norm_lstm_forward_recurrence",                           \
                             ln_lstm_forward_kernel<NB_, CT_>, plan, p, stream);
  HASTE_LAUNCH(4, 1) HASTE_LAUNCH(4, 2) HASTE_LAUNCH(4, 4)
  HASTE_LAUNCH(8, 1) HASTE_LAUNCH(8, 2) HASTE_LAUNCH(8, 4)
  HASTE_LAUNCH(16, 1) HASTE_LAUNCH(16, 2) HASTE_LAUNCH(16, 4)
  HASTE_LAUNCH(32, 1) HASTE_LAUNCH(32, 2) HASTE_LAUNCH(32, 4)
  HASTE_LAUNCH(64, 1) HASTE_LAUNCH(64, 2) HASTE_LAUNCH(64, 4)
#undef HASTE_LAUNCH
  return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
}

int haste_hip_layer_norm_lstm_backward_f32(int steps, int batch_size, int input_size,
                                           int hidden_size,
                                           const float* W_t, const float* R_t, const float* b,
                                           const float* x_t, const float* h, const float* c,
                                           const float* dh_new, const float* dc_new,
                                           float* dx, float* dW, float* dR, float* db,
                                           float* dh, float* dc,
                                           float* act_Wx, const float* gamma1, float* dgamma1,
                                           float* act_Wx_norm, float* act_Rh,
                                           const float* gamma2, float* dgamma2,
                                           const float* cache2,
                                           const float* gamma_h, const float* beta_h,
                                           float* dgamma_h, float* dbeta_h,
                                           const float* cache3,
                                           float* act_c_norm,
                                           const float* zoneout_mask, void* stream_) {
  (void)b;
  (void)beta_h;
  const int T = steps, N = batch_size, C = input_size, H = hidden_size;
  HASTE_HIP_REQUIRE(T > 0 && N > 0 && C > 0 && H > 0);
  HASTE_HIP_REQUIRE(W_t && R_t && x_t && h && c && dh_new && dc_new);
  HASTE_HIP_REQUIRE(dx && dW && dR && db && dh && dc && act_Wx && gamma1 && dgamma1);
  HASTE_HIP_REQUIRE(act_Wx_norm && act_Rh && gamma2 && dgamma2 && cache2 && gamma_h);
  HASTE_HIP_REQUIRE(dgamma_h && dbeta_h && cache3 && act_c_norm);
  hipStream_t stream = as_stream(stream_);
  // per row: 10 column-sum accumulators of 16 floats (or the partial tiles, whichever is more) + 10 sums
  const BackwardTile tile = pick_backward_tile(4 * H, N, H, 10 * 16, 10, true);
  if (!tile.ok)
    return layer_norm_lstm_backward_streamed(stream, T, N, C, H, W_t, R_t, x_t, h, c, dh_new, dc_new,
                                             dx, dW, dR, db, dh, dc, act_Wx, gamma1, dgamma1,
                                             act_Wx_norm, act_Rh, gamma2, dgamma2, cache2, gamma_h,
                                             dgamma_h, dbeta_h, cache3, act_c_norm, zoneout_mask);
  const int gx = tile.gx, gy = tile.gy;
  const int NB = tile.nb;
  // one tagged row exchange: [groups][2] buffers of 8-byte words, counted in floats
  const size_t part_floats = (size_t)gy * 2 * tagged_row_words(gx, NB, 10) * 2;
  const size_t col_floats = (size_t)gy * 10 * H;
  const size_t col_floats4 = (col_floats + 3) / 4 * 4;

  Workspace ws;
  const size_t xd_floats = exchange_floats(64 * gx, NB, gy, kPolledTiles);
  HASTE_HIP_PROPAGATE(get_workspace(stream, (part_floats + col_floats4 + xd_floats) * sizeof(float), &ws));
  HASTE_HIP_PROPAGATE(check_and_clear_abort(stream, &ws));

  LnLstmBwdParams p;
  p.T = T; p.N = N; p.H = H;
  p.R_t = R_t; p.c = c; p.dh_new = dh_new; p.dc_new = dc_new;
  p.db = db; p.dh = dh; p.dc = dc; p.v = act_Wx_norm; p.act_Rh = act_Rh;
  p.gamma2 = gamma2; p.dgamma2 = dgamma2; p.cache2 = cache2;
  p.gamma_h = gamma_h; p.dgamma_h = dgamma_h; p.dbeta_h = dbeta_h; p.cache3 = cache3;
  p.act_c_norm = act_c_norm; p.zoneout_mask = zoneout_mask;
  p.part = reinterpret_cast<unsigned long long*>(ws.scratch);
  p.col_partial = ws.scratch + part_floats;
  p.xd = ws.scratch + part_floats + col_floats4;
  // Short tiles park the inputs of a step in LDS when there is room: [2][18][NB * 16] floats.
  const size_t park_bytes = (size_t)2 * kLnLstmBwdInputs * NB * 16 * sizeof(float);
  const bool parked = NB <= 8 && tile.reg_groups == 0 && tile.lds_bytes + park_bytes <= kMaxLdsBytes;
  LaunchPlan plan;
  HASTE_HIP_PROPAGATE(plan_launch(stream, ws, gx, gy, tile.nb, tile.lds_bytes + (parked ? park_bytes : 0),
                                  3u * (unsigned)T + 1, &plan));
  p.ls = plan.shape;
  int rc = HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  const char* name = "layer_norm_lstm_backward_recurrence";
#define HASTE_LAUNCH_BWD_RESIDENT(NB_)                                                          \
  (tile.reg_groups == 8    ? launch_persistent(name, ln_lstm_backward_kernel<NB_, 8>, plan, p, stream)  \
   : tile.reg_groups == 16 ? launch_persistent(name, ln_lstm_backward_kernel<NB_, 16>, plan, p, stream) \
   : tile.reg_groups == 24 ? launch_persistent(name, ln_lstm_backward_kernel<NB_, 24>, plan, p, stream) \
                           : launch_persistent(name, ln_lstm_backward_kernel<NB_, 32>, plan, p, stream))
  if (tile.reg_groups > 0) {
    if (NB == 16) rc = HASTE_LAUNCH_BWD_RESIDENT(16);
    else if (NB == 32) rc = HASTE_LAUNCH_BWD_RESIDENT(32);
    else if (NB == 64) rc = HASTE_LAUNCH_BWD_RESIDENT(64);
  }
#undef HASTE_LAUNCH_BWD_RESIDENT
  else if (NB == 4 && parked) rc = launch_persistent(name, ln_lstm_backward_kernel<4, 0, true>, plan, p, stream);
  else if (NB == 8 && parked) rc = launch_persistent(name, ln_lstm_backward_kernel<8, 0, true>, plan, p, stream);
  else if (NB == 4) rc = launch_persistent(name, ln_lstm_backward_kernel<4>, plan, p, stream);
  else if (NB == 8) rc = launch_persistent(name, ln_lstm_backward_kernel<8>, plan, p, stream);
  else if (NB == 16) rc = launch_persistent(name, ln_lstm_backward_kernel<16>, plan, p, stream);
  else if (NB == 32) rc = launch_persistent(name, ln_lstm_backward_kernel<32>, plan, p, stream);
  else if (NB == 64) rc = launch_persistent(name, ln_lstm_backward_kernel<64>, plan, p, stream);
  HASTE_HIP_PROPAGATE(rc);

  // Gradient through the norm of x*W (in place over act_Wx), then the batched products.
  const int TN = T * N;
  HASTE_HIP_PROPAGATE(layer_norm_backward(stream, TN, 4 * H, gamma1, act_Wx, act_Wx_norm, act_Wx,
                                          dgamma1, nullptr));
  HASTE_HIP_PROPAGATE(gemm_f32_pair(stream, C, H, 4 * H, TN, x_t, TN, act_Wx, 4 * H, dW, 4 * H,
                                    h, H, act_Rh, 4 * H, dR, 4 * H, true));
  HASTE_HIP_PROPAGATE(gemm_f32(stream, false, TN, C, 4 * H, act_Wx, 4 * H, W_t, C, dx, C, false));
  return HASTE_HIP_OK;
}

}  // extern "C"
