// The backward recurrence of 4-row batch tiles in scattered form, for any cell whose step is
// "pointwise gradients of the gates, then dh = (gate gradients) * R_t": the kernel, and what a
// cell has to supply (its pointwise step, its inputs, its outputs).
#pragma once

#include "recurrent.h"

namespace haste_hip {

// See "scattered partial sums" in recurrent.h: a workgroup owns 16 hidden units; the first
// wavefront of a set (the owner) does the pointwise step (Cell: gate gradients, state
// gradients, bias sums) on the sums of the pieces
// of dh for those units and hands the gate gradients of every (row, unit) -- one MFMA
// operand register of four floats per lane -- to the other wavefronts of its set through polled words of
// LDS; every wavefront multiplies them with the rows of R_t that belong to the workgroup's
// units and its own 64*CTN output columns (weights in registers) and publishes the pieces of
// the partial sums.  The second wavefront (the helper) also requests the owner's inputs two
// steps ahead and parks them in LDS, and writes the caller's copy of the gate gradients: those
// come from and go to memory that is cold in this launch, and a wavefront's loads return in
// order -- requested by a wavefront that gathers they would stand before the polls of its next
// gather.  The owner, the third and the fourth wavefront gather.
// Cell::pieces(p): the pieces, [batch tiles][2][gx owners][16*CTN producers][64].
// The sets take the workgroup's wavefronts alternately (see set_index).
//
// A Cell supplies
//   Params                 the kernel's arguments: T, N, H, R_t [G*H, H], zoneout_mask, db_partial
//                          [batch tiles][kSums*H], ls, and whatever the cell reads and writes
//   kGates                 gate gradients per element that dh contracts over (rows of R_t per unit)
//   kInputs, kSums         inputs per element and step; column sums per unit (bias gradients)
//   pieces(p)              the exchange area
//   request(p, in, e, ve)  loads the inputs of element e = (t*N + row)*H + unit, ve = (t*N + row)*4H + unit
//   load_state / store_state(p, e)   the gradients carried from step to step, e = row*H + unit
//   prepare(sv)            the part of a step that does not depend on the gathered sums
//   step(act, zoneout, sums)         the rest: returns the MFMA operand (kGates gate gradients,
//                          further components for store_copy), adds to the column sums
//   add_gathered(sum)      dh of the next step = what step() kept + the gathered sums
//   store_copy(p, t, row, unit, a)   the caller's copy of the gate gradients
//   add_sums(p, col, s)    column sum `col` (of kSums*H) of the whole batch
// HALF: the product runs on the half matrix cores (scatter_product_half), for cells whose
// tensors are half; everything else of the step stays in fp32.
template <class Cell, int CTN, int SETS, bool HALF = false>
__global__ __launch_bounds__(256 * SETS, 1)
void scatter_backward_kernel(typename Cell::Params p) {
  using S = ScatterShape<CTN>;
  constexpr int HSB = 16;
  constexpr int NP = S::kProducers;
  constexpr int G = Cell::kGates;
  constexpr int kInputs = Cell::kInputs;
  constexpr int kSums = Cell::kSums;
  static_assert(kInputs <= 12 && G <= 4, "LDS parking areas, operand register");
  __shared__ unsigned int s_role;
  __shared__ unsigned int s_flag;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const Role role = take_role(p.ls, &s_role);
  if (!role.active) return;

  const int H = p.H, N = p.N, T = p.T, gx = p.ls.gx;
  const int set = set_index<SETS>();
  const int wave = set_wave<SETS>();
  const int lane = threadIdx.x & 63;
  const int set_tid = wave * 64 + lane;
  const int cw = role.cw;
  const int j0 = cw * HSB;
  const int bt = role.bt * SETS + set;  // this set's batch tile
  const int n0 = bt * 4;
  const int rows_here = (N - n0) < 4 ? (N - n0) : 4;  // <= 0: a set without rows
  const size_t NH = (size_t)N * H;
  // wavefronts whose output columns exist
  const int live_waves = (H + S::kColumns - 1) / S::kColumns;
  const bool owner = wave == 0, helper = wave == 1;

  // LDS of this set: the owner's operand by step parity and reader; the other gathering
  // wavefronts' sums by step parity; the parked inputs by step parity; the step each parking
  // area holds.
  float* set_lds = lds + (size_t)set * kScatterSetFloats;
  float (*s_hand)[3][64 * 4] = reinterpret_cast<float (*)[3][64 * 4]>(set_lds);
  float (*s_part)[2][64 * 4] = reinterpret_cast<float (*)[2][64 * 4]>(set_lds + kScatterHandFloats);
  float (*s_park)[kInputs][64] =
      reinterpret_cast<float (*)[kInputs][64]>(set_lds + kScatterHandFloats + kScatterPartFloats);
  unsigned int* s_parked = reinterpret_cast<unsigned int*>(set_lds + kScatterHandFloats + kScatterPartFloats +
                                                           kScatterParkFloats);

  GroupSync gs;
  group_sync_init(gs, p.ls, role);

  const int tile_floats = gx * NP * S::kPieceFloats;
  float* xp = Cell::pieces(p) + (size_t)bt * kScatterTiles * tile_floats;
  const TileBuffer xpb = make_tile_buffer(xp, kScatterTiles * tile_floats);

  // The wavefront's weights: rows (gate c, unit j0 + a) of R_t, columns (wave*CTN + ct)*64 + lane.
  float wreg[HALF ? 1 : 16][G][CTN];
  half4_t whalf[HALF ? 16 : 1][CTN];
#pragma unroll
  for (int a = 0; a < 16; ++a)
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int ct = 0; ct < CTN; ++ct) {
        const int unit = j0 + a, col = (wave * CTN + ct) * 64 + lane;
        const bool ok = c < G && unit < H && col < H;
        if (c < G || HALF) {
          const float x = p.R_t[ok ? ((size_t)c * H + unit) * H + col : 0];
          if constexpr (HALF) whalf[a][ct][c] = (_Float16)(ok ? x : 0.f);
          else wreg[a][c < G ? c : 0][ct] = ok ? x : 0.f;
        }
      }

  // The pieces this lane publishes: columns (wave*CTN + ct)*64 + lane belong to owner col/16,
  // whose piece from this producer keeps the 4 rows of unit col%16 at float 4*(col%16).
  int pub_off[CTN];
  bool pub_ok[CTN];
#pragma unroll
  for (int ct = 0; ct < CTN; ++ct) {
    const int col = (wave * CTN + ct) * 64 + lane;
    const int o = col >> 4;
    pub_ok[ct] = o < gx;
    pub_off[ct] = ((pub_ok[ct] ? o : 0) * NP + cw) * S::kPieceFloats + (col & 15) * 4;
  }
  // All pieces start out with the tag their first publication does not have.  One real barrier:
  // nobody polls before everybody has set up.
  {
    const float stale = __uint_as_float(1u ^ scatter_tag(0));
#pragma unroll
    for (int ct = 0; ct < CTN; ++ct)
      if (pub_ok[ct])
        for (int b = 0; b < kScatterTiles; ++b)
          store_exchanged4(gs, xp + (size_t)b * tile_floats + pub_off[ct], stale, stale, stale, stale);
    // the padding of this workgroup's own row of pieces (producers that do not exist) holds
    // zeros: it is added up with the rest
    for (int i = set_tid; i < (NP - gx) * S::kPieceFloats; i += 256)
      for (int b = 0; b < kScatterTiles; ++b)
        store_exchanged(gs, xp + (size_t)b * tile_floats + (cw * NP + gx) * S::kPieceFloats + i, 0.f);
    const float u = unwritten_value();
    for (int i = set_tid; i < (int)(kScatterHandFloats + kScatterPartFloats); i += 256) set_lds[i] = u;
    if (set_tid < 2) s_parked[set_tid] = 0u;
  }

  // Pointwise ownership (owner; the helper loads the inputs of the same elements): lane
  // 16*g + u handles batch row n0 + scatter_row(g), unit j0 + u.
  const int pr = scatter_row(lane >> 4), pu = lane & 15;
  const int pn = n0 + pr, pj = j0 + pu;
  const bool act = pr < rows_here && pj < H;
  const size_t row = act ? (size_t)pn : 0, unit = act ? (size_t)pj : 0;
  // The MFMA operand's lanes: lane 4*u + r holds the gate gradients of (row r, unit u).
  const int mr = lane & 3, mu = lane >> 2;
  const bool zoneout = p.zoneout_mask != nullptr;
  Cell cell;
  cell.load_state(p, row * H + unit, owner && act);
  float sums[kSums];
#pragma unroll
  for (int g = 0; g < kSums; ++g) sums[g] = 0.f;

  // Step inputs that do not depend on the recurrence.  Every lane of the helper loads (lanes
  // without an element some valid address: their values are never used).
  float in[kInputs];
#pragma unroll
  for (int i = 0; i < kInputs; ++i) in[i] = 1.f;
  auto request = [&](int t) {
    const size_t tt = t >= 0 ? t : 0;
    Cell::request(p, in, tt * NH + row * H + unit, (tt * N + row) * 4 * H + unit, zoneout);
  };
  // step index d (0 .. T-1) works on time step T-1-d; its inputs are parked in area d%2,
  // marked with d+1
  auto park = [&](int d) {
#pragma unroll
    for (int i = 0; i < kInputs; ++i) s_park[d & 1][i][lane] = in[i];
    if (lane == 0) s_parked[d & 1] = (unsigned int)d + 1u;
  };
  group_arrive(gs);  // also: the LDS of the set is set up
  group_wait(gs);
  if (helper) {
    request(T - 1);
    park(0);
    request(T - 2);
  }

  const bool steps = rows_here > 0;
  const bool multiplies = wave < live_waves;
  const int owner_off = cw * NP * S::kPieceFloats;  // this workgroup's row of pieces
  // The sums of the pieces published at step d, as far as this wavefront gathers them.
  auto gather_own = [&](int d) {
    PieceGather<S::kOwnerLoads> pieces;
    pieces.request(xpb, (d & 1) * tile_floats + owner_off, 0, gx);
    return pieces;
  };
  auto gather_other = [&](int d) {
    PieceGather<S::kOtherLoads> pieces;
    pieces.request(xpb, (d & 1) * tile_floats + owner_off, S::kOwnerLoads + (wave - 2) * S::kOtherLoads, gx);
    const float4_t sum = publishable4(pieces.finish(gs, xpb, scatter_tag(d)));
    *reinterpret_cast<float4_t*>(&s_part[d & 1][wave - 2][lane * 4]) = sum;
  };
  auto all_sums = [&](PieceGather<S::kOwnerLoads>& pieces, int d) {
    float4_t sum = pieces.finish(gs, xpb, scatter_tag(d));
    float4_t s2, s3;
    take_lds4_pair(gs, reinterpret_cast<float4_t*>(&s_part[d & 1][0][lane * 4]),
                   reinterpret_cast<float4_t*>(&s_part[d & 1][1][lane * 4]), s2, s3);
    sum += s2;
    sum += s3;
    return scatter_lane_groups(sum);
  };
  for (int d = 0; steps && d < T; ++d) {
    const int t = T - 1 - d;
    float4_t a;
    if (owner) {
      // dh of this step: what the step before left here plus the pieces every producer
      // published at that step.  Requested first; what does not depend on it is done meanwhile.
      PieceGather<S::kOwnerLoads> pieces;
      if (d > 0) pieces = gather_own(d - 1);
      // the inputs the helper parked
      {
        volatile unsigned int* mark = &s_parked[d & 1];
        unsigned int seen = *mark;
        poll_until_written(gs, [&] { __builtin_amdgcn_s_sleep(1); seen = *mark; },
                           [&] { return seen == (unsigned int)d + 1u; });
      }
      float sv[kInputs];
#pragma unroll
      for (int i = 0; i < kInputs; ++i) sv[i] = s_park[d & 1][i][lane];
      cell.prepare(sv);
      if (d > 0) cell.add_gathered(all_sums(pieces, d - 1));
      const float4_t dv = cell.step(act, zoneout, sums);
      // to the lanes of the MFMA operand: for the other wavefronts through LDS, for this one
      // across its lanes (lane 4*u + r takes from lane 16*scatter_row(r) + u)
      const float4_t ap = publishable4(dv);
      for (int r = 0; r < 3; ++r) *reinterpret_cast<float4_t*>(&s_hand[d & 1][r][(4 * pu + pr) * 4]) = ap;
      const int from = (16 * scatter_row(mr) + mu) * 4;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        a[g] = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(dv[g])));
    } else {
      // The helper parks the inputs of the next step, requested a step ago, while it waits for
      // the owner (who has read those of the step before this one: it handed over its operand
      // afterwards).  The third and fourth wavefront gather their shares of the owner's pieces.
      if (helper) park(d + 1);
      else if (d > 0) gather_other(d - 1);
      // The owner's gate gradients, through LDS.  Every wavefront takes them, also one without
      // output columns: a share of pieces that is all padding never waits, and nothing else
      // would keep such a wavefront from running steps ahead of the owner that reads its sums.
      a = take_lds4(gs, reinterpret_cast<float4_t*>(&s_hand[d & 1][wave - 1][lane * 4]));
    }

    if (multiplies) {
      float4_t acc[2][CTN];
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int ct = 0; ct < CTN; ++ct) acc[c][ct] = float4_t{0.f, 0.f, 0.f, 0.f};
      if constexpr (HALF) scatter_product_half<G, CTN>(a, whalf, acc);
      else scatter_product<G, CTN>(a, wreg, acc);
      float* tile_pub = xp + (size_t)(d & 1) * tile_floats;
      const unsigned int tag = scatter_tag(d);
#pragma unroll
      for (int ct = 0; ct < CTN; ++ct) {
        const float4_t s = tagged4(acc[0][ct] + acc[1][ct], tag);
        if (pub_ok[ct]) store_exchanged4(gs, tile_pub + pub_off[ct], s.x, s.y, s.z, s.w);
      }
    }
    if (helper) {
      // The caller's copy: nobody in the launch waits for it.
      if (mr < rows_here && j0 + mu < H) Cell::store_copy(p, t, (size_t)(n0 + mr), (size_t)(j0 + mu), a);
      request(t - 2);
    }
  }

  // the sums the last step left
  if (steps && wave >= 2) gather_other(T - 1);
  if (owner && steps) {
    PieceGather<S::kOwnerLoads> pieces = gather_own(T - 1);
    cell.add_gathered(all_sums(pieces, T - 1));
    if (act) cell.store_state(p, (size_t)pn * H + pj);
  }

  // Column sums (bias gradients): the rows of this tile are in the four lane groups (fixed
  // order), parked per tile; the last workgroup of the column block to finish adds the tiles in
  // order.
  if (owner) {
#pragma unroll
    for (int g = 0; g < kSums; ++g) {
      float s = act ? sums[g] : 0.f;
      s += __shfl_xor(s, 32, 64);  // rows 0 + 1 (lane groups 0, 2), rows 2 + 3 (lane groups 1, 3)
      s += __shfl_xor(s, 16, 64);
      if (lane < 16 && pj < H) store_agent(&p.db_partial[(size_t)bt * kSums * H + g * H + pj], s);
    }
  }
  if (column_last_arrival(p.ls.cb, cw, (unsigned)p.ls.gy, &s_flag)) {
    const int tid = threadIdx.x;
    if (tid < kSums * HSB && j0 + tid % HSB < H) {
      const int col = (tid / HSB) * H + j0 + tid % HSB;
      Cell::add_sums(p, col, sum_over_tiles(p.db_partial + col, (size_t)kSums * H, p.ls.gy * SETS));
    }
  }
}


// Launches the kernel for `sets` sets per workgroup and hidden size H <= 512.
template <class Cell, bool HALF = false>
int launch_scatter_backward(const char* name, int H, int sets, const LaunchPlan& plan, typename Cell::Params& p,
                            hipStream_t stream) {
  if (H <= 256)
    return sets == 2 ? launch_persistent(name, scatter_backward_kernel<Cell, 1, 2, HALF>, plan, p, stream)
                     : launch_persistent(name, scatter_backward_kernel<Cell, 1, 1, HALF>, plan, p, stream);
  return sets == 2 ? launch_persistent(name, scatter_backward_kernel<Cell, 2, 2, HALF>, plan, p, stream)
                   : launch_persistent(name, scatter_backward_kernel<Cell, 2, 1, HALF>, plan, p, stream);
}

}  // namespace haste_hip
