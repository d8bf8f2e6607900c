// Device-side building blocks of the persistent recurrence kernels.
//
// A recurrence kernel is one launch that runs all T steps (an ordinary launch whose grid
// is checked against what the chip can hold at once).  The grid is (column workgroups) x
// (batch tiles): a workgroup owns `HS` hidden units (all of their gate columns) for the NB
// batch rows of its tile, keeps its slice of the recurrent weight matrix in LDS for the
// whole launch, and per step multiplies the tile's rows of the exchanged activation (h_t
// forward, the gate gradients backward) with that slice on the MFMA units.  Workgroups that
// share a batch tile form a group and hand each step's activations to each other through
// tiles in device memory whose consumers poll for the data itself (or, at set-up, through
// per-workgroup flag words); different batch tiles never wait for each other.
#pragma once

#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <utility>

#include "common.h"

namespace haste_hip {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));


// Gate nonlinearities on the hardware exp2 and reciprocal (about 1 ulp each): absolute
// error around 1e-7, the size of one fp32 rounding of the result.
__device__ __forceinline__ float exp_f(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269504088896341f);
}
__device__ __forceinline__ float sigmoid_f(float x) {
  return __builtin_amdgcn_rcpf(1.0f + exp_f(-x));
}
// Small arguments use the odd series (truncation below 1e-7 for |x| < 0.25), which keeps
// the relative accuracy that 1 - 2/(exp(2x)+1) loses to cancellation there.
__device__ __forceinline__ float tanh_f(float x) {
  const float x2 = x * x;
  const float series =
      x * (1.0f + x2 * (-0.333333333f + x2 * (0.133333333f + x2 * -0.0539682540f)));
  const float wide = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + exp_f(2.0f * x));
  return fabsf(x) < 0.25f ? series : wide;
}
__device__ __forceinline__ float d_sigmoid_f(float y) { return y * (1.0f - y); }
__device__ __forceinline__ float d_tanh_f(float y) { return 1.0f - y * y; }

// ---- Exchange between workgroups inside one launch --------------------------------
// The 8 XCDs of the chip have separate L2 caches, every CU has its own L1.  Data one
// workgroup writes and another reads in the same launch is always READ with agent-scope
// loads (the sc1 form of the load instructions): they never trust the reader's L1, which
// nothing invalidates between the steps of a launch and which may still hold what the
// address contained two steps ago; they are served by the L2 when the line was written
// through that L2, and otherwise come from the memory side.  How the data is WRITTEN
// depends on where the readers are: when a whole group sits on one XCD an ordinary store
// is enough (the shared L2 is the meeting point, ~0.25 us one way); when the group spans
// XCDs the store is agent scope too (written through to the memory side, ~0.4 us one
// way).  Everything else uses ordinary cached accesses: no cache-wide write-back or
// invalidate is needed at a step boundary.
__device__ __forceinline__ float load_exchanged(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16-byte aligned p.
__device__ __forceinline__ float4_t load_exchanged4(const float* p) {
  const unsigned long long* q = reinterpret_cast<const unsigned long long*>(p);
  const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  float4_t v;
  v.x = __uint_as_float((unsigned int)lo);
  v.y = __uint_as_float((unsigned int)(lo >> 32));
  v.z = __uint_as_float((unsigned int)hi);
  v.w = __uint_as_float((unsigned int)(hi >> 32));
  return v;
}

// A workgroup of 512 threads (SETS == 2) holds two sets of 256 threads (four wavefronts) that
// work on batch tiles of their own.  The sets take the workgroup's wavefronts alternately:
// wavefronts land on the CU's four SIMDs round-robin, so each set gets two SIMDs of its own
// and the products of one set never delay the pointwise work of the other (measured: sets
// of four consecutive wavefronts, which share all four SIMDs, are 12 % slower per step).
// set_thread: thread index inside the set (0..255); set_wave: wavefront inside the set.
// (Both are the same in every lane of a wavefront, which the compiler cannot see from
// threadIdx: told so, it keeps what is derived from them -- tile addresses, buffer resources
// -- in scalar registers instead of wrapping every buffer load in a loop over the distinct
// resources its lanes might hold.)
template <int SETS>
__device__ __forceinline__ int set_index() {
  return SETS == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)((threadIdx.x >> 6) & 1));
}
template <int SETS>
__device__ __forceinline__ int set_wave() {
  return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> (SETS == 1 ? 6 : 7)));
}
template <int SETS>
__device__ __forceinline__ int set_thread() {
  return SETS == 1 ? (int)threadIdx.x : (int)(((threadIdx.x >> 7) << 6) | (threadIdx.x & 63));
}

// What the host tells a persistent kernel about its launch.
struct LaunchShape {
  ControlBlock* cb;
  unsigned int* host_status;   // pinned host word the kernel reports an abort to
  unsigned int spin_limit;     // polls before a barrier wait gives up
  unsigned int epoch;          // step flags of this launch count up from here
  unsigned int ticket_base;    // per-XCD tickets of this launch count up from here
  int gx, gy;                  // column workgroups per group, number of groups (batch tiles)
  int tile_rows;               // batch rows per group (the kernel's NB)
  int xcd_local;               // 1: group g is the set of workgroups running on XCD g
  int per_xcd;                 // workgroups this launch places on every XCD (xcd_local)
  unsigned long long xcc_map;  // 4 bits per hardware XCC id: which group runs there (xcd_local)
  int absent;                  // workgroups the barriers wait for although nobody plays them
                               // (0 except in the test of the time-out path)
};

// The part of the problem a workgroup works on.
struct Role {
  int cw;       // column workgroup index inside the group
  int bt;       // group = batch tile
  bool active;  // false: nothing to do (surplus workgroup of an XCD-local launch)
};

__device__ __forceinline__ unsigned int xcc_id() {
  unsigned int v;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
  return v & 0xfu;
}

// Cross-XCD launches use the grid coordinates.  XCD-local launches fill every CU with one
// workgroup; a workgroup reads which XCD it runs on and draws a ticket there: XCD x hosts
// batch tile x and the ticket is the column index.  If an XCD turns out to host more
// workgroups than the launch assumed, the launch is aborted (bounded waits, error status).
// `word` is a word of LDS.  Called by all threads.
__device__ __forceinline__ Role take_role(const LaunchShape& ls, unsigned int* word) {
  Role r;
  if (!ls.xcd_local) {
    r.cw = blockIdx.x;
    r.bt = blockIdx.y;
    r.active = true;
    return r;
  }
  if (threadIdx.x == 0) {
    const unsigned int xcc = xcc_id();
    const unsigned int ticket =
        __hip_atomic_fetch_add(&ls.cb->xcd_ticket[xcc * kCounterStride], 1u, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT) - ls.ticket_base;
    if (ticket >= (unsigned int)ls.per_xcd) {
      __hip_atomic_store(&ls.cb->abort_flag[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(ls.host_status, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      *word = 0xffffffffu;
    } else {
      *word = ((unsigned int)((ls.xcc_map >> (4 * xcc)) & 0xfull) << 16) | ticket;
    }
  }
  __syncthreads();
  const unsigned int w = *word;
  r.bt = (int)(w >> 16);
  r.cw = (int)(w & 0xffffu);
  r.active = w != 0xffffffffu && r.bt < ls.gy && r.cw < ls.gx;
  return r;
}

// Per-workgroup view of its group's step barrier: one flag word per workgroup holding
// the number of arrivals it has made (offset by a per-launch epoch so that the words
// never need clearing).  Arriving is one store; waiting is one wavefront reading the
// group's flags side by side, so no read-modify-write traffic is serialised.
struct GroupSync {
  unsigned int* flags;         // this group's flag words, one per workgroup
  unsigned int* abort_flag;    // device-wide: some wait gave up
  unsigned int* host_status;   // pinned host word mirrored from abort_flag
  unsigned int group_size;
  unsigned int my_index;
  unsigned int epoch;          // value of the flags after `arrivals` arrivals is epoch + arrivals
  unsigned int arrivals;
  unsigned int spin_limit;
  bool same_xcd;               // every workgroup of the group shares one L2
};

__device__ __forceinline__ void group_sync_init(GroupSync& g, const LaunchShape& ls, const Role& r) {
  g.flags = &ls.cb->step_flags[r.bt * ls.gx];
  g.abort_flag = &ls.cb->abort_flag[0];
  g.host_status = ls.host_status;
  g.group_size = (unsigned int)(ls.gx + ls.absent);
  g.my_index = (unsigned int)r.cw;
  g.epoch = ls.epoch;
  g.arrivals = 0;
  g.spin_limit = ls.spin_limit;
  g.same_xcd = ls.xcd_local != 0;
}

__device__ __forceinline__ void store_exchanged(const GroupSync& g, float* p, float v) {
  if (g.same_xcd) *p = v;
  else __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 8-byte aligned p.
__device__ __forceinline__ void store_exchanged2(const GroupSync& g, float* p, float a, float b) {
  if (g.same_xcd) {
    *reinterpret_cast<float2*>(p) = make_float2(a, b);
    return;
  }
  const unsigned long long bits =
      (unsigned long long)__float_as_uint(a) | ((unsigned long long)__float_as_uint(b) << 32);
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), bits, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// 16-byte aligned p.
__device__ __forceinline__ void store_exchanged4(const GroupSync& g, float* p, float a, float b,
                                                 float c, float d) {
  if (g.same_xcd) {
    *reinterpret_cast<float4_t*>(p) = float4_t{a, b, c, d};
    return;
  }
  store_exchanged2(g, p, a, b);
  store_exchanged2(g, p + 2, c, d);
}

// Counts the workgroup as arrived once every exchanged store its threads have issued
// has completed.  Called by all threads.
__device__ __forceinline__ void group_arrive(GroupSync& g) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  g.arrivals += 1;
  if (threadIdx.x == 0) {
    if (g.same_xcd)
      *reinterpret_cast<volatile unsigned int*>(&g.flags[g.my_index]) = g.epoch + g.arrivals;
    else
      __hip_atomic_store(&g.flags[g.my_index], g.epoch + g.arrivals, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Blocks until every workgroup of the group has made as many arrivals as this one.
// The wait is bounded: after spin_limit polls (or when another workgroup has given
// up) it raises the abort flag and returns, so that every wavefront still reaches the
// end of the kernel.  Called by all threads; exchanged loads may follow directly.
__device__ __forceinline__ void group_wait(GroupSync& g) {
  if (threadIdx.x < 64) {
    const unsigned int target = g.epoch + g.arrivals;
    unsigned int spins = 0;
    for (;;) {
      bool ok = true;
      for (unsigned int i = threadIdx.x; i < g.group_size; i += 64) {
        const unsigned int f =
            __hip_atomic_load(&g.flags[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = ok && (int)(f - target) >= 0;
      }
      if (__all(ok)) break;
      __builtin_amdgcn_s_sleep(1);
      ++spins;
      if ((spins & 255u) == 0u) {
        unsigned int ab = __hip_atomic_load(g.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (spins >= g.spin_limit && threadIdx.x == 0) {
          __hip_atomic_store(g.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(g.host_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        if (ab != 0u || spins >= g.spin_limit) break;
      }
    }
  }
  __syncthreads();
}

// Publishing without cache-wide fences: agent-scope stores (store_agent) before an arrival,
// agent-scope loads (load_exchanged) after it (release / acquire fences at agent scope would
// write back and invalidate whole caches instead).
__device__ __forceinline__ void store_agent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// True in the last of the `gy` workgroups with column index `cw` (one per batch tile) to
// call it; data is published with store_agent before and read with load_exchanged after
// the call.  Lets every column block
// finish its own column sums instead of one workgroup finishing all of them.
__device__ __forceinline__ bool column_last_arrival(ControlBlock* cb, int cw, unsigned int gy,
                                                    unsigned int* flag) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned int old = __hip_atomic_fetch_add(&cb->tile_counter[cw], 1u, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
    const bool last = old == gy - 1;
    if (last)
      __hip_atomic_store(&cb->tile_counter[cw], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last ? 1u : 0u;
  }
  __syncthreads();
  return *flag != 0u;
}

// base[0] + base[stride] + ... (gy terms, in that order), read with agent-scope loads that
// are issued eight at a time.
__device__ __forceinline__ float sum_over_tiles(const float* base, size_t stride, int gy) {
  float s = 0.f;
  for (int b0 = 0; b0 < gy; b0 += 8) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = b0 + i < gy ? load_exchanged(base + (size_t)(b0 + i) * stride) : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += v[i];
  }
  return s;
}

__device__ __forceinline__ int round_up(int x, int m) { return (x + m - 1) / m * m; }

// LDS image of a weight slice: element (k, col) of a [Kpad x NCOLS] slice lives at
// float index (((k/16)*4 + (k%16)/4) * NCOLS + col) * 4 + k%4, i.e. the 4 consecutive
// k a lane feeds to 4 consecutive 16x16x4 MFMAs are one 16-byte LDS read, and the 16
// lanes of a k-quarter read 16 consecutive such vectors (no bank conflicts).
__device__ __forceinline__ int slice_index(int k, int col, int ncols) {
  return ((((k >> 4) << 2) + ((k & 15) >> 2)) * ncols + col) * 4 + (k & 3);
}

// Fills the resident slice.  `offset(k, col)` is the element's index in `src` (and in
// `mask`, when DropConnect is fused) or -1 for padding; the four columns of an aligned
// column quad must be adjacent in memory whenever the quad's first and last are valid
// (true for the gate-block layouts of R and R_t).  A thread takes 4 consecutive k of one
// column quad: four 16-byte loads, all issued before the first use (several items per
// thread are in flight at once), a 4x4 transpose in registers, four 16-byte LDS stores.
// `fast`: src (and mask) are 16-byte aligned, every valid quad starts at a multiple of 4
// elements and no quad is partly valid (row lengths and column origins are multiples of
// 4); otherwise the slice is filled element by element.
template <int NCOLS, class OffsetFn>
__device__ __forceinline__ void fill_slice(float* w_lds, int Kpad, const float* __restrict__ src,
                                           const float* __restrict__ mask, float scale, bool fast,
                                           OffsetFn offset) {
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  if (!fast) {
    for (int idx = tid; idx < Kpad * NCOLS; idx += nthreads) {
      const int k = idx / NCOLS, col = idx % NCOLS;
      const long long off = offset(k, col);
      float w = 0.f;
      if (off >= 0) {
        w = src[off];
        if (mask != nullptr) w = w * mask[off] * scale;
      }
      w_lds[slice_index(k, col, NCOLS)] = w;
    }
    return;
  }
  constexpr int QUADS = NCOLS / 4;
  constexpr int UNROLL = 4;
  const int items = (Kpad / 4) * QUADS;
  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  for (int base = tid; base < items; base += nthreads * UNROLL) {
    float4_t v[UNROLL][4];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int item = base + nthreads * u;
      const int k4 = item / QUADS, col = (item % QUADS) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const long long o0 = item < items ? offset(4 * k4 + i, col) : -1;
        const long long o3 = item < items ? offset(4 * k4 + i, col + 3) : -1;
        const bool whole = o0 >= 0 && o3 >= 0;
        float4_t w = *reinterpret_cast<const float4_t*>(src + (whole ? o0 : 0));
        if (mask != nullptr)
          w = w * *reinterpret_cast<const float4_t*>(mask + (whole ? o0 : 0)) * scale;
        v[u][i] = whole ? w : zero4;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int item = base + nthreads * u;
      if (item < items) {
        const int k4 = item / QUADS, col = (item % QUADS) * 4;
        float* dst = w_lds + ((size_t)k4 * NCOLS + col) * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c)
          *reinterpret_cast<float4_t*>(dst + 4 * c) =
              float4_t{v[u][0][c], v[u][1][c], v[u][2][c], v[u][3][c]};
      }
    }
  }
}

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(std::integral_constant<int, i>) for i = 0 .. N-1, unrolled at compile time (MFMA
// broadcast selectors must be immediates).
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// MFMAs of k-groups [g_abs, g_abs+CHUNK): one straight-line block (no branches, so the
// accumulators stay in the matrix unit's registers).  The LDS reads of the slice columns
// run kTallLdsAhead blocks ahead of the MFMAs that use them; a scheduling barrier keeps each
// read where it is issued (the compiler would otherwise sink it to just before its use and
// the wavefront would wait out the LDS latency once per block).  Consecutive MFMAs go to
// different accumulators (two per output tile, alternating by k-group): with one output
// tile per wavefront a block is two k-groups whose MFMAs alternate, so that none waits for
// the result of the one before it.
constexpr int kTallLdsAhead = 2;

// Keeps the two MFMAs issued before it ahead of those issued after it (an empty statement
// the compiler cannot move accumulator updates across): the compiler otherwise lines up the
// four dependent MFMAs of one k-group, each of which waits for the one before it.
__device__ __forceinline__ void pin_mfma_pair(float4_t& a, float4_t& b) {
  asm volatile("" : "+a"(a), "+a"(b));
}

template <int RT, int CT, int CHUNK>
__device__ __forceinline__ void mfma_chunk(const float* w_lds, int g_abs,
                                           const float4_t (&av)[CHUNK][RT],
                                           float4_t (&acc0)[RT][CT], float4_t (&acc1)[RT][CT]) {
  constexpr int NCOLS = 16 * CT;
  constexpr int P = (RT * CT == 1 && CHUNK % 2 == 0) ? 2 : 1;  // k-groups per block
  constexpr int BLOCKS = CHUNK / P;
  constexpr int AHEAD = BLOCKS < kTallLdsAhead ? BLOCKS : kTallLdsAhead;
  const int lane = threadIdx.x & 63;
  const int row = lane & 15;
  const int kq = lane >> 4;
  const float* wp0 = w_lds + ((g_abs * 4 + kq) * NCOLS + row) * 4;
  float4_t b[CHUNK][CT];
  auto read_block = [&](auto bc) {
    constexpr int B = decltype(bc)::value;
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        b[B * P + p][ct] = *reinterpret_cast<const float4_t*>(wp0 + (B * P + p) * 4 * NCOLS * 4 + ct * 64);
  };
  static_for<AHEAD>(read_block);
  static_for<BLOCKS>([&](auto bc) {
    constexpr int B = decltype(bc)::value;
    if constexpr (B + AHEAD < BLOCKS) {
      read_block(std::integral_constant<int, B + AHEAD>{});
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
#pragma unroll
      for (int p = 0; p < P; ++p) {
        constexpr int G0 = B * P;
        float4_t (&acc)[RT][CT] = ((G0 + p) & 1) ? acc1 : acc0;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[G0 + p][rt][c], b[G0 + p][ct][c],
                                                               acc[rt][ct], 0, 0, 0);
      }
      if constexpr (P == 2) pin_mfma_pair(acc0[0][0], acc1[0][0]);
    }
  });
}

// The same MFMAs for k-groups whose slice rows the lanes hold in registers: lane (kq, row)
// keeps in breg[j][ct] what mfma_chunk reads from the slice in LDS for its wavefront's
// j-th k-group (see load_resident_rows).
template <int RT, int CT, int CHUNK, int REG, int FIRST>
__device__ __forceinline__ void mfma_chunk_resident(const float4_t (&breg)[REG][CT],
                                                    const float4_t (&av)[CHUNK][RT],
                                                    float4_t (&acc0)[RT][CT], float4_t (&acc1)[RT][CT]) {
  static_assert(FIRST + CHUNK <= REG, "chunk beyond the resident rows");
  constexpr int P = (RT * CT == 1 && CHUNK % 2 == 0) ? 2 : 1;  // k-groups whose MFMAs alternate
#pragma unroll
  for (int g0 = 0; g0 < CHUNK; g0 += P)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
#pragma unroll
      for (int p = 0; p < P; ++p) {
        float4_t (&acc)[RT][CT] = ((g0 + p) & 1) ? acc1 : acc0;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[g0 + p][rt][c], breg[FIRST + g0 + p][ct][c],
                                                               acc[rt][ct], 0, 0, 0);
      }
      if constexpr (P == 2) pin_mfma_pair(acc0[0][0], acc1[0][0]);
    }
}

// A slice too large for LDS keeps the first REG k-groups of every wavefront's share in
// that wavefront's registers and the rest in LDS, compacted: LDS k-group w*(groups-REG) + j
// is k-group w*groups + REG + j of the contraction (groups = Kpad/64 per wavefront).
__device__ __forceinline__ int resident_split_k(int k_lds, int groups, int reg_groups) {
  const int lds_groups = groups - reg_groups;
  const int gl = k_lds >> 4;
  return ((gl / lds_groups) * groups + reg_groups + gl % lds_groups) * 16 + (k_lds & 15);
}

// Loads the register-resident rows of this wavefront: `offset(k, col)` as for fill_slice,
// `mask` and `scale` likewise (DropConnect).
template <int REG, int CT, class OffsetFn>
__device__ __forceinline__ void load_resident_rows(float4_t (&breg)[REG][CT], int groups,
                                                   const float* __restrict__ src,
                                                   const float* __restrict__ mask, float scale,
                                                   OffsetFn offset) {
  const int lane = threadIdx.x & 63;
  const int wave = (threadIdx.x >> 6) & 3;
  const int col0 = lane & 15, kq = lane >> 4;
#pragma unroll
  for (int j = 0; j < REG; ++j)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int k = (wave * groups + j) * 16 + kq * 4;
      float w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const long long off = offset(k + i, ct * 16 + col0);
        w[i] = src[off >= 0 ? off : 0];
        if (mask != nullptr) w[i] = w[i] * mask[off >= 0 ? off : 0] * scale;
        if (off < 0) w[i] = 0.f;
      }
      breg[j][ct] = float4_t{w[0], w[1], w[2], w[3]};
    }
}

// Writes this wavefront's accumulators to red[wave][16*RT][16*CT] in LDS.
template <int RT, int CT>
__device__ __forceinline__ void store_partials(float* red, const float4_t (&acc)[RT][CT]) {
  constexpr int NCOLS = 16 * CT;
  constexpr int NB = 16 * RT;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  float* base = red + wave * NB * NCOLS;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int col = ct * 16 + (lane & 15);
      const int r0 = rt * 16 + (lane >> 4) * 4;
      base[(r0 + 0) * NCOLS + col] = acc[rt][ct].x;
      base[(r0 + 1) * NCOLS + col] = acc[rt][ct].y;
      base[(r0 + 2) * NCOLS + col] = acc[rt][ct].z;
      base[(r0 + 3) * NCOLS + col] = acc[rt][ct].w;
    }
}

// ---- batch tiles of 4 or 8 rows ----------------------------------------------------
// A 16x16x4 MFMA spends its full time on 16 rows however few are real.  Short tiles use
// the 16-block 4x4x1 MFMA instead, with the A operand of one block broadcast to a group
// of blocks (CBSZ/ABID): one instruction multiplies 4 batch rows by MC = 16, 32 or 64
// slice columns for KS = 4, 2 or 1 values of k (lane group l/MC takes the k-th value),
// so the matrix unit's time scales with the rows in steps of 4.

// Sums across lane groups.  swap_add16(a, b): lanes of the even 16-lane rows get a(row) +
// a(row+1), lanes of the odd rows b(row-1) + b(row), each from the lanes at the same position
// in the two rows.  swap_add32 is the same for the two halves of the wavefront.
__device__ __forceinline__ float swap_add16(float a, float b) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap_add32(float a, float b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int CT>
struct ShortTileShape {
  static constexpr int NCOLS = 16 * CT;
  static constexpr int CBSZ = NCOLS % 64 == 0 ? 4 : (NCOLS % 32 == 0 ? 3 : 2);
  static constexpr int NBC = 1 << CBSZ;   // 4-column blocks sharing one A block
  static constexpr int MC = 4 * NBC;      // slice columns per MFMA
  static constexpr int KS = 16 / NBC;     // k values per MFMA = lane groups with sums of their own
  static constexpr int CTN = NCOLS / MC;  // MFMAs side by side to cover the slice columns
};

// ---- the product of one step, for any tile height ------------------------------------
// NB batch rows (4, 8, or a multiple of 16) by 16*CT slice columns.  kPartials partial
// tiles of [NB][16*CT] floats are left in `red` by tile_product; sum_product adds them in a
// fixed order.
template <int NB, int CT>
struct ProductTile {
  static_assert(NB == 4 || NB == 8 || NB % 16 == 0, "unsupported tile height");
  static constexpr bool kShort = NB < 16;
  static constexpr int NCOLS = 16 * CT;
  static constexpr int kPartials = 4;  // one per wavefront
  static constexpr int kRedFloats = kPartials * NB * NCOLS;
};

// ---- exchange tiles ------------------------------------------------------------------
// What a step's product reads from the other workgroups (h[t], or the gate gradients of
// step t) is kept by its producers in a copy laid out for the consumers: per batch tile
// [Kpad/4][NB rows][4 consecutive k].  A wavefront's operand load is then one contiguous
// kilobyte (rows of the public [N, K] layout would make each 4-lane group touch 4 lines),
// needs no bounds checks (rows and k beyond the problem are kept at zero by whoever owns
// them) and producers write 16 bytes at a time.  Two tiles alternate by step parity: a
// workgroup may publish step t+1 while a slower one still reads step t.
__device__ __forceinline__ int xchg_index(int k, int row, int nb) {
  return ((k >> 2) * nb + row) * 4 + (k & 3);
}

// The two tiles of a group as a buffer resource: 16-byte loads that are served by the L2
// (agent scope, the reader's L1 is never consulted: it may hold the tile's previous
// contents) and return zero beyond the end.
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
struct TileBuffer {
  __amdgpu_buffer_rsrc_t rsrc;
};

__device__ __forceinline__ TileBuffer make_tile_buffer(float* tiles, int floats) {
  TileBuffer b;
  b.rsrc = __builtin_amdgcn_make_buffer_rsrc(tiles, 0, floats * 4, 0x00020000);
  return b;
}

// float_index: multiple of 4.
__device__ __forceinline__ float4_t load_tile4(const TileBuffer& b, int float_index) {
  constexpr int kAgentScope = 16;  // the sc1 bit of the cache policy
  const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(b.rsrc, float_index * 4, 0, kAgentScope);
  return float4_t{__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z),
                  __uint_as_float(v.w)};
}

// ---- polled exchange tiles -------------------------------------------------------------
// The step barrier costs a store acknowledgement (the producer may only raise its flag
// once its data has landed), a flag round trip and then the operand load itself.  Polled
// tiles drop the flags: an element that has not been published yet holds a bit pattern no
// producer ever stores (all ones, a NaN that publishable() maps to the canonical NaN), and
// the consumers' operand loads are themselves the wait: a wavefront re-issues the loads of
// a chunk until none of its elements is unwritten.  What a consumer has seen of step s
// therefore tells it that every producer of those elements had finished step s-1.
//
// kPolledTiles tiles rotate.  The tile read at step s is reset to "unwritten" by its
// owners during step s+1 (once their workgroup has seen all of step s+1's data, nobody can
// still be reading step s), and is written again at the earliest two steps later, behind an
// s_waitcnt vmcnt(0) that the reset has long satisfied: a consumer that has seen what an
// owner published at that point is guaranteed to see the reset as well, so a stale value
// of four steps ago can never pass for new data.
constexpr unsigned int kUnwrittenBits = 0xffffffffu;
constexpr int kPolledTiles = 4;

__device__ __forceinline__ float unwritten_value() { return __uint_as_float(kUnwrittenBits); }
__device__ __forceinline__ float publishable(float v) {
  return __float_as_uint(v) == kUnwrittenBits ? __uint_as_float(0x7fc00000u) : v;
}

// True (in every lane) when no lane of the wavefront holds an unwritten element.
template <int A, int B>
__device__ __forceinline__ bool all_written(const float4_t (&av)[A][B]) {
  unsigned int m = 0u;
#pragma unroll
  for (int a = 0; a < A; ++a)
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const unsigned int x = __float_as_uint(av[a][b].x), y = __float_as_uint(av[a][b].y);
      const unsigned int z = __float_as_uint(av[a][b].z), w = __float_as_uint(av[a][b].w);
      const unsigned int xy = x > y ? x : y, zw = z > w ? z : w;
      const unsigned int q = xy > zw ? xy : zw;
      m = m > q ? m : q;
    }
  return __all(m != kUnwrittenBits) != 0;
}

// Re-issues `load()` until `written()`; gives up (abort flag, host status) after the launch's
// spin limit or when another workgroup has given up, so that every wavefront still reaches
// the end of the kernel.
template <class LoadFn, class WrittenFn>
__device__ __forceinline__ void poll_until_written(const GroupSync& g, LoadFn&& load, WrittenFn&& written) {
  unsigned int spins = 0;
  while (!written()) {
    ++spins;
    if ((spins & 255u) == 0u) {
      const unsigned int ab = __hip_atomic_load(g.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (spins >= g.spin_limit && (threadIdx.x & 63) == 0) {
        __hip_atomic_store(g.abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(g.host_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      if (ab != 0u || spins >= g.spin_limit) break;
    }
    asm volatile("" ::: "memory");  // the loads must really be issued again
    load();
  }
}

// 16x16x4 path: A operands of k-groups [g_abs, g_abs+CHUNK) from an exchange tile of
// 16*RT rows.  Lane l holds row l%16 (of each 16-row block) and k = 16 g + 4 (l/16) .. +3.
template <int RT, int CHUNK>
__device__ __forceinline__ void load_tile_chunk(const TileBuffer& xb, int tile_off, int g_abs,
                                                int g_end, float4_t (&av)[CHUNK][RT]) {
  constexpr int NB = 16 * RT;
  const int lane = threadIdx.x & 63;
  // Every caller stays inside its wavefront's share (g_abs + CHUNK <= g_end), so the loads
  // carry no conditions: selects among the MFMAs would be time the matrix unit stands still.
  (void)g_end;
  const int base = tile_off + ((lane >> 4) * NB + (lane & 15)) * 4 + g_abs * 16 * NB;
#pragma unroll
  for (int gi = 0; gi < CHUNK; ++gi)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) av[gi][rt] = load_tile4(xb, base + (gi * 4 * NB + rt * 16) * 4);
}

struct NoResidentRows {};

// REG > 0: the first REG k-groups of every wavefront's share take their slice rows from
// `breg` (registers), the others from the compacted slice in LDS (resident_split_k).
template <int RT, int CT, int CHUNK, bool POLLED, int REG = 0, class Resident = NoResidentRows>
__device__ __forceinline__ void tall_tile_product(const TileBuffer& xb, int tile_off, int Kpad,
                                                  const float* w_lds, float* red,
                                                  const GroupSync* gs,
                                                  const Resident* breg = nullptr) {
  static_assert(REG % CHUNK == 0, "resident rows: whole chunks");
  const int wave = threadIdx.x >> 6;
  const int groups = Kpad >> 6;  // k-groups of 16 per wavefront
  const int lds_groups = groups - REG;
  const int full = lds_groups / CHUNK;
  int g = wave * groups;         // k-group of the operand tile
  int gl = wave * lds_groups;    // k-group of the slice in LDS
  const int g_end = g + groups;
  float4_t acc[RT][CT], acc1[RT][CT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = acc1[rt][ct] = float4_t{0.f, 0.f, 0.f, 0.f};

  if (REG > 0 || full > 0) {
    // Two operand buffers that swap roles chunk by chunk (no copies): while the MFMAs of
    // one run, the loads of the next chunk fill the other.  The poll comes before those
    // loads are issued: with them in flight the compiler could not tell whether the poll's
    // re-load had completed and would wait for the oldest of them before the MFMAs.
    float4_t buf0[CHUNK][RT], buf1[CHUNK][RT];
    load_tile_chunk<RT, CHUNK>(xb, tile_off, g, g_end, buf0);
    auto stage = [&](float4_t (&cur)[CHUNK][RT], float4_t (&nxt)[CHUNK][RT], bool more, auto&& mfmas) {
      if constexpr (POLLED)
        poll_until_written(*gs, [&] { load_tile_chunk<RT, CHUNK>(xb, tile_off, g, g_end, cur); },
                           [&] { return all_written(cur); });
      if (more) load_tile_chunk<RT, CHUNK>(xb, tile_off, g + CHUNK, g_end, nxt);
      mfmas(cur);
      g += CHUNK;
    };
    constexpr int RC = REG / CHUNK;  // chunks with register-resident slice rows
    if constexpr (REG > 0) {
      static_for<RC>([&](auto ic) {
        constexpr int CI = decltype(ic)::value;
        auto mfmas = [&](const float4_t (&cur)[CHUNK][RT]) {
          mfma_chunk_resident<RT, CT, CHUNK, REG, CI * CHUNK>(*breg, cur, acc, acc1);
        };
        if constexpr (CI % 2 == 0) stage(buf0, buf1, CI + 1 < RC || full > 0, mfmas);
        else stage(buf1, buf0, CI + 1 < RC || full > 0, mfmas);
      });
    }
    auto lds_mfmas = [&](const float4_t (&cur)[CHUNK][RT]) {
      mfma_chunk<RT, CT, CHUNK>(w_lds, gl, cur, acc, acc1);
      gl += CHUNK;
    };
    float4_t (&first)[CHUNK][RT] = RC % 2 == 0 ? buf0 : buf1;
    float4_t (&second)[CHUNK][RT] = RC % 2 == 0 ? buf1 : buf0;
    int c = 0;
    for (; c + 1 < full; c += 2) {
      stage(first, second, true, lds_mfmas);
      stage(second, first, c + 2 < full, lds_mfmas);
    }
    if (c < full) stage(first, second, false, lds_mfmas);
  }
  for (; g < g_end; ++g, ++gl) {
    float4_t one[1][RT];
    load_tile_chunk<RT, 1>(xb, tile_off, g, g_end, one);
    if constexpr (POLLED)
      poll_until_written(*gs, [&] { load_tile_chunk<RT, 1>(xb, tile_off, g, g_end, one); },
                         [&] { return all_written(one); });
    mfma_chunk<RT, CT, 1>(w_lds, gl, one, acc, acc1);
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[rt][ct] += acc1[rt][ct];
  store_partials<RT, CT>(red, acc);
}

// 4x4x1 path: A operands of CH super-groups s0, s0+4, ... (64 k each) from an exchange
// tile of 4*RB rows.  Lane l = 4*block + r holds row 4*rb + r; block g*NBC + a holds the
// four k of float4 index 16 s + a*KS + g, which makes the KS lane groups of one MFMA read
// adjacent float4 rows of the slice in LDS.
template <int RB, int CT, int CH>
__device__ __forceinline__ void load_tile_rows4(const TileBuffer& xb, int tile_off, int s0,
                                                float4_t (&av)[CH][RB]) {
  using S = ShortTileShape<CT>;
  constexpr int NB = 4 * RB;
  const int lane = threadIdx.x & 63;
  const int block = lane >> 2;
  const int k4 = (block % S::NBC) * S::KS + block / S::NBC;
  const int base = tile_off + (k4 * NB + (lane & 3)) * 4;
#pragma unroll
  for (int ci = 0; ci < CH; ++ci)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      av[ci][rb] = load_tile4(xb, base + ((s0 + 4 * ci) * 16 * NB + 4 * rb) * 4);
}

// MFMAs of the CH super-groups s, s+4, ... for the operand layout of load_tile_rows4.
// One 16-byte LDS read per (super-group, abid, column tile) feeds 4*RB MFMAs; the reads
// run kLdsAhead steps ahead of the MFMAs that use them, across super-group boundaries.
// Consecutive MFMAs on one output tile alternate between two accumulators.
constexpr int kLdsAhead = 3;

// HALF: on the half matrix cores -- the four k of an operand register are the four k of one
// v_mfma_f32_4x4x4_16B_f16 (both operands rounded to half: a cell whose tensors are half),
// one MFMA where the fp32 form issues four.
template <int RB, int CT, int CH, bool HALF = false>
__device__ __forceinline__ void mfma_tile_rows4(const float* w_lds, int s,
                                                const float4_t (&av)[CH][RB],
                                                float4_t (&acc0)[RB][ShortTileShape<CT>::CTN],
                                                float4_t (&acc1)[RB][ShortTileShape<CT>::CTN]) {
  using S = ShortTileShape<CT>;
  constexpr int STEPS = CH * S::NBC;
  const int lane = threadIdx.x & 63;
  const float* wp = w_lds + ((16 * s + lane / S::MC) * S::NCOLS + lane % S::MC) * 4;
  // step i = (super-group i / NBC, abid i % NBC): float offset of its slice rows from wp
  auto step_offset = [](int i) {
    return ((i / S::NBC) * 64 + (i % S::NBC) * S::KS) * S::NCOLS * 4;
  };
  float4_t b[STEPS][S::CTN];
  static_for<(kLdsAhead < STEPS ? kLdsAhead : STEPS)>([&](auto ic) {
    constexpr int I = decltype(ic)::value;
#pragma unroll
    for (int ct = 0; ct < S::CTN; ++ct)
      b[I][ct] = *reinterpret_cast<const float4_t*>(wp + step_offset(I) + ct * S::MC * 4);
  });
  half4_t ah[HALF ? CH : 1][RB];
  if constexpr (HALF) {
#pragma unroll
    for (int ci = 0; ci < CH; ++ci)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int e = 0; e < 4; ++e) ah[ci][rb][e] = (_Float16)av[ci][rb][e];
  }
  static_for<STEPS>([&](auto ic) {
    constexpr int I = decltype(ic)::value;
    constexpr int A = I % S::NBC;
    constexpr int CI = I / S::NBC;
    if constexpr (I + kLdsAhead < STEPS) {
#pragma unroll
      for (int ct = 0; ct < S::CTN; ++ct)
        b[I + kLdsAhead][ct] = *reinterpret_cast<const float4_t*>(
            wp + step_offset(I + kLdsAhead) + ct * S::MC * 4);
      // keep the read here: the scheduler would otherwise sink it to just before its use
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (HALF) {
#pragma unroll
      for (int ct = 0; ct < S::CTN; ++ct) {
        half4_t bh;
#pragma unroll
        for (int e = 0; e < 4; ++e) bh[e] = (_Float16)b[I][ct][e];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          if constexpr (I % 2 == 0)
            acc0[rb][ct] = __builtin_amdgcn_mfma_f32_4x4x4f16(ah[CI][rb], bh, acc0[rb][ct], S::CBSZ, A, 0);
          else
            acc1[rb][ct] = __builtin_amdgcn_mfma_f32_4x4x4f16(ah[CI][rb], bh, acc1[rb][ct], S::CBSZ, A, 0);
        }
      }
      return;
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ct = 0; ct < S::CTN; ++ct)
        acc0[rb][ct] = __builtin_amdgcn_mfma_f32_4x4x1f32(av[CI][rb].x, b[I][ct].x, acc0[rb][ct], S::CBSZ, A, 0);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ct = 0; ct < S::CTN; ++ct)
        acc1[rb][ct] = __builtin_amdgcn_mfma_f32_4x4x1f32(av[CI][rb].y, b[I][ct].y, acc1[rb][ct], S::CBSZ, A, 0);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ct = 0; ct < S::CTN; ++ct)
        acc0[rb][ct] = __builtin_amdgcn_mfma_f32_4x4x1f32(av[CI][rb].z, b[I][ct].z, acc0[rb][ct], S::CBSZ, A, 0);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int ct = 0; ct < S::CTN; ++ct)
        acc1[rb][ct] = __builtin_amdgcn_mfma_f32_4x4x1f32(av[CI][rb].w, b[I][ct].w, acc1[rb][ct], S::CBSZ, A, 0);
  });
}

// ---- work beside the wait ------------------------------------------------------------
// A step of a recurrence is a chain (wait for the exchanged operand, product, pointwise math,
// publish) during most of which the matrix unit of the wavefront's SIMD is idle.  A product
// that does not depend on the recurrence can be issued while the wavefront waits: the input
// projection x[t] * W of a forward pass.  Its B operand comes from registers (no LDS reads
// compete with the resident slice), its MFMAs accumulate into the accumulators the recurrent
// product continues with -- always all of the projection first, then the recurrent product,
// so the sums do not depend on timing -- and between batches of them the wavefront looks at
// the operand loads it is polling.
struct NoSideWork {
  static constexpr int kBatches = 0;
  static constexpr bool kExtraTile = false;
};

// x[t][4 rows of a batch tile][C] * W[C][16*CT slice columns] on the 4x4x1 path, the
// contraction split over the four wavefronts of a set like the recurrent product's: this
// wavefront takes the XSG super-groups (64 k each) wave, wave + 4, ...  A lane keeps the weights
// its MFMAs need in registers for the whole launch: 4 * CT * XSG floats, i.e. 128 for a
// 64-column slice and C = 512 (two wavefronts per SIMD leave 256 registers per lane).
// SPLIT (a GRU: the candidate gate needs x*W and h*R apart): the projection's last column tile
// accumulates into a tile of its own instead of the recurrent product's, which the product
// leaves behind the slice's tiles in the partial tile (column tile CTN).
template <int CT, int XSG, bool SPLIT = false>
struct InputProjection {
  using S = ShortTileShape<CT>;
  static constexpr bool kExtraTile = SPLIT;
  float4_t extra0, extra1;   // SPLIT: the sums of the last column tile
  static constexpr int kSteps = XSG * S::NBC;   // one step: 4 * CTN MFMAs on one A block
  static constexpr int kStepsPerBatch = 4;
  static constexpr int kBatches = (kSteps + kStepsPerBatch - 1) / kStepsPerBatch;
  float w[XSG][S::NBC][S::CTN][4];
  float4_t xa[XSG];          // this step's A operands
  const float* xp[XSG];      // where the lane's operands of the next step to load are
  bool valid[XSG];           // the lane's k exist (k < C)
  size_t step_stride;        // floats between consecutive steps of x

  // `wave`: wavefront inside the set.  Column `col` of the slice is column gcol(col) of W
  // (row length `row_len`), or does not exist (gcol < 0).  Lane l = 4*block + r multiplies
  // row n0 + r (rows beyond N read row N-1: their results are never used).
  template <class ColFn>
  __device__ __forceinline__ void setup(const float* __restrict__ W, const float* __restrict__ x,
                                        int C, int N, int row_len, int wave, int n0, ColFn gcol) {
    const int lane = threadIdx.x & 63;
    const int g = lane / S::MC;
    step_stride = (size_t)N * C;
    int row = n0 + (lane & 3);
    row = row < N ? row : N - 1;
    const int block = lane >> 2;
    const int k4 = (block % S::NBC) * S::KS + block / S::NBC;
#pragma unroll
    for (int xs = 0; xs < XSG; ++xs) {
      const int kx = 64 * (wave + 4 * xs) + 4 * k4;
      valid[xs] = kx < C;
      xp[xs] = x + (size_t)row * C + (valid[xs] ? kx : 0);
#pragma unroll
      for (int a = 0; a < S::NBC; ++a)
#pragma unroll
        for (int ct = 0; ct < S::CTN; ++ct) {
          const long long col = gcol(ct * S::MC + lane % S::MC);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            // every lane loads (some valid element where its own does not exist), so that the
            // loads carry no branches and are all in flight at once
            const int k = 64 * (wave + 4 * xs) + 4 * (a * S::KS + g) + c;
            const bool exists = k < C && col >= 0;
            const float loaded = W[exists ? (size_t)k * row_len + col : 0];
            w[xs][a][ct][c] = exists ? loaded : 0.f;
          }
        }
    }
  }

  // Requests the operands of the next step (C is a multiple of 4 and x 16-byte aligned).
  __device__ __forceinline__ void request() {
#pragma unroll
    for (int xs = 0; xs < XSG; ++xs) {
      xa[xs] = *reinterpret_cast<const float4_t*>(xp[xs]);
      xp[xs] += step_stride;
    }
  }

  // Waits until everything this wavefront has requested or stored has completed -- the
  // operands of the next step among it -- and finishes those (lanes whose k do not exist
  // contribute zeros: their loads read some valid element).  The operands pass through the
  // wait as its outputs, and through an empty statement afterwards: left to itself the compiler
  // touches them, and so waits for them, at the top of the next step, where its wait also covers
  // whatever was stored since -- the publication, the caller's copies -- with the matrix
  // units idle (0.6 us per step).
  __device__ __forceinline__ void settle() {
#pragma unroll
    for (int xs = 0; xs < XSG; ++xs) asm volatile("s_waitcnt vmcnt(0)" : "+v"(xa[xs]) : : "memory");
#pragma unroll
    for (int xs = 0; xs < XSG; ++xs) {
      if (!valid[xs]) xa[xs] = float4_t{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+v"(xa[xs]));
    }
  }

  __device__ __forceinline__ void begin() { extra0 = extra1 = float4_t{0.f, 0.f, 0.f, 0.f}; }

  template <int B>
  __device__ __forceinline__ void batch(float4_t (&acc0)[1][S::CTN], float4_t (&acc1)[1][S::CTN]) {
    static_for<kStepsPerBatch>([&](auto ic) {
      constexpr int I = B * kStepsPerBatch + decltype(ic)::value;
      if constexpr (I < kSteps) {
        constexpr int XS = I / S::NBC;
        constexpr int A = I % S::NBC;
        // component c of the operand goes to accumulator c % 2; the last tile to the extra one
        static_for<4>([&](auto cc) {
          constexpr int C4 = decltype(cc)::value;
          const float xc = xa[XS][C4];
#pragma unroll
          for (int ct = 0; ct < S::CTN; ++ct) {
            float4_t& acc = (SPLIT && ct == S::CTN - 1) ? (C4 % 2 == 0 ? extra0 : extra1)
                                                        : (C4 % 2 == 0 ? acc0[0][ct] : acc1[0][ct]);
            acc = __builtin_amdgcn_mfma_f32_4x4x1f32(xc, w[XS][A][ct][C4], acc, S::CBSZ, A, 0);
          }
        });
      }
    });
  }
};

// One 4-row accumulator tile to its place in a partial tile: the KS lane groups hold sums over
// different k of the same elements; they are added here, and every lane stores 4/KS of the 4
// rows.  q: the tile's first row at this lane's column; `pitch`: floats per row.
template <int KS, bool TAGGED>
__device__ __forceinline__ void store_tile_sum(float* q, int pitch, float4_t v, int lane) {
  if constexpr (KS == 4) {
    // lane group 0, 1, 2, 3 ends up with row 0, 2, 1, 3
    const float xz = swap_add16(v.x, v.z), yw = swap_add16(v.y, v.w);
    float r = swap_add32(xz, yw);
    if constexpr (TAGGED) r = publishable(r);
    const int g = lane >> 4;
    q[(((g & 1) << 1) | (g >> 1)) * pitch] = r;
  } else if constexpr (KS == 2) {
    // lane group 0: rows 0 and 2; lane group 1: rows 1 and 3
    float r0 = swap_add32(v.x, v.y), r1 = swap_add32(v.z, v.w);
    if constexpr (TAGGED) { r0 = publishable(r0); r1 = publishable(r1); }
    const int g = lane >> 5;
    q[g * pitch] = r0;
    q[(g + 2) * pitch] = r1;
  } else {
    if constexpr (TAGGED) v = float4_t{publishable(v.x), publishable(v.y), publishable(v.z), publishable(v.w)};
    q[0] = v.x;
    q[pitch] = v.y;
    q[2 * pitch] = v.z;
    q[3 * pitch] = v.w;
  }
}

// Product of a short exchange tile: red[wave][4*RB][16*CT] <- this wavefront's partial tile
// (accumulator element r of acc[rb][ct] in lane l is row 4*rb + r, column ct*MC + l%MC, of
// the k that lane group l/MC took).  The operand
// loads of chunk c+1 (CH super-groups) are issued before the MFMAs of chunk c; the two
// register buffers alternate so that nothing is copied.  The four wavefronts are those of one
// 256-thread set of the workgroup.  TAGGED: the partial tiles are themselves polled by their
// readers (take_product), so no element may carry the "unwritten" pattern.
// RED_CT: column tiles of a partial tile's rows (more than CT when the side work leaves a tile of
// its own behind the slice's).
template <int RB, int CT, int CH, bool POLLED, bool TAGGED = false, class Side = NoSideWork, bool HALF = false,
          int RED_CT = CT>
__device__ __forceinline__ void short_exchange_product(const TileBuffer& xb, int tile_off, int Kpad,
                                                       const float* w_lds, float* red,
                                                       const GroupSync* gs, Side* side = nullptr) {
  using S = ShortTileShape<CT>;
  constexpr int NB = 4 * RB;
  const int lane = threadIdx.x & 63;
  const int wave = set_wave<TAGGED ? 2 : 1>();  // polled partial tiles: two sets
  const int s_end = Kpad >> 6;
  const int mine = (s_end - wave + 3) >> 2;  // super-groups wave, wave+4, ...
  // A wavefront without a share of k waits for nobody, so nothing would keep it from running
  // steps ahead of the readers of its partial tile: it leaves no partial tile at all.
  if (TAGGED && mine == 0) return;
  const int chunks = mine / CH;
  float4_t acc0[RB][S::CTN], acc1[RB][S::CTN];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ct = 0; ct < S::CTN; ++ct) acc0[rb][ct] = acc1[rb][ct] = float4_t{0.f, 0.f, 0.f, 0.f};

  int s = wave;
  if constexpr (Side::kExtraTile) side->begin();
  if constexpr (Side::kBatches > 0) {
    static_assert(RB == 1 && POLLED, "side work: polled 4-row tiles");
    // no operand chunk to look at between the batches: the side work runs on its own
    if (chunks == 0)
      static_for<Side::kBatches>([&](auto b) { side->template batch<decltype(b)::value>(acc0, acc1); });
  }
  if (chunks > 0) {
    float4_t buf0[CH][RB], buf1[CH][RB];
    load_tile_rows4<RB, CT, CH>(xb, tile_off, s, buf0);
    if constexpr (Side::kBatches > 0) {
      // The side work, in batches; after every second one a look at the first chunk's loads
      // (re-issued while some element is still unwritten).  How often makes no difference
      // (looks after every batch, every fourth, none: 3.26-3.33 us per step at N = 64,
      // C = H = 512): with the projection the step is bound by the rate of the 4x4x1 MFMAs.
      bool seen = false;
      static_for<Side::kBatches>([&](auto b) {
        side->template batch<decltype(b)::value>(acc0, acc1);
        if (decltype(b)::value % 2 == 1 && !seen) {
          seen = all_written(buf0);
          if (!seen) {
            asm volatile("" ::: "memory");
            load_tile_rows4<RB, CT, CH>(xb, tile_off, s, buf0);
          }
        }
      });
    }
    int c = 0;
    for (;;) {
      if (c + 1 < chunks) load_tile_rows4<RB, CT, CH>(xb, tile_off, s + 4 * CH, buf1);
      if constexpr (POLLED)
        poll_until_written(*gs, [&] { load_tile_rows4<RB, CT, CH>(xb, tile_off, s, buf0); },
                           [&] { return all_written(buf0); });
      mfma_tile_rows4<RB, CT, CH, HALF>(w_lds, s, buf0, acc0, acc1);
      s += 4 * CH;
      if (++c == chunks) break;
      if (c + 1 < chunks) load_tile_rows4<RB, CT, CH>(xb, tile_off, s + 4 * CH, buf0);
      if constexpr (POLLED)
        poll_until_written(*gs, [&] { load_tile_rows4<RB, CT, CH>(xb, tile_off, s, buf1); },
                           [&] { return all_written(buf1); });
      mfma_tile_rows4<RB, CT, CH, HALF>(w_lds, s, buf1, acc0, acc1);
      s += 4 * CH;
      if (++c == chunks) break;
    }
  }
  for (; s < s_end; s += 4) {
    float4_t one[1][RB];
    load_tile_rows4<RB, CT, 1>(xb, tile_off, s, one);
    if constexpr (POLLED)
      poll_until_written(*gs, [&] { load_tile_rows4<RB, CT, 1>(xb, tile_off, s, one); },
                         [&] { return all_written(one); });
    mfma_tile_rows4<RB, CT, 1, HALF>(w_lds, s, one, acc0, acc1);
  }

  // The KS lane groups hold partial sums of the same elements: they are added here, so that a
  // wavefront leaves one partial tile, and every lane stores 4/KS of the 4 rows.
  constexpr int PITCH = 16 * RED_CT;
  float* base = red + (wave * NB) * PITCH + lane % S::MC;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ct = 0; ct < S::CTN; ++ct)
      store_tile_sum<S::KS, TAGGED>(base + (4 * rb) * PITCH + ct * S::MC, PITCH, acc0[rb][ct] + acc1[rb][ct], lane);
  if constexpr (Side::kExtraTile) {
    static_assert(RED_CT * 16 >= (S::CTN + 1) * S::MC, "no room for the side work's tile");
    store_tile_sum<S::KS, TAGGED>(base + S::CTN * S::MC, PITCH, side->extra0 + side->extra1, lane);
  }
}

// red <- partial tiles of tile[NB rows, Kpad] * slice[Kpad, 16*CT]; the exchange tile
// starts at float `tile_off` of `xb`.  LONG_K selects deeper prefetch for contractions much
// longer than the hidden size (the backward passes).
// POLLED: the tile is a polled exchange tile (see above) and `gs` supplies the bounds of the
// wait; otherwise the caller has waited at the group's step barrier and `gs` is unused.
// REG > 0 (tall tiles): the slice is split between registers and LDS, see tall_tile_product.
template <int NB, int CT, bool LONG_K, bool POLLED = false, bool TAGGED = false, class Side = NoSideWork,
          int REG = 0, class Resident = NoResidentRows, bool HALF = false, int RED_CT = CT>
__device__ __forceinline__ void tile_product(const TileBuffer& xb, int tile_off, int Kpad,
                                             const float* w_lds, float* red,
                                             const GroupSync* gs = nullptr, Side* side = nullptr,
                                             const Resident* breg = nullptr) {
  if constexpr (ProductTile<NB, CT>::kShort) {
    static_assert(REG == 0, "register-resident slice rows exist for tall tiles only");
    short_exchange_product<NB / 4, CT, LONG_K ? 4 : 2, POLLED, TAGGED, Side, HALF, RED_CT>(xb, tile_off, Kpad,
                                                                                            w_lds, red, gs, side);
  } else {
    static_assert(!HALF, "the product on the half matrix cores exists for short tiles only");
    static_assert(!TAGGED, "polled partial tiles exist for short tiles only");
    static_assert(Side::kBatches == 0, "side work exists for short tiles only");
    constexpr int RT = NB / 16;
    // k-groups of operands per load (two loads in flight).  Measured at H = 512: a forward share
    // (8 groups per wavefront) in one piece, a backward share (32 groups) in two, are 9-10 %
    // faster per step than pieces of 4 / 8 at 16 rows, pieces of 8 than 4 at 32 rows; twice
    // that is slower again.
    constexpr int CHUNK0 = LONG_K ? (RT == 1 ? 16 : (RT == 2 ? 8 : 2)) : (RT >= 4 ? 2 : 8);
    constexpr int CHUNK = (REG % CHUNK0 != 0) ? 8 : CHUNK0;  // REG: a multiple of 8
    tall_tile_product<RT, CT, CHUNK, POLLED, REG, Resident>(xb, tile_off, Kpad, w_lds, red, gs, breg);
  }
}

// Zeroes this workgroup's share of its group's exchange tiles: float4 rows
// [first4, first4 + count4) of [Kpad/4][NB][4], in each of the n_tiles tiles.  The stores have completed
// when it returns.  Called by all threads of the workgroup.
template <int SETS = 1>
__device__ __forceinline__ void zero_tile_share(const GroupSync& g, float* tiles, int tile_floats,
                                                int nb, int first4, int count4, int n_tiles = 2) {
  // the threads of one set share the work (two sets: each has tiles of its own)
  for (int i = set_thread<SETS>(); i < count4 * nb; i += 256) {
    float* q = tiles + ((size_t)first4 * nb + i) * 4;
    for (int b = 0; b < n_tiles; ++b) store_exchanged4(g, q + (size_t)b * tile_floats, 0.f, 0.f, 0.f, 0.f);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
}

// Element (row, col) of the product: the partial tiles written by tile_product, added
// pairwise in a fixed order.
template <int NB, int CT>
__device__ __forceinline__ float sum_product(const float* red, int row, int col) {
  using P = ProductTile<NB, CT>;
  constexpr int STRIDE = NB * P::NCOLS;
  const float* p = red + row * P::NCOLS + col;
  float v[P::kPartials];
#pragma unroll
  for (int i = 0; i < P::kPartials; ++i) v[i] = p[i * STRIDE];
#pragma unroll
  for (int w = P::kPartials / 2; w > 0; w >>= 1)
#pragma unroll
    for (int i = 0; i < w; ++i) v[i] = v[2 * i] + v[2 * i + 1];
  return v[0];
}

// ---- polled partial tiles -------------------------------------------------------------
// A workgroup may hold two independent batch tiles: two 256-thread sets that share the
// resident slice and are at different points of their steps, so that one set's product
// runs while the other waits for its exchange.  Such a set cannot use the workgroup barrier
// between its product and the threads that consume it.  Its partial tiles are polled
// instead, like the exchange tiles: every element starts out unwritten, the product stores
// publishable values (TAGGED), and the one thread that consumes an element re-reads it
// until it is written and resets it afterwards.  Two such areas alternate by step: a
// wavefront can only get to the product of step s+2 once every workgroup has finished step
// s+1, for which the consumers of this set had to publish the results of step s -- after
// their resets (LDS operations of a wavefront complete in order, and the reset is waited
// for here).
//
// Partial tiles that a TAGGED product of contraction length Kpad writes: those of the
// wavefronts that have a share of k.
template <int CT>
__device__ __forceinline__ int live_partials(int Kpad) {
  return (Kpad >> 6) < 4 ? (Kpad >> 6) : 4;
}

// out[g] = element (row, col0 + g * col_stride) of the product, partials added in
// sum_product's order.  Called by whole wavefronts; lanes with !mine take no part.  Only the
// first `live` partial tiles are ever written (live_partials()): the others hold zeros.
template <int NB, int CT, int G>
__device__ __forceinline__ void take_product(const GroupSync& gs, float* red, int row, int col0,
                                             int col_stride, bool mine, int live, float (&out)[G]) {
  using P = ProductTile<NB, CT>;
  constexpr int STRIDE = NB * P::NCOLS;
  float* p = red + row * P::NCOLS + col0;
  // Every lane reads (lanes that take no part: some valid address) and the reads carry no
  // conditions, so that all of them are in flight at once.
  const float* q = mine ? p : red;
  float v[G][P::kPartials];
  auto load = [&] {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < P::kPartials; ++i) v[g][i] = q[g * col_stride + i * STRIDE];
  };
  auto written = [&] {
    unsigned int m = 0u;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < P::kPartials; ++i) {
        const unsigned int x = __float_as_uint(v[g][i]);
        m = m > x ? m : x;
      }
    return __all(!mine || m != kUnwrittenBits) != 0;
  };
  load();
  poll_until_written(gs, [&] { __builtin_amdgcn_s_sleep(1); load(); }, written);
  if (mine) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < P::kPartials; ++i)
        p[g * col_stride + i * STRIDE] = i < live ? unwritten_value() : 0.f;
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int w = P::kPartials / 2; w > 0; w >>= 1)
#pragma unroll
      for (int i = 0; i < w; ++i) v[g][i] = v[g][2 * i] + v[g][2 * i + 1];
    out[g] = v[g][0];
  }
}

// Sets up the two polled areas of partial tiles of one set: the tiles that products write
// start out unwritten, the others hold zeros for good.  A workgroup barrier must follow
// before the first product.
template <int NB, int CT>
__device__ __forceinline__ void reset_partials(float* red, int live) {
  using P = ProductTile<NB, CT>;
  constexpr int TILE = NB * P::NCOLS;
  for (int i = set_thread<2>(); i < 2 * P::kRedFloats; i += 256)
    red[i] = (i % P::kRedFloats) / TILE < live ? unwritten_value() : 0.f;
}

// ---- scattered partial sums (backward recurrences, 4-row tiles) --------------------------
// The backward step dh = dv * R_t contracts over the gate gradients of ALL hidden units.  A
// workgroup that owns output units must therefore gather the whole of dv (4 gates wide) from
// every other workgroup before its matrix units can start.  The scattered form turns the
// ownership round: a workgroup contracts over the gate gradients it has just computed itself
// -- the G gates of its 16 units, a single MFMA operand register per lane -- against the rows
// of R_t that belong to those units and ALL H columns, and hands every owner its 4 x 16 piece
// of the partial sums; the owner adds the pieces of all producers in index order.  What
// crosses between workgroups is H wide instead of G*H wide, the products wait for nothing
// remote, and a wavefront's share of R_t (its 64*CTN output columns, the workgroup's 16*G
// rows) lives in registers for the whole launch, so the step has no LDS traffic to speak of.
//
// Pieces: per 4-row batch tile two tiles (alternating by step) of [owner][producer][unit][row]
// floats (a piece is 64 floats).  Producers are padded to kProducers per owner; the padding
// holds zeros for good and its tags are not looked at.  A piece is polled like the exchange tiles above
// -- the owner's loads are themselves the wait -- but what marks an element as written is a
// TAG in its lowest mantissa bit: the use count of its slot, modulo 2.  A piece written at
// step d (tile d%2, tag (d/2)%2) is read at step d+1 and written again at step d+2, with the
// other tag, so what the slot held before can never pass for new data and nothing has to be
// reset in between (resetting the pieces cost as much L2 write bandwidth as publishing them:
// 512 KiB per XCD and step each at H = 512, 800 cycles of a 6 400-cycle step).  At step d+2 the
// producer's workgroup has seen the sums of step d+1, which every producer publishes only after
// its workgroup has finished reading step d, so the slot is free.  The price is the last bit
// of each partial sum (a relative 6e-8, below the rounding of the sum of 32 of them); an
// infinite partial sum tagged 1 reads as NaN, a NaN stays NaN.
//
// Agent-scope loads are not combined across lanes: every lane's access is a request of its
// own to the L2 (a gather of 32 pieces with one float per lane and load took 3 500 cycles,
// 1.7 per request).  So the pieces are read 16 bytes per lane -- lane 16*g + u the four rows of
// unit u from the producers 4*i + g -- and by three wavefronts of the set at once (the owner
// and the two that have no other duties between their publication and the owner's operand),
// each adding up its share of the producers; the owner adds the three sums, and its four lane
// groups then add theirs to each other so that each ends up with one row: the pointwise work
// of the owner runs on lane 16*g + u = (row scatter_row(g), unit u), and the gate gradients
// go to the lanes of the MFMA operand (lane 4*unit + row) from there.
template <int CTN>
struct ScatterShape {
  static constexpr int kColumns = 64 * CTN;     // output columns of one wavefront
  static constexpr int kProducers = 16 * CTN;   // producers per owner, padded (H <= 256 * CTN)
  static constexpr int kPieceFloats = 64;
  static constexpr int kLoads = kProducers / 4;              // 16-byte loads per lane, all producers
  static constexpr int kOwnerLoads = 2;                      // ... of which the owner issues these
  static constexpr int kOtherLoads = (kLoads - kOwnerLoads) / 2;  // ... and two others these each
};

constexpr int kScatterTiles = 2;
inline size_t scatter_tile_floats(int gx, int ctn) { return (size_t)gx * 16 * ctn * 64; }
// LDS of a set: the owner wavefront's operand for the three other wavefronts, by step parity;
// the sums of the two other gathering wavefronts, by step parity; up to 12 parked inputs per
// lane of the owner, by step parity; which step each parking area holds.
constexpr size_t kScatterHandFloats = 2 * 3 * 64 * 4;
constexpr size_t kScatterPartFloats = 2 * 2 * 64 * 4;
constexpr size_t kScatterParkFloats = 2 * 12 * 64;
constexpr size_t kScatterSetFloats = kScatterHandFloats + kScatterPartFloats + kScatterParkFloats + 4;

// The batch row (of the tile's four) that lane group g of the owner ends up with.
__device__ __forceinline__ int scatter_row(int g) { return ((g & 1) << 1) | (g >> 1); }

// The tag of the pieces published at step d, and a value carrying a tag.
__device__ __forceinline__ unsigned int scatter_tag(int d) { return ((unsigned int)d >> 1) & 1u; }
// (A NaN stays one: what arithmetic produces is a quiet NaN, whose top mantissa bit is set.)
__device__ __forceinline__ float tagged(float v, unsigned int tag) {
  return __uint_as_float((__float_as_uint(v) & ~1u) | tag);
}
__device__ __forceinline__ float4_t tagged4(const float4_t& v, unsigned int tag) {
  return float4_t{tagged(v.x, tag), tagged(v.y, tag), tagged(v.z, tag), tagged(v.w, tag)};
}

// A wavefront's share of an owner's gather: NLW consecutive groups of four producers, starting
// with group `first`, of the pieces that start at float `owner_off` of `xb`.  Lane 16*g + u
// ends up with the four rows of unit u summed over producers 4*i + g of its groups, added in
// index order, once all of them carry the tag `tag`.  request() issues the loads; finish()
// waits, polls and adds, so that work that does not depend on the sums can stand in between.
// `gx`: producers that exist.
template <int NLW>
struct PieceGather {
  float4_t v[NLW];
  int base;
  bool real[NLW];

  __device__ __forceinline__ void load(const TileBuffer& xb) {
#pragma unroll
    for (int i = 0; i < NLW; ++i) v[i] = load_tile4(xb, base + i * 256);
  }
  __device__ __forceinline__ void request(const TileBuffer& xb, int owner_off, int first, int gx) {
    const int lane = threadIdx.x & 63;
    base = owner_off + (4 * first + (lane >> 4)) * 64 + (lane & 15) * 4;
#pragma unroll
    for (int i = 0; i < NLW; ++i) real[i] = 4 * (first + i) + (lane >> 4) < gx;
    load(xb);
  }
  __device__ __forceinline__ float4_t finish(const GroupSync& gs, const TileBuffer& xb, unsigned int tag) {
    auto written = [&] {
      unsigned int m = 0u;
#pragma unroll
      for (int i = 0; i < NLW; ++i) {
        const unsigned int q = (__float_as_uint(v[i].x) ^ tag) | (__float_as_uint(v[i].y) ^ tag) |
                               (__float_as_uint(v[i].z) ^ tag) | (__float_as_uint(v[i].w) ^ tag);
        m |= real[i] ? q : 0u;
      }
      return __all((m & 1u) == 0u) != 0;
    };
    poll_until_written(gs, [&] { load(xb); }, written);
    float4_t s = v[0];
#pragma unroll
    for (int i = 1; i < NLW; ++i) s += v[i];
    return s;
  }
};

// The owner's last step: its four lane groups hold sums over different producers of the same
// elements; lane groups 0, 1, 2, 3 end up with the totals of rows 0, 2, 1, 3 (scatter_row).
__device__ __forceinline__ float scatter_lane_groups(const float4_t& s) {
  return swap_add32(swap_add16(s.x, s.z), swap_add16(s.y, s.w));
}

// Reads 16-byte words of LDS that other wavefronts publish (every element written with a
// publishable value) until they are written, and resets them to "unwritten" for their next
// use.  The reset is not waited for: the LDS operations of a wavefront complete in order, so it
// has landed before anything this wavefront reads from LDS afterwards, and whoever writes the
// word again has first seen something this wavefront published after such a read.
__device__ __forceinline__ float4_t take_lds4(const GroupSync& gs, float4_t* q) {
  float4_t got[1][1];
  got[0][0] = *q;
  poll_until_written(gs, [&] { __builtin_amdgcn_s_sleep(1); got[0][0] = *q; }, [&] { return all_written(got); });
  const float u = unwritten_value();
  *q = float4_t{u, u, u, u};
  return got[0][0];
}
__device__ __forceinline__ void take_lds4_pair(const GroupSync& gs, float4_t* q0, float4_t* q1, float4_t& v0,
                                               float4_t& v1) {
  float4_t got[2][1];
  got[0][0] = *q0;
  got[1][0] = *q1;
  poll_until_written(gs, [&] { __builtin_amdgcn_s_sleep(1); got[0][0] = *q0; got[1][0] = *q1; },
                     [&] { return all_written(got); });
  const float u = unwritten_value();
  *q0 = float4_t{u, u, u, u};
  *q1 = float4_t{u, u, u, u};
  v0 = got[0][0];
  v1 = got[1][0];
}

__device__ __forceinline__ float4_t publishable4(const float4_t& v) {
  return float4_t{publishable(v.x), publishable(v.y), publishable(v.z), publishable(v.w)};
}

// acc[c%2][ct] += a[c] (the operand of row l%4, k = 4*(l/4) + c, broadcast block by block)
// times the lane's weights w[block][c][ct], for the G components in use: 16 * G * CTN MFMAs,
// consecutive ones on different accumulators.
template <int G, int CTN>
__device__ __forceinline__ void scatter_product(const float4_t& a, const float (&w)[16][G][CTN],
                                                float4_t (&acc)[2][CTN]) {
  static_for<16>([&](auto bc) {
    constexpr int A = decltype(bc)::value;
#pragma unroll
    for (int c = 0; c < G; ++c)
#pragma unroll
      for (int ct = 0; ct < CTN; ++ct)
        acc[c & 1][ct] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[c], w[A][c][ct], acc[c & 1][ct], 4, A, 0);
  });
}

// The same product on the half matrix cores (a cell whose tensors are half: the gate gradients
// are rounded to half, as such a cell stores them, and the weights are exact in half): the G
// gate gradients of an element are the four k of one v_mfma_f32_4x4x4_16B_f16, so a unit takes
// one MFMA per column tile instead of G -- 16 * CTN in all.  w[block][ct]: the lane's weights of
// the block's unit for gates 0 .. 3 (zero beyond G).

template <int G, int CTN>
__device__ __forceinline__ void scatter_product_half(const float4_t& a, const half4_t (&w)[16][CTN],
                                                     float4_t (&acc)[2][CTN]) {
  half4_t ah;
#pragma unroll
  for (int c = 0; c < 4; ++c) ah[c] = c < G ? (_Float16)a[c] : (_Float16)0.f;
  static_for<16>([&](auto bc) {
    constexpr int A = decltype(bc)::value;
#pragma unroll
    for (int ct = 0; ct < CTN; ++ct)
      acc[A & 1][ct] = __builtin_amdgcn_mfma_f32_4x4x4f16(ah, w[A][ct], acc[A & 1][ct], 4, A, 0);
  });
}

// ---- one batch row -----------------------------------------------------------------------
// With a single batch row the step's product is a matrix-vector product.  The 4-row MFMA tile
// spends three quarters of the matrix unit's time on padding and, like any tile, reads the
// whole slice from LDS every step (128 KiB at H = 512: 0.45 us at the LDS's rate).  The
// single-row kernels keep the slice in REGISTERS instead: 256 threads, a thread owns one of 64
// slice columns (16 hidden units x up to 4 gates: column c is gate c/16, unit c%16) and a
// quarter of k (wavefront w: k in [w*KW, (w+1)*KW), KW = Kpad/4 <= KW_MAX), i.e. up to 128
// weights, and a step is up to 128 FMAs per thread against h, which the wavefront polls from
// the exchange tile ([4 polled tiles][Kpad] for the one row), parks in LDS and reads back as
// broadcast 16-byte reads.
constexpr int kSingleRowUnits = 16;
constexpr int kSingleRowCols = 64;
// The forward kernels add a fifth wavefront that parks the next steps' inputs in LDS:
// [2][5][16] floats behind the role word.
constexpr int kSingleRowThreads = 320;
constexpr size_t kSingleRowParkBytes = (size_t)(2 * 5 * kSingleRowUnits + 3) * sizeof(float);

// Dynamic LDS of a single-row kernel: [4][KW_MAX] a wavefront's share of h, [2][4][64]
// partial sums by step parity and wavefront, one word for the role (no static LDS:
// launch_persistent sizes the dynamic limit for kernels without any).
inline size_t single_row_lds_bytes(int kw_max) {
  return ((size_t)4 * kw_max + 2 * 4 * kSingleRowCols + 4) * sizeof(float);
}
inline int single_row_kw_max(int Kpad) { return Kpad <= 128 ? 32 : (Kpad <= 256 ? 64 : 128); }

// The thread's weights: column `lane` of the slice, k = wave*KW + i.  `col` is the column's
// offset inside a row of `src` (row length `row_len`), valid: the column exists.
template <int KW_MAX>
__device__ __forceinline__ void single_row_weights(float (&w)[KW_MAX], const float* __restrict__ src,
                                                   const float* __restrict__ mask, float scale,
                                                   int KW, int K, int row_len, int col, bool valid) {
  const int wave = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < KW_MAX; ++i) {
    const int k = wave * KW + i;
    float v = 0.f;
    if (i < KW && k < K && valid) {
      const size_t o = (size_t)k * row_len + col;
      v = src[o];
      if (mask != nullptr) v = v * mask[o] * scale;
    }
    w[i] = v;
  }
}

// This thread's part of the step's product: its column, its wavefront's quarter of k.  The
// wavefront's share of the polled tile starts at float `off` of `xb`; h_wave: the wavefront's
// KW_MAX floats of LDS, zero beyond KW (so no step of the loop is conditional).
template <int KW_MAX>
__device__ __forceinline__ float single_row_product(const GroupSync& gs, const TileBuffer& xb, int off,
                                                    int KW, float* h_wave, const float (&w)[KW_MAX]) {
  const int lane = threadIdx.x & 63;
  const bool loads = 4 * lane < KW;  // lanes 0 .. KW/4-1 poll four k each
  float4_t hv[1][1];
  auto load = [&] { hv[0][0] = loads ? load_tile4(xb, off + 4 * lane) : float4_t{0.f, 0.f, 0.f, 0.f}; };
  load();
  poll_until_written(gs, load, [&] { return all_written(hv); });
  if (loads) *reinterpret_cast<float4_t*>(&h_wave[4 * lane]) = hv[0][0];
  // LDS operations of a wavefront complete in order: the reads below see the store above.
  float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
  for (int i = 0; i < KW_MAX; i += 4) {
    const float4_t h4 = *reinterpret_cast<const float4_t*>(&h_wave[i]);
    acc0 = fmaf(w[i], h4.x, acc0);
    acc1 = fmaf(w[i + 1], h4.y, acc1);
    acc0 = fmaf(w[i + 2], h4.z, acc0);
    acc1 = fmaf(w[i + 3], h4.w, acc1);
  }
  return acc0 + acc1;
}

// ---- host side ---------------------------------------------------------------------
// Partial tiles slice_product leaves in LDS (ProductTile<nb, ct>::kPartials).
inline int product_partials(int nb, int ct) {
  (void)nb;
  (void)ct;
  return 4;
}

// LDS bytes of a forward kernel (slice [Kpad x 16*ct] + the partial tiles of nb rows).
inline size_t fwd_lds_bytes(int H, int nb, int ct) {
  const int Kpad = (H + 63) / 64 * 64;
  return ((size_t)Kpad * 16 * ct + (size_t)product_partials(nb, ct) * nb * 16 * ct) * sizeof(float);
}

// LDS bytes of a kernel that runs an 8-row tile as two sets of 4 rows: the slice
// [Kpad x 16*ct] and, per set, two polled areas of partial tiles.
inline size_t paired_lds_bytes(int Kpad, int ct) {
  return ((size_t)Kpad * 16 * ct + 4 * (size_t)product_partials(4, ct) * 4 * 16 * ct) * sizeof(float);
}

// Host-side plan of a persistent launch: fills `shape` and the grid for (gx, gy).
// An XCD-local launch is used when every group fits on one XCD (gx <= CUs per XCD,
// gy <= XCDs); it fills the chip with one workgroup per CU (the LDS request is raised so
// that two cannot share a CU) and lets the kernel sort the workgroups by XCD.
struct LaunchPlan {
  dim3 grid;
  size_t lds_bytes;
  LaunchShape shape;
  int threads = 256;  // 512: two 256-thread sets per workgroup
};

inline bool xcd_local_fits(int gx, int gy) {
  const int cus = device_cu_count(), xcds = device_xcd_count();
  return xcds > 0 && cus % xcds == 0 && gy <= xcds && gx <= cus / xcds;
}

inline int plan_launch(hipStream_t stream, const Workspace& ws, int gx, int gy, int tile_rows,
                       size_t lds_bytes, unsigned int epochs, LaunchPlan* plan) {
  plan->shape.cb = ws.control;
  plan->shape.host_status = ws.host_status_dev;
  plan->shape.spin_limit = spin_limit();
  plan->shape.absent = test_absent_workgroups();
  plan->shape.gx = gx;
  plan->shape.gy = gy;
  plan->shape.tile_rows = tile_rows;
  plan->shape.ticket_base = 0;
  plan->shape.per_xcd = 0;
  plan->shape.xcc_map = 0;
  HASTE_HIP_PROPAGATE(reserve_epochs(stream, epochs, &plan->shape.epoch));
  HASTE_HIP_PROPAGATE(xcd_layout_ready(stream));
  const int cus = device_cu_count(), xcds = device_xcd_count();
  if (xcds > 0 && cus % xcds == 0 && gy <= xcds && gx <= cus / xcds) {
    plan->shape.xcd_local = 1;
    plan->shape.per_xcd = cus / xcds;
    plan->shape.xcc_map = device_xcc_logical_map();
    HASTE_HIP_PROPAGATE(reserve_tickets(stream, (unsigned)plan->shape.per_xcd, &plan->shape.ticket_base));
    plan->grid = dim3((unsigned)cus);
    const size_t one_per_cu = 84 * 1024;  // more than half of a CU's LDS
    plan->lds_bytes = lds_bytes > one_per_cu ? lds_bytes : one_per_cu;
  } else {
    plan->shape.xcd_local = 0;
    plan->grid = dim3((unsigned)gx, (unsigned)gy);
    plan->lds_bytes = lds_bytes;
  }
  return HASTE_HIP_OK;
}

// Dynamic LDS a persistent kernel may ask for: the 160 KiB of a gfx950 workgroup less room
// for the kernels' few statically allocated words (role, flag), which count against the
// same limit.  A kernel without static LDS may ask for all of it.
constexpr size_t kWorkgroupLdsBytes = 160 * 1024;
constexpr size_t kMaxLdsBytes = kWorkgroupLdsBytes - 256;

// Launches a persistent kernel whose workgroups wait for each other, so all of them must
// be resident at once: the grid is checked against what the chip can hold.  It is an
// ordinary launch, not hipLaunchCooperativeKernel: the cooperative queue can be held by only
// one process per device at a time (a second process gets hipErrorIllegalState), which
// would make the library unusable from several workers sharing a GPU.  Two persistent kernels
// of this process on different streams are ordered one after the other (see
// order_persistent_launches) because two half-resident grids could starve each other; the
// bounded step-barrier waits cover everything else (another process's long kernel).
template <typename KernelT, typename ParamsT>
int launch_persistent(const char* name, KernelT kernel, const LaunchPlan& plan, ParamsT& params,
                      hipStream_t stream) {
  // The kernel's LDS limit and its occupancy at this request are looked up once per process
  // and device: single-step callers (Iterate) launch the same kernel over and over.  The
  // limit is a property of the kernel, not of the launch, and is only ever raised.
  struct Known { size_t limit = 0; std::map<size_t, int> per_cu; };
  static std::mutex known_mutex;
  static std::map<std::pair<const void*, int>, Known> known;
  int device = 0;
  HASTE_HIP_TRY(hipGetDevice(&device));
  const void* fn = reinterpret_cast<const void*>(kernel);
  std::lock_guard<std::mutex> lock(known_mutex);
  Known& k = known[std::make_pair(fn, device)];
  if (k.limit < plan.lds_bytes) {
    const size_t limit = plan.lds_bytes > kMaxLdsBytes ? plan.lds_bytes : kMaxLdsBytes;
    HASTE_HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)limit));
    k.limit = limit;
  }
  auto found = k.per_cu.find(plan.lds_bytes);
  if (found == k.per_cu.end()) {
    int blocks = 0;
    HASTE_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, plan.threads, plan.lds_bytes));
    found = k.per_cu.emplace(plan.lds_bytes, blocks).first;
  }
  const int per_cu = found->second;
  const long long capacity = (long long)per_cu * device_cu_count();
  if ((long long)plan.grid.x * plan.grid.y > capacity) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  // wait for the last launch, launch, become the last launch: as one step among host threads
  PersistentLaunchOrder in_order;
  HASTE_HIP_PROPAGATE(order_persistent_launches(stream, true));
  {
    ScopedKernelTimer timer(name, stream);
    kernel<<<plan.grid, dim3((unsigned)plan.threads), plan.lds_bytes, stream>>>(params);
    HASTE_HIP_TRY(hipGetLastError());
  }
  HASTE_HIP_PROPAGATE(order_persistent_launches(stream, false));
  return HASTE_HIP_OK;
}


// Floats of the exchange tiles (2 behind a step barrier, kPolledTiles when polled) of every
// group (batch tile) for contraction length K.
inline size_t exchange_floats(int K, int nb, int gy, int n_tiles = 2) {
  const size_t Kpad = (size_t)(K + 63) / 64 * 64;
  return (size_t)n_tiles * Kpad * nb * gy;
}

// Geometry of a forward recurrence: nb batch rows and hs hidden units per workgroup
// (their gate columns fill ct 16-column tiles), gx column workgroups, gy batch tiles.
struct ForwardTile {
  int nb, ct, hs, gx, gy;
  size_t lds_bytes;
  bool ok;
  int reg_groups;  // k-groups of the slice that every wavefront keeps in registers
};

constexpr int kTileHeights[] = {4, 8, 16, 32, 64};

// Prefers a geometry whose groups each fit on one XCD (shortest tiles first, which
// spreads a small batch over the most XCDs; then the most column workgroups), else the
// cross-XCD geometry with the most parallelism that fits the chip.  `extra_lds_per_row` is
// what the cell needs in LDS per batch row beyond the slice and the partial tiles.
// `wide_first`: 4-row tiles take the fewest column workgroups instead.  The layer-norm cells,
// whose steps also exchange row statistics among all workgroups of a group (every workgroup
// reads every other's slots), are 10-25 % faster per step that way (N <= 32, H = 64 .. 256;
// with 8-row tiles it depends on H, and the plain cells are 10-20 % slower).
// `resident_max_ct` > 0: the kernel can keep part of a slice that exceeds LDS in registers
// (tiles of 16 rows and more, 8 or 16 hidden units per workgroup in at most that many column
// tiles; a multiple of 8 k-groups per wavefront, at most 128 registers per lane).  Tried when no
// geometry fits LDS alone.
inline ForwardTile pick_forward_tile(int gates, int N, int H, size_t extra_lds_per_row,
                                     size_t lds_limit = kMaxLdsBytes, bool wide_first = false,
                                     int resident_max_ct = 0) {
  const int cus = device_cu_count();
  ForwardTile best;
  best.ok = false;
  best.reg_groups = 0;
  for (int pass = 0; pass < 2 && !best.ok; ++pass) {
    const int hs_order_local[] = {4, 8, 16};
    const int hs_order_wide[] = {16, 8, 4};
    const int hs_order_cross[] = {8, 16, 4};
    for (int nb : kTileHeights) {
      for (int i = 0; i < 3 && !best.ok; ++i) {
        const int hs = pass == 0 ? (wide_first && nb == 4 ? hs_order_wide[i] : hs_order_local[i])
                                 : hs_order_cross[i];
        const int ct = (gates * hs + 15) / 16;
        const int gx = (H + hs - 1) / hs, gy = (N + nb - 1) / nb;
        const size_t lds = fwd_lds_bytes(H, nb, ct) + extra_lds_per_row * nb;
        if (lds > lds_limit || gy > kMaxGroups || gx * gy > kMaxWorkgroups) continue;
        if (pass == 0 ? !xcd_local_fits(gx, gy) : (long long)gx * gy > cus) continue;
        best = ForwardTile{nb, ct, hs, gx, gy, lds, true, 0};
      }
      if (best.ok) break;
    }
  }
  if (best.ok || resident_max_ct <= 0) return best;
  const int groups = (H + 63) / 64;  // k-groups of 16 per wavefront
  for (int nb : kTileHeights) {
    if (nb < 16) continue;
    for (int hs : {8, 16}) {
      const int ct = (gates * hs + 15) / 16;
      const int gx = (H + hs - 1) / hs, gy = (N + nb - 1) / nb;
      if (ct > resident_max_ct || gy > kMaxGroups || (long long)gx * gy > cus) continue;
      const size_t group_bytes = (size_t)4 * 16 * 16 * ct * sizeof(float);  // one k-group of each wavefront
      const size_t other = (size_t)product_partials(nb, ct) * nb * 16 * ct * sizeof(float) +
                           extra_lds_per_row * nb;
      if (other >= lds_limit) continue;
      const int fit = (int)((lds_limit - other) / group_bytes);
      if (fit >= groups) continue;  // fits LDS: the passes above decide
      const int reg_groups = (groups - fit + 7) / 8 * 8;
      if (reg_groups * ct > 32 || reg_groups >= groups) continue;
      best = ForwardTile{nb, ct, hs, gx, gy, (size_t)(groups - reg_groups) * group_bytes + other, true,
                         reg_groups};
      return best;
    }
  }
  return best;
}

// Geometry of a backward recurrence: 16 hidden units and nb batch rows per workgroup.
struct BackwardTile {
  int nb, gx, gy;
  size_t lds_bytes;
  bool ok;
  int reg_groups;  // k-groups of the slice that every wavefront keeps in registers
};

// The most k-groups (of 16) of its share of the slice that a wavefront keeps in registers.
constexpr int kMaxResidentGroups = 32;

// K = gates*H is the contraction length.  Per batch row the kernel needs, beyond the
// slice, max(`reduce_floats_per_row`, the partial tiles) + `extra_floats_per_row` floats.
// `resident_rows`: the kernel can keep part of a slice that exceeds LDS in registers (tiles
// of 16 rows and more; a multiple of 8 k-groups per wavefront, at most kMaxResidentGroups).
inline BackwardTile pick_backward_tile(int K, int N, int H, size_t reduce_floats_per_row,
                                       size_t extra_floats_per_row, bool resident_rows = false) {
  const int cus = device_cu_count();
  const int gx = (H + 15) / 16;
  const int Kpad = (K + 63) / 64 * 64;
  const int groups = Kpad / 64;                // per wavefront
  const size_t group_bytes = 4 * 16 * 16 * sizeof(float);  // one k-group of each wavefront
  BackwardTile best;
  best.ok = false;
  for (int pass = 0; pass < 2 && !best.ok; ++pass) {
    for (int nb : kTileHeights) {
      const int gy = (N + nb - 1) / nb;
      size_t per_row = (size_t)product_partials(nb, 1) * 16;
      if (per_row < reduce_floats_per_row) per_row = reduce_floats_per_row;
      per_row += extra_floats_per_row;
      const size_t other = per_row * nb * sizeof(float);
      size_t lds = (size_t)Kpad * 16 * sizeof(float) + other;
      int reg_groups = 0;
      if (lds > kMaxLdsBytes && resident_rows && nb >= 16 && other < kMaxLdsBytes) {
        const int fit = (int)((kMaxLdsBytes - other) / group_bytes);
        reg_groups = (groups - fit + 7) / 8 * 8;
        if (reg_groups > kMaxResidentGroups || reg_groups >= groups) continue;  // some of the slice stays in LDS
        lds = (size_t)(groups - reg_groups) * group_bytes + other;
      }
      if (lds > kMaxLdsBytes || gy > kMaxGroups || gx * gy > kMaxWorkgroups) continue;
      if (pass == 0 ? !xcd_local_fits(gx, gy) : (long long)gx * gy > cus) continue;
      best = BackwardTile{nb, gx, gy, lds, true, reg_groups};
      break;
    }
  }
  return best;
}

}  // namespace haste_hip
