// Device-side building blocks of the persistent recurrence kernels.
//
// A recurrence kernel is one cooperative launch that runs all T steps.  The grid is
// (column workgroups) x (batch tiles): a workgroup owns `HS` hidden units (all of
// their gate columns) for the 16*RT batch rows of its tile, keeps its slice of the
// recurrent weight matrix in LDS for the whole launch, and per step multiplies the
// tile's rows of the exchanged activation (h_t forward, the gate gradients backward)
// with that slice on the MFMA units.  Workgroups that share a batch tile form a
// group and synchronise once per exchange through a counter in device memory;
// different batch tiles never wait for each other.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"

namespace haste_hip {

typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr unsigned int kSpinLimit = 1u << 24;  // polls before a barrier wait gives up

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float d_sigmoid_f(float y) { return y * (1.0f - y); }
__device__ __forceinline__ float d_tanh_f(float y) { return 1.0f - y * y; }

// ---- Exchange between workgroups inside one launch --------------------------------
// The 8 XCDs of the chip have separate L2 caches, so data one workgroup writes and
// another reads in the same launch must not rest in an L2.  Such data is written and
// read with agent-scope accesses (the sc1 forms of global_store / global_load, which
// go to the memory side), and everything else uses ordinary cached accesses: no
// cache-wide write-back or invalidate is needed at a step boundary.
__device__ __forceinline__ void store_exchanged(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
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
};

__device__ __forceinline__ void group_sync_init(GroupSync& g, ControlBlock* cb, unsigned int group,
                                                unsigned int group_size, unsigned int my_index,
                                                unsigned int epoch, unsigned int* host_status,
                                                unsigned int spin_limit) {
  g.flags = &cb->step_flags[group * group_size];
  g.abort_flag = &cb->abort_flag[0];
  g.host_status = host_status;
  g.group_size = group_size;
  g.my_index = my_index;
  g.epoch = epoch;
  g.arrivals = 0;
  g.spin_limit = spin_limit;
}

// Counts the workgroup as arrived once every exchanged store its threads have issued
// has completed.  Called by all threads.
__device__ __forceinline__ void group_arrive(GroupSync& g) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  g.arrivals += 1;
  if (threadIdx.x == 0)
    __hip_atomic_store(&g.flags[g.my_index], g.epoch + g.arrivals, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
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

// True in exactly one workgroup of the launch: the last to call it.  Stores made by
// the other workgroups before their call are visible to that workgroup afterwards.
// `flag` is a word of LDS.  Called by all threads.
__device__ __forceinline__ bool grid_last_arrival(ControlBlock* cb, unsigned int total_workgroups,
                                                  unsigned int* flag) {
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    const unsigned int old = __hip_atomic_fetch_add(&cb->grid_exit_counter[0], 1u, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
    const bool last = old == total_workgroups - 1;
    if (last) {
      __hip_atomic_store(&cb->grid_exit_counter[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    }
    *flag = last ? 1u : 0u;
  }
  __syncthreads();
  return *flag != 0u;
}

__device__ __forceinline__ int round_up(int x, int m) { return (x + m - 1) / m * m; }

// LDS image of a weight slice: element (k, col) of a [Kpad x NCOLS] slice lives at
// float index (((k/16)*4 + (k%16)/4) * NCOLS + col) * 4 + k%4, i.e. the 4 consecutive
// k a lane feeds to 4 consecutive 16x16x4 MFMAs are one 16-byte LDS read, and the 16
// lanes of a k-quarter read 16 consecutive such vectors (no bank conflicts).
__device__ __forceinline__ int slice_index(int k, int col, int ncols) {
  return ((((k >> 4) << 2) + ((k & 15) >> 2)) * ncols + col) * 4 + (k & 3);
}

// Guarded 4-float read of exchanged data: elements beyond `valid` read as zero.
__device__ __forceinline__ float4_t load_a4(const float* p, int valid, bool vec_ok) {
  float4_t v = {0.f, 0.f, 0.f, 0.f};
  if (valid >= 4 && vec_ok) {
    v = load_exchanged4(p);
  } else {
    if (valid > 0) v.x = load_exchanged(p);
    if (valid > 1) v.y = load_exchanged(p + 1);
    if (valid > 2) v.z = load_exchanged(p + 2);
    if (valid > 3) v.w = load_exchanged(p + 3);
  }
  return v;
}

// acc[rt][ct] += A[16*RT rows, K] * slice[K, 16*CT] for this wavefront's quarter of K.
// `a` points at row 0 of the batch tile (row stride a_ld floats, K contiguous);
// rows >= rows_valid and k >= K read as zero.  The four wavefronts of the workgroup
// each take Kpad/4 consecutive k; the caller adds their accumulators.
// Accumulator element r of acc[rt][ct] in lane l is row 16*rt + 4*(l/16) + r,
// column 16*ct + l%16.
template <int RT, int CT, int CHUNK>
__device__ __forceinline__ void slice_matmul(const float* __restrict__ a, int a_ld, int rows_valid,
                                             int K, int Kpad, const float* w_lds, bool vec_ok,
                                             float4_t (&acc)[RT][CT]) {
  constexpr int NCOLS = 16 * CT;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int row = lane & 15;
  const int kq = lane >> 4;
  const int groups = Kpad >> 6;  // k-groups of 16 per wavefront
  const int g_first = wave * groups;

  for (int g0 = 0; g0 < groups; g0 += CHUNK) {
    float4_t av[CHUNK][RT];
#pragma unroll
    for (int gi = 0; gi < CHUNK; ++gi) {
      const int k = (g_first + g0 + gi) * 16 + kq * 4;
      const bool live = g0 + gi < groups;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int rr = rt * 16 + row;
        const int valid = (live && rr < rows_valid) ? (K - k) : 0;
        av[gi][rt] = load_a4(a + (size_t)rr * a_ld + k, valid, vec_ok);
      }
    }
#pragma unroll
    for (int gi = 0; gi < CHUNK; ++gi) {
      if (g0 + gi < groups) {
        const int kg = g_first + g0 + gi;
        const float* wp = w_lds + ((kg * 4 + kq) * NCOLS + row) * 4;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const float4_t b = *reinterpret_cast<const float4_t*>(wp + ct * 64);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[gi][rt].x, b.x, acc[rt][ct], 0, 0, 0);
            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[gi][rt].y, b.y, acc[rt][ct], 0, 0, 0);
            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[gi][rt].z, b.z, acc[rt][ct], 0, 0, 0);
            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[gi][rt].w, b.w, acc[rt][ct], 0, 0, 0);
          }
        }
      }
    }
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

// Sum over the four wavefronts of element (row, col) written by store_partials.
template <int RT, int CT>
__device__ __forceinline__ float sum_partials(const float* red, int row, int col) {
  constexpr int NCOLS = 16 * CT;
  constexpr int NB = 16 * RT;
  const float* p = red + row * NCOLS + col;
  return (p[0] + p[NB * NCOLS]) + (p[2 * NB * NCOLS] + p[3 * NB * NCOLS]);
}

// ---- host side ---------------------------------------------------------------------
// LDS bytes of a forward kernel (slice [Kpad x 16*CT] + 4 wavefront partial tiles).
inline size_t fwd_lds_bytes(int H, int RT, int CT) {
  const int Kpad = (H + 63) / 64 * 64;
  return ((size_t)Kpad * 16 * CT + 4 * 16 * RT * 16 * CT) * sizeof(float);
}

inline size_t bwd_lds_bytes(int K, int RT) {
  const int Kpad = (K + 63) / 64 * 64;
  const size_t red = (size_t)4 * 16 * RT * 16;
  return ((size_t)Kpad * 16 + red) * sizeof(float);
}

template <typename KernelT, typename ParamsT>
int launch_persistent(const char* name, KernelT kernel, dim3 grid, size_t lds_bytes, ParamsT& params,
                      hipStream_t stream) {
  HASTE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  int per_cu = 0;
  HASTE_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, lds_bytes));
  const long long capacity = (long long)per_cu * device_cu_count();
  if ((long long)grid.x * grid.y > capacity) return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  void* args[] = {&params};
  ScopedKernelTimer timer(name, stream);
  HASTE_HIP_TRY(hipLaunchCooperativeKernel(reinterpret_cast<const void*>(kernel), grid, dim3(256),
                                           args, (unsigned int)lds_bytes, stream));
  return HASTE_HIP_OK;
}

constexpr size_t kMaxLdsBytes = 160 * 1024;  // LDS per workgroup on gfx950


}  // namespace haste_hip
