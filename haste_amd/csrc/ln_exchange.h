// Row statistics across workgroups, for layer norm inside a persistent recurrence.
//
// A normalised row spans the columns of every workgroup in a group.  Each workgroup
// reduces its own columns of each of its NB rows, publishes a few floats per row to
// a small exchange buffer in device memory (agent-scope stores), the group passes a
// step barrier, and then every workgroup combines all contributions in the same fixed
// order, so all of them obtain bit-identical statistics.
//
// Forward: contributions are (mean, sum of squared deviations) of the workgroup's own
// columns, merged pairwise with Chan's update, which keeps the two-pass accuracy of
// reference lib/layer_norm_forward_gpu.cu.cc:45-77 without a second exchange.
// Backward: contributions are the three sums of lib/layer_norm_backward_gpu.cu.cc:49-78.
#pragma once

#include "recurrent.h"

namespace haste_hip {

constexpr float kLnEps = 1e-5f;

// Sum over the W consecutive lanes (W a power of two, segment aligned to W).
template <int W>
__device__ __forceinline__ float segment_sum(float v) {
#pragma unroll
  for (int off = W / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ void load_exchanged2(const float* p, float& a, float& b) {
  const unsigned long long bits = __hip_atomic_load(
      reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  a = __uint_as_float((unsigned int)bits);
  b = __uint_as_float((unsigned int)(bits >> 32));
}

struct Moments { float n, mean, m2; };

// Chan's pairwise update; either side may be empty (n == 0).
__device__ __forceinline__ Moments merge_moments(const Moments a, const Moments b) {
  if (b.n == 0.f) return a;
  if (a.n == 0.f) return b;
  Moments r;
  r.n = a.n + b.n;
  const float delta = b.mean - a.mean;
  r.mean = a.mean + delta * (b.n / r.n);
  r.m2 = a.m2 + b.m2 + delta * delta * (a.n * b.n / r.n);
  return r;
}

// part: this group's buffer, [gx][NB][2] floats holding each workgroup's (mean, m2) of its
// columns of each row.  Workgroup cw contributed `full_count` columns, the last one
// `last_count`.  Writes (mean, 1/sqrt(var + eps)) of the whole row (D columns) to
// out[row*2 .. +1] in LDS.  Called by all 256 threads after the barrier that follows the
// publication; the caller synchronises the workgroup before reading `out`.
template <int NB>
__device__ __forceinline__ void merge_row_moments(const float* part, int gx, float full_count,
                                                  float last_count, float D, float* out) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  for (int row = wave; row < NB; row += 4) {
    Moments acc = {0.f, 0.f, 0.f};
    for (int cw = lane; cw < gx; cw += 64) {
      Moments m;
      load_exchanged2(part + ((size_t)cw * NB + row) * 2, m.mean, m.m2);
      m.n = (cw == gx - 1) ? last_count : full_count;
      acc = merge_moments(acc, m);
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      Moments o;
      o.n = __shfl_xor(acc.n, off, 64);
      o.mean = __shfl_xor(acc.mean, off, 64);
      o.m2 = __shfl_xor(acc.m2, off, 64);
      acc = (lane & off) ? merge_moments(o, acc) : merge_moments(acc, o);
    }
    if (lane == 0) {
      out[row * 2 + 0] = acc.mean;
      out[row * 2 + 1] = 1.0f / sqrtf(acc.m2 / D + kLnEps);
    }
  }
}

// part: [gx][NB][4] floats, each workgroup's (s0, s1, s2, unused) per row.  Writes the
// three row sums to out[row*4 .. +2] in LDS.  Same calling rules as merge_row_moments.
template <int NB>
__device__ __forceinline__ void sum_row_partials(const float* part, int gx, float* out) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  for (int row = wave; row < NB; row += 4) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
    for (int cw = lane; cw < gx; cw += 64) {
      const float4_t v = load_exchanged4(part + ((size_t)cw * NB + row) * 4);
      s0 += v.x;
      s1 += v.y;
      s2 += v.z;
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      s0 += __shfl_xor(s0, off, 64);
      s1 += __shfl_xor(s1, off, 64);
      s2 += __shfl_xor(s2, off, 64);
    }
    if (lane == 0) {
      out[row * 4 + 0] = s0;
      out[row * 4 + 1] = s1;
      out[row * 4 + 2] = s2;
    }
  }
}

}  // namespace haste_hip
