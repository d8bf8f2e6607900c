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

#include <type_traits>

#include "recurrent.h"

namespace haste_hip {

constexpr float kLnEps = 1e-5f;

// Cross-lane moves inside a row of 16 lanes on the data-parallel-primitive path of the
// VALU (a few cycles; a shuffle through the LDS crossbar costs over a hundred).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// Sum over the W consecutive lanes (W a power of two up to 16, segment aligned to W); every
// lane of the segment receives it.  Pairs are formed by quad permutes (lane^1, lane^2), then
// by mirroring the half row and the row: once the lanes of a quad (half row) agree, lane i and
// lane 7-i (15-i) hold the sums of the two halves.
template <int W>
__device__ __forceinline__ float segment_sum(float v) {
  static_assert(W == 1 || W == 2 || W == 4 || W == 8 || W == 16, "segment within a row of 16 lanes");
  if (W >= 2) v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
  if (W >= 4) v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
  if (W >= 8) v += dpp_move<0x141>(v);   // row_half_mirror
  if (W >= 16) v += dpp_move<0x140>(v);  // row_mirror
  return v;
}

// Sum over all 64 lanes, the same value in every lane: rows of 16 as above, then the four
// row sums in lane order.
__device__ __forceinline__ float wave_sum(float v) {
  v = segment_sum<16>(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
}

// Sums over the lanes of a wavefront of W values at once, valid in lane 0 at least.
// `first_row_only`: only the first 16 lanes hold anything that counts, and every one of them
// receives the sums of those.  One branch for all values, so that their chains of cross-lane
// adds interleave instead of each waiting out its own hazards.
template <int W>
__device__ __forceinline__ void lanes_sums(float (&v)[W], bool first_row_only) {
  if (first_row_only) {
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = segment_sum<16>(v[i]);
  } else {
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = wave_sum(v[i]);
  }
}
__device__ __forceinline__ float lanes_sum(float v, bool first_row_only) {
  float one[1] = {v};
  lanes_sums<1>(one, first_row_only);
  return one[0];
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

// ---- tagged row exchange ---------------------------------------------------------------
// The same exchanges without a step barrier.  Every float travels in an 8-byte word next to
// a 32-bit tag that names the use (launch epoch + running count), so a reader knows from the
// word itself whether it has been published: it re-issues its loads until every tag matches.
// Two buffers alternate by use parity: a workgroup publishes use u+2 only after it has read
// every contribution to use u+1, and those were published after their authors had read use u,
// so nobody can still be reading the words that use u+2 overwrites.  Layout of one buffer:
// [gx][NB] slots of WS words (W values, padded to an even count so that a slot
// is written and read with 16-byte accesses); a workgroup's slots share lines with nobody.
template <int W> struct RowSlot { static constexpr int kWords = (W + 1) / 2 * 2; };

__host__ __device__ __forceinline__ size_t tagged_row_words(int gx, int nb, int w) {
  return (size_t)gx * nb * ((w + 1) / 2 * 2);
}

typedef unsigned int uint4_row_t __attribute__((ext_vector_type(4)));

template <int W>
__device__ __forceinline__ void publish_row(const GroupSync& g, unsigned long long* buffer, int nb,
                                            int cw, int row, const float (&v)[W], unsigned int tag) {
  constexpr int WS = RowSlot<W>::kWords;
  unsigned long long* q = buffer + ((size_t)cw * nb + row) * WS;
#pragma unroll
  for (int i = 0; i < WS; i += 2) {
    uint4_row_t u;
    u.x = __float_as_uint(v[i]);
    u.y = tag;
    u.z = i + 1 < W ? __float_as_uint(v[i + 1 < W ? i + 1 : i]) : 0u;
    u.w = tag;
    if (g.same_xcd) {
      // An ordinary store (the slot stays in the XCD's L2, where its readers look).  Not a
      // volatile one: that compiles to a system-scope store followed by a wait for its
      // acknowledgement -- and for that of everything stored before it -- 1.2 us per exchange.
      *reinterpret_cast<uint4_row_t*>(q + i) = u;
      asm volatile("" ::: "memory");
    } else {
      __hip_atomic_store(q + i, (unsigned long long)u.x | ((unsigned long long)u.y << 32),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(q + i + 1, (unsigned long long)u.z | ((unsigned long long)u.w << 32),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// Zeroes this workgroup's slots of both buffers (a tag of zero is never expected); called
// before the launch's initial barrier.
__device__ __forceinline__ void clear_row_words(const GroupSync& g, unsigned long long* both, int gx,
                                                int cw, int nb, int w) {
  const int ws = (w + 1) / 2 * 2;
  for (int i = threadIdx.x; i < 2 * nb * ws; i += 256) {
    unsigned long long* q = both + (size_t)(i / (nb * ws)) * tagged_row_words(gx, nb, w) +
                            (size_t)cw * nb * ws + i % (nb * ws);
    if (g.same_xcd) *reinterpret_cast<volatile unsigned long long*>(q) = 0ull;
    else __hip_atomic_store(q, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Loads the slot of (cw, row) until all of its words carry `tag` (`have` false: nothing to
// load).  `slots` is a buffer resource over the buffer (16-byte agent-scope loads, never
// served by this CU's L1).  The whole wavefront polls together, backing off briefly between
// attempts (all workgroups of the group poll the same few lines); bounded like every wait of
// the launch.
template <int W>
__device__ __forceinline__ void load_row_polled(const GroupSync& g, const TileBuffer& slots, int nb,
                                                int cw, int row, bool have, unsigned int tag,
                                                float (&v)[W]) {
  constexpr int WS = RowSlot<W>::kWords;
  const int word = ((have ? cw : 0) * nb + row) * WS;
  bool ok = !have;
  auto load = [&] {
    // All of a slot's loads are issued before any tag is looked at, and the tags are combined
    // without branches: with `&&` the compiler makes a load wait for the previous one's tag.
    uint4_t u[WS / 2];
#pragma unroll
    for (int i = 0; i < WS; i += 2)
      u[i / 2] = __builtin_amdgcn_raw_buffer_load_b128(slots.rsrc, (word + i) * 8, 0, 16);
    unsigned int differ = 0u;
#pragma unroll
    for (int i = 0; i < WS; i += 2) {
      v[i] = __uint_as_float(u[i / 2].x);
      if (i + 1 < W) v[i + 1 < W ? i + 1 : i] = __uint_as_float(u[i / 2].z);
      differ |= (u[i / 2].y ^ tag) | (u[i / 2].w ^ tag);
    }
    ok = !have || differ == 0u;
  };
  if (have) load();
    poll_until_written(g, [&] { __builtin_amdgcn_s_sleep(1); load(); }, [&] { return __all(ok) != 0; });
}

// N slots per lane at once (word offsets `word`, slots a lane does not have: have[i] false),
// all loads in flight together and re-issued until every tag matches.  Values of slots a lane
// does not have come back as zeros.
template <int W, int N>
__device__ __forceinline__ void load_slots_polled(const GroupSync& g, const TileBuffer& slots,
                                                  const int (&word)[N], const bool (&have)[N],
                                                  unsigned int tag, float (&v)[N][W]) {
  constexpr int WS = RowSlot<W>::kWords;
  bool ok = false;
  auto load = [&] {
    uint4_t u[N][WS / 2];
#pragma unroll
    for (int n = 0; n < N; ++n)
#pragma unroll
      for (int i = 0; i < WS; i += 2)
        u[n][i / 2] = __builtin_amdgcn_raw_buffer_load_b128(slots.rsrc, ((have[n] ? word[n] : 0) + i) * 8, 0, 16);
    unsigned int differ = 0u;
#pragma unroll
    for (int n = 0; n < N; ++n) {
      unsigned int d = 0u;
#pragma unroll
      for (int i = 0; i < WS; i += 2) {
        v[n][i] = have[n] ? __uint_as_float(u[n][i / 2].x) : 0.f;
        if (i + 1 < W) v[n][i + 1 < W ? i + 1 : i] = have[n] ? __uint_as_float(u[n][i / 2].z) : 0.f;
        d |= (u[n][i / 2].y ^ tag) | (u[n][i / 2].w ^ tag);
      }
      differ |= have[n] ? d : 0u;
    }
    ok = differ == 0u;
  };
  load();
  poll_until_written(g, [&] { __builtin_amdgcn_s_sleep(1); load(); }, [&] { return __all(ok) != 0; });
}

// The rows whose moments a wavefront gathers through LDS (row = wave + 4 i) are taken up to
// eight at a time: one poll for all of them instead of a round trip per row (tiles of 32 and
// 64 rows have eight and sixteen rows per wavefront, and across XCDs a round trip is
// microseconds): LayerNormLSTM forward, T = 100, N = 128, H = 640 4.99 -> 2.65 ms, N = 64,
// H = 1024 3.20 -> 2.52.  The backward sums (3 or 10 values per slot) stay one row per poll:
// batched four rows at a time they were 7-12 % slower.
template <int NB, int W>
struct RowBatch {
  static constexpr int kRowsPerWave = (NB + 3) / 4;
  static constexpr int kMax = W <= 3 ? 8 : 4;
  static constexpr int kRows = kRowsPerWave < kMax ? kRowsPerWave : kMax;
};

// Row statistics from a tagged buffer ([gx][NB][2] words holding each workgroup's (mean, m2)
// of its `full_count` columns, `last_count` for the last one): the merged mean is the weighted
// mean of the means, the merged m2 the sum of m2_i + n_i (mean_i - mean)^2 -- the pairwise
// update of merge_moments written out for all parts at once, as two plain sums.  Writes
// (mean, 1/sqrt(var + eps)) of the whole row (D columns) to out[row*2 .. +1] in LDS; the
// caller synchronises the workgroup before reading `out`.  Called by all 256 threads.
template <int NB>
__device__ __forceinline__ void merge_row_moments_polled(const GroupSync& g,
                                                         unsigned long long* buffer, int gx,
                                                         unsigned int tag, float full_count,
                                                         float last_count, float D, float* out) {
  constexpr int RB = RowBatch<NB, 2>::kRows;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const TileBuffer slots = make_tile_buffer(reinterpret_cast<float*>(buffer),
                                            (int)tagged_row_words(gx, NB, 2) * 2);
  const bool narrow = gx <= 16;
  const float inv_D = 1.0f / D;
  for (int r0 = wave; r0 < NB; r0 += 4 * RB) {
    // what the first two chunks of 64 column workgroups published is kept for the second pass
    // (a reload is another round trip); further chunks are loaded again
    float kept[2][RB][2], s1[RB], s2[RB];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      s1[i] = s2[i] = 0.f;
      kept[0][i][0] = kept[0][i][1] = kept[1][i][0] = kept[1][i][1] = 0.f;
    }
    auto slots_of = [&](int c0, int (&word)[RB], bool (&have)[RB]) {
      const int cw = c0 + lane;
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        const int row = r0 + 4 * i;
        have[i] = cw < gx && row < NB;
        word[i] = (cw * NB + row) * 2;
      }
    };
    auto count = [&](int c0) {
      const int cw = c0 + lane;
      return cw < gx ? ((cw == gx - 1) ? last_count : full_count) : 0.f;
    };
    // first pass: the weighted means (chunks 0 and 1 at compile-time indices, so that what is
    // kept stays in registers)
    static_for<2>([&](auto cc) {
      constexpr int C = decltype(cc)::value;
      if (C * 64 < gx) {
        int word[RB];
        bool have[RB];
        slots_of(C * 64, word, have);
        load_slots_polled<2, RB>(g, slots, word, have, tag, kept[C]);
        const float n = count(C * 64);
#pragma unroll
        for (int i = 0; i < RB; ++i) s1[i] += n * kept[C][i][0];
      }
    });
    for (int c0 = 128; c0 < gx; c0 += 64) {
      int word[RB];
      bool have[RB];
      float v[RB][2];
      slots_of(c0, word, have);
      load_slots_polled<2, RB>(g, slots, word, have, tag, v);
      const float n = count(c0);
#pragma unroll
      for (int i = 0; i < RB; ++i) s1[i] += n * v[i][0];
    }
    lanes_sums<RB>(s1, narrow);
    // second pass: the squared deviations
    static_for<2>([&](auto cc) {
      constexpr int C = decltype(cc)::value;
      if (C * 64 < gx) {
        const float n = count(C * 64);
#pragma unroll
        for (int i = 0; i < RB; ++i) {
          const float d = kept[C][i][0] - s1[i] * inv_D;
          s2[i] += n > 0.f ? kept[C][i][1] + n * d * d : 0.f;
        }
      }
    });
    for (int c0 = 128; c0 < gx; c0 += 64) {  // seen before
      int word[RB];
      bool have[RB];
      float v[RB][2];
      slots_of(c0, word, have);
      load_slots_polled<2, RB>(g, slots, word, have, tag, v);
      const float n = count(c0);
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        const float d = v[i][0] - s1[i] * inv_D;
        s2[i] += n > 0.f ? v[i][1] + n * d * d : 0.f;
      }
    }
    lanes_sums<RB>(s2, narrow);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        const int row = r0 + 4 * i;
        if (row < NB) {
          out[row * 2 + 0] = s1[i] * inv_D;
          // the hardware's reciprocal square root (1 ulp), as the reference's rsqrt
          // (lib/layer_norm_forward_gpu.cu.cc:77)
          out[row * 2 + 1] = __builtin_amdgcn_rsqf(s2[i] * inv_D + kLnEps);
        }
      }
    }
  }
}

// sum_row_partials over a tagged buffer (slots holding (s0, s1, s2)).
template <int NB>
__device__ __forceinline__ void sum_row_partials_polled(const GroupSync& g,
                                                        unsigned long long* buffer, int gx,
                                                        unsigned int tag, float* out) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const TileBuffer slots = make_tile_buffer(reinterpret_cast<float*>(buffer),
                                            (int)tagged_row_words(gx, NB, 3) * 2);
  for (int row = wave; row < NB; row += 4) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
    for (int c0 = 0; c0 < gx; c0 += 64) {
      const int cw = c0 + lane;
      float v[3];
      load_row_polled<3>(g, slots, NB, cw, row, cw < gx, tag, v);
      if (cw < gx) {
        s0 += v[0];
        s1 += v[1];
        s2 += v[2];
      }
    }
    float s[3] = {s0, s1, s2};
    lanes_sums<3>(s, gx <= 16);
    if (lane == 0) {
      out[row * 4 + 0] = s[0];
      out[row * 4 + 1] = s[1];
      out[row * 4 + 2] = s[2];
    }
  }
}

// ---- gathers that stay inside the wavefront ---------------------------------------------
// The threads that work on the elements of a row are HS consecutive lanes (thread / HS is the
// row, HS a power of two up to 16), and they are the only ones that need the row's statistics.
// So those lanes gather them: lane c of the segment reads the slots of the column workgroups
// c, c + HS, ... and the segment adds up with DPP row operations, after which every lane of
// the segment holds the row's totals -- no LDS, no workgroup barrier, and wavefronts without
// elements do not take part.  Every workgroup adds in the same order, so all of them obtain
// bit-identical results.  For rows of at most 4 * HS parts, and more for narrow workgroups
// (row_gather_in_wavefront); longer rows take the gathers further up, which put all 64 lanes of
// a wavefront on one row and hand the result over through LDS.
// Workgroups of 8 or 4 units whose tile keeps at least two (8 units) or all four wavefronts
// busy gather rows of up to 16 * HS parts this way, all of a lane's slots in one poll: their
// rows are the long ones (H > 512: 72 to 128 parts), and through LDS every wavefront polls
// for four to sixteen rows.  LayerNormLSTM forward, T = 100: N = 64, H = 768 2.03 -> 1.69 ms,
// N = 128, H = 1024 3.59 -> 2.99, N = 32, H = 1024 1.66 -> 1.28; tiles that leave more
// wavefronts idle lose that way (N = 8, H >= 576: +11 %; N = 64, H = 128: +7 %).
template <int HS, int NB>
__device__ __forceinline__ bool row_gather_in_wavefront(int gx) {
  return gx <= 4 * HS || (HS <= 8 && NB * HS >= (HS == 8 ? 128 : 256) && gx <= 16 * HS);
}
// The backward passes, whose slots hold 3 or 10 values: with more than two slots per lane the
// gather inside the wavefront only pays for tiles of 32 rows and more, where the other form
// has a wavefront poll for eight or sixteen rows one after the other (LayerNormLSTM backward,
// T = 100: N = 64, H = 1024 on 16-row tiles 3.27 -> 2.89 ms with the hand-over through LDS,
// N = 128, H = 640 on 32-row tiles 2.62 -> 2.88).
template <int HS>
__device__ __forceinline__ bool row_sums_gather_in_wavefront(int gx, int nb) {
  return gx <= 2 * HS || (gx <= 4 * HS && nb >= 32);
}

// The slots of `row` from the column workgroups cw0, cw0 + step, ... (NCH of them, those beyond
// gx skipped), all loads in flight together and re-issued until every tag matches.
template <int W, int NCH>
__device__ __forceinline__ void load_row_chunks_polled(const GroupSync& g, const TileBuffer& slots,
                                                       int nb, int cw0, int step, int gx, int row,
                                                       bool have_row, unsigned int tag,
                                                       float (&v)[NCH][W]) {
  constexpr int WS = RowSlot<W>::kWords;
  bool have[NCH];
  int word[NCH];
#pragma unroll
  for (int ch = 0; ch < NCH; ++ch) {
    const int cw = cw0 + ch * step;
    have[ch] = have_row && cw < gx;
    word[ch] = have[ch] ? (cw * nb + row) * WS : 0;
  }
  bool ok = false;
  auto load = [&] {
    uint4_t u[NCH][WS / 2];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
      for (int i = 0; i < WS; i += 2)
        u[ch][i / 2] = __builtin_amdgcn_raw_buffer_load_b128(slots.rsrc, (word[ch] + i) * 8, 0, 16);
    unsigned int differ = 0u;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      unsigned int d = 0u;
#pragma unroll
      for (int i = 0; i < WS; i += 2) {
        v[ch][i] = have[ch] ? __uint_as_float(u[ch][i / 2].x) : 0.f;
        if (i + 1 < W) v[ch][i + 1 < W ? i + 1 : i] = have[ch] ? __uint_as_float(u[ch][i / 2].z) : 0.f;
        d |= (u[ch][i / 2].y ^ tag) | (u[ch][i / 2].w ^ tag);
      }
      differ |= have[ch] ? d : 0u;
    }
    ok = differ == 0u;
  };
  load();
  poll_until_written(g, [&] { __builtin_amdgcn_s_sleep(1); load(); }, [&] { return __all(ok) != 0; });
}

// Totals of the W values of `row` over all gx column workgroups, in every lane of the row's
// segment.  have_row: the thread works on an element of the tile (the others get zeros).
template <int HS, int W>
__device__ __forceinline__ void gather_row_sums(const GroupSync& g, unsigned long long* buffer, int nb,
                                                int gx, unsigned int tag, int row, bool have_row,
                                                float (&sum)[W]) {
#pragma unroll
  for (int i = 0; i < W; ++i) sum[i] = 0.f;
  if (__builtin_amdgcn_ballot_w64(have_row) == 0ull) return;
  const TileBuffer slots = make_tile_buffer(reinterpret_cast<float*>(buffer),
                                            (int)tagged_row_words(gx, nb, W) * 2);
  const int c = (int)threadIdx.x % HS;
  auto add = [&](auto nch, int cw0) {
    constexpr int NCH = decltype(nch)::value;
    float v[NCH][W];
    load_row_chunks_polled<W, NCH>(g, slots, nb, cw0, HS, gx, row, have_row, tag, v);
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
      for (int i = 0; i < W; ++i) sum[i] += v[ch][i];
  };
  if (gx <= HS) add(std::integral_constant<int, 1>{}, c);
  else if (gx <= 2 * HS) add(std::integral_constant<int, 2>{}, c);
  else add(std::integral_constant<int, 4>{}, c);
#pragma unroll
  for (int i = 0; i < W; ++i) sum[i] = segment_sum<HS>(sum[i]);
}

// Mean and 1/sqrt(var + eps) of `row` (D columns) from the (mean, m2) that the column
// workgroups published for their `full_count` columns (`last_count` for the last one): the
// weighted mean of the means first, then the sum of m2_i + n_i (mean_i - mean)^2.
template <int HS>
__device__ __forceinline__ void gather_row_moments(const GroupSync& g, unsigned long long* buffer,
                                                   int nb, int gx, unsigned int tag, float full_count,
                                                   float last_count, float D, int row, bool have_row,
                                                   float& mean_out, float& invstd_out) {
  mean_out = 0.f;
  invstd_out = 0.f;
  if (__builtin_amdgcn_ballot_w64(have_row) == 0ull) return;
  const TileBuffer slots = make_tile_buffer(reinterpret_cast<float*>(buffer),
                                            (int)tagged_row_words(gx, nb, 2) * 2);
  const int c = (int)threadIdx.x % HS;
  const float inv_D = 1.0f / D;
  auto count = [&](int cw) { return cw < gx ? (cw == gx - 1 ? last_count : full_count) : 0.f; };
  auto finish = [&](float m2) {
    // the hardware's reciprocal square root (1 ulp), as the reference's rsqrt
    // (lib/layer_norm_forward_gpu.cu.cc:77)
    invstd_out = __builtin_amdgcn_rsqf(m2 * inv_D + kLnEps);
  };
  auto both = [&](auto nch) {
    constexpr int NCH = decltype(nch)::value;
    float v[NCH][2];
    load_row_chunks_polled<2, NCH>(g, slots, nb, c, HS, gx, row, have_row, tag, v);
    float s1 = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) s1 += count(c + ch * HS) * v[ch][0];
    mean_out = segment_sum<HS>(s1) * inv_D;
    float s2 = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      const float d = v[ch][0] - mean_out;
      s2 += v[ch][1] + count(c + ch * HS) * d * d;   // a skipped chunk: 0 + 0 * d * d
    }
    finish(segment_sum<HS>(s2));
  };
  if (gx <= HS) both(std::integral_constant<int, 1>{});
  else if (gx <= 2 * HS) both(std::integral_constant<int, 2>{});
  else if (HS > 8 || gx <= 4 * HS) both(std::integral_constant<int, 4>{});
  else if constexpr (HS <= 8) {
    // narrow workgroups (8 or 4 units): rows of up to 16 * HS parts, all slots of a lane in one poll
    if (gx <= 8 * HS) both(std::integral_constant<int, 8>{});
    else both(std::integral_constant<int, 16>{});
  }
}

// Row sums of W values per slot from a tagged buffer: out[row * RowSlot<W>::kWords + i] in LDS.
// Same calling rules as sum_row_partials_polled.
template <int NB, int W>
__device__ __forceinline__ void sum_row_values_polled(const GroupSync& g, unsigned long long* buffer,
                                                      int gx, unsigned int tag, float* out) {
  constexpr int WS = RowSlot<W>::kWords;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const TileBuffer slots = make_tile_buffer(reinterpret_cast<float*>(buffer),
                                            (int)tagged_row_words(gx, NB, W) * 2);
  for (int row = wave; row < NB; row += 4) {
    float s[W];
#pragma unroll
    for (int i = 0; i < W; ++i) s[i] = 0.f;
    for (int c0 = 0; c0 < gx; c0 += 64) {
      const int cw = c0 + lane;
      float v[W];
      load_row_polled<W>(g, slots, NB, cw, row, cw < gx, tag, v);
      if (cw < gx) {
#pragma unroll
        for (int i = 0; i < W; ++i) s[i] += v[i];
      }
    }
    lanes_sums<W>(s, gx <= 16);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < W; ++i) out[row * WS + i] = s[i];
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
