// fp32 MFMA GEMM for gfx950: C[M,N] = op(A)[M,K] * B[K,N] (+ C).
//
// Replaces the cuBLAS sgemm calls of the reference (lib/blas.h:48-61): the
// time-fused input projection x*W (lib/lstm_forward_gpu.cu.cc:340-348) and the
// three batched backward products dW, dR, dx (lib/lstm_backward_gpu.cu.cc:374-402).
//
// Design: 128x128 output tile per 256-thread workgroup (4 wavefronts, each a 64x64
// quadrant = 2x2 v_mfma_f32_32x32x2_f32 tiles), K consumed 16 at a time through a
// double-buffered LDS stage.  Both operand tiles sit in LDS k-major, so a wavefront
// reads the 32 consecutive floats of one k for each half of its lanes, which is the
// operand layout of the 32x32x2 instruction and is bank-conflict free.
//
// Work distribution: output tiles are handed out in rounds of one tile per CU for as
// long as whole rounds remain; the tiles of the last, partial round (all tiles, when
// there are fewer tiles than CUs: dW, dR with K = T*N) are cut along K into pieces so
// that the pieces again fill the chip evenly.  Pieces park partial tiles; a second,
// bandwidth-bound kernel adds the pieces of a tile in index order, so results do not
// depend on scheduling.  Whole tiles are numbered so that each XCD (one L2) works on a
// contiguous run of them; the pieces follow, dealt round-robin over the XCDs.
#include "common.h"

namespace haste_hip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int BN = 128;
constexpr int BK = 16;
constexpr int LDB = BN + 4;
constexpr int B_STAGE = BK * LDB;
constexpr int kXcds = 8;

// Operand panels are read through buffer resources: a 16-byte load at any 4-byte aligned
// offset, elements beyond the resource's range read as zero and never fault.  That keeps the
// K loop free of branches (the compiler can then overlap the loads of the next step with the
// MFMAs of this one); `valid` (how many of the four elements belong to the problem) is applied
// with selects.
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_panel(const float* base, long long floats) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)(floats * 4), 0x00020000);
}

// The load is issued here; `valid` is applied by masked4() when the data is used, so that
// nothing waits for the load in between.
__device__ __forceinline__ uint4_t load4_raw(__amdgpu_buffer_rsrc_t panel, long long float_offset,
                                             int valid) {
  const unsigned int off = valid > 0 ? (unsigned int)(float_offset * 4) : 0x7ffffff0u;
  return __builtin_amdgcn_raw_buffer_load_b128(panel, off, 0, 0);
}

__device__ __forceinline__ float4_t masked4(uint4_t u, int valid) {
  float4_t v;
  v.x = valid > 0 ? __uint_as_float(u.x) : 0.f;
  v.y = valid > 1 ? __uint_as_float(u.y) : 0.f;
  v.z = valid > 2 ? __uint_as_float(u.z) : 0.f;
  v.w = valid > 3 ? __uint_as_float(u.w) : 0.f;
  return v;
}

// One BM x 128 output tile over the K range [k_begin, k_end): BM = 128 (each wavefront a
// 64x64 quadrant) or 64 (each a 32x64 quadrant) for outputs too small to fill the chip with
// 128-row tiles.  part == null: the tile goes to C (+= when accumulate); otherwise the whole
// [BM][BN] partial tile is parked at `part`.  `smem`: 2 * (BK * (BM + 4) + B_STAGE) floats.
template <bool TRANS_A, int BM, bool INTERIOR = false>
__device__ __forceinline__ void gemm_tile(int M, int N, int K,
                                          const float* __restrict__ A, int lda,
                                          const float* __restrict__ B, int ldb,
                                          float* __restrict__ C, int ldc, int accumulate,
                                          int tm, int tn, int k_begin, int k_end,
                                          float* __restrict__ part, float* smem) {
  // A tile k-major in LDS: leading dimension BM+2 when it is written with transposing
  // scalar stores (bank-conflict free), BM+4 when written with 16-byte stores.
  constexpr int LDA = TRANS_A ? BM + 4 : BM + 2;
  constexpr int A_STAGE = BK * (BM + 4);
  constexpr int MI = BM / 64;       // 32x32 MFMA tiles per wavefront along M
  constexpr int A_PASSES = BM / 64; // passes of 256 threads to load the A tile
  float* As = smem;
  float* Bs = smem + 2 * A_STAGE;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = (wave >> 1) * (32 * MI);
  const int wn = (wave & 1) * 64;

  float16_t acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  uint4_t a_raw[A_PASSES], b_raw[2];
  int a_valid[A_PASSES], b_valid[2];
  // A tile stored [K][M] in memory: one pass covers (256*4/BM) k-rows of BM columns.
  constexpr int TA_ROWS = 1024 / BM;
  constexpr int TA_COLS = BM / 4;

  // This workgroup's operand panels: its BM rows (TRANS_A: columns) of A and its 128 columns
  // of B, all of K.  Offsets below are in floats from the panel's first element.
  const int rows_here = (M - m0) < BM ? (M - m0) : BM;
  const int cols_here = (N - n0) < BN ? (N - n0) : BN;
  const __amdgpu_buffer_rsrc_t a_panel =
      TRANS_A ? make_panel(A + m0, (long long)(K - 1) * lda + rows_here)
              : make_panel(A + (size_t)m0 * lda, (long long)(rows_here - 1) * lda + K);
  const __amdgpu_buffer_rsrc_t b_panel = make_panel(B + n0, (long long)(K - 1) * ldb + cols_here);

  // INTERIOR (every tile whole, K and the K pieces multiples of BK): a thread's offsets into
  // the panels are fixed and the step enters as the instruction's scalar offset, so that a
  // step's loads cost no vector instruction besides themselves (everything the vector units
  // do in this loop is time the matrix units stand still).
  unsigned int a_voff[A_PASSES], b_voff[2];
#pragma unroll
  for (int i = 0; i < A_PASSES; ++i)
    a_voff[i] = TRANS_A ? (unsigned int)((((tid / TA_COLS) + TA_ROWS * i) * lda + (tid % TA_COLS) * 4) * 4)
                        : (unsigned int)((((tid >> 2) + 64 * i) * lda + (tid & 3) * 4) * 4);
#pragma unroll
  for (int i = 0; i < 2; ++i) b_voff[i] = (unsigned int)((((tid >> 5) + 8 * i) * ldb + (tid & 31) * 4) * 4);

  auto load_global = [&](int kk) {
    if constexpr (INTERIOR) {
      const int a_soff = TRANS_A ? kk * lda * 4 : kk * 4;
      const int b_soff = kk * ldb * 4;
#pragma unroll
      for (int i = 0; i < A_PASSES; ++i) {
        a_valid[i] = 4;
        a_raw[i] = __builtin_amdgcn_raw_buffer_load_b128(a_panel, a_voff[i], a_soff, 0);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        b_valid[i] = 4;
        b_raw[i] = __builtin_amdgcn_raw_buffer_load_b128(b_panel, b_voff[i], b_soff, 0);
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      if (TRANS_A) {
        const int ak = (tid / TA_COLS) + TA_ROWS * i;
        const int am = (tid % TA_COLS) * 4;
        const int k = kk + ak;
        a_valid[i] = INTERIOR ? 4 : ((k < k_end) ? (rows_here - am) : 0);
        a_raw[i] = load4_raw(a_panel, (long long)k * lda + am, a_valid[i]);
      } else {
        const int arow = (tid >> 2) + 64 * i;
        const int ak = (tid & 3) * 4;
        const int k = kk + ak;
        a_valid[i] = INTERIOR ? 4 : ((arow < rows_here) ? (k_end - k) : 0);
        a_raw[i] = load4_raw(a_panel, (long long)arow * lda + k, a_valid[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int bk = (tid >> 5) + 8 * i;
      const int bn = (tid & 31) * 4;
      const int k = kk + bk;
      b_valid[i] = INTERIOR ? 4 : ((k < k_end) ? (cols_here - bn) : 0);
      b_raw[i] = load4_raw(b_panel, (long long)k * ldb + bn, b_valid[i]);
    }
  };

  auto store_lds = [&](int buf) {
    float* as = As + buf * A_STAGE;
    float* bs = Bs + buf * B_STAGE;
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const float4_t a = masked4(a_raw[i], a_valid[i]);
      if (TRANS_A) {
        const int ak = (tid / TA_COLS) + TA_ROWS * i;
        const int am = (tid % TA_COLS) * 4;
        *reinterpret_cast<float4_t*>(as + ak * LDA + am) = a;
      } else {
        const int arow = (tid >> 2) + 64 * i;
        const int ak = (tid & 3) * 4;
        as[(ak + 0) * LDA + arow] = a.x;
        as[(ak + 1) * LDA + arow] = a.y;
        as[(ak + 2) * LDA + arow] = a.z;
        as[(ak + 3) * LDA + arow] = a.w;
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int bk = (tid >> 5) + 8 * i;
      const int bn = (tid & 31) * 4;
      *reinterpret_cast<float4_t*>(bs + bk * LDB + bn) = masked4(b_raw[i], b_valid[i]);
    }
  };

  auto compute = [&](int buf) {
    const float* as = As + buf * A_STAGE + (lane >> 5) * LDA + wm + (lane & 31);
    const float* bs = Bs + buf * B_STAGE + (lane >> 5) * LDB + wn + (lane & 31);
    // The LDS reads of K pair k2+2 are issued before the MFMAs of pair k2.
    float b_nxt[2], a_nxt[MI];
    b_nxt[0] = bs[0];
    b_nxt[1] = bs[32];
#pragma unroll
    for (int i = 0; i < MI; ++i) a_nxt[i] = as[32 * i];
#pragma unroll
    for (int k2 = 0; k2 < BK; k2 += 2) {
      const float b0 = b_nxt[0], b1 = b_nxt[1];
      float av[MI];
#pragma unroll
      for (int i = 0; i < MI; ++i) av[i] = a_nxt[i];
      if (k2 + 2 < BK) {
        b_nxt[0] = bs[(k2 + 2) * LDB];
        b_nxt[1] = bs[(k2 + 2) * LDB + 32];
#pragma unroll
        for (int i = 0; i < MI; ++i) a_nxt[i] = as[(k2 + 2) * LDA + 32 * i];
        // keep the reads here: the scheduler would otherwise sink them to just before their use
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], b0, acc[i][0], 0, 0, 0);
        acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], b1, acc[i][1], 0, 0, 0);
      }
    }
  };

  if (k_begin < k_end) {
    load_global(k_begin);
    store_lds(0);
    __syncthreads();
    int buf = 0;
    for (int kk = k_begin; kk < k_end; kk += BK) {
      const bool more = kk + BK < k_end;
      if (more) load_global(kk + BK);
      compute(buf);
      if (more) store_lds(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
  }

  // Output element (row, col) of accumulator register e in a 32x32 tile:
  // col = lane % 32, row = 8*(e/4) + 4*(lane/32) + e%4.
  const int col_in = lane & 31;
  const int row_in = (lane >> 5) * 4;
  if (part == nullptr) {
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn + 32 * j + col_in;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = m0 + wm + 32 * i + 8 * (e >> 2) + row_in + (e & 3);
          if (row < M && col < N) {
            float* p = C + (size_t)row * ldc + col;
            *p = accumulate ? (*p + acc[i][j][e]) : acc[i][j][e];
          }
        }
      }
    return;
  }

  // A K piece: park the whole [BM][BN] partial tile (rows and columns beyond the problem
  // hold zeros); a second, bandwidth-bound kernel adds a tile's pieces in order (the kernel
  // boundary makes them visible, so no cache-wide fence is needed here).
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = wn + 32 * j + col_in;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = wm + 32 * i + 8 * (e >> 2) + row_in + (e & 3);
        part[row * BN + col] = acc[i][j][e];
      }
    }
}

// Runs one tile (or K piece of a tile) with the loop that fits it: whole tiles whose K range
// is a multiple of BK need no masks (gemm_tile's INTERIOR), the tiles on the edges of a ragged
// problem do.
template <bool TRANS_A, int BM>
__device__ __forceinline__ void gemm_any_tile(int M, int N, int K, const float* __restrict__ A, int lda,
                                              const float* __restrict__ B, int ldb,
                                              float* __restrict__ C, int ldc, int accumulate,
                                              int tm, int tn, int k_begin, int k_end,
                                              float* __restrict__ part, float* smem) {
  const bool whole = M - tm * BM >= BM && N - tn * BN >= BN && (k_end - k_begin) % BK == 0;
  if (whole)
    gemm_tile<TRANS_A, BM, true>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, tm, tn, k_begin, k_end, part, smem);
  else
    gemm_tile<TRANS_A, BM, false>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, tm, tn, k_begin, k_end, part, smem);
}

template <bool TRANS_A, int BM>
__global__ __launch_bounds__(256, 2)
void gemm_f32_kernel(int M, int N, int K,
                     const float* __restrict__ A, int lda,
                     const float* __restrict__ B, int ldb,
                     float* __restrict__ C, int ldc, int accumulate,
                     int tiles_n, int whole_tiles, int splits, int k_per_split,
                     float* __restrict__ partial) {
  __shared__ __attribute__((aligned(16))) float smem[2 * BK * (BM + 4) + 2 * B_STAGE];
  // Workgroups [0, whole_tiles) compute one whole tile each.  Ids are handed to the XCDs
  // round-robin; XCD x gets the x-th contiguous chunk of the tile list so that neighbours
  // in the list share an L2.  Workgroups from whole_tiles on compute one K piece of one of
  // the remaining tiles: piece j = id - whole_tiles is split j % splits of tile
  // whole_tiles + j / splits, and parks its result at partial + j * BM * BN.
  const int id = blockIdx.x;
  int tile, k_begin, k_end;
  float* part = nullptr;
  if (id < whole_tiles) {
    const int q = whole_tiles / kXcds, r = whole_tiles % kXcds;
    const int xcd = id % kXcds, local = id / kXcds;
    tile = xcd * q + (xcd < r ? xcd : r) + local;
    k_begin = 0;
    k_end = K;
  } else {
    // Pieces that read the same rows of A -- the same split of the tiles of one row of tiles --
    // form a group, and the groups are dealt to the XCDs (workgroup ids go to them round-robin)
    // so that a group's pieces have consecutive places on one XCD: its rows of A then come
    // from HBM once and from that XCD's L2 afterwards.  (dx of the headline shape, 4 tiles per
    // row: 245 -> 100 MiB fetched.)  Groups beyond the last whole round of 8, and lists that do
    // not consist of whole rows of tiles, keep the plain order.  Where a piece's result is
    // parked does not depend on the order.
    const int j = id - whole_tiles;
    const int rest = (int)gridDim.x - whole_tiles;          // pieces
    int t = j / splits, split = j % splits;                 // plain order
    if ((rest / splits) % tiles_n == 0 && whole_tiles % tiles_n == 0) {
      const int groups = rest / tiles_n;                    // (row of tiles, split) pairs
      const int dealt = groups / kXcds * kXcds * tiles_n;   // pieces in whole rounds of groups
      int group, member;
      if (j < dealt) {
        const int xcd = j % kXcds, place = j / kXcds;
        group = place / tiles_n * kXcds + xcd;
        member = place % tiles_n;
      } else {
        group = (groups / kXcds) * kXcds + (j - dealt) / tiles_n;
        member = (j - dealt) % tiles_n;
      }
      t = (group / splits) * tiles_n + member;
      split = group % splits;
    }
    tile = whole_tiles + t;
    k_begin = split * k_per_split;
    k_end = (k_begin + k_per_split < K) ? (k_begin + k_per_split) : K;
    part = partial + ((size_t)t * splits + split) * BM * BN;
  }
  gemm_any_tile<TRANS_A, BM>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, tile / tiles_n, tile % tiles_n,
                             k_begin, k_end, part, smem);
}

// Two products with the same N and K in one launch (dW = x^T dv and dR = h^T dv of a backward
// pass): A1 row-major [M1,K], A2 stored transposed [K,M2].  Their tiles form one list, every
// tile cut into `splits` K pieces (splits == 1: whole tiles); piece j of the list parks its
// result at partial + j * BM * BN.  One launch of twice the tiles needs half the pieces per
// tile to fill the chip, i.e. half the partial-tile traffic.
struct GemmPair {
  int M1, M2, N, K;
  const float* A1; int lda1; const float* B1; int ldb1; float* C1; int ldc1;
  const float* A2; int lda2; const float* B2; int ldb2; float* C2; int ldc2;
  int accumulate, tiles_n, tiles_m1, splits, k_per_split;
  float* partial;
};

template <int BM>
__global__ __launch_bounds__(256, 2)
void gemm_f32_pair_kernel(GemmPair p) {
  __shared__ __attribute__((aligned(16))) float smem[2 * BK * (BM + 4) + 2 * B_STAGE];
  const int j = blockIdx.x;
  const int tile = j / p.splits;
  const int k_begin = (j % p.splits) * p.k_per_split;
  const int k_end = (k_begin + p.k_per_split < p.K) ? (k_begin + p.k_per_split) : p.K;
  float* part = p.splits > 1 ? p.partial + (size_t)j * BM * BN : nullptr;
  const int tm = tile / p.tiles_n, tn = tile % p.tiles_n;
  if (tm < p.tiles_m1)
    gemm_any_tile<false, BM>(p.M1, p.N, p.K, p.A1, p.lda1, p.B1, p.ldb1, p.C1, p.ldc1, p.accumulate,
                             tm, tn, k_begin, k_end, part, smem);
  else
    gemm_any_tile<true, BM>(p.M2, p.N, p.K, p.A2, p.lda2, p.B2, p.ldb2, p.C2, p.ldc2, p.accumulate,
                            tm - p.tiles_m1, tn, k_begin, k_end, part, smem);
}

// For the split tiles (tile index whole_tiles + blockIdx.x): C tile (+)= sum over its
// `splits` pieces of partial[(blockIdx.x * splits + piece)][BM][BN], pieces added in index
// order.  blockIdx.y selects 8 of the tile's rows; a thread owns 4 consecutive columns.
template <int BM>
__global__ __launch_bounds__(256)
void split_reduce_kernel(int M, int N, int splits, int tiles_n, int whole_tiles,
                         const float* __restrict__ partial, float* __restrict__ C, int ldc,
                         int accumulate, int vec_ok) {
  const int tile = whole_tiles + blockIdx.x;
  const int tm = tile / tiles_n, tn = tile % tiles_n;
  const int r = blockIdx.y * 8 + (threadIdx.x >> 5);
  const int c = (threadIdx.x & 31) * 4;
  const int row = tm * BM + r, col = tn * BN + c;
  if (r >= BM || row >= M || col >= N) return;
  const float* p = partial + ((size_t)blockIdx.x * splits) * BM * BN + r * BN + c;
  float4_t s = *reinterpret_cast<const float4_t*>(p);
  for (int sp = 1; sp < splits; ++sp)
    s += *reinterpret_cast<const float4_t*>(p + (size_t)sp * BM * BN);
  float* out = C + (size_t)row * ldc + col;
  if (vec_ok && col + 3 < N) {
    float4_t* o = reinterpret_cast<float4_t*>(out);
    *o = accumulate ? (*o + s) : s;
  } else {
    const float v[4] = {s.x, s.y, s.z, s.w};
    for (int i = 0; i < 4 && col + i < N; ++i) out[i] = accumulate ? (out[i] + v[i]) : v[i];
  }
}

// The same for the tile list of gemm_f32_pair_kernel: tile rows below tiles_m1 belong to the
// first product.
template <int BM>
__global__ __launch_bounds__(256)
void split_reduce_pair_kernel(int M1, int M2, int N, int splits, int tiles_n, int tiles_m1,
                              const float* __restrict__ partial, float* __restrict__ C1, int ldc1,
                              float* __restrict__ C2, int ldc2, int accumulate, int vec_ok) {
  const int tile = blockIdx.x;
  int tm = tile / tiles_n;
  const int tn = tile % tiles_n;
  const bool second = tm >= tiles_m1;
  if (second) tm -= tiles_m1;
  const int M = second ? M2 : M1;
  float* C = second ? C2 : C1;
  const int ldc = second ? ldc2 : ldc1;
  const int r = blockIdx.y * 8 + (threadIdx.x >> 5);
  const int c = (threadIdx.x & 31) * 4;
  const int row = tm * BM + r, col = tn * BN + c;
  if (r >= BM || row >= M || col >= N) return;
  const float* p = partial + ((size_t)blockIdx.x * splits) * BM * BN + r * BN + c;
  float4_t s = *reinterpret_cast<const float4_t*>(p);
  for (int sp = 1; sp < splits; ++sp)
    s += *reinterpret_cast<const float4_t*>(p + (size_t)sp * BM * BN);
  float* out = C + (size_t)row * ldc + col;
  if (vec_ok && col + 3 < N) {
    float4_t* o = reinterpret_cast<float4_t*>(out);
    *o = accumulate ? (*o + s) : s;
  } else {
    const float v[4] = {s.x, s.y, s.z, s.w};
    for (int i = 0; i < 4 && col + i < N; ++i) out[i] = accumulate ? (out[i] + v[i]) : v[i];
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// How a product is cut into workgroups (depends on the shape only).
struct GemmPlan {
  int bm, tiles_n, whole_tiles, rest, splits, k_per_split, pieces;
  size_t scratch_bytes;
};

GemmPlan plan_gemm(int M, int N, int K) {
  GemmPlan g;
  g.tiles_n = (N + BN - 1) / BN;
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;

  // Tile height: 64 rows only when the output has no more than that.
  g.bm = M <= 64 ? 64 : 128;
  const int tiles_m = (M + g.bm - 1) / g.bm;
  const long long tiles = (long long)tiles_m * g.tiles_n;

  // Whole rounds of one tile per CU run unsplit; the `rest` tiles of the last round are each
  // cut into `splits` K pieces.  In units of the time one CU needs for one whole tile, s
  // pieces per tile cost ceil(rest*s/CUs)/s for the arithmetic plus 0.25*rest*s/K for
  // writing and re-reading the partial tiles (128 KiB per piece at the chip's memory rate
  // against 2*128*128*K flops at one CU's MFMA rate); a launch that consists of fewer than
  // two pieces per CU pays 20 % more (a lone workgroup cannot hide its own load latency;
  // measured 5-9 % between 1 and 2 pieces per CU at 128 x 8192 x 2048 with the traffic term).
  // The cheapest s is taken, a piece keeping at least 64 of K.  The choice depends on the
  // shape only, so results are reproducible.
  const long long whole = tiles >= cus ? tiles / cus * cus : 0;
  g.rest = (int)(tiles - whole);
  int splits = 1;
  if (g.rest > 0) {
    const int k_iters = (K + BK - 1) / BK;
    int s_max = k_iters / 4;
    if (s_max > 64) s_max = 64;
    auto cost = [&](int s) {
      const long long pieces = (long long)g.rest * s;
      double c = (double)((pieces + cus - 1) / cus) / s;
      if (whole == 0 && pieces < 2LL * cus) c *= 1.2;
      if (s > 1) c += 0.25 * (double)g.rest * s / K;
      return c;
    };
    // At most four pieces per CU: that bounds the partial tiles of any product (64 KiB a
    // piece) by a size callers who lend the library its scratch memory can plan for.
    double best = cost(1);
    for (int s = 2; s <= s_max && (long long)g.rest * s <= 4LL * cus; ++s)
      if (cost(s) < best - 1e-9) { best = cost(s); splits = s; }
  }
  g.k_per_split = (K + splits - 1) / splits;
  g.k_per_split = (g.k_per_split + BK - 1) / BK * BK;
  g.splits = (K + g.k_per_split - 1) / g.k_per_split;
  const bool split = g.splits > 1;
  // Unsplit "rest" tiles are ordinary whole tiles.
  g.whole_tiles = split ? (int)whole : (int)tiles;
  g.pieces = split ? g.rest * g.splits : 0;
  g.scratch_bytes = (size_t)g.pieces * g.bm * BN * sizeof(float);
  return g;
}

}  // namespace

size_t gemm_f32_scratch_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  // Which kernel runs also depends on the operands' alignment: room for either.
  const size_t tiled = plan_gemm(M, N, K).scratch_bytes;
  const size_t skinny = gemm_f32_skinny_shape(false, M, N, K) ? gemm_f32_skinny_scratch_bytes(M, N, K) : 0;
  return tiled > skinny ? tiled : skinny;
}

namespace {
int gemm_f32_once(hipStream_t stream, bool trans_a, int M, int N, int K,
                  const float* A, int lda, const float* B, int ldb,
                  float* C, int ldc, bool accumulate, size_t scratch_offset);
}  // namespace

// A workgroup of the tile kernel addresses its operand panels (its rows of A, its columns of
// B, all of K) with 32-bit byte offsets, so a panel must stay under 2 GiB.  A longer
// contraction -- the dW and dR products of a backward pass contract over T*N with rows of 4H
// floats, 2 GiB from T*N*H = 2^27 on -- is cut into runs of K that fit, each accumulating into
// C; where the cuts fall depends on the shape only.
int gemm_f32(hipStream_t stream, bool trans_a, int M, int N, int K,
             const float* A, int lda, const float* B, int ldb,
             float* C, int ldc, bool accumulate, size_t scratch_offset) {
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0);
  HASTE_HIP_REQUIRE(A != nullptr && B != nullptr && C != nullptr);
  HASTE_HIP_REQUIRE(lda >= (trans_a ? M : K) && ldb >= N && ldc >= N);
  const long long limit = (1ll << 29) - 256;  // floats a panel may span
  long long run = (limit - BN) / ldb;
  if (trans_a) {
    const long long a_run = (limit - 128) / lda;
    run = a_run < run ? a_run : run;
  } else if (128ll * lda + K >= limit) {
    run = 0;  // 128 rows of A alone exceed the limit
  }
  if (run >= K) return gemm_f32_once(stream, trans_a, M, N, K, A, lda, B, ldb, C, ldc, accumulate, scratch_offset);
  run = run / 1024 * 1024;
  if (run <= 0) {
    set_error_text("gemm: a row of an operand is too long for the kernel's 32-bit panel offsets "
                   "(leading dimension of 2^19 floats or more per 1024 rows)");
    return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  }
  for (long long k0 = 0; k0 < K; k0 += run) {
    const int kc = (int)(K - k0 < run ? K - k0 : run);
    const float* a = trans_a ? A + (size_t)k0 * lda : A + k0;
    HASTE_HIP_PROPAGATE(gemm_f32_once(stream, trans_a, M, N, kc, a, lda, B + (size_t)k0 * ldb, ldb, C, ldc,
                                      accumulate || k0 > 0, scratch_offset));
  }
  return HASTE_HIP_OK;
}

namespace {
int gemm_f32_once(hipStream_t stream, bool trans_a, int M, int N, int K,
                  const float* A, int lda, const float* B, int ldb,
                  float* C, int ldc, bool accumulate, size_t scratch_offset) {
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0);
  HASTE_HIP_REQUIRE(A != nullptr && B != nullptr && C != nullptr);
  HASTE_HIP_REQUIRE(lda >= (trans_a ? M : K) && ldb >= N && ldc >= N);
  HASTE_HIP_REQUIRE((long long)((M + 63) / 64) * ((N + BN - 1) / BN) < (1ll << 26));
  if (gemm_f32_skinny_applies(trans_a, M, N, K, A, lda, B, ldb, C, ldc))
    return gemm_f32_skinny(stream, M, N, K, A, lda, B, ldb, C, ldc, accumulate, scratch_offset);
  const GemmPlan g = plan_gemm(M, N, K);
  const int bm = g.bm, tiles_n = g.tiles_n, whole_tiles = g.whole_tiles, rest = g.rest;
  const int splits = g.splits, k_per_split = g.k_per_split, pieces = g.pieces;
  const bool split = splits > 1;

  // The partial tiles live `scratch_offset` bytes (a multiple of 16) into the stream's
  // scratch buffer; callers that keep data of their own in front of them say so.
  Workspace ws;
  float* partial = nullptr;
  if (split) {
    HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + g.scratch_bytes, &ws));
    partial = ws.scratch + scratch_offset / sizeof(float);
  }
  // A workgroup addresses its operand panels (its rows of A, its columns of B, all of K)
  // with 32-bit byte offsets.
  HASTE_HIP_REQUIRE(((long long)(trans_a ? K : bm) * lda + (trans_a ? bm : K)) * 4 < (1ll << 31));
  HASTE_HIP_REQUIRE(((long long)K * ldb + BN) * 4 < (1ll << 31));
  dim3 grid((unsigned)(whole_tiles + pieces)), block(256);
  ScopedKernelTimer timer("gemm_f32", stream);
#define HASTE_GEMM_LAUNCH(TA_, BM_)                                                          \
  if (trans_a == TA_ && bm == BM_)                                                           \
    gemm_f32_kernel<TA_, BM_><<<grid, block, 0, stream>>>(                                   \
        M, N, K, A, lda, B, ldb, C, ldc, accumulate ? 1 : 0, tiles_n, whole_tiles, splits,   \
        k_per_split, partial);
  HASTE_GEMM_LAUNCH(false, 128) HASTE_GEMM_LAUNCH(false, 64)
  HASTE_GEMM_LAUNCH(true, 128) HASTE_GEMM_LAUNCH(true, 64)
#undef HASTE_GEMM_LAUNCH
  HASTE_HIP_TRY(hipGetLastError());
  if (split) {
    const int vec = (ldc % 4 == 0) && aligned16(C);
    const dim3 rgrid((unsigned)rest, (unsigned)(bm / 8));
    if (bm == 128)
      split_reduce_kernel<128><<<rgrid, dim3(256), 0, stream>>>(
          M, N, splits, tiles_n, whole_tiles, partial, C, ldc, accumulate ? 1 : 0, vec);
    else
      split_reduce_kernel<64><<<rgrid, dim3(256), 0, stream>>>(
          M, N, splits, tiles_n, whole_tiles, partial, C, ldc, accumulate ? 1 : 0, vec);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}
}  // namespace

// C1[M1,N] (+)= A1[M1,K] * B1 and C2[M2,N] (+)= A2^T * B2 (A2 stored [K,M2]) in one launch when
// together they have fewer tiles than the chip has CUs (then each alone would be cut into
// twice the pieces); otherwise two ordinary products.  `products` of the timer: 2.
int gemm_f32_pair(hipStream_t stream, int M1, int M2, int N, int K, const float* A1, int lda1,
                  const float* B1, int ldb1, float* C1, int ldc1, const float* A2, int lda2,
                  const float* B2, int ldb2, float* C2, int ldc2, bool accumulate) {
  HASTE_HIP_REQUIRE(M1 > 0 && M2 > 0 && N > 0 && K > 0 && A1 && B1 && C1 && A2 && B2 && C2);
  HASTE_HIP_REQUIRE(lda1 >= K && lda2 >= M2 && ldb1 >= N && ldb2 >= N && ldc1 >= N && ldc2 >= N);
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const int tiles_n = (N + BN - 1) / BN;
  const int tiles_m1 = (M1 + 127) / 128, tiles_m2 = (M2 + 127) / 128;
  const long long tiles = (long long)(tiles_m1 + tiles_m2) * tiles_n;
  const bool panels_ok = ((long long)128 * lda1 + K) * 4 < (1ll << 31) && ((long long)K * lda2 + 128) * 4 < (1ll << 31) &&
                         ((long long)K * ldb1 + BN) * 4 < (1ll << 31) && ((long long)K * ldb2 + BN) * 4 < (1ll << 31);
  if (tiles >= cus || M1 <= 64 || M2 <= 64 || !panels_ok) {
    HASTE_HIP_PROPAGATE(gemm_f32(stream, false, M1, N, K, A1, lda1, B1, ldb1, C1, ldc1, accumulate));
    return gemm_f32(stream, true, M2, N, K, A2, lda2, B2, ldb2, C2, ldc2, accumulate);
  }
  // The cost model of plan_gemm for a list in which every tile is cut.
  const int k_iters = (K + BK - 1) / BK;
  int s_max = k_iters / 4;
  if (s_max > 64) s_max = 64;
  auto cost = [&](int s) {
    const long long pieces = tiles * s;
    double c = (double)((pieces + cus - 1) / cus) / s;
    if (pieces < 2LL * cus) c *= 1.2;
    if (s > 1) c += 0.25 * (double)tiles * s / K;
    return c;
  };
  int splits = 1;
  double best = cost(1);
  for (int s = 2; s <= s_max && tiles * s <= 4LL * cus; ++s)
    if (cost(s) < best - 1e-9) { best = cost(s); splits = s; }
  int k_per_split = (K + splits - 1) / splits;
  k_per_split = (k_per_split + BK - 1) / BK * BK;
  splits = (K + k_per_split - 1) / k_per_split;

  GemmPair p;
  p.M1 = M1; p.M2 = M2; p.N = N; p.K = K;
  p.A1 = A1; p.lda1 = lda1; p.B1 = B1; p.ldb1 = ldb1; p.C1 = C1; p.ldc1 = ldc1;
  p.A2 = A2; p.lda2 = lda2; p.B2 = B2; p.ldb2 = ldb2; p.C2 = C2; p.ldc2 = ldc2;
  p.accumulate = accumulate ? 1 : 0;
  p.tiles_n = tiles_n; p.tiles_m1 = tiles_m1; p.splits = splits; p.k_per_split = k_per_split;
  p.partial = nullptr;
  if (splits > 1) {
    Workspace ws;
    HASTE_HIP_PROPAGATE(get_workspace(stream, (size_t)tiles * splits * 128 * BN * sizeof(float), &ws));
    p.partial = ws.scratch;
  }
  ScopedKernelTimer timer("gemm_f32", stream, 2);
  gemm_f32_pair_kernel<128><<<dim3((unsigned)(tiles * splits)), dim3(256), 0, stream>>>(p);
  HASTE_HIP_TRY(hipGetLastError());
  if (splits > 1) {
    const int vec = (ldc1 % 4 == 0) && (ldc2 % 4 == 0) && aligned16(C1) && aligned16(C2);
    split_reduce_pair_kernel<128><<<dim3((unsigned)tiles, 16), dim3(256), 0, stream>>>(
        M1, M2, N, splits, tiles_n, tiles_m1, p.partial, C1, ldc1, C2, ldc2, p.accumulate, vec);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

// The product as its K pieces, for a consumer that adds them itself (in piece order): only the
// tile kernel is launched.  Possible when every tile of the product is cut into pieces and
// the output is one tile high; *splits == 0 otherwise (nothing launched).  Element (row, col)
// of piece s lies at partial[((col / 128 * splits + s) * bm + row) * 128 + col % 128]; valid
// until the next product on the stream.
int gemm_f32_pieces(hipStream_t stream, int M, int N, int K, const float* A, int lda,
                    const float* B, int ldb, size_t scratch_offset, const float** partial,
                    int* splits, int* bm) {
  *splits = 0;
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0 && A != nullptr && B != nullptr);
  HASTE_HIP_REQUIRE(lda >= K && ldb >= N);
  const GemmPlan g = plan_gemm(M, N, K);
  if (g.splits <= 1 || g.whole_tiles != 0 || M > g.bm) return HASTE_HIP_OK;
  if (((long long)g.bm * lda + K) * 4 >= (1ll << 31) || ((long long)K * ldb + BN) * 4 >= (1ll << 31))
    return HASTE_HIP_OK;
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + g.scratch_bytes, &ws));
  float* part = ws.scratch + scratch_offset / sizeof(float);
  dim3 grid((unsigned)g.pieces), block(256);
  ScopedKernelTimer timer("gemm_f32", stream);
  if (g.bm == 128)
    gemm_f32_kernel<false, 128><<<grid, block, 0, stream>>>(M, N, K, A, lda, B, ldb, nullptr, 0, 0, g.tiles_n,
                                                            0, g.splits, g.k_per_split, part);
  else
    gemm_f32_kernel<false, 64><<<grid, block, 0, stream>>>(M, N, K, A, lda, B, ldb, nullptr, 0, 0, g.tiles_n,
                                                           0, g.splits, g.k_per_split, part);
  HASTE_HIP_TRY(hipGetLastError());
  *partial = part;
  *splits = g.splits;
  *bm = g.bm;
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_f32(int trans_a, int M, int N, int K,
                                  const float* A, int lda, const float* B, int ldb,
                                  float* C, int ldc, int accumulate, void* stream) {
  return haste_hip::gemm_f32(haste_hip::as_stream(stream), trans_a != 0, M, N, K, A, lda, B, ldb,
                             C, ldc, accumulate != 0);
}
