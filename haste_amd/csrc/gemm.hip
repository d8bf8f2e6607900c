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
// operand layout of the 32x32x2 instruction and is bank-conflict free.  Small
// outputs with a long K (dW, dR: K = T*N) are split along K over several workgroups;
// the last workgroup to arrive at a tile adds the partial sums in a fixed order, so
// results do not depend on arrival order.  Workgroup ids are remapped so that each
// XCD (one L2) works on a contiguous run of tiles.
#include "common.h"

namespace haste_hip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int BM = 128;
constexpr int BN = 128;
constexpr int BK = 16;
constexpr int LDA_ROWMAJOR = BM + 2;  // A tile written with transposing scalar stores
constexpr int LDA_KMAJOR = BM + 4;    // A tile written with 16-byte stores
constexpr int LDB = BN + 4;
constexpr int A_STAGE = BK * (BM + 4);
constexpr int B_STAGE = BK * LDB;
constexpr int kXcds = 8;

__device__ __forceinline__ float4_t load4_guarded(const float* p, int valid, bool vec_ok) {
  float4_t v = {0.f, 0.f, 0.f, 0.f};
  if (valid >= 4 && vec_ok) {
    v = *reinterpret_cast<const float4_t*>(p);
  } else {
    if (valid > 0) v.x = p[0];
    if (valid > 1) v.y = p[1];
    if (valid > 2) v.z = p[2];
    if (valid > 3) v.w = p[3];
  }
  return v;
}

template <bool TRANS_A>
__global__ __launch_bounds__(256, 2)
void gemm_f32_kernel(int M, int N, int K,
                     const float* __restrict__ A, int lda,
                     const float* __restrict__ B, int ldb,
                     float* __restrict__ C, int ldc, int accumulate,
                     int tiles_n, int total_blocks, int splits, int k_per_split,
                     int a_vec_ok, int b_vec_ok,
                     float* __restrict__ partial, unsigned int* tile_counter) {
  __shared__ __attribute__((aligned(16))) float smem[2 * A_STAGE + 2 * B_STAGE];
  __shared__ unsigned int s_arrival;
  float* As = smem;
  float* Bs = smem + 2 * A_STAGE;
  constexpr int LDA = TRANS_A ? LDA_KMAJOR : LDA_ROWMAJOR;

  // Workgroup ids are handed to the XCDs round-robin; give XCD x the x-th contiguous
  // chunk of the tile list so that neighbours in the list share an L2.
  const int id = blockIdx.x;
  const int q = total_blocks / kXcds, r = total_blocks % kXcds;
  const int xcd = id % kXcds, local = id / kXcds;
  const int nid = xcd * q + (xcd < r ? xcd : r) + local;
  const int split = nid % splits;
  const int tile = nid / splits;
  const int tm = tile / tiles_n, tn = tile % tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;
  const int k_begin = split * k_per_split;
  const int k_end = (k_begin + k_per_split < K) ? (k_begin + k_per_split) : K;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = (wave >> 1) * 64;
  const int wn = (wave & 1) * 64;

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  float4_t a_reg[2], b_reg[2];

  auto load_global = [&](int kk) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (TRANS_A) {
        const int ak = (tid >> 5) + 8 * i;
        const int am = (tid & 31) * 4;
        const int k = kk + ak, m = m0 + am;
        const int valid = (k < k_end) ? (M - m) : 0;
        a_reg[i] = load4_guarded(A + (size_t)k * lda + m, valid, a_vec_ok);
      } else {
        const int arow = (tid >> 2) + 64 * i;
        const int ak = (tid & 3) * 4;
        const int m = m0 + arow, k = kk + ak;
        const int valid = (m < M) ? (k_end - k) : 0;
        a_reg[i] = load4_guarded(A + (size_t)m * lda + k, valid, a_vec_ok);
      }
      const int bk = (tid >> 5) + 8 * i;
      const int bn = (tid & 31) * 4;
      const int k = kk + bk, n = n0 + bn;
      const int valid = (k < k_end) ? (N - n) : 0;
      b_reg[i] = load4_guarded(B + (size_t)k * ldb + n, valid, b_vec_ok);
    }
  };

  auto store_lds = [&](int buf) {
    float* as = As + buf * A_STAGE;
    float* bs = Bs + buf * B_STAGE;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (TRANS_A) {
        const int ak = (tid >> 5) + 8 * i;
        const int am = (tid & 31) * 4;
        *reinterpret_cast<float4_t*>(as + ak * LDA + am) = a_reg[i];
      } else {
        const int arow = (tid >> 2) + 64 * i;
        const int ak = (tid & 3) * 4;
        as[(ak + 0) * LDA + arow] = a_reg[i].x;
        as[(ak + 1) * LDA + arow] = a_reg[i].y;
        as[(ak + 2) * LDA + arow] = a_reg[i].z;
        as[(ak + 3) * LDA + arow] = a_reg[i].w;
      }
      const int bk = (tid >> 5) + 8 * i;
      const int bn = (tid & 31) * 4;
      *reinterpret_cast<float4_t*>(bs + bk * LDB + bn) = b_reg[i];
    }
  };

  auto compute = [&](int buf) {
    const float* as = As + buf * A_STAGE + (lane >> 5) * LDA + wm + (lane & 31);
    const float* bs = Bs + buf * B_STAGE + (lane >> 5) * LDB + wn + (lane & 31);
#pragma unroll
    for (int k2 = 0; k2 < BK; k2 += 2) {
      const float a0 = as[k2 * LDA];
      const float a1 = as[k2 * LDA + 32];
      const float b0 = bs[k2 * LDB];
      const float b1 = bs[k2 * LDB + 32];
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
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
  if (splits == 1) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
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

  // Split-K: park the partial tile, then the last arrival folds all partials of the
  // tile into C in split order.
  const size_t tile_elems = (size_t)BM * BN;
  float* part_tile = partial + ((size_t)tile * splits + split) * tile_elems;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = wn + 32 * j + col_in;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int rr = wm + 32 * i + 8 * (e >> 2) + row_in + (e & 3);
        part_tile[rr * BN + c] = acc[i][j][e];
      }
    }
  __threadfence();
  __syncthreads();
  if (tid == 0) s_arrival = atomicAdd(&tile_counter[tile], 1u);
  __syncthreads();
  if (s_arrival != (unsigned)(splits - 1)) return;
  __threadfence();
  const float* base = partial + (size_t)tile * splits * tile_elems;
  for (int idx = tid; idx < BM * BN; idx += 256) {
    const int rr = idx / BN, c = idx % BN;
    const int row = m0 + rr, col = n0 + c;
    if (row < M && col < N) {
      float s = 0.f;
      for (int sp = 0; sp < splits; ++sp) s += base[(size_t)sp * tile_elems + idx];
      float* p = C + (size_t)row * ldc + col;
      *p = accumulate ? (*p + s) : s;
    }
  }
  if (tid == 0) tile_counter[tile] = 0u;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

int gemm_f32(hipStream_t stream, bool trans_a, int M, int N, int K,
             const float* A, int lda, const float* B, int ldb,
             float* C, int ldc, bool accumulate) {
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0);
  HASTE_HIP_REQUIRE(A != nullptr && B != nullptr && C != nullptr);
  HASTE_HIP_REQUIRE(lda >= (trans_a ? M : K) && ldb >= N && ldc >= N);
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = (N + BN - 1) / BN;
  const long long tiles = (long long)tiles_m * tiles_n;
  HASTE_HIP_REQUIRE(tiles < (1ll << 30));
  const int cus = device_cu_count();

  // Split K when the output alone cannot occupy the chip and K is long.
  int splits = 1;
  if (cus > 0 && tiles * 2 <= cus && K >= 1024 && tiles <= 4096) {
    splits = (int)((cus + tiles - 1) / tiles);
    const int max_by_k = K / 256;
    if (splits > max_by_k) splits = max_by_k;
    if (splits > 32) splits = 32;
    if (splits < 1) splits = 1;
  }
  int k_per_split = (K + splits - 1) / splits;
  k_per_split = (k_per_split + BK - 1) / BK * BK;
  splits = (K + k_per_split - 1) / k_per_split;

  Workspace ws;
  float* partial = nullptr;
  unsigned int* tile_counter = nullptr;
  if (splits > 1) {
    const size_t bytes = (size_t)tiles * splits * BM * BN * sizeof(float);
    HASTE_HIP_PROPAGATE(get_workspace(stream, bytes, &ws));
    partial = ws.scratch;
    tile_counter = ws.control->tile_counter;
  }
  const int a_vec_ok = aligned16(A) && (lda % 4 == 0) && (k_per_split % 4 == 0);
  const int b_vec_ok = aligned16(B) && (ldb % 4 == 0);
  const int total = (int)(tiles * splits);
  dim3 grid((unsigned)total), block(256);
  ScopedKernelTimer timer("gemm_f32", stream);
  if (trans_a) {
    gemm_f32_kernel<true><<<grid, block, 0, stream>>>(
        M, N, K, A, lda, B, ldb, C, ldc, accumulate ? 1 : 0, tiles_n, total, splits,
        k_per_split, a_vec_ok, b_vec_ok, partial, tile_counter);
  } else {
    gemm_f32_kernel<false><<<grid, block, 0, stream>>>(
        M, N, K, A, lda, B, ldb, C, ldc, accumulate ? 1 : 0, tiles_n, total, splits,
        k_per_split, a_vec_ok, b_vec_ok, partial, tile_counter);
  }
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_f32(int trans_a, int M, int N, int K,
                                  const float* A, int lda, const float* B, int ldb,
                                  float* C, int ldc, int accumulate, void* stream) {
  return haste_hip::gemm_f32(haste_hip::as_stream(stream), trans_a != 0, M, N, K, A, lda, B, ldb,
                             C, ldc, accumulate != 0);
}
