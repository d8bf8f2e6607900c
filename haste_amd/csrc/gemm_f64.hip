// C[M,N] (+)= op(A)[M,K] * B[K,N] in double precision on the fp64 matrix cores
// (v_mfma_f64_16x16x4_f64): what the `double` instantiations of the reference get from
// cublasDgemm (lib/blas.h:48-61).
//
// Bound: MFMA (fp64 peak 78.6 TFLOP/s), algorithmic flops 2*M*N*K.  A workgroup of four
// wavefronts owns a 64 x 64 tile of C; a wavefront owns 32 x 32 of it as 2 x 2 MFMA tiles.
// Operand panels of 32 k go through LDS k-major ([k][m], [k][n]): the lanes of one MFMA
// operand read 16 consecutive doubles of one k row.  A product with few tiles and a long
// contraction (the recurrent product of one step: 64 x 512 x 2048 is 8 tiles) is cut along K
// into pieces, each a workgroup of its own, which park partial results in the stream's scratch
// buffer; a second kernel adds a tile's pieces in index order.  How a product is cut depends
// on its shape only, so results are reproducible.  Lane layout of the instruction (checked on
// the hardware): a = A[i = lane%16][k = lane/16], b = B[k = lane/16][j = lane%16],
// d[r] = D[i = 4*r + lane/16][j = lane%16].
#include "common.h"

namespace haste_hip {
namespace {

typedef double double4_t __attribute__((ext_vector_type(4)));

constexpr int DM = 64, DN = 64, DK = 32;
constexpr int DPITCH = 64 + 1;  // doubles per k row in LDS (odd: the transposing stores of A spread over the banks)

template <bool TRANS_A>
__global__ __launch_bounds__(256)
void gemm_f64_kernel(int M, int N, int K, const double* __restrict__ A, int lda,
                     const double* __restrict__ B, int ldb, double* __restrict__ C, int ldc,
                     int accumulate, int k_per_piece, double* __restrict__ part) {
  __shared__ double As[DK][DPITCH];
  __shared__ double Bs[DK][DPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * DM, n0 = blockIdx.x * DN;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  double4_t acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) acc[a][b] = double4_t{0.0, 0.0, 0.0, 0.0};

  // A thread's 8 elements of each operand panel.  The panel of step k0 + DK is requested before
  // the MFMAs of step k0, so that the loads' latency (what a step of this short loop costs
  // otherwise) passes beside them.
  double ra[8], rb[8];
  auto request = [&](int k0) {
    if (TRANS_A) {
      const int gk = k0 + (tid >> 3), m8 = (tid & 7) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int gm = m0 + m8 + i;
        ra[i] = (gm < M && gk < K) ? A[(size_t)gk * lda + gm] : 0.0;
      }
    } else {
      const int gm = m0 + (tid >> 2), k8 = (tid & 3) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int gk = k0 + k8 + i;
        ra[i] = (gm < M && gk < K) ? A[(size_t)gm * lda + gk] : 0.0;
      }
    }
    const int gk = k0 + (tid >> 3), n8 = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int gn = n0 + n8 + i;
      rb[i] = (gn < N && gk < K) ? B[(size_t)gk * ldb + gn] : 0.0;
    }
  };
  auto park = [&]() {
    if (TRANS_A) {
      const int k = tid >> 3, m8 = (tid & 7) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) As[k][m8 + i] = ra[i];
    } else {
      const int m = tid >> 2, k8 = (tid & 3) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) As[k8 + i][m] = ra[i];
    }
    const int k = tid >> 3, n8 = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) Bs[k][n8 + i] = rb[i];
  };

  // this workgroup's piece of the contraction; request() and the loop below see its end as K
  const int k_begin = blockIdx.z * k_per_piece;
  K = k_begin + k_per_piece < K ? k_begin + k_per_piece : K;
  if (part != nullptr) {  // piece z parks [M][N] at part + z * M * N
    C = part + (size_t)blockIdx.z * M * N;
    ldc = N;
    accumulate = 0;
  }
  request(k_begin);
  for (int k0 = k_begin; k0 < K; k0 += DK) {
    park();
    __syncthreads();
    if (k0 + DK < K) request(k0 + DK);
#pragma unroll
    for (int kk = 0; kk < DK; kk += 4) {
      const int k = kk + (lane >> 4), o = lane & 15;
      const double a0 = As[k][wm + o], a1 = As[k][wm + 16 + o];
      const double b0 = Bs[k][wn + o], b1 = Bs[k][wn + 16 + o];
      acc[0][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b1, acc[1][1], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int gm = m0 + wm + 16 * a + 4 * r + (lane >> 4);
        const int gn = n0 + wn + 16 * b + (lane & 15);
        if (gm < M && gn < N) {
          double* p = C + (size_t)gm * ldc + gn;
          *p = accumulate ? *p + acc[a][b][r] : acc[a][b][r];
        }
      }
}

// C (+)= the pieces of every element, added in index order.
__global__ __launch_bounds__(256)
void gemm_f64_reduce_kernel(int M, int N, int pieces, const double* __restrict__ part,
                            double* __restrict__ C, int ldc, int accumulate) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)M * N) return;
  double s = part[i];
  for (int z = 1; z < pieces; ++z) s += part[(size_t)z * M * N + i];
  double* out = C + (i / N) * ldc + i % N;
  *out = accumulate ? *out + s : s;
}

// Pieces a product is cut into along K: as many as fill about one workgroup per CU, a piece
// keeping at least 4 panels of the contraction; products of 128 tiles and more are not cut.
void plan_f64(int M, int N, int K, int* pieces, int* k_per_piece) {
  const long long tiles = (long long)((M + DM - 1) / DM) * ((N + DN - 1) / DN);
  int s = 1;
  if (tiles < 128) {
    s = (int)(256 / tiles);
    const int most = K / (4 * DK);
    s = s < most ? s : most;
    s = s < 64 ? s : 64;
    s = s > 1 ? s : 1;
  }
  int per = (K + s - 1) / s;
  per = (per + DK - 1) / DK * DK;
  *k_per_piece = per;
  *pieces = (K + per - 1) / per;
}

}  // namespace

size_t gemm_f64_scratch_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int pieces, per;
  plan_f64(M, N, K, &pieces, &per);
  return pieces > 1 ? (size_t)pieces * M * N * sizeof(double) : 0;
}

// The partial results of a cut product lie `scratch_offset` bytes (a multiple of 16) into the
// stream's scratch buffer.
int gemm_f64(hipStream_t stream, bool trans_a, int M, int N, int K, const double* A, int lda,
             const double* B, int ldb, double* C, int ldc, bool accumulate, size_t scratch_offset) {
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0 && A && B && C);
  HASTE_HIP_REQUIRE(lda >= (trans_a ? M : K) && ldb >= N && ldc >= N);
  int pieces, per;
  plan_f64(M, N, K, &pieces, &per);
  const dim3 grid((unsigned)((N + DN - 1) / DN), (unsigned)((M + DM - 1) / DM), (unsigned)pieces);
  HASTE_HIP_REQUIRE(grid.y < 65536u);
  double* part = nullptr;
  if (pieces > 1) {
    Workspace ws;
    HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + (size_t)pieces * M * N * sizeof(double), &ws));
    part = reinterpret_cast<double*>(reinterpret_cast<char*>(ws.scratch) + scratch_offset);
  }
  ScopedKernelTimer timer("gemm_f64", stream);
  if (trans_a)
    gemm_f64_kernel<true><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, per, part);
  else
    gemm_f64_kernel<false><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, per, part);
  HASTE_HIP_TRY(hipGetLastError());
  if (pieces > 1) {
    const size_t n = (size_t)M * N;
    gemm_f64_reduce_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(M, N, pieces, part, C, ldc,
                                                                                         accumulate ? 1 : 0);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_f64(int trans_a, int M, int N, int K, const double* A, int lda,
                                  const double* B, int ldb, double* C, int ldc, int accumulate,
                                  void* stream) {
  return haste_hip::gemm_f64(haste_hip::as_stream(stream), trans_a != 0, M, N, K, A, lda, B, ldb,
                             C, ldc, accumulate != 0, 0);
}
