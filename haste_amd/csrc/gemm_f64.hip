// C[M,N] (+)= op(A)[M,K] * B[K,N] in double precision on the fp64 matrix cores
// (v_mfma_f64_16x16x4_f64): what the `double` instantiations of the reference get from
// cublasDgemm (lib/blas.h:48-61).
//
// Bound: MFMA (fp64 peak 78.6 TFLOP/s), algorithmic flops 2*M*N*K.  A workgroup of four
// wavefronts owns a 64 x 64 tile of C; a wavefront owns 32 x 32 of it as 2 x 2 MFMA tiles.
// Operand panels of 16 k go through LDS k-major ([k][m], [k][n]): the lanes of one MFMA
// operand read 16 consecutive doubles of one k row.  The contraction is never split, so the
// result does not depend on the launch geometry.  Lane layout of the instruction (checked on
// the hardware): a = A[i = lane%16][k = lane/16], b = B[k = lane/16][j = lane%16],
// d[r] = D[i = 4*r + lane/16][j = lane%16].
#include "common.h"

namespace haste_hip {
namespace {

typedef double double4_t __attribute__((ext_vector_type(4)));

constexpr int DM = 64, DN = 64, DK = 16;
constexpr int DPITCH = 64 + 4;  // doubles per k row in LDS

template <bool TRANS_A>
__global__ __launch_bounds__(256)
void gemm_f64_kernel(int M, int N, int K, const double* __restrict__ A, int lda,
                     const double* __restrict__ B, int ldb, double* __restrict__ C, int ldc,
                     int accumulate) {
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

  for (int k0 = 0; k0 < K; k0 += DK) {
    // A panel -> As[k][m]
    if (TRANS_A) {
      const int k = tid >> 4, m4 = (tid & 15) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gm = m0 + m4 + i, gk = k0 + k;
        As[k][m4 + i] = (gm < M && gk < K) ? A[(size_t)gk * lda + gm] : 0.0;
      }
    } else {
      const int m = tid >> 2, k4 = (tid & 3) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gm = m0 + m, gk = k0 + k4 + i;
        As[k4 + i][m] = (gm < M && gk < K) ? A[(size_t)gm * lda + gk] : 0.0;
      }
    }
    {
      const int k = tid >> 4, n4 = (tid & 15) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gn = n0 + n4 + i, gk = k0 + k;
        Bs[k][n4 + i] = (gn < N && gk < K) ? B[(size_t)gk * ldb + gn] : 0.0;
      }
    }
    __syncthreads();
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

}  // namespace

int gemm_f64(hipStream_t stream, bool trans_a, int M, int N, int K, const double* A, int lda,
             const double* B, int ldb, double* C, int ldc, bool accumulate) {
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0 && A && B && C);
  HASTE_HIP_REQUIRE(lda >= (trans_a ? M : K) && ldb >= N && ldc >= N);
  const dim3 grid((unsigned)((N + DN - 1) / DN), (unsigned)((M + DM - 1) / DM));
  HASTE_HIP_REQUIRE(grid.y < 65536u);
  ScopedKernelTimer timer("gemm_f64", stream);
  if (trans_a)
    gemm_f64_kernel<true><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate);
  else
    gemm_f64_kernel<false><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_f64(int trans_a, int M, int N, int K, const double* A, int lda,
                                  const double* B, int ldb, double* C, int ldc, int accumulate,
                                  void* stream) {
  return haste_hip::gemm_f64(haste_hip::as_stream(stream), trans_a != 0, M, N, K, A, lda, B, ldb,
                             C, ldc, accumulate != 0);
}
