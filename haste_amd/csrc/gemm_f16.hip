// C[M,N] (+)= op(A)[M,K] * B[K,N] with IEEE half operands and result, accumulated in fp32 on
// the matrix cores (v_mfma_f32_32x32x8_f16): what the `half` instantiation of the reference's
// GRU gets from cublasHgemm (lib/blas.h:48-61, lib/gru_forward_gpu.cu.cc:373).
//
// Bound: MFMA, algorithmic flops 2*M*N*K.  A workgroup of four wavefronts owns a 64 x 64 tile
// of C, one 32 x 32 MFMA tile per wavefront.  Operand panels of 16 k go through LDS with k
// contiguous ([m][k], [n][k]), so a lane reads the four consecutive k of its row / column as
// one 8-byte load.  Lane layout of the instruction: a = A[i = lane%32][k = 4*(lane/32)..+3],
// b = B[k = 4*(lane/32)..+3][j = lane%32], d[e] = D[i = 8*(e/4) + 4*(lane/32) + e%4][j = lane%32].
// The contraction is never split: the result does not depend on the launch geometry.
#include "common.h"

namespace haste_hip {
namespace {

typedef _Float16 half_t;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int HM = 64, HN = 64, HK = 16;
constexpr int HPITCH = HK + 4;  // halves per row in LDS (40 bytes: 8-byte aligned groups of 4)

template <bool TRANS_A>
__global__ __launch_bounds__(256)
void gemm_f16_kernel(int M, int N, int K, const half_t* __restrict__ A, int lda,
                     const half_t* __restrict__ B, int ldb, half_t* __restrict__ C, int ldc,
                     int accumulate) {
  __shared__ __attribute__((aligned(8))) half_t As[HM][HPITCH];
  __shared__ __attribute__((aligned(8))) half_t Bs[HN][HPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * HM, n0 = blockIdx.x * HN;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  float16_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;

  for (int k0 = 0; k0 < K; k0 += HK) {
    if (TRANS_A) {
      const int k = tid >> 4, m4 = (tid & 15) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gm = m0 + m4 + i, gk = k0 + k;
        As[m4 + i][k] = (gm < M && gk < K) ? A[(size_t)gk * lda + gm] : half_t(0);
      }
    } else {
      const int m = tid >> 2, k4 = (tid & 3) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gm = m0 + m, gk = k0 + k4 + i;
        As[m][k4 + i] = (gm < M && gk < K) ? A[(size_t)gm * lda + gk] : half_t(0);
      }
    }
    {
      const int k = tid >> 4, n4 = (tid & 15) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int gn = n0 + n4 + i, gk = k0 + k;
        Bs[n4 + i][k] = (gn < N && gk < K) ? B[(size_t)gk * ldb + gn] : half_t(0);
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HK; kk += 8) {
      const int k = kk + 4 * (lane >> 5), o = lane & 31;
      const half4_t a = *reinterpret_cast<const half4_t*>(&As[wm + o][k]);
      const half4_t b = *reinterpret_cast<const half4_t*>(&Bs[wn + o][k]);
      acc = __builtin_amdgcn_mfma_f32_32x32x8f16(a, b, acc, 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int gm = m0 + wm + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
    const int gn = n0 + wn + (lane & 31);
    if (gm < M && gn < N) {
      half_t* p = C + (size_t)gm * ldc + gn;
      *p = (half_t)(accumulate ? (float)*p + acc[e] : acc[e]);
    }
  }
}

}  // namespace

int gemm_f16(hipStream_t stream, bool trans_a, int M, int N, int K, const void* A, int lda,
             const void* B, int ldb, void* C, int ldc, bool accumulate) {
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0 && A && B && C);
  HASTE_HIP_REQUIRE(lda >= (trans_a ? M : K) && ldb >= N && ldc >= N);
  const dim3 grid((unsigned)((N + HN - 1) / HN), (unsigned)((M + HM - 1) / HM));
  HASTE_HIP_REQUIRE(grid.y < 65536u);
  ScopedKernelTimer timer("gemm_f16", stream);
  const half_t* a = static_cast<const half_t*>(A);
  const half_t* b = static_cast<const half_t*>(B);
  half_t* c = static_cast<half_t*>(C);
  if (trans_a)
    gemm_f16_kernel<true><<<grid, dim3(256), 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc, accumulate);
  else
    gemm_f16_kernel<false><<<grid, dim3(256), 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc, accumulate);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_f16(int trans_a, int M, int N, int K, const void* A, int lda,
                                  const void* B, int ldb, void* C, int ldc, int accumulate,
                                  void* stream) {
  return haste_hip::gemm_f16(haste_hip::as_stream(stream), trans_a != 0, M, N, K, A, lda, B, ldb,
                             C, ldc, accumulate != 0);
}
