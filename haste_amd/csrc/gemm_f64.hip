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
typedef double double2_t __attribute__((ext_vector_type(2)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
constexpr unsigned int kNowhere = 0x7ffffff0u;  // an offset beyond any buffer resource's range: the load returns zeros

constexpr int DM = 64, DN = 64, DK = 32;
constexpr int DPITCH = 64 + 1;  // doubles per k row in LDS (odd: the transposing stores of A spread over the banks)

template <bool TRANS_A>
__global__ __launch_bounds__(256)
void gemm_f64_kernel(int M, int N, int K, const double* __restrict__ A, int lda,
                     const double* __restrict__ B, int ldb, double* __restrict__ C, int ldc,
                     int accumulate, int k_per_piece, double* __restrict__ part, int panels_ok) {
  __shared__ double As[DK][DPITCH];
  __shared__ double Bs[DK][DPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * DM, n0 = blockIdx.x * DN;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  // A workgroup whose columns (and, with A stored transposed, rows) are all inside the problem
  // and whose piece of K is whole panels loads through buffer resources, 16 bytes at a time and
  // without a branch: rows of A beyond M lie beyond the resource's range and read as zero.
  // Otherwise every element is loaded under its own bounds check (one branch each).
  const int piece_begin = blockIdx.z * k_per_piece;
  const int piece_end = piece_begin + k_per_piece < K ? piece_begin + k_per_piece : K;
  const bool fast = panels_ok != 0 && (piece_end - piece_begin) % DK == 0 && n0 + DN <= N &&
                    (!TRANS_A || m0 + DM <= M);
  const __amdgpu_buffer_rsrc_t pa = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<double*>(A), 0,
      fast ? (int)((TRANS_A ? (long long)(K - 1) * lda + M : (long long)(M - 1) * lda + K) * 8) : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t pb = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<double*>(B), 0, fast ? (int)(((long long)(K - 1) * ldb + N) * 8) : 0, 0x00020000);
  const unsigned int a_voff = TRANS_A ? (unsigned int)(((tid >> 3) * lda + m0 + (tid & 7) * 8) * 8)
                                      : (unsigned int)(((m0 + (tid >> 2)) * lda + (tid & 3) * 8) * 8);
  const unsigned int b_voff = (unsigned int)(((tid >> 3) * ldb + n0 + (tid & 7) * 8) * 8);
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
    if (fast) {
      const int sa = TRANS_A ? k0 * lda * 8 : k0 * 8, sb = k0 * ldb * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const double2_t va = __builtin_bit_cast(double2_t, __builtin_amdgcn_raw_buffer_load_b128(pa, a_voff + 16 * i, sa, 0));
        const double2_t vb = __builtin_bit_cast(double2_t, __builtin_amdgcn_raw_buffer_load_b128(pb, b_voff + 16 * i, sb, 0));
        ra[2 * i] = va[0];
        ra[2 * i + 1] = va[1];
        rb[2 * i] = vb[0];
        rb[2 * i + 1] = vb[1];
      }
      return;
    }
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
  const int k_begin = piece_begin;
  K = piece_end;
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

// ---- The product of one step of the step-wise regime: at most 64 rows (the batch), a few
// hundred to a few thousand columns and as long a contraction.  The tile kernel above gives
// it a handful of tiles whose workgroups walk their K range panel by panel, a load latency
// each; here everything a wavefront needs is requested at once and goes from memory straight
// into the MFMA operand registers -- no LDS, no barrier before the last sum.
//   * A workgroup takes 16 columns, all rows (RB blocks of 16) and k_per_wg of the contraction;
//     its four wavefronts take a quarter of that each and their blocks are added through LDS
//     in wavefront order; the workgroups of a column block leave [chunk][M][N] for the consumer
//     to add in chunk order.
//   * v_mfma_f64_16x16x4_f64 wants A[row = lane % 16][k = lane / 16] and B[k = lane / 16]
//     [col = lane % 16] of a lane.  Which four k one instruction contracts is free as long as
//     both operands agree: a lane loads A[row][k0 + 2 q], A[row][k0 + 2 q + 1] (q = lane / 16)
//     with one 16-byte load and the two B elements of the same k, and a stage of 8 k is two
//     instructions per row block, one on the even and one on the odd k.
//   * Rounds of four stages alternate between two register sets, the next round's loads in
//     flight while this one's MFMAs run.  Stages beyond a wavefront's range are loaded from an
//     offset beyond the buffer resources' range (zeros, no traffic), as are columns beyond N,
//     rows beyond M and B's k beyond K; A's k beyond K (the next row) is masked.
constexpr int kRoundStages = 4;   // stages of 8 k per round and wavefront

template <int RB>
__global__ __launch_bounds__(256)
void skinny_f64_kernel(int M, int N, int K, const double* __restrict__ A, int lda,
                       const double* __restrict__ B, int ldb, double* __restrict__ part, int k_per_wg) {
  __shared__ double red[3][RB][4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int kb = blockIdx.y * k_per_wg;
  const int ke = kb + k_per_wg < K ? kb + k_per_wg : K;
  const int kw = k_per_wg / 4;  // a multiple of 8
  const int kws = kb + wave * kw;
  const int kwe = kws + kw < ke ? kws + kw : ke;  // <= kws: a wavefront without work

  const __amdgpu_buffer_rsrc_t pa = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<double*>(A), 0, (int)(((long long)(M - 1) * lda + K) * 8), 0x00020000);
  const __amdgpu_buffer_rsrc_t pb = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<double*>(B), 0, (int)(((long long)(K - 1) * ldb + N) * 8), 0x00020000);
  unsigned int a_voff[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) a_voff[rb] = (unsigned int)(((16 * rb + c) * lda + 2 * q) * 8);
  const unsigned int b_voff = n0 + c < N ? (unsigned int)((2 * q * ldb + n0 + c) * 8) : kNowhere;
  const unsigned int b_next = (unsigned int)(ldb * 8);

  double2_t a[2][kRoundStages][RB];
  double b[2][kRoundStages][2];
  double4_t acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) acc[rb] = double4_t{0.0, 0.0, 0.0, 0.0};

  auto request = [&](auto set_c, int k_first) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int s = 0; s < kRoundStages; ++s) {
      const int k0 = k_first + 8 * s;
      const bool in = k0 < kwe;  // the same for a whole wavefront
      unsigned int ob = in ? b_voff : kNowhere, ob1 = in ? b_voff + b_next : kNowhere;
      asm volatile("" : "+v"(ob), "+v"(ob1));
      b[SET][s][0] = __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(pb, ob, k0 * ldb * 8, 0));
      b[SET][s][1] = __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(pb, ob1, k0 * ldb * 8, 0));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        unsigned int oa = in ? a_voff[rb] : kNowhere;
        asm volatile("" : "+v"(oa));
        a[SET][s][rb] = __builtin_bit_cast(double2_t, __builtin_amdgcn_raw_buffer_load_b128(pa, oa, k0 * 8, 0));
      }
    }
  };
  auto multiply = [&](auto set_c, int k_first) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int s = 0; s < kRoundStages; ++s) {
      const int left = K - (k_first + 8 * s + 2 * q);  // of this lane's two k, how many exist
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const double a0 = left > 0 ? a[SET][s][rb][0] : 0.0;
        acc[rb] = __builtin_amdgcn_mfma_f64_16x16x4f64(a0, b[SET][s][0], acc[rb], 0, 0, 0);
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const double a1 = left > 1 ? a[SET][s][rb][1] : 0.0;
        acc[rb] = __builtin_amdgcn_mfma_f64_16x16x4f64(a1, b[SET][s][1], acc[rb], 0, 0, 0);
      }
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  constexpr int kRound = 8 * kRoundStages;
  request(Set0{}, kws);
  for (int k = kws; k < kwe; k += 2 * kRound) {
    request(Set1{}, k + kRound);
    multiply(Set0{}, k);
    if (k + kRound >= kwe) break;
    request(Set0{}, k + 2 * kRound);
    multiply(Set1{}, k + kRound);
  }

  if (wave > 0) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave - 1][rb][e][lane] = acc[rb][e];
  }
  __syncthreads();
  if (wave > 0 || n0 + c >= N) return;
  double* out = part + (size_t)blockIdx.y * M * N + n0 + c;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int row = 16 * rb + 4 * e + q;
      const double sum = ((acc[rb][e] + red[0][rb][e][lane]) + red[1][rb][e][lane]) + red[2][rb][e][lane];
      if (row < M) out[(size_t)row * N] = sum;
    }
}

// k_per_wg: 256 (a wavefront then has two rounds, everything in flight at once) unless that
// leaves CUs without a workgroup (then 128), and never more than 8 chunks for the consumer.
void plan_skinny_f64(int M, int N, int K, int* chunks, int* k_per_wg) {
  (void)M;
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const long long col_blocks = (N + 15) / 16;
  int per = 256;
  if (col_blocks * ((K + 255) / 256) < cus) per = 128;
  const int least = ((K + 7) / 8 + 31) / 32 * 32;  // at most 8 chunks
  if (per < least) per = least;
  const int whole = (K + 31) / 32 * 32;
  if (per > whole) per = whole;
  *k_per_wg = per;
  *chunks = (K + per - 1) / per;
}

// The operands fit the 32-bit byte offsets of a buffer resource.
int panels_fit(bool trans_a, int M, int N, int K, int lda, int ldb) {
  const long long a = trans_a ? (long long)K * lda + M : (long long)M * lda + K, b = (long long)K * ldb + N;
  return a * 8 < (1ll << 31) - 64 && b * 8 < (1ll << 31) - 64 ? 1 : 0;
}

bool skinny_f64_applies(int M, int N, int K, int lda, int ldb) {
  return M <= 64 && ((long long)M * lda + K) * 8 < (1ll << 31) - 64 && ((long long)K * ldb + N) * 8 < (1ll << 31) - 64 &&
         (long long)ldb * 8 < (1ll << 28);
}

}  // namespace

size_t gemm_f64_scratch_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int pieces, per;
  plan_f64(M, N, K, &pieces, &per);
  size_t tiled = pieces > 1 ? (size_t)pieces * M * N * sizeof(double) : 0;
  if (M <= 64) {
    plan_skinny_f64(M, N, K, &pieces, &per);
    const size_t skinny = (size_t)pieces * M * N * sizeof(double);
    tiled = tiled > skinny ? tiled : skinny;
  }
  return tiled;
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
    gemm_f64_kernel<true><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, per, part,
                                                          panels_fit(true, M, N, K, lda, ldb));
  else
    gemm_f64_kernel<false><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, per, part,
                                                           panels_fit(false, M, N, K, lda, ldb));
  HASTE_HIP_TRY(hipGetLastError());
  if (pieces > 1) {
    const size_t n = (size_t)M * N;
    gemm_f64_reduce_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(M, N, pieces, part, C, ldc,
                                                                                         accumulate ? 1 : 0);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

// The product left as chunks of its contraction, [chunk][M][N] in the stream's scratch buffer,
// for a consumer that adds them itself in chunk order (one launch less per step than adding
// them here); *chunks == 0, and nothing launched, when the product is not cut.  Valid until the
// next product on the stream.
int gemm_f64_chunks(hipStream_t stream, int M, int N, int K, const double* A, int lda, const double* B,
                    int ldb, size_t scratch_offset, const double** partial, int* chunks) {
  *chunks = 0;
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0 && A && B);
  HASTE_HIP_REQUIRE(lda >= K && ldb >= N);
  int pieces, per;
  const bool skinny = skinny_f64_applies(M, N, K, lda, ldb);
  if (skinny) plan_skinny_f64(M, N, K, &pieces, &per);
  else plan_f64(M, N, K, &pieces, &per);
  if (!skinny && pieces <= 1) return HASTE_HIP_OK;
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + (size_t)pieces * M * N * sizeof(double), &ws));
  double* part = reinterpret_cast<double*>(reinterpret_cast<char*>(ws.scratch) + scratch_offset);
  if (skinny) {
    const dim3 grid((unsigned)((N + 15) / 16), (unsigned)pieces);
    ScopedKernelTimer timer("gemm_f64_skinny", stream);
    if (M <= 16) skinny_f64_kernel<1><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, part, per);
    else if (M <= 32) skinny_f64_kernel<2><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, part, per);
    else skinny_f64_kernel<4><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, part, per);
    HASTE_HIP_TRY(hipGetLastError());
  } else {
    const dim3 grid((unsigned)((N + DN - 1) / DN), (unsigned)((M + DM - 1) / DM), (unsigned)pieces);
    HASTE_HIP_REQUIRE(grid.y < 65536u);
    ScopedKernelTimer timer("gemm_f64", stream);
    gemm_f64_kernel<false><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, nullptr, 0, 0, per, part,
                                                           panels_fit(false, M, N, K, lda, ldb));
    HASTE_HIP_TRY(hipGetLastError());
  }
  *partial = part;
  *chunks = pieces;
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_f64(int trans_a, int M, int N, int K, const double* A, int lda,
                                  const double* B, int ldb, double* C, int ldc, int accumulate,
                                  void* stream) {
  return haste_hip::gemm_f64(haste_hip::as_stream(stream), trans_a != 0, M, N, K, A, lda, B, ldb,
                             C, ldc, accumulate != 0, 0);
}
