// C[M,N] (+)= A[M,K] * B[K,N] for M <= 128: the recurrent product of one step (h_t * R,
// delta_t * R^T) when R is streamed from HBM every step (stepwise.hip) and the batch is
// small.  Replaces the per-step cublasSgemm of the reference
// (lib/lstm_forward_gpu.cu.cc:232-242, lib/lstm_backward_gpu.cu.cc:281-291).
//
// Bound: HBM.  Algorithmic bytes 4*K*N (B is read exactly once; A and C are M rows).  The
// 128 x 128 tile kernel of gemm.hip gives such a product a handful of tiles and pushes B
// through LDS; here B goes from HBM straight into the MFMA operand registers: a lane loads 16
// bytes (four consecutive columns of one k row), a wavefront 1 KiB of whole 256- or 512-byte
// row segments, and the four components feed four MFMAs whose output columns are therefore
// interleaved by 4 -- which is exactly a 16-byte store per lane in the epilogue.  M <= 16
// uses v_mfma_f32_16x16x4_f32 (4 k rows x 64 columns per load), M <= 32 v_mfma_f32_32x32x2_f32
// (2 k rows x 128 columns); the matrix cores then need 128 / 256 cycles per KiB of B, below
// the 330 cycles a CU's share of 8 TB/s allows.  M <= 64 carries two blocks of 32 rows on the
// same B registers: bound by the matrix cores, but still without LDS traffic or tile pieces.  The four wavefronts of a workgroup split the
// workgroup's k range and add their tiles through LDS in wavefront order; workgroups split K
// further (enough of them to keep every CU's memory pipeline full); their tiles are added in
// chunk order by a second small kernel, or by the consumer of the product itself
// (gemm_f32_skinny_chunks): deterministic, no atomics.
#include "common.h"

namespace haste_hip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

template <int MT> struct SkinnyShape;
template <> struct SkinnyShape<16> {
  static constexpr int kStep = 4, kCols = 64;
  typedef float4_t Acc;
  static __device__ __forceinline__ Acc mfma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  // row of accumulator element e held by `lane`
  static __device__ __forceinline__ int row(int lane, int e) { return 4 * (lane >> 4) + e; }
  static constexpr int kAccElems = 4;
};
template <> struct SkinnyShape<32> {
  static constexpr int kStep = 2, kCols = 128;
  typedef float16_t Acc;
  static __device__ __forceinline__ Acc mfma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int lane, int e) {
    return 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
  }
  static constexpr int kAccElems = 16;
};

constexpr int kUnroll = 8;  // load instructions in flight per wavefront and operand

// MT: rows of one MFMA tile (16 or 32); RB: row blocks of MT rows a wavefront carries (the
// B registers are shared between them), so a workgroup covers MT*RB rows of A.
template <int MT, int RB>
__global__ __launch_bounds__(256)
void skinny_kernel(int M, int N, int K, const float* __restrict__ A, int lda,
                   const float* __restrict__ B, int ldb, float* __restrict__ C, int ldc,
                   int accumulate, int k_per_wg, float* __restrict__ partial) {
  typedef SkinnyShape<MT> S;
  typedef typename S::Acc Acc;
  __shared__ __attribute__((aligned(16))) float red[3][MT][S::kCols];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * S::kCols;
  const int chunk = blockIdx.y;
  const int kb_wg = chunk * k_per_wg;
  const int ke_wg = kb_wg + k_per_wg < K ? kb_wg + k_per_wg : K;
  const int k_per_wave = ((k_per_wg + 3) / 4 + 7) / 8 * 8;
  const int kb = kb_wg + wave * k_per_wave;
  const int ke = kb + k_per_wave < ke_wg ? kb + k_per_wave : ke_wg;

  const int i = lane % MT, kq = lane / MT;
  const int m0 = blockIdx.z * (MT * RB);  // more than MT*RB rows: one grid layer per group of rows
  const int col = n0 + 4 * (lane % MT);
  const bool col_ok = col < N;
  // Out-of-range lanes load from a valid address and drop the value.
  bool row_ok[RB];
  const float* ap[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    row_ok[rb] = m0 + rb * MT + i < M;
    ap[rb] = A + (size_t)(row_ok[rb] ? m0 + rb * MT + i : 0) * lda;
  }
  const float* bp = B + (col_ok ? col : 0);

  Acc acc[RB][4];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int e = 0; e < S::kAccElems; ++e) acc[rb][c][e] = 0.f;

  // A batch is kUnroll MFMA steps.  Which k a lane contributes at which step is free as long
  // as both operands agree: lane group kq takes the run of kUnroll consecutive k starting at
  // k + kUnroll*kq, one per step, so its A values are two 16-byte loads of consecutive k and
  // every B load instruction still covers whole row segments.
  for (int k = kb; k < ke; k += S::kStep * kUnroll) {
    const int k_mine = k + kUnroll * kq;
    float4_t b[kUnroll];
    float4_t a4[RB][kUnroll / 4];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < kUnroll / 4; ++j) {
        const int g = k_mine + 4 * j;
        const bool ok = g < ke;
        const float4_t av = *reinterpret_cast<const float4_t*>(ap[rb] + (ok ? g : kb));
        a4[rb][j] = (ok && row_ok[rb]) ? av : float4_t{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int r = k_mine + u;
      const bool ok = r < ke;
      const float4_t bv = *reinterpret_cast<const float4_t*>(bp + (size_t)(ok ? r : kb) * ldb);
      b[u] = (ok && col_ok) ? bv : float4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const float a = a4[rb][u / 4][u % 4];
        acc[rb][0] = S::mfma(a, b[u].x, acc[rb][0]);
        acc[rb][1] = S::mfma(a, b[u].y, acc[rb][1]);
        acc[rb][2] = S::mfma(a, b[u].z, acc[rb][2]);
        acc[rb][3] = S::mfma(a, b[u].w, acc[rb][3]);
      }
  }

  // Element e of the four accumulators = four consecutive columns of one row.  The
  // wavefronts' tiles are added through LDS, one row block at a time.
  const int cslot = 4 * (lane % MT);
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    if (rb > 0) __syncthreads();  // wavefront 0 has read the previous block's tiles
    if (wave > 0) {
#pragma unroll
      for (int e = 0; e < S::kAccElems; ++e)
        *reinterpret_cast<float4_t*>(&red[wave - 1][S::row(lane, e)][cslot]) =
            float4_t{acc[rb][0][e], acc[rb][1][e], acc[rb][2][e], acc[rb][3][e]};
    }
    __syncthreads();
    if (wave == 0 && col_ok) {
#pragma unroll
      for (int e = 0; e < S::kAccElems; ++e) {
        const int in_block = S::row(lane, e);
        const int row = m0 + rb * MT + in_block;
        if (row >= M) continue;
        float4_t s = float4_t{acc[rb][0][e], acc[rb][1][e], acc[rb][2][e], acc[rb][3][e]};
        s += *reinterpret_cast<const float4_t*>(&red[0][in_block][cslot]);
        s += *reinterpret_cast<const float4_t*>(&red[1][in_block][cslot]);
        s += *reinterpret_cast<const float4_t*>(&red[2][in_block][cslot]);
        if (partial != nullptr) {
          *reinterpret_cast<float4_t*>(partial + ((size_t)chunk * M + row) * N + col) = s;
        } else {
          float4_t* o = reinterpret_cast<float4_t*>(C + (size_t)row * ldc + col);
          *o = accumulate ? (*o + s) : s;
        }
      }
    }
  }
}

// C (+)= sum over chunks of partial[chunk][M][N], chunks added in index order.
__global__ __launch_bounds__(256)
void skinny_reduce_kernel(int M, int N, int chunks, const float* __restrict__ partial,
                          float* __restrict__ C, int ldc, int accumulate) {
  const size_t q = blockIdx.x * (size_t)256 + threadIdx.x;  // index of a group of 4 columns
  const size_t per_row = (size_t)N / 4;
  if (q >= per_row * M) return;
  const size_t row = q / per_row, col = (q % per_row) * 4;
  float4_t s = float4_t{0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < chunks; ++k)
    s += *reinterpret_cast<const float4_t*>(partial + ((size_t)k * M + row) * N + col);
  float4_t* o = reinterpret_cast<float4_t*>(C + row * ldc + col);
  *o = accumulate ? (*o + s) : s;
}

struct SkinnyPlan {
  int mt, rb, row_groups, col_blocks, chunks, k_per_wg;  // MFMA tile rows, row blocks, grid layers
};

SkinnyPlan plan_skinny(int M, int N, int K) {
  SkinnyPlan p;
  p.mt = M <= 16 ? 16 : 32;
  p.rb = M <= 32 ? 1 : 2;
  p.row_groups = (M + p.mt * p.rb - 1) / (p.mt * p.rb);
  const int cols = 4 * p.mt;
  p.col_blocks = (N + cols - 1) / cols;
  // Enough workgroups for about three per CU (measured: four is no faster at 268 MB of B and
  // slower when B fits the memory-side cache), a workgroup keeping at least 128 of K.
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  int chunks = (3 * cus + p.col_blocks * p.row_groups - 1) / (p.col_blocks * p.row_groups);
  const int most = (K + 127) / 128;
  if (chunks > most) chunks = most;
  if (chunks < 1) chunks = 1;
  p.k_per_wg = (K + chunks - 1) / chunks;
  p.k_per_wg = (p.k_per_wg + 31) / 32 * 32;  // four wavefronts x a multiple of 8
  p.chunks = (K + p.k_per_wg - 1) / p.k_per_wg;
  return p;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

void launch_skinny(const SkinnyPlan& p, dim3 grid, hipStream_t stream, int M, int N, int K,
                   const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                   int accumulate, float* partial) {
  if (p.mt == 16)
    skinny_kernel<16, 1><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, p.k_per_wg, partial);
  else if (p.rb == 1)
    skinny_kernel<32, 1><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, p.k_per_wg, partial);
  else
    skinny_kernel<32, 2><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, B, ldb, C, ldc, accumulate, p.k_per_wg, partial);
}

}  // namespace

bool gemm_f32_skinny_shape(bool trans_a, int M, int N, int K) {
  if (trans_a || M > 128 || N % 4 != 0 || K % 4 != 0 || K < 64 || (long long)K * N < (1ll << 16)) return false;
  // 33..128 rows (65 and up as two grid layers of 64) are bound by the matrix cores; measured
  // against the tile kernel they win while B is small (the tile kernel then has too few tiles and pays for its pieces): up to 6 Mi
  // elements, e.g. the reverse step of H = 1024 (4096 x 1024).
  return M <= 32 || (long long)K * N <= 6ll * (1 << 20);
}

size_t gemm_f32_skinny_scratch_bytes(int M, int N, int K) {
  return (size_t)plan_skinny(M, N, K).chunks * M * N * sizeof(float);
}

bool gemm_f32_skinny_applies(bool trans_a, int M, int N, int K, const float* A, int lda,
                             const float* B, int ldb, const float* C, int ldc) {
  return gemm_f32_skinny_shape(trans_a, M, N, K) && lda % 4 == 0 && ldb % 4 == 0 && ldc % 4 == 0 &&
         aligned16(A) && aligned16(B) && aligned16(C);
}

// The streaming kernel alone: leaves `*chunks` partial results [chunk][M][N] at `*partial`
// (in the stream's scratch buffer, valid until the next product on the stream) for a consumer
// that adds them itself, in chunk order.
int gemm_f32_skinny_chunks(hipStream_t stream, int M, int N, int K, const float* A, int lda,
                           const float* B, int ldb, size_t scratch_offset, const float** partial,
                           int* chunks) {
  const SkinnyPlan p = plan_skinny(M, N, K);
  Workspace ws;
  HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + (size_t)p.chunks * M * N * sizeof(float), &ws));
  float* part = ws.scratch + scratch_offset / sizeof(float);
  const dim3 grid((unsigned)p.col_blocks, (unsigned)p.chunks, (unsigned)p.row_groups);
  ScopedKernelTimer timer("gemm_f32_skinny", stream);
  launch_skinny(p, grid, stream, M, N, K, A, lda, B, ldb, nullptr, 0, 0, part);
  HASTE_HIP_TRY(hipGetLastError());
  *partial = part;
  *chunks = p.chunks;
  return HASTE_HIP_OK;
}

int gemm_f32_skinny(hipStream_t stream, int M, int N, int K, const float* A, int lda,
                    const float* B, int ldb, float* C, int ldc, bool accumulate,
                    size_t scratch_offset) {
  const SkinnyPlan p = plan_skinny(M, N, K);
  float* partial = nullptr;
  if (p.chunks > 1) {
    Workspace ws;
    HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + gemm_f32_skinny_scratch_bytes(M, N, K), &ws));
    partial = ws.scratch + scratch_offset / sizeof(float);
  }
  const dim3 grid((unsigned)p.col_blocks, (unsigned)p.chunks, (unsigned)p.row_groups);
  {
    ScopedKernelTimer timer("gemm_f32_skinny", stream);
    launch_skinny(p, grid, stream, M, N, K, A, lda, B, ldb, C, ldc, accumulate ? 1 : 0, partial);
    HASTE_HIP_TRY(hipGetLastError());
  }
  if (partial != nullptr) {
    ScopedKernelTimer timer("gemm_f32_skinny_reduce", stream);
    const size_t groups = (size_t)M * (N / 4);
    skinny_reduce_kernel<<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, stream>>>(
        M, N, p.chunks, partial, C, ldc, accumulate ? 1 : 0);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

}  // namespace haste_hip
