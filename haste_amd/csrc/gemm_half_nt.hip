// C[M,N] (+)= A[M,K] * Bt[N,K]^T with half operands, fp32 accumulation and an fp32 result, on
// the half matrix cores of gfx950 (v_mfma_f32_32x32x16_f16): the products of the half GRU
// (reference lib/gru_forward_gpu.cu.cc:340-348 with T = __half, lib/gru_backward_gpu.cu.cc:374-409),
// whose recurrences run in fp32 (gru_half.hip).  A may also be an fp32 tensor, rounded to half as
// it is staged (the gate gradients a backward recurrence has just written).
//
// Bound: MFMA (half peak 2.5 PFLOP/s), algorithmic flops 2*M*N*K.  Both operands have the
// contraction index contiguous -- what the instruction wants of a lane, eight consecutive k
// of one row -- so a tile goes from global memory to LDS to the operand registers in 16-byte
// pieces with no transposition anywhere; callers transpose the operand that is not laid out
// that way once (transpose_to_half).  128 x 128 tile per 256-thread workgroup, each wavefront a
// 64 x 64 quadrant as 2 x 2 MFMA tiles, 64 k per step through a double-buffered LDS stage.  A
// row of an LDS tile is 8 chunks of 8 halves; chunk c of row r sits at position c ^ ((r >> 1) & 7),
// which makes the 16 rows x one chunk that a quarter of a wavefront reads (and the 8 rows x 8
// chunks it writes) cover all 64 banks.  Lane layout of the instruction: a = A[i = lane%32]
// [k = 8*(lane/32) .. +7], b = Bt[j = lane%32][the same k], d[e] = D[i = 8*(e/4) + 4*(lane/32) +
// e%4][j = lane%32].
//
// A product with fewer tiles than three quarters of the CUs is cut along K into pieces (each at least 256 k)
// that park [M][N] partial results in the stream's scratch buffer; a second kernel adds them in
// index order.  The cut depends on the shape only: results are reproducible.
#include "common.h"

namespace haste_hip {
namespace {

typedef _Float16 half_t;
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));

constexpr int QM = 128, QN = 128, QK = 64;
constexpr int kTileChunks = 128 * 8;           // 16-byte chunks of one operand tile
constexpr unsigned int kNowhere = 0x7ffffff0u;  // an offset beyond any panel: the load returns zeros

__device__ __forceinline__ int lds_chunk(int row, int c) { return row * 8 + (c ^ ((row >> 1) & 7)); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t panel(const void* base, long long bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ uint4_t pack8(float4_t lo, float4_t hi) {
  half8_t h;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    h[e] = (half_t)lo[e];
    h[4 + e] = (half_t)hi[e];
  }
  return __builtin_bit_cast(uint4_t, h);
}

// One 128 x 128 tile over k in [k_begin, k_end); K % 8 == 0, rows 16-byte aligned.
template <bool A_FLOAT>
__global__ __launch_bounds__(256, 2)
void gemm_half_nt_kernel(int M, int N, int K, const void* __restrict__ A, int lda,
                         const half_t* __restrict__ Bt, int ldb, float* __restrict__ C, int ldc,
                         int accumulate, int tiles_n, int tiles, int k_per_piece,
                         float* __restrict__ partial) {
  __shared__ __attribute__((aligned(16))) uint4_t lds[2][2][kTileChunks];  // [buffer][A, B][chunk]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int piece = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const int m0 = (tile / tiles_n) * QM, n0 = (tile % tiles_n) * QN;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int k_begin = piece * k_per_piece;
  const int k_end = k_begin + k_per_piece < K ? k_begin + k_per_piece : K;

  const int rows_a = M - m0 < QM ? M - m0 : QM, rows_b = N - n0 < QN ? N - n0 : QN;
  constexpr int ASZ = A_FLOAT ? 4 : 2;
  const __amdgpu_buffer_rsrc_t pa =
      panel(static_cast<const char*>(A) + (size_t)m0 * lda * ASZ, ((long long)(rows_a - 1) * lda + K) * ASZ);
  const __amdgpu_buffer_rsrc_t pb = panel(Bt + (size_t)n0 * ldb, ((long long)(rows_b - 1) * ldb + K) * 2);

  // A thread's four chunks of each tile: chunk c = tid % 8 of rows tid / 8 + 32 * i.  Two
  // steps of operands are kept in flight in two register sets (a step's 512 cycles of MFMAs
  // are a fraction of a load's latency).  An fp32 A stays as loaded until it is parked:
  // converted at the request it would make the request wait for its own loads.
  const int c = tid & 7, r = tid >> 3;
  constexpr int AR = A_FLOAT ? 8 : 4;
  uint4_t ra[2][AR], rb[2][4];
  // A thread's offsets into the panels are fixed; the step enters as the loads' scalar offset
  // (which the range check ignores: chunks beyond the end of K, in the last step of a ragged K
  // only, get an offset beyond the panel instead).  The offsets pass through an empty asm
  // statement: left to see the select, the compiler puts every load behind a branch of its own
  // and a wait for all loads before it (8192^3: 565 -> 814 TFLOP/s without them).  Loads issued
  // straight from the fixed offsets, with nothing between them, are slower again (783): more
  // loads in flight are not what the step lacks.
  unsigned int va[4], vb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    va[i] = (unsigned int)(((size_t)(r + 32 * i) * lda + 8 * c) * ASZ);
    vb[i] = (unsigned int)(((size_t)(r + 32 * i) * ldb + 8 * c) * 2);
  }
  auto request = [&](auto set_c, int k0) {
    constexpr int SET = decltype(set_c)::value;
    const int sa = k0 * ASZ, sb = k0 * 2;
    const bool gone = k0 + 8 * c >= k_end;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      unsigned int oa = gone ? kNowhere : va[i], ob = gone ? kNowhere : vb[i];
      asm volatile("" : "+v"(oa), "+v"(ob));
      if constexpr (A_FLOAT) {
        ra[SET][2 * i] = __builtin_amdgcn_raw_buffer_load_b128(pa, oa, sa, 0);
        ra[SET][2 * i + 1] = __builtin_amdgcn_raw_buffer_load_b128(pa, oa + 16, sa, 0);
      } else {
        ra[SET][i] = __builtin_amdgcn_raw_buffer_load_b128(pa, oa, sa, 0);
      }
      rb[SET][i] = __builtin_amdgcn_raw_buffer_load_b128(pb, ob, sb, 0);
    }
  };
  auto park = [&](auto set_c) {
    constexpr int SET = decltype(set_c)::value;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (A_FLOAT)
        lds[SET][0][lds_chunk(r + 32 * i, c)] = pack8(__builtin_bit_cast(float4_t, ra[SET][2 * i]),
                                                      __builtin_bit_cast(float4_t, ra[SET][2 * i + 1]));
      else
        lds[SET][0][lds_chunk(r + 32 * i, c)] = ra[SET][i];
      lds[SET][1][lds_chunk(r + 32 * i, c)] = rb[SET][i];
    }
  };

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  auto compute = [&](int buf) {
#pragma unroll
    for (int ks = 0; ks < QK / 16; ++ks) {
      const int cc = 2 * ks + (lane >> 5), o = lane & 31;
      half8_t a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = __builtin_bit_cast(half8_t, lds[buf][0][lds_chunk(wm + 32 * i + o, cc)]);
        b[i] = __builtin_bit_cast(half8_t, lds[buf][1][lds_chunk(wn + 32 * i + o, cc)]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  };
  // step at k0 from LDS buffer / register set CUR: request the step after the next one into the
  // set this step was parked from, multiply, park the next step (its loads were issued a step ago)
  auto step = [&](auto cur_c, int k0) {
    constexpr int CUR = decltype(cur_c)::value;
    if (k0 + 2 * QK < k_end) request(cur_c, k0 + 2 * QK);
    compute(CUR);
    if (k0 + QK < k_end) park(std::integral_constant<int, 1 - CUR>{});
    __syncthreads();
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  if (k_begin < k_end) {
    request(Set0{}, k_begin);
    if (k_begin + QK < k_end) request(Set1{}, k_begin + QK);
    park(Set0{});
    __syncthreads();
    for (int k0 = k_begin; k0 < k_end; k0 += 2 * QK) {
      step(Set0{}, k0);
      if (k0 + QK < k_end) step(Set1{}, k0 + QK);
    }
  }

  float* out = C;
  int ld = ldc, add = accumulate;
  if (partial != nullptr) {  // piece z parks [M][N] at partial + z * M * N
    out = partial + (size_t)piece * M * N;
    ld = N;
    add = 0;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn + 32 * j + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm + 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (row < M && col < N) {
          float* p = out + (size_t)row * ld + col;
          *p = add ? *p + acc[i][j][e] : acc[i][j][e];
        }
      }
    }
}

// C (+)= the pieces of every element, added in index order.
__global__ __launch_bounds__(256)
void gemm_half_nt_reduce_kernel(int M, int N, int pieces, const float* __restrict__ part,
                                float* __restrict__ C, int ldc, int accumulate) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)M * N) return;
  float s = part[i];
  for (int z = 1; z < pieces; ++z) s += part[(size_t)z * M * N + i];
  float* out = C + (i / N) * ldc + i % N;
  *out = accumulate ? *out + s : s;
}

void plan_half_nt(int M, int N, int K, int* pieces, int* k_per_piece) {
  const long long tiles = (long long)((M + QM - 1) / QM) * ((N + QN - 1) / QN);
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  int s = 1;
  // three quarters of a workgroup per CU: at the shapes of a GRU step with N = 64, T = 100,
  // C = H = 512, two per CU costs dx (200 tiles) 47 us in three pieces against 32 us whole, and
  // dW, dR (48 tiles) as much in ten pieces as in four
  const long long want = (long long)cus * 3 / 4;
  if (tiles < want) {
    s = (int)((want + tiles - 1) / tiles);
    const int most = K / 256;
    s = s < most ? s : most;
    s = s > 1 ? s : 1;
  }
  int per = (K + s - 1) / s;
  per = (per + QK - 1) / QK * QK;
  *k_per_piece = per;
  *pieces = (K + per - 1) / per;
}

// in[rows, cols] (float or half) -> out[cols, rows] in half, 64 x 64 tiles through LDS.
template <typename T>
__global__ __launch_bounds__(256)
void transpose_to_half_kernel(int rows, int cols, const T* __restrict__ in, half_t* __restrict__ out,
                              int tiles_c) {
  __shared__ float tile[64][65];
  const int r0 = (blockIdx.x / tiles_c) * 64, c0 = (blockIdx.x % tiles_c) * 64;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int rr = r0 + ly + 4 * i, cc = c0 + lx;
    tile[ly + 4 * i][lx] = (rr < rows && cc < cols) ? (float)in[(size_t)rr * cols + cc] : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int cc = c0 + ly + 4 * i, rr = r0 + lx;
    if (cc < cols && rr < rows) out[(size_t)cc * rows + rr] = (half_t)tile[lx][ly + 4 * i];
  }
}

}  // namespace

bool gemm_half_nt_applies(bool a_float, int M, int N, int K, const void* A, int lda, const void* Bt,
                          int ldb) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0) return false;
  const int asz = a_float ? 4 : 2;
  if ((reinterpret_cast<uintptr_t>(A) & 15u) != 0 || (reinterpret_cast<uintptr_t>(Bt) & 15u) != 0) return false;
  if (((long long)lda * asz) % 16 != 0 || ((long long)ldb * 2) % 16 != 0) return false;
  // a workgroup addresses its panels (128 rows, all of K) with 32-bit offsets
  return ((long long)QM * lda + K) * asz < (1ll << 31) && ((long long)QN * ldb + K) * 2 < (1ll << 31) &&
         (long long)((M + QM - 1) / QM) * ((N + QN - 1) / QN) * 64 < (1ll << 30);
}

size_t gemm_half_nt_scratch_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int pieces, per;
  plan_half_nt(M, N, K, &pieces, &per);
  return pieces > 1 ? (size_t)pieces * M * N * sizeof(float) : 0;
}

// The partial results of a cut product lie `scratch_offset` bytes (a multiple of 16) into the
// stream's scratch buffer.
int gemm_half_nt(hipStream_t stream, bool a_float, int M, int N, int K, const void* A, int lda,
                 const void* Bt, int ldb, float* C, int ldc, bool accumulate, size_t scratch_offset) {
  HASTE_HIP_REQUIRE(A != nullptr && Bt != nullptr && C != nullptr && lda >= K && ldb >= K && ldc >= N);
  HASTE_HIP_REQUIRE(gemm_half_nt_applies(a_float, M, N, K, A, lda, Bt, ldb));
  int pieces, per;
  plan_half_nt(M, N, K, &pieces, &per);
  const int tiles_n = (N + QN - 1) / QN, tiles = ((M + QM - 1) / QM) * tiles_n;
  float* part = nullptr;
  if (pieces > 1) {
    Workspace ws;
    HASTE_HIP_PROPAGATE(get_workspace(stream, scratch_offset + (size_t)pieces * M * N * sizeof(float), &ws));
    part = reinterpret_cast<float*>(reinterpret_cast<char*>(ws.scratch) + scratch_offset);
  }
  const dim3 grid((unsigned)(tiles * pieces));
  const half_t* b = static_cast<const half_t*>(Bt);
  ScopedKernelTimer timer("gemm_half_nt", stream);
  if (a_float)
    gemm_half_nt_kernel<true><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, b, ldb, C, ldc, accumulate ? 1 : 0,
                                                              tiles_n, tiles, per, part);
  else
    gemm_half_nt_kernel<false><<<grid, dim3(256), 0, stream>>>(M, N, K, A, lda, b, ldb, C, ldc, accumulate ? 1 : 0,
                                                               tiles_n, tiles, per, part);
  HASTE_HIP_TRY(hipGetLastError());
  if (pieces > 1) {
    const size_t n = (size_t)M * N;
    gemm_half_nt_reduce_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(M, N, pieces, part, C, ldc,
                                                                                             accumulate ? 1 : 0);
    HASTE_HIP_TRY(hipGetLastError());
  }
  return HASTE_HIP_OK;
}

int transpose_to_half(hipStream_t stream, bool in_float, int rows, int cols, const void* in, void* out) {
  HASTE_HIP_REQUIRE(rows > 0 && cols > 0 && in != nullptr && out != nullptr);
  const long long tiles_c = (cols + 63) / 64, tiles_r = (rows + 63) / 64;
  HASTE_HIP_REQUIRE(tiles_c * tiles_r < (1ll << 31));
  const dim3 grid((unsigned)(tiles_c * tiles_r));
  if (in_float)
    transpose_to_half_kernel<float><<<grid, dim3(256), 0, stream>>>(rows, cols, static_cast<const float*>(in),
                                                                    static_cast<half_t*>(out), (int)tiles_c);
  else
    transpose_to_half_kernel<half_t><<<grid, dim3(256), 0, stream>>>(rows, cols, static_cast<const half_t*>(in),
                                                                     static_cast<half_t*>(out), (int)tiles_c);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

}  // namespace haste_hip

extern "C" int haste_hip_gemm_half_nt(int a_is_float, int M, int N, int K, const void* A, int lda,
                                      const void* Bt, int ldb, float* C, int ldc, int accumulate,
                                      void* stream) {
  using namespace haste_hip;
  HASTE_HIP_REQUIRE(M > 0 && N > 0 && K > 0 && A != nullptr && Bt != nullptr && C != nullptr);
  if (!gemm_half_nt_applies(a_is_float != 0, M, N, K, A, lda, Bt, ldb)) {
    set_error_text("gemm_half_nt: K and the leading dimensions must be multiples of 8 halves (16 bytes), the "
                   "operands 16-byte aligned, and 128 rows of an operand span less than 2 GiB");
    return HASTE_HIP_ERROR_UNSUPPORTED_SIZE;
  }
  return gemm_half_nt(as_stream(stream), a_is_float != 0, M, N, K, A, lda, Bt, ldb, C, ldc, accumulate != 0, 0);
}
