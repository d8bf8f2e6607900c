// out[cols, rows] = in[rows, cols]: the layout change the backward passes ask their
// callers for (x[T*N, C] -> x_t[C, T*N], W -> W_t, R -> R_t; reference
// frameworks/pytorch/lstm.py:84-86, and cublasSgeam in benchmarks/benchmark_lstm.cc:417-445).
//
// Bound: HBM.  Algorithmic bytes 2 * rows * cols * 4.  A workgroup moves a 64 x 64 tile
// through LDS: rows of the tile are read as 256-byte segments, the transposed rows are
// written as 256-byte segments; the 65-float row pitch keeps both LDS phases conflict free.
#include "common.h"

namespace haste_hip {
namespace {

constexpr int TT = 64;

template <typename T>
__global__ __launch_bounds__(256)
void transpose_kernel(int rows, int cols, const T* __restrict__ in, T* __restrict__ out,
                      int tiles_c) {
  __shared__ T tile[TT][TT + 1];
  const int tr = blockIdx.x / tiles_c, tc = blockIdx.x % tiles_c;
  const int r0 = tr * TT, c0 = tc * TT;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
  T v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = r0 + ly + 4 * i, c = c0 + lx;
    v[i] = (r < rows && c < cols) ? in[(size_t)r * cols + c] : T(0);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) tile[ly + 4 * i][lx] = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = c0 + ly + 4 * i, r = r0 + lx;
    if (c < cols && r < rows) out[(size_t)c * rows + r] = tile[lx][ly + 4 * i];
  }
}

// Up to three transposes in one launch: the tiles of the matrices are numbered one after the
// other.  The callers of a backward pass need x_t, W_t and R_t together, and at the sizes of W
// and R (a few MiB) a launch of its own costs more than the copy.
struct TransposeJob {
  int rows, cols, tiles_c, first_tile;
  const float* in;
  float* out;
};
struct TransposeJobs {
  TransposeJob job[3];
};

__global__ __launch_bounds__(256)
void transpose3_kernel(TransposeJobs jobs) {
  __shared__ float tile[TT][TT + 1];
  const int b = blockIdx.x;
  const int which = b >= jobs.job[2].first_tile ? 2 : (b >= jobs.job[1].first_tile ? 1 : 0);
  const TransposeJob j = jobs.job[which];
  const int local = b - j.first_tile;
  const int r0 = (local / j.tiles_c) * TT, c0 = (local % j.tiles_c) * TT;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
  float v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = r0 + ly + 4 * i, c = c0 + lx;
    v[i] = (r < j.rows && c < j.cols) ? j.in[(size_t)r * j.cols + c] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) tile[ly + 4 * i][lx] = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = c0 + ly + 4 * i, r = r0 + lx;
    if (c < j.cols && r < j.rows) j.out[(size_t)c * j.rows + r] = tile[lx][ly + 4 * i];
  }
}

template <typename T>
int transpose(const char* name, int rows, int cols, const T* in, T* out, hipStream_t stream) {
  HASTE_HIP_REQUIRE(rows > 0 && cols > 0 && in != nullptr && out != nullptr && in != out);
  const long long tiles_r = (rows + TT - 1) / TT;
  const long long tiles_c = (cols + TT - 1) / TT;
  HASTE_HIP_REQUIRE(tiles_r * tiles_c < (1ll << 31));
  ScopedKernelTimer timer(name, stream);
  transpose_kernel<T><<<dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, stream>>>(
      rows, cols, in, out, (int)tiles_c);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

}  // namespace
}  // namespace haste_hip

extern "C" int haste_hip_transpose_f32(int rows, int cols, const float* in, float* out,
                                       void* stream) {
  return haste_hip::transpose("transpose_f32", rows, cols, in, out, haste_hip::as_stream(stream));
}

extern "C" int haste_hip_transpose3_f32(int rows0, int cols0, const float* in0, float* out0,
                                        int rows1, int cols1, const float* in1, float* out1,
                                        int rows2, int cols2, const float* in2, float* out2,
                                        void* stream) {
  using namespace haste_hip;
  const int rows[3] = {rows0, rows1, rows2}, cols[3] = {cols0, cols1, cols2};
  const float* in[3] = {in0, in1, in2};
  float* out[3] = {out0, out1, out2};
  TransposeJobs jobs;
  long long tiles = 0;
  for (int i = 0; i < 3; ++i) {
    HASTE_HIP_REQUIRE(rows[i] > 0 && cols[i] > 0 && in[i] != nullptr && out[i] != nullptr &&
                      in[i] != out[i]);
    const long long tiles_r = (rows[i] + TT - 1) / TT, tiles_c = (cols[i] + TT - 1) / TT;
    jobs.job[i] = TransposeJob{rows[i], cols[i], (int)tiles_c, (int)tiles, in[i], out[i]};
    tiles += tiles_r * tiles_c;
    HASTE_HIP_REQUIRE(tiles < (1ll << 31));
  }
  ScopedKernelTimer timer("transpose3_f32", as_stream(stream));
  transpose3_kernel<<<dim3((unsigned)tiles), dim3(256), 0, as_stream(stream)>>>(jobs);
  HASTE_HIP_TRY(hipGetLastError());
  return HASTE_HIP_OK;
}

extern "C" int haste_hip_transpose_f64(int rows, int cols, const double* in, double* out,
                                       void* stream) {
  return haste_hip::transpose("transpose_f64", rows, cols, in, out, haste_hip::as_stream(stream));
}

// IEEE binary16 elements, passed as void*.
extern "C" int haste_hip_transpose_f16(int rows, int cols, const void* in, void* out, void* stream) {
  return haste_hip::transpose("transpose_f16", rows, cols, static_cast<const _Float16*>(in),
                              static_cast<_Float16*>(out), haste_hip::as_stream(stream));
}
