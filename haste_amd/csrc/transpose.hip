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

extern "C" int haste_hip_transpose_f64(int rows, int cols, const double* in, double* out,
                                       void* stream) {
  return haste_hip::transpose("transpose_f64", rows, cols, in, out, haste_hip::as_stream(stream));
}

// IEEE binary16 elements, passed as void*.
extern "C" int haste_hip_transpose_f16(int rows, int cols, const void* in, void* out, void* stream) {
  return haste_hip::transpose("transpose_f16", rows, cols, static_cast<const _Float16*>(in),
                              static_cast<_Float16*>(out), haste_hip::as_stream(stream));
}
