// Shared declarations of the header-only adapters in include/haste/*.h.
#pragma once

#include <hip/hip_runtime_api.h>
#include <hip/hip_fp16.h>

#if __has_include(<hipblas/hipblas.h>)
#include <hipblas/hipblas.h>
#else
typedef void* hipblasHandle_t;
#endif

#include "../haste_hip.h"

namespace haste {
namespace v0 {
namespace detail {

// State every RNN pass object keeps: the problem size, the stream all of its work
// goes to, and the status of its last Run().
struct PassState {
  bool training;
  int batch_size;
  int input_size;
  int hidden_size;
  hipStream_t stream;
  int status;
};

inline void* stream_arg(hipStream_t s) { return reinterpret_cast<void*>(s); }

// The C entry points behind a class instantiated for T.  As in the reference, only the
// types the library is built for can be used (float and double, e.g.
// lib/lstm_forward_gpu.cu.cc:368-369, and __half for the GRU, lib/gru_forward_gpu.cu.cc:373);
// any other T fails to compile here.
template<typename T> struct Abi;
template<> struct Abi<float> {
  static constexpr auto lstm_forward = &haste_hip_lstm_forward_f32;
  static constexpr auto lstm_backward = &haste_hip_lstm_backward_f32;
  static constexpr auto lstm_forward_iterate = &haste_hip_lstm_forward_iterate_f32;
  static constexpr auto lstm_backward_iterate = &haste_hip_lstm_backward_iterate_f32;
  static constexpr auto gru_forward = &haste_hip_gru_forward_f32;
  static constexpr auto gru_backward = &haste_hip_gru_backward_f32;
  static constexpr auto gru_forward_iterate = &haste_hip_gru_forward_iterate_f32;
  static constexpr auto gru_backward_iterate = &haste_hip_gru_backward_iterate_f32;
  static constexpr auto layer_norm_forward = &haste_hip_layer_norm_forward_f32;
  static constexpr auto layer_norm_backward = &haste_hip_layer_norm_backward_f32;
  static constexpr auto layer_norm_lstm_forward = &haste_hip_layer_norm_lstm_forward_f32;
  static constexpr auto layer_norm_lstm_backward = &haste_hip_layer_norm_lstm_backward_f32;
  static constexpr auto layer_norm_gru_forward = &haste_hip_layer_norm_gru_forward_f32;
  static constexpr auto layer_norm_gru_backward = &haste_hip_layer_norm_gru_backward_f32;
  static constexpr auto indrnn_forward = &haste_hip_indrnn_forward_f32;
  static constexpr auto indrnn_backward = &haste_hip_indrnn_backward_f32;
  static constexpr auto layer_norm_indrnn_forward = &haste_hip_layer_norm_indrnn_forward_f32;
  static constexpr auto layer_norm_indrnn_backward = &haste_hip_layer_norm_indrnn_backward_f32;
};
template<> struct Abi<double> {
  static constexpr auto lstm_forward = &haste_hip_lstm_forward_f64;
  static constexpr auto lstm_backward = &haste_hip_lstm_backward_f64;
  static constexpr auto lstm_forward_iterate = &haste_hip_lstm_forward_iterate_f64;
  static constexpr auto lstm_backward_iterate = &haste_hip_lstm_backward_iterate_f64;
  static constexpr auto gru_forward = &haste_hip_gru_forward_f64;
  static constexpr auto gru_backward = &haste_hip_gru_backward_f64;
  static constexpr auto gru_forward_iterate = &haste_hip_gru_forward_iterate_f64;
  static constexpr auto gru_backward_iterate = &haste_hip_gru_backward_iterate_f64;
  static constexpr auto layer_norm_forward = &haste_hip_layer_norm_forward_f64;
  static constexpr auto layer_norm_backward = &haste_hip_layer_norm_backward_f64;
  static constexpr auto layer_norm_lstm_forward = &haste_hip_layer_norm_lstm_forward_f64;
  static constexpr auto layer_norm_lstm_backward = &haste_hip_layer_norm_lstm_backward_f64;
  static constexpr auto layer_norm_gru_forward = &haste_hip_layer_norm_gru_forward_f64;
  static constexpr auto layer_norm_gru_backward = &haste_hip_layer_norm_gru_backward_f64;
  static constexpr auto indrnn_forward = &haste_hip_indrnn_forward_f64;
  static constexpr auto indrnn_backward = &haste_hip_indrnn_backward_f64;
  static constexpr auto layer_norm_indrnn_forward = &haste_hip_layer_norm_indrnn_forward_f64;
  static constexpr auto layer_norm_indrnn_backward = &haste_hip_layer_norm_indrnn_backward_f64;
};

template<> struct Abi<__half> {
  static constexpr auto gru_forward = &haste_hip_gru_forward_f16;
  static constexpr auto gru_backward = &haste_hip_gru_backward_f16;
  static constexpr auto gru_forward_iterate = &haste_hip_gru_forward_iterate_f16;
  static constexpr auto gru_backward_iterate = &haste_hip_gru_backward_iterate_f16;
};

}  // namespace detail
}  // namespace v0
}  // namespace haste
