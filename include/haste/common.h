// Shared declarations of the header-only adapters in include/haste/*.h.
#pragma once

#include <hip/hip_runtime_api.h>

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

}  // namespace detail
}  // namespace v0
}  // namespace haste
