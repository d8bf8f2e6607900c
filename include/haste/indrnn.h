// haste::v0::indrnn — drop-in for reference lib/haste/indrnn.h:25-87.
#pragma once

#include "common.h"

namespace haste {
namespace v0 {
namespace indrnn {

template<typename T>
class ForwardPass {
  public:
    ForwardPass(
        const bool training,
        const int batch_size,
        const int input_size,
        const int hidden_size,
        const hipblasHandle_t& blas_handle,
        const hipStream_t& stream = 0)
        : data_{training, batch_size, input_size, hidden_size, stream, HASTE_HIP_OK} {
      (void)blas_handle;
    }

    ~ForwardPass() {}

    // W[C,H] u[H] b[H] x[T,N,C]; h[T+1,N,H] with slot 0 preset; workspace[T,N,H] receives x*W.
    void Run(
        const int steps,
        const T* W,
        const T* u,
        const T* b,
        const T* x,
        T* h,
        T* workspace,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::indrnn_forward(
          data_.training, steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W, u, b, x, h, workspace, zoneout_prob, zoneout_mask, detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

template<typename T>
class BackwardPass {
  public:
    BackwardPass(
        const int batch_size,
        const int input_size,
        const int hidden_size,
        const hipblasHandle_t& blas_handle,
        const hipStream_t& stream = 0)
        : data_{true, batch_size, input_size, hidden_size, stream, HASTE_HIP_OK} {
      (void)blas_handle;
    }

    ~BackwardPass() {}

    // W_t[H,C] u[H] b[H] x_t[C,T,N] h[T+1,N,H] dh_new[T+1,N,H]; dx[T,N,C] and dW[C,H]
    // assigned; du[H], db[H] accumulated into; dh[N,H] in/out; workspace[T,N,H] scratch.
    void Run(
        const int steps,
        const T* W_t,
        const T* u,
        const T* b,
        const T* x_t,
        const T* h,
        const T* dh_new,
        T* dx,
        T* dW,
        T* du,
        T* db,
        T* dh,
        T* workspace,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::indrnn_backward(
          steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, u, b, x_t, h, dh_new, dx, dW, du, db, dh, workspace, zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

}  // namespace indrnn
}  // namespace v0
}  // namespace haste
