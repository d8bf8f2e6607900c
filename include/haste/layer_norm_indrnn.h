// haste::v0::layer_norm_indrnn — drop-in for reference lib/haste/layer_norm_indrnn.h:25-90.
#pragma once

#include "common.h"
#include "layer_norm.h"

namespace haste {
namespace v0 {
namespace layer_norm_indrnn {

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

    // As indrnn::ForwardPass::Run; act_Wx[T,N,H] receives x*W and workspace its norm
    // (layer_norm1: T*N rows of H, gamma and cache used).
    void Run(
        const int steps,
        const T* W,
        const T* u,
        const T* b,
        const T* x,
        T* h,
        T* workspace,
        T* act_Wx,
        layer_norm::ForwardPass<T>& layer_norm1,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::layer_norm_indrnn_forward(
          data_.training, steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W, u, b, x, h, workspace, act_Wx, layer_norm1.gamma(), layer_norm1.cache(),
          zoneout_prob, zoneout_mask, detail::stream_arg(data_.stream));
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

    // As indrnn::BackwardPass::Run; layer_norm1 (x = act_Wx) supplies gamma and dgamma.
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
        layer_norm::BackwardPass<T>& layer_norm1,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::layer_norm_indrnn_backward(
          steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, u, b, x_t, h, dh_new, dx, dW, du, db, dh, workspace,
          layer_norm1.x(), layer_norm1.gamma(), layer_norm1.dgamma(), zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

}  // namespace layer_norm_indrnn
}  // namespace v0
}  // namespace haste
