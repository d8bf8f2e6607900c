// haste::v0::layer_norm_gru — drop-in for reference lib/haste/layer_norm_gru.h:25-204.
#pragma once

#include "common.h"
#include "layer_norm.h"

namespace haste {
namespace v0 {
namespace layer_norm_gru {

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

    // W[C,3H] R[H,3H] bx,br[3H] x[T,N,C]; h[T+1,N,H]; v[T,N,4H] (null when not training);
    // act_Wx[T,N,3H] receives x*W, tmp_Wx_norm[T,N,3H] its norm, act_Rh[T,N,3H] h*R before
    // its norm; tmp_Rh_norm is unused (may be null).
    void Run(
        const int steps,
        const T* W,
        const T* R,
        const T* bx,
        const T* br,
        const T* x,
        T* h,
        T* v,
        T* act_Wx,
        layer_norm::ForwardPass<T>& layer_norm1,
        T* tmp_Wx_norm,
        T* act_Rh,
        layer_norm::ForwardPass<T>& layer_norm2,
        T* tmp_Rh_norm,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::layer_norm_gru_forward(
          data_.training, steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W, R, bx, br, x, h, v, act_Wx, layer_norm1.gamma(), layer_norm1.cache(), tmp_Wx_norm,
          act_Rh, layer_norm2.gamma(), layer_norm2.cache(), tmp_Rh_norm,
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

    // Shapes as in gru::BackwardPass::Run.  layer_norm1 (x = act_Wx) and layer_norm2
    // (x = act_Rh) supply gamma, dgamma, the saved pre-norm activations and the caches.
    // dp, dq end up holding the gradients w.r.t. the pre-norm activations.
    void Run(
        const int steps,
        const T* W_t,
        const T* R_t,
        const T* bx,
        const T* br,
        const T* x_t,
        const T* h,
        const T* v,
        const T* dh_new,
        T* dx,
        T* dW,
        T* dR,
        T* dbx,
        T* dbr,
        T* dh,
        T* dp,
        T* dq,
        layer_norm::BackwardPass<T>& layer_norm1,
        layer_norm::BackwardPass<T>& layer_norm2,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::layer_norm_gru_backward(
          steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, R_t, bx, br, x_t, h, v, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq,
          layer_norm1.x(), layer_norm1.gamma(), layer_norm1.dgamma(),
          layer_norm2.x(), layer_norm2.gamma(), layer_norm2.dgamma(), layer_norm2.cache(),
          zoneout_mask, detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

}  // namespace layer_norm_gru
}  // namespace v0
}  // namespace haste
