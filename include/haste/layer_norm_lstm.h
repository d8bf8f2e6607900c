// haste::v0::layer_norm_lstm — drop-in for reference lib/haste/layer_norm_lstm.h:25-205.
#pragma once

#include "common.h"
#include "layer_norm.h"

namespace haste {
namespace v0 {
namespace layer_norm_lstm {

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

    // W[C,4H] R[H,4H] b[4H] x[T,N,C]; h,c[T+1,N,H] with slot 0 preset.
    // act_Wx[T,N,4H] receives x*W; act_Wx_norm[T,N,4H] its norm, then (training) the gate
    // activations; act_Rh[T,N,4H] receives h*R before its norm; act_c_norm[T,N,H] the
    // normalised cell state.  layer_norm1 spans T*N rows of 4H, layer_norm2 T*N rows of 4H
    // (one step at a time), layer_norm3 T*N rows of H; only their gamma/beta/cache are
    // used.  tmp_Rh is unused (may be null).
    void Run(
        const int steps,
        const T* W,
        const T* R,
        const T* b,
        const T* x,
        T* h,
        T* c,
        T* act_Wx,
        T* tmp_Rh,
        layer_norm::ForwardPass<T>& layer_norm1,
        T* act_Wx_norm,
        T* act_Rh,
        layer_norm::ForwardPass<T>& layer_norm2,
        layer_norm::ForwardPass<T>& layer_norm3,
        T* act_c_norm,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::layer_norm_lstm_forward(
          data_.training, steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W, R, b, x, h, c, act_Wx, tmp_Rh,
          layer_norm1.gamma(), layer_norm1.cache(), act_Wx_norm, act_Rh,
          layer_norm2.gamma(), layer_norm2.cache(),
          layer_norm3.gamma(), layer_norm3.beta(), layer_norm3.cache(), act_c_norm,
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

    // Shapes as in lstm::BackwardPass::Run.  act_Wx, act_Wx_norm, act_Rh are consumed.
    // layer_norm1 (x = act_Wx), layer_norm2 (x = act_Rh), layer_norm3 (x = c[1:]) supply
    // gamma, the gradient accumulators dgamma/dbeta and the forward caches.
    void Run(
        const int steps,
        const T* W_t,
        const T* R_t,
        const T* b,
        const T* x_t,
        const T* h,
        const T* c,
        const T* dh_new,
        const T* dc_new,
        T* dx,
        T* dW,
        T* dR,
        T* db,
        T* dh,
        T* dc,
        T* act_Wx,
        layer_norm::BackwardPass<T>& layer_norm1,
        T* act_Wx_norm,
        T* act_Rh,
        layer_norm::BackwardPass<T>& layer_norm2,
        layer_norm::BackwardPass<T>& layer_norm3,
        T* act_c_norm,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::layer_norm_lstm_backward(
          steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, R_t, b, x_t, h, c, dh_new, dc_new, dx, dW, dR, db, dh, dc,
          act_Wx, layer_norm1.gamma(), layer_norm1.dgamma(), act_Wx_norm, act_Rh,
          layer_norm2.gamma(), layer_norm2.dgamma(), layer_norm2.cache(),
          layer_norm3.gamma(), layer_norm3.beta(), layer_norm3.dgamma(), layer_norm3.dbeta(),
          layer_norm3.cache(), act_c_norm, zoneout_mask, detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

}  // namespace layer_norm_lstm
}  // namespace v0
}  // namespace haste
