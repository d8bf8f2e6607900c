// haste::v0::gru — drop-in for reference lib/haste/gru.h:25-228.
#pragma once

#include "common.h"

namespace haste {
namespace v0 {
namespace gru {

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

    // One step.  W[C,3H] R[H,3H] bx,br[3H] x[N,C] h[N,H] -> h_out[N,H]; v[N,4H];
    // tmp_Wx[N,3H]; tmp_Rh unused.
    void Iterate(
        const T* W,
        const T* R,
        const T* bx,
        const T* br,
        const T* x,
        const T* h,
        T* h_out,
        T* v,
        T* tmp_Wx,
        T* tmp_Rh,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::gru_forward_iterate(
          data_.training, data_.batch_size, data_.input_size, data_.hidden_size,
          W, R, bx, br, x, h, h_out, v, tmp_Wx, tmp_Rh, zoneout_prob, zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    // W[C,3H] R[H,3H] bx,br[3H] x[T,N,C]; h[T+1,N,H] with slot 0 preset; v[T,N,4H]
    // (z, r, g, Rh_g+br_g; may be null when not training); tmp_Wx[T,N,3H] receives x*W;
    // tmp_Rh unused (may be null); zoneout_mask[T,N,H] or null.
    void Run(
        const int steps,
        const T* W,
        const T* R,
        const T* bx,
        const T* br,
        const T* x,
        T* h,
        T* v,
        T* tmp_Wx,
        T* tmp_Rh,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::gru_forward(
          data_.training, steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W, R, bx, br, x, h, v, tmp_Wx, tmp_Rh, zoneout_prob, zoneout_mask,
          detail::stream_arg(data_.stream));
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

    void Iterate(
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
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::gru_backward_iterate(
          data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, R_t, bx, br, x_t, h, v, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq, zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    // W_t[3H,C] R_t[3H,H] x_t[C,T,N] h[T+1,N,H] v[T,N,4H] dh_new[T+1,N,H];
    // dx[T,N,C] assigned; dW,dR,dbx,dbr accumulated into; dh[N,H] in/out;
    // dp,dq[T,N,3H] scratch that receives the gate gradients.
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
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::gru_backward(
          steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, R_t, bx, br, x_t, h, v, dh_new, dx, dW, dR, dbx, dbr, dh, dp, dq, zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

}  // namespace gru
}  // namespace v0
}  // namespace haste
