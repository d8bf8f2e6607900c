// haste::v0::lstm — drop-in for reference lib/haste/lstm.h:25-283.
#pragma once

#include "common.h"

namespace haste {
namespace v0 {
namespace lstm {

template<typename T>
class ForwardPass {
  public:
    // training: true if a backward pass will follow (v then returns the gate activations).
    // blas_handle is ignored.  stream: where all work is enqueued.
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

    // Never blocks: completion follows stream order.
    ~ForwardPass() {}

    // One step.  W[C,4H] R[H,4H] b[4H] x[N,C] h,c[N,H] -> h_out,c_out[N,H]; v[N,4H];
    // tmp_Rh is unused.  h_out/c_out may alias h/c.
    void Iterate(
        const hipStream_t& stream,
        const T* W,
        const T* R,
        const T* b,
        const T* x,
        const T* h,
        const T* c,
        T* h_out,
        T* c_out,
        T* v,
        T* tmp_Rh,
        const float zoneout_prob,
        const T* zoneout_mask) {
      // `stream` is where the caller produced the inputs and will consume the outputs;
      // the step itself runs on the stream given to the constructor.
      void* mine = detail::stream_arg(data_.stream);
      void* theirs = detail::stream_arg(stream);
      data_.status = haste_hip_stream_order(theirs, mine);
      if (data_.status != HASTE_HIP_OK) return;
      data_.status = detail::Abi<T>::lstm_forward_iterate(
          data_.training, data_.batch_size, data_.input_size, data_.hidden_size,
          W, R, b, x, h, c, h_out, c_out, v, tmp_Rh, zoneout_prob, zoneout_mask, mine);
      if (data_.status != HASTE_HIP_OK) return;
      data_.status = haste_hip_stream_order(mine, theirs);
    }

    // All steps.  W[C,4H] R[H,4H] b[4H] x[T,N,C]; h,c[T+1,N,H] with slot 0 preset by the
    // caller; v[T,N,4H]; tmp_Rh[N,4H] unused (may be null); zoneout_mask[T,N,H] or null.
    void Run(
        const int steps,
        const T* W,
        const T* R,
        const T* b,
        const T* x,
        T* h,
        T* c,
        T* v,
        T* tmp_Rh,
        const float zoneout_prob,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::lstm_forward(
          data_.training, steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W, R, b, x, h, c, v, tmp_Rh, zoneout_prob, zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    // HASTE_HIP_OK or the error code of the last Run()/Iterate().
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

    // One step, in reverse order of the forward steps.  Shapes as in Run with T = 1.
    void Iterate(
        const hipStream_t& stream,
        const T* W_t,
        const T* R_t,
        const T* b,
        const T* x_t,
        const T* h,
        const T* c,
        const T* c_new,
        const T* dh_new,
        const T* dc_new,
        T* dx,
        T* dW,
        T* dR,
        T* db,
        T* dh,
        T* dc,
        T* v,
        const T* zoneout_mask) {
      void* mine = detail::stream_arg(data_.stream);
      void* theirs = detail::stream_arg(stream);
      data_.status = haste_hip_stream_order(theirs, mine);
      if (data_.status != HASTE_HIP_OK) return;
      data_.status = detail::Abi<T>::lstm_backward_iterate(
          data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, R_t, b, x_t, h, c, c_new, dh_new, dc_new, dx, dW, dR, db, dh, dc, v, zoneout_mask,
          mine);
      if (data_.status != HASTE_HIP_OK) return;
      data_.status = haste_hip_stream_order(mine, theirs);
    }

    // W_t[4H,C] R_t[4H,H] b[4H] x_t[C,T,N] h,c[T+1,N,H] dh_new,dc_new[T+1,N,H];
    // dx[T,N,C] assigned; dW[C,4H] dR[H,4H] db[4H] accumulated into; dh,dc[N,H] zero on
    // entry, gradients of the initial state on return; v[T,N,4H] consumed.
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
        T* v,
        const T* zoneout_mask) {
      data_.status = detail::Abi<T>::lstm_backward(
          steps, data_.batch_size, data_.input_size, data_.hidden_size,
          W_t, R_t, b, x_t, h, c, dh_new, dc_new, dx, dW, dR, db, dh, dc, v, zoneout_mask,
          detail::stream_arg(data_.stream));
    }

    int last_status() const { return data_.status; }
    // After the caller has synchronized the stream: HASTE_HIP_OK, or the error of a kernel of
    // this stream that gave up a bounded wait (see haste_hip_stream_status).
    int stream_status() const { return haste_hip_stream_status(detail::stream_arg(data_.stream)); }

  private:
    detail::PassState data_;
};

}  // namespace lstm
}  // namespace v0
}  // namespace haste
