// haste::v0::layer_norm — drop-in for reference lib/haste/layer_norm.h:24-91.
#pragma once

#include <cassert>

#include "common.h"

namespace haste {
namespace v0 {
namespace layer_norm {

template<typename T>
class ForwardPass {
  public:
    // batch_size rows of hidden_size columns.  gamma[hidden_size]; beta[hidden_size] or
    // null (no shift); cache[batch_size,2] receives (mean, 1/std) per row.
    ForwardPass(
        const int batch_size,
        const int hidden_size,
        const T* gamma,
        const T* beta,
        T* cache)
        : batch_size_(batch_size), hidden_size_(hidden_size), gamma_(gamma), beta_(beta),
          cache_(cache), partial_(0), status_(HASTE_HIP_OK) {}

    // Normalises all rows: y = (x - mean) / std * gamma (+ beta).
    void Run(const hipStream_t& stream, const T* x, T* y) {
      RunPartial(stream, batch_size_, x, y);
    }

    // Normalises the next `minibatch` rows; consecutive calls walk forward through the
    // rows (and the cache) until batch_size rows have been consumed.
    void RunPartial(
        const hipStream_t& stream,
        const int minibatch,
        const T* x,
        T* y) {
      assert(partial_ + minibatch <= batch_size_);
      status_ = detail::Abi<T>::layer_norm_forward(
          minibatch, hidden_size_, gamma_, beta_, x, y, cache_ ? cache_ + partial_ * 2 : nullptr,
          detail::stream_arg(stream));
      partial_ += minibatch;
    }

    int last_status() const { return status_; }

    // Read access for the fused LayerNorm RNN passes.
    int batch_size() const { return batch_size_; }
    int hidden_size() const { return hidden_size_; }
    const T* gamma() const { return gamma_; }
    const T* beta() const { return beta_; }
    T* cache() const { return cache_; }

  private:
    const int batch_size_;
    const int hidden_size_;
    const T* gamma_;
    const T* beta_;
    T* cache_;
    int partial_;
    int status_;
};

template<typename T>
class BackwardPass {
  public:
    // x[batch_size,hidden_size] is the input the forward pass normalised; dgamma (and
    // dbeta unless null) are accumulated into; cache as written by the forward pass.
    BackwardPass(
        const int batch_size,
        const int hidden_size,
        const T* gamma,
        const T* beta,
        const T* x,
        T* dgamma,
        T* dbeta,
        T* cache)
        : batch_size_(batch_size), hidden_size_(hidden_size), gamma_(gamma), beta_(beta), x_(x),
          dgamma_(dgamma), dbeta_(dbeta), cache_(cache), partial_(batch_size),
          status_(HASTE_HIP_OK) {}

    // dx may alias dy.
    void Run(const hipStream_t& stream, const T* dy, T* dx) {
      RunPartial(stream, batch_size_, dy, dx);
    }

    // Processes the previous `minibatch` rows; consecutive calls walk backward from the
    // last row, mirroring the forward cursor.
    void RunPartial(
        const hipStream_t& stream,
        const int minibatch,
        const T* dy,
        T* dx) {
      assert(partial_ - minibatch >= 0);
      const int first = partial_ - minibatch;
      status_ = detail::Abi<T>::layer_norm_backward(
          minibatch, hidden_size_, gamma_, x_ + static_cast<long long>(first) * hidden_size_, dy,
          dx, dgamma_, (beta_ && dbeta_) ? dbeta_ : nullptr, cache_ ? cache_ + first * 2 : nullptr,
          detail::stream_arg(stream));
      partial_ = first;
    }

    int last_status() const { return status_; }

    int batch_size() const { return batch_size_; }
    int hidden_size() const { return hidden_size_; }
    const T* gamma() const { return gamma_; }
    const T* beta() const { return beta_; }
    const T* x() const { return x_; }
    T* dgamma() const { return dgamma_; }
    T* dbeta() const { return dbeta_; }
    T* cache() const { return cache_; }

  private:
    const int batch_size_;
    const int hidden_size_;
    const T* gamma_;
    const T* beta_;
    const T* x_;
    T* dgamma_;
    T* dbeta_;
    T* cache_;
    int partial_;
    int status_;
};

}  // namespace layer_norm
}  // namespace v0
}  // namespace haste
