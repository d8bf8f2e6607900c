// libhaste-compatible C++ API on top of libhaste_hip.so (MI355X / gfx950).
//
// Source-compatible with the reference's lib/haste.h:16-34: the same namespaces,
// class templates, constructor and Run() parameter lists, with the CUDA handle and
// stream types replaced by their HIP counterparts (hipblasHandle_t, hipStream_t).
//
// Conventions (reference lib/haste.h:18-26): T = time steps, N = batch size,
// C = input size, H = hidden size; tensors are row-major with the rightmost index
// fastest; every pointer is device memory and non-null unless stated otherwise.
//
// Differences a caller can observe:
//  * T = float and T = double for every class, T = __half for the GRU, as in the
//    reference (the persistent MFMA kernels are float; double and half run step-wise);
//  * all work is enqueued on the stream given to the constructor (0 = the null
//    stream) and completes in stream order; destructors never block;
//  * the BLAS handle is accepted and ignored (the library has its own MFMA GEMM);
//  * Run() reports failures through last_status() instead of silently ignoring them;
//    failures inside a kernel (a bounded wait that ran out) are reported by
//    stream_status(), to be called after synchronizing the stream;
//  * layer_norm::BackwardPass recomputes the row statistics, its cache is not read
//    except by the fused LayerNormLSTM/GRU kernels.
#pragma once

#include "haste/gru.h"
#include "haste/indrnn.h"
#include "haste/layer_norm.h"
#include "haste/layer_norm_gru.h"
#include "haste/layer_norm_indrnn.h"
#include "haste/layer_norm_lstm.h"
#include "haste/lstm.h"
