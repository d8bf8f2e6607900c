/* C ABI of libhaste_hip.so: the MI355X (gfx950) implementation of the fused-RNN
 * hot path behind the libhaste C++ API.
 *
 * Every entry point takes plain ints, floats and device pointers; `stream` is a
 * hipStream_t passed as void* (NULL = the null stream).  All work is enqueued on
 * that stream and the call returns without waiting for it.  All tensors are
 * caller-allocated device memory, row-major, rightmost index fastest
 * (T steps, N batch, C input size, H hidden size), exactly as the reference
 * documents them in lib/haste.h:18-26.  Return value: 0 on success, otherwise one
 * of the HASTE_HIP_ERROR_* codes; nothing is launched when an argument check fails.
 *
 * Each *_forward / *_backward entry point is what the corresponding
 * haste::v0::<cell>::ForwardPass<float>::Run / BackwardPass<float>::Run binds to
 * (see include/haste/ *.h for the header-only C++ adapters).
 */
#ifndef HASTE_HIP_H_
#define HASTE_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HASTE_HIP_OK 0
#define HASTE_HIP_ERROR_INVALID_ARGUMENT 1  /* null pointer, non-positive dimension */
#define HASTE_HIP_ERROR_UNSUPPORTED_SIZE 2  /* recurrent slice does not fit on chip / in the grid */
#define HASTE_HIP_ERROR_RUNTIME 3           /* a HIP runtime call failed */
#define HASTE_HIP_ERROR_STEP_BARRIER 4      /* an earlier persistent kernel gave up waiting at its step barrier */

/* Library version as major*10000 + minor*100 + patch. */
int haste_hip_version(void);

/* Human-readable text for a return code. */
const char* haste_hip_error_string(int code);

/* Text of the last HIP runtime error seen by the calling thread ("" if none). */
const char* haste_hip_last_runtime_error(void);

/* Largest hidden size whose recurrent weight slice the persistent kernels can keep
 * on chip (in LDS, or in LDS and registers) in both directions for `gates` gate blocks
 * (4 LSTM, 3 GRU) and `batch_size` rows on the current device; 0 if none.  Larger hidden sizes are accepted as well: the cells then
 * stream the recurrent matrix from HBM every step (one GEMM plus row-wise norm and pointwise
 * kernels per step, as the reference does). */
int haste_hip_max_hidden_size(int gates, int batch_size);

/* How Run would lay the persistent recurrences of a cell with `gates` gate blocks (4 LSTM, 3 GRU)
 * out for this batch and hidden size on a device of `cus` compute units in `xcds` XCDs that take
 * workgroups evenly (cus == 0: the current device as the library found it; xcds == 0: no
 * placement by XCD).  Touches no device when cus > 0.  plan[0..7] describes the forward
 * recurrence, plan[8..15] the backward one: {found (0: the cell streams the recurrent matrix
 * from HBM every step instead; the rest are then 0), batch rows per tile, hidden units per
 * workgroup, 16-column tiles of the weight slice, column workgroups, batch tiles, groups of 16
 * contraction rows per wavefront kept in registers, such groups in a wavefront's whole share}.
 * No counterpart in the reference (its kernels have one geometry); for capacity planning and
 * for tests of the geometry search. */
int haste_hip_plan_tiles(int cus, int xcds, int gates, int batch_size, int hidden_size, int* plan);

/* Drops this thread's cached per-stream workspaces on the current device (frees
 * device memory; the caller must have synchronized the streams that used them). */
int haste_hip_release_workspaces(void);

/* Status of the persistent kernels launched on `stream` so far; call it after synchronizing
 * the stream.  HASTE_HIP_OK, or HASTE_HIP_ERROR_STEP_BARRIER when one of them gave up (a
 * bounded wait for another workgroup ran out, or an XCD hosted more workgroups than the launch
 * had been promised): the outputs of that launch, and of library launches that were already
 * queued behind it on the device, are invalid, although the calls that enqueued them returned
 * HASTE_HIP_OK (they return before the kernels run).  Reporting clears the condition (the
 * control block is wiped in stream order; after an XCD placement failure later launches use
 * the placement-independent exchange path) and haste_hip_last_runtime_error() says which of
 * the two it was.  Without this call the condition is reported by the next entry point
 * called on the stream.  The reference has no error reporting to replace (its Run methods
 * return void). */
int haste_hip_stream_status(void* stream);

/* Caller-owned scratch memory.  By default the library keeps one workspace per (device,
 * stream) that it allocates on first use and grows on demand (hipMalloc, and on growth a
 * stream synchronization and hipFree, inside Run).  A caller who wants every byte in its
 * own allocator, or who records calls into a HIP graph, lends the stream a buffer instead:
 * `memory` is device memory, 256-byte aligned, of `bytes` bytes, which stays valid and is
 * used by nothing else until it is replaced or taken back (memory == NULL: back to a
 * library-owned workspace); the call synchronizes `stream` if the stream has a workspace in
 * use.  With a lent buffer no entry point allocates, frees or synchronizes; a call that needs
 * more than `bytes` returns HASTE_HIP_ERROR_UNSUPPORTED_SIZE (the size in
 * haste_hip_last_runtime_error()) before it launches anything that uses the workspace.
 * The reference's contract being honoured: every buffer, tmp_Rh included, is the caller's
 * (lib/haste/lstm.h:98-117).
 *
 * haste_hip_workspace_bytes: an upper bound of what any cell, direction and scalar type
 * (but for the half GRU, below) needs for (T, N, C, H) on the current device (for the stand-alone layer norm: T = 1,
 * N = rows, C = H = dim): 64 MiB for the partial tiles of split GEMMs plus terms in N*H,
 * H*H and T*N.  haste_hip_workspace_high_water: what the calls made on `stream` so far
 * have actually needed (after a rehearsal of the same calls, the exact size to lend). */
size_t haste_hip_workspace_bytes(int time_steps, int batch_size, int input_size, int hidden_size);

/* The same bound for haste_hip_gru_{forward,forward_dropconnect,backward}_f16, which over more
 * than one step stage fp32 copies of their tensors in the workspace (4 bytes per element of
 * every tensor of the call) in front of what the fp32 passes they run ask for.  No counterpart
 * in the reference. */
size_t haste_hip_gru_half_workspace_bytes(int time_steps, int batch_size, int input_size,
                                          int hidden_size);
int haste_hip_set_workspace(void* stream, void* memory, size_t bytes);
int haste_hip_workspace_high_water(void* stream, size_t* bytes);

/* Makes everything enqueued on `then` after this call wait for everything enqueued on
 * `first` before it (an event recorded on `first`, waited for on `then`); no-op when both
 * name the same stream.  Counterpart of the event hand-over around the reference's
 * lstm::ForwardPass::Iterate(stream, ...) (lib/lstm_forward_gpu.cu.cc:171-175,203-206). */
int haste_hip_stream_order(void* first, void* then);

/* Per-kernel timing, off by default.  While enabled, every kernel the library
 * launches is bracketed by a pair of HIP events recorded on the stream the kernel
 * runs on.  haste_hip_profile_read waits for those events and returns, for the kernel
 * called `name` ("gemm_f32", "lstm_forward_recurrence", "lstm_backward_recurrence", ...),
 * the summed duration in milliseconds and the number of launches since the last reset (a
 * launch that fuses two products, dW and dR of the LSTM backward pass, counts as two).
 * The reference has only cudaEvent timers in its benchmarks
 * (benchmarks/benchmark_lstm.cc:49-63); this is their in-library counterpart. */
int haste_hip_profile_enable(int on);
int haste_hip_profile_reset(void);
int haste_hip_profile_read(const char* name, double* total_ms, int* launches);

/* C[M,N] = op(A)[M,K] * B[K,N] (+ C if accumulate != 0); fp32 MFMA.
 * trans_a == 0: A is [M,K] with leading dimension lda; trans_a != 0: A is stored
 * as [K,M] with leading dimension lda.  Replaces the cuBLAS calls the reference
 * makes through lib/blas.h:48-61. */
int haste_hip_gemm_f32(int trans_a, int M, int N, int K,
                       const float* A, int lda, const float* B, int ldb,
                       float* C, int ldc, int accumulate, void* stream);

/* out[cols,rows] = in[rows,cols] (in != out).  The backward entry points take x, W and R
 * transposed by the caller (x_t[C,T*N], W_t, R_t), as the reference's do
 * (lib/haste/lstm.h:230-247); its benchmark produces them with cublasSgeam inside the timed
 * region (benchmarks/benchmark_lstm.cc:417-445).  This is that helper. */
int haste_hip_transpose_f32(int rows, int cols, const float* in, float* out, void* stream);

/* The same for three matrices in one launch: a backward pass needs x_t, W_t and R_t together
 * (lib/haste/lstm.h:230-247), and W and R are small enough that a launch each costs more than
 * the copy (the reference's benchmark issues one cublasSgeam per matrix,
 * benchmarks/benchmark_lstm.cc:417-445). */
int haste_hip_transpose3_f32(int rows0, int cols0, const float* in0, float* out0,
                             int rows1, int cols1, const float* in1, float* out1,
                             int rows2, int cols2, const float* in2, float* out2, void* stream);

/* ---- LSTM ----------------------------------------------------------------
 * reference lib/haste/lstm.h:118-129 (ForwardPass::Run), lib/lstm_forward_gpu.cu.cc:313-366.
 * W[C,4H] R[H,4H] b[4H] x[T,N,C] h,c[T+1,N,H] (slot 0 preset by the caller)
 * v[T,N,4H] (training: activations i,g,f,o on return) tmp_Rh[N,4H] (unused scratch,
 * may be NULL) zoneout_mask[T,N,H] or NULL. */
int haste_hip_lstm_forward_f32(int training, int steps, int batch_size, int input_size,
                               int hidden_size,
                               const float* W, const float* R, const float* b, const float* x,
                               float* h, float* c, float* v, float* tmp_Rh,
                               float zoneout_prob, const float* zoneout_mask, void* stream);

/* Same, with DropConnect fused into the load of R: the recurrence uses
 * R[i] * dropconnect_mask[i] * dropconnect_scale.  The reference applies this in
 * Python before calling the op (frameworks/pytorch/lstm.py:252); mask NULL = plain R. */
int haste_hip_lstm_forward_dropconnect_f32(int training, int steps, int batch_size,
                                           int input_size, int hidden_size,
                                           const float* W, const float* R, const float* b,
                                           const float* x, float* h, float* c, float* v,
                                           float zoneout_prob, const float* zoneout_mask,
                                           const float* dropconnect_mask, float dropconnect_scale,
                                           void* stream);

/* reference lib/haste/lstm.h:248-265 (BackwardPass::Run), lib/lstm_backward_gpu.cu.cc:319-405.
 * W_t[4H,C] R_t[4H,H] b[4H] (unused) x_t[C,T,N] h,c[T+1,N,H] dh_new,dc_new[T+1,N,H]
 * dx[T,N,C] (assigned) dW[C,4H] dR[H,4H] db[4H] (accumulated into) dh,dc[N,H] (in/out,
 * zero on entry, d h0 / d c0 on return) v[T,N,4H] (in: activations, out: gate gradients)
 * zoneout_mask[T,N,H] or NULL. */
int haste_hip_lstm_backward_f32(int steps, int batch_size, int input_size, int hidden_size,
                                const float* W_t, const float* R_t, const float* b,
                                const float* x_t, const float* h, const float* c,
                                const float* dh_new, const float* dc_new,
                                float* dx, float* dW, float* dR, float* db,
                                float* dh, float* dc, float* v,
                                const float* zoneout_mask, void* stream);

/* Single-step variants: reference lib/haste/lstm.h:73-86 (ForwardPass::Iterate,
 * lib/lstm_forward_gpu.cu.cc:140-208) and lib/haste/lstm.h:201-219 (BackwardPass::Iterate,
 * lib/lstm_backward_gpu.cu.cc:143-244).  Shapes are those of the all-steps entry points
 * with T = 1, except that the states before and after the step are separate [N,H]
 * buffers: x[N,C] h,c[N,H] -> h_out,c_out[N,H] (h_out may alias h, c_out may alias c),
 * v[N,4H], zoneout_mask[N,H] or NULL.  Backward: x_t[C,N], h,c = states before the step,
 * c_new = cell state after it, dh_new,dc_new[N,H] upstream gradients of the states the
 * step produced, dx[N,C] assigned, dW,dR,db accumulated, dh,dc[N,H] in/out, v in/out. */
int haste_hip_lstm_forward_iterate_f32(int training, int batch_size, int input_size,
                                       int hidden_size,
                                       const float* W, const float* R, const float* b,
                                       const float* x, const float* h, const float* c,
                                       float* h_out, float* c_out, float* v, float* tmp_Rh,
                                       float zoneout_prob, const float* zoneout_mask,
                                       void* stream);
int haste_hip_lstm_backward_iterate_f32(int batch_size, int input_size, int hidden_size,
                                        const float* W_t, const float* R_t, const float* b,
                                        const float* x_t, const float* h, const float* c,
                                        const float* c_new, const float* dh_new,
                                        const float* dc_new, float* dx, float* dW, float* dR,
                                        float* db, float* dh, float* dc, float* v,
                                        const float* zoneout_mask, void* stream);

/* ---- GRU -------------------------------------------------------------------
 * reference lib/haste/gru.h:86-98, lib/gru_forward_gpu.cu.cc:314-371.
 * W[C,3H] R[H,3H] bx,br[3H] x[T,N,C] h[T+1,N,H] v[T,N,4H] = (z,r,g,Rh_g+br_g)
 * (training only; may be NULL otherwise) tmp_Wx[T,N,3H] tmp_Rh[N,3H] (unused, may be NULL). */
int haste_hip_gru_forward_f32(int training, int steps, int batch_size, int input_size,
                              int hidden_size,
                              const float* W, const float* R, const float* bx, const float* br,
                              const float* x, float* h, float* v, float* tmp_Wx, float* tmp_Rh,
                              float zoneout_prob, const float* zoneout_mask, void* stream);

/* GRU forward with DropConnect fused into the load of R (frameworks/pytorch/gru.py:257). */
int haste_hip_gru_forward_dropconnect_f32(int training, int steps, int batch_size,
                                          int input_size, int hidden_size,
                                          const float* W, const float* R, const float* bx,
                                          const float* br, const float* x, float* h, float* v,
                                          float* tmp_Wx, float zoneout_prob,
                                          const float* zoneout_mask,
                                          const float* dropconnect_mask, float dropconnect_scale,
                                          void* stream);

/* reference lib/haste/gru.h:191-209, lib/gru_backward_gpu.cu.cc:321-409.
 * dp,dq[T,N,3H] are outputs/scratch; dbx,dbr,dW,dR accumulated; dx assigned; dh in/out. */
int haste_hip_gru_backward_f32(int steps, int batch_size, int input_size, int hidden_size,
                               const float* W_t, const float* R_t, const float* bx,
                               const float* br, const float* x_t, const float* h, const float* v,
                               const float* dh_new, float* dx, float* dW, float* dR,
                               float* dbx, float* dbr, float* dh, float* dp, float* dq,
                               const float* zoneout_mask, void* stream);

/* Single-step variants: reference lib/haste/gru.h:72-84 (ForwardPass::Iterate,
 * lib/gru_forward_gpu.cu.cc:159-212) and lib/haste/gru.h:172-189 (BackwardPass::Iterate,
 * lib/gru_backward_gpu.cu.cc:167-250).  x[N,C] h[N,H] -> h_out[N,H] (may alias h),
 * v[N,4H], tmp_Wx[N,3H].  Backward: x_t[C,N], h = state before the step, v[N,4H],
 * dh_new[N,H] upstream gradient of the state the step produced, dp,dq[N,3H]. */
int haste_hip_gru_forward_iterate_f32(int training, int batch_size, int input_size,
                                      int hidden_size,
                                      const float* W, const float* R, const float* bx,
                                      const float* br, const float* x, const float* h,
                                      float* h_out, float* v, float* tmp_Wx, float* tmp_Rh,
                                      float zoneout_prob, const float* zoneout_mask,
                                      void* stream);
int haste_hip_gru_backward_iterate_f32(int batch_size, int input_size, int hidden_size,
                                       const float* W_t, const float* R_t, const float* bx,
                                       const float* br, const float* x_t, const float* h,
                                       const float* v, const float* dh_new, float* dx, float* dW,
                                       float* dR, float* dbx, float* dbr, float* dh, float* dp,
                                       float* dq, const float* zoneout_mask, void* stream);

/* ---- Layer norm --------------------------------------------------------------
 * reference lib/haste/layer_norm.h:30-49, lib/layer_norm_forward_gpu.cu.cc:96-150.
 * y = (x-mean)*invstd*gamma (+beta if non-NULL), eps 1e-5, biased variance;
 * cache[rows,2] = (mean, invstd) (may be NULL). */
int haste_hip_layer_norm_forward_f32(int rows, int dim, const float* gamma, const float* beta,
                                     const float* x, float* y, float* cache, void* stream);

/* reference lib/haste/layer_norm.h:63-79, lib/layer_norm_backward_gpu.cu.cc:101-165.
 * dx may alias dy.  dgamma (and dbeta if non-NULL) are accumulated into.  Statistics
 * are recomputed from x; `cache` is accepted for signature parity and not read. */
int haste_hip_layer_norm_backward_f32(int rows, int dim, const float* gamma, const float* x,
                                      const float* dy, float* dx, float* dgamma, float* dbeta,
                                      const float* cache, void* stream);

/* The same computation as haste_hip_layer_norm_backward_f32 for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  The workgroups' partial column sums go
 * to a fixed 16 MiB array inside the library's device image (one copy per GPU, held until the
 * process ends) instead of the stream's workspace, and the call makes no hipMalloc / hipFree
 * and creates no events.  Limits: dim <= 4096 (1024 when dim is not a multiple of 4 or a
 * pointer is not 16-byte aligned) and min(ceil(rows/4), 2 x compute units) x 2 x dim <= 4 Mi
 * floats; beyond them HASTE_HIP_ERROR_UNSUPPORTED_SIZE with the reason in
 * haste_hip_last_runtime_error().  All calls on one GPU share the array: calls that overlap
 * on one GPU (different streams, or threads) race; calls on one stream are ordered. */
int haste_hip_layer_norm_backward_noalloc_f32(int rows, int dim, const float* gamma,
                                              const float* x, const float* dy, float* dx,
                                              float* dgamma, float* dbeta, const float* cache,
                                              void* stream);

/* ---- LayerNorm LSTM ----------------------------------------------------------
 * reference lib/haste/layer_norm_lstm.h:75-92, lib/layer_norm_lstm_forward_gpu.cu.cc:276-340.
 * The three layer_norm::ForwardPass objects of the reference are passed flattened:
 * ln1 (on xW, rows T*N, dim 4H): gamma1[4H], cache1[T*N,2];
 * ln2 (on hR per step):          gamma2[4H], cache2[T*N,2];
 * ln3 (on c per step, dim H):    gamma_h[H], beta_h[H], cache3[T*N,2]. */
int haste_hip_layer_norm_lstm_forward_f32(int training, int steps, int batch_size,
                                          int input_size, int hidden_size,
                                          const float* W, const float* R, const float* b,
                                          const float* x, float* h, float* c,
                                          float* act_Wx, float* tmp_Rh,
                                          const float* gamma1, float* cache1,
                                          float* act_Wx_norm, float* act_Rh,
                                          const float* gamma2, float* cache2,
                                          const float* gamma_h, const float* beta_h, float* cache3,
                                          float* act_c_norm,
                                          float zoneout_prob, const float* zoneout_mask,
                                          void* stream);

/* reference lib/haste/layer_norm_lstm.h:160-183, lib/layer_norm_lstm_backward_gpu.cu.cc:255-352.
 * act_Wx, act_Wx_norm, act_Rh are consumed (overwritten with gradients); act_c_norm is
 * read.  dgamma1, dgamma2 [4H], dgamma_h, dbeta_h [H] are accumulated into.
 * cache2, cache3 [T*N,2] are the (mean, 1/std) caches the forward pass wrote for the
 * per-step norms (the reference's layer_norm2 / layer_norm3 objects hold them). */
int haste_hip_layer_norm_lstm_backward_f32(int steps, int batch_size, int input_size,
                                           int hidden_size,
                                           const float* W_t, const float* R_t, const float* b,
                                           const float* x_t, const float* h, const float* c,
                                           const float* dh_new, const float* dc_new,
                                           float* dx, float* dW, float* dR, float* db,
                                           float* dh, float* dc,
                                           float* act_Wx, const float* gamma1, float* dgamma1,
                                           float* act_Wx_norm, float* act_Rh,
                                           const float* gamma2, float* dgamma2,
                                           const float* cache2,
                                           const float* gamma_h, const float* beta_h,
                                           float* dgamma_h, float* dbeta_h,
                                           const float* cache3,
                                           float* act_c_norm,
                                           const float* zoneout_mask, void* stream);

/* ---- LayerNorm GRU -----------------------------------------------------------
 * reference lib/haste/layer_norm_gru.h:72-88, lib/layer_norm_gru_forward_gpu.cu.cc:242-305. */
int haste_hip_layer_norm_gru_forward_f32(int training, int steps, int batch_size,
                                         int input_size, int hidden_size,
                                         const float* W, const float* R, const float* bx,
                                         const float* br, const float* x, float* h, float* v,
                                         float* act_Wx, const float* gamma1, float* cache1,
                                         float* tmp_Wx_norm, float* act_Rh,
                                         const float* gamma2, float* cache2, float* tmp_Rh_norm,
                                         float zoneout_prob, const float* zoneout_mask,
                                         void* stream);

/* reference lib/haste/layer_norm_gru.h:164-184, lib/layer_norm_gru_backward_gpu.cu.cc:219-310.
 * act_Wx / act_Rh are the pre-norm activations saved by the forward pass (the `x` of the
 * reference's layer_norm1 / layer_norm2 BackwardPass objects). dp, dq are overwritten
 * with the gradients w.r.t. the pre-norm activations, as in the reference.
 * cache2 [T*N,2] is the (mean, 1/std) cache the forward pass wrote for the per-step norm. */
int haste_hip_layer_norm_gru_backward_f32(int steps, int batch_size, int input_size,
                                          int hidden_size,
                                          const float* W_t, const float* R_t, const float* bx,
                                          const float* br, const float* x_t, const float* h,
                                          const float* v, const float* dh_new,
                                          float* dx, float* dW, float* dR, float* dbx, float* dbr,
                                          float* dh, float* dp, float* dq,
                                          const float* act_Wx, const float* gamma1, float* dgamma1,
                                          const float* act_Rh, const float* gamma2, float* dgamma2,
                                          const float* cache2,
                                          const float* zoneout_mask, void* stream);

/* ---- IndRNN --------------------------------------------------------------------
 * reference lib/haste/indrnn.h:37-47, lib/indrnn_forward_gpu.cu.cc:114-210.
 * W[C,H] u[H] b[H] x[T,N,C] h[T+1,N,H] workspace[T,N,H]. */
int haste_hip_indrnn_forward_f32(int training, int steps, int batch_size, int input_size,
                                 int hidden_size,
                                 const float* W, const float* u, const float* b, const float* x,
                                 float* h, float* workspace,
                                 float zoneout_prob, const float* zoneout_mask, void* stream);

/* reference lib/haste/indrnn.h:66-80, lib/indrnn_backward_gpu.cu.cc:122-207.
 * dW[C,H] and dx are assigned; du, db accumulated; dh in/out; workspace[T,N,H] out. */
int haste_hip_indrnn_backward_f32(int steps, int batch_size, int input_size, int hidden_size,
                                  const float* W_t, const float* u, const float* b,
                                  const float* x_t, const float* h, const float* dh_new,
                                  float* dx, float* dW, float* du, float* db, float* dh,
                                  float* workspace, const float* zoneout_mask, void* stream);

/* ---- LayerNorm IndRNN ----------------------------------------------------------
 * reference lib/haste/layer_norm_indrnn.h:37-49, lib/layer_norm_indrnn_forward_gpu.cu.cc:114-213. */
int haste_hip_layer_norm_indrnn_forward_f32(int training, int steps, int batch_size,
                                            int input_size, int hidden_size,
                                            const float* W, const float* u, const float* b,
                                            const float* x, float* h, float* workspace,
                                            float* act_Wx, const float* gamma1, float* cache1,
                                            float zoneout_prob, const float* zoneout_mask,
                                            void* stream);

/* reference lib/haste/layer_norm_indrnn.h:68-83, lib/layer_norm_indrnn_backward_gpu.cu.cc:122-209. */
int haste_hip_layer_norm_indrnn_backward_f32(int steps, int batch_size, int input_size,
                                             int hidden_size,
                                             const float* W_t, const float* u, const float* b,
                                             const float* x_t, const float* h,
                                             const float* dh_new,
                                             float* dx, float* dW, float* du, float* db, float* dh,
                                             float* workspace,
                                             const float* act_Wx, const float* gamma1,
                                             float* dgamma1,
                                             const float* zoneout_mask, void* stream);

/* ---- double precision -------------------------------------------------------------
 * The reference instantiates every class for double as well (e.g.
 * lib/lstm_forward_gpu.cu.cc:368-369, lib/gru_forward_gpu.cu.cc:374-375,
 * lib/layer_norm_forward_gpu.cu.cc:152-153, lib/indrnn_forward_gpu.cu.cc:212-213).  These are
 * what haste::v0::<cell>::ForwardPass<double>::Run / BackwardPass<double>::Run (and Iterate)
 * bind to: same arguments, shapes and semantics as the *_f32 entry points above, tensors in
 * double; zoneout_prob and dropconnect_scale stay float as in the reference's signatures.
 * Every step is a GEMM on the fp64 matrix cores plus row-wise / pointwise kernels, for any
 * hidden size. */
int haste_hip_gemm_f64(int trans_a, int M, int N, int K,
                       const double* A, int lda, const double* B, int ldb,
                       double* C, int ldc, int accumulate, void* stream);
int haste_hip_transpose_f64(int rows, int cols, const double* in, double* out, void* stream);
int haste_hip_lstm_forward_f64(int training, int steps, int batch_size, int input_size,
                               int hidden_size,
                               const double* W, const double* R, const double* b, const double* x,
                               double* h, double* c, double* v, double* tmp_Rh,
                               float zoneout_prob, const double* zoneout_mask, void* stream);
int haste_hip_lstm_forward_dropconnect_f64(int training, int steps, int batch_size,
                                           int input_size, int hidden_size,
                                           const double* W, const double* R, const double* b,
                                           const double* x, double* h, double* c, double* v,
                                           float zoneout_prob, const double* zoneout_mask,
                                           const double* dropconnect_mask, float dropconnect_scale,
                                           void* stream);
int haste_hip_lstm_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                                const double* W_t, const double* R_t, const double* b,
                                const double* x_t, const double* h, const double* c,
                                const double* dh_new, const double* dc_new,
                                double* dx, double* dW, double* dR, double* db,
                                double* dh, double* dc, double* v,
                                const double* zoneout_mask, void* stream);
int haste_hip_lstm_forward_iterate_f64(int training, int batch_size, int input_size,
                                       int hidden_size,
                                       const double* W, const double* R, const double* b,
                                       const double* x, const double* h, const double* c,
                                       double* h_out, double* c_out, double* v, double* tmp_Rh,
                                       float zoneout_prob, const double* zoneout_mask,
                                       void* stream);
int haste_hip_lstm_backward_iterate_f64(int batch_size, int input_size, int hidden_size,
                                        const double* W_t, const double* R_t, const double* b,
                                        const double* x_t, const double* h, const double* c,
                                        const double* c_new, const double* dh_new,
                                        const double* dc_new, double* dx, double* dW, double* dR,
                                        double* db, double* dh, double* dc, double* v,
                                        const double* zoneout_mask, void* stream);
int haste_hip_gru_forward_f64(int training, int steps, int batch_size, int input_size,
                              int hidden_size,
                              const double* W, const double* R, const double* bx, const double* br,
                              const double* x, double* h, double* v, double* tmp_Wx, double* tmp_Rh,
                              float zoneout_prob, const double* zoneout_mask, void* stream);
int haste_hip_gru_forward_dropconnect_f64(int training, int steps, int batch_size,
                                          int input_size, int hidden_size,
                                          const double* W, const double* R, const double* bx,
                                          const double* br, const double* x, double* h, double* v,
                                          double* tmp_Wx, float zoneout_prob,
                                          const double* zoneout_mask,
                                          const double* dropconnect_mask, float dropconnect_scale,
                                          void* stream);
int haste_hip_gru_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                               const double* W_t, const double* R_t, const double* bx,
                               const double* br, const double* x_t, const double* h, const double* v,
                               const double* dh_new, double* dx, double* dW, double* dR,
                               double* dbx, double* dbr, double* dh, double* dp, double* dq,
                               const double* zoneout_mask, void* stream);
int haste_hip_gru_forward_iterate_f64(int training, int batch_size, int input_size,
                                      int hidden_size,
                                      const double* W, const double* R, const double* bx,
                                      const double* br, const double* x, const double* h,
                                      double* h_out, double* v, double* tmp_Wx, double* tmp_Rh,
                                      float zoneout_prob, const double* zoneout_mask,
                                      void* stream);
int haste_hip_gru_backward_iterate_f64(int batch_size, int input_size, int hidden_size,
                                       const double* W_t, const double* R_t, const double* bx,
                                       const double* br, const double* x_t, const double* h,
                                       const double* v, const double* dh_new, double* dx, double* dW,
                                       double* dR, double* dbx, double* dbr, double* dh, double* dp,
                                       double* dq, const double* zoneout_mask, void* stream);
int haste_hip_layer_norm_forward_f64(int rows, int dim, const double* gamma, const double* beta,
                                     const double* x, double* y, double* cache, void* stream);
int haste_hip_layer_norm_backward_f64(int rows, int dim, const double* gamma, const double* x,
                                      const double* dy, double* dx, double* dgamma, double* dbeta,
                                      const double* cache, void* stream);
int haste_hip_layer_norm_lstm_forward_f64(int training, int steps, int batch_size,
                                          int input_size, int hidden_size,
                                          const double* W, const double* R, const double* b,
                                          const double* x, double* h, double* c,
                                          double* act_Wx, double* tmp_Rh,
                                          const double* gamma1, double* cache1,
                                          double* act_Wx_norm, double* act_Rh,
                                          const double* gamma2, double* cache2,
                                          const double* gamma_h, const double* beta_h, double* cache3,
                                          double* act_c_norm,
                                          float zoneout_prob, const double* zoneout_mask,
                                          void* stream);
int haste_hip_layer_norm_lstm_backward_f64(int steps, int batch_size, int input_size,
                                           int hidden_size,
                                           const double* W_t, const double* R_t, const double* b,
                                           const double* x_t, const double* h, const double* c,
                                           const double* dh_new, const double* dc_new,
                                           double* dx, double* dW, double* dR, double* db,
                                           double* dh, double* dc,
                                           double* act_Wx, const double* gamma1, double* dgamma1,
                                           double* act_Wx_norm, double* act_Rh,
                                           const double* gamma2, double* dgamma2,
                                           const double* cache2,
                                           const double* gamma_h, const double* beta_h,
                                           double* dgamma_h, double* dbeta_h,
                                           const double* cache3,
                                           double* act_c_norm,
                                           const double* zoneout_mask, void* stream);
int haste_hip_layer_norm_gru_forward_f64(int training, int steps, int batch_size,
                                         int input_size, int hidden_size,
                                         const double* W, const double* R, const double* bx,
                                         const double* br, const double* x, double* h, double* v,
                                         double* act_Wx, const double* gamma1, double* cache1,
                                         double* tmp_Wx_norm, double* act_Rh,
                                         const double* gamma2, double* cache2, double* tmp_Rh_norm,
                                         float zoneout_prob, const double* zoneout_mask,
                                         void* stream);
int haste_hip_layer_norm_gru_backward_f64(int steps, int batch_size, int input_size,
                                          int hidden_size,
                                          const double* W_t, const double* R_t, const double* bx,
                                          const double* br, const double* x_t, const double* h,
                                          const double* v, const double* dh_new,
                                          double* dx, double* dW, double* dR, double* dbx, double* dbr,
                                          double* dh, double* dp, double* dq,
                                          const double* act_Wx, const double* gamma1, double* dgamma1,
                                          const double* act_Rh, const double* gamma2, double* dgamma2,
                                          const double* cache2,
                                          const double* zoneout_mask, void* stream);
int haste_hip_indrnn_forward_f64(int training, int steps, int batch_size, int input_size,
                                 int hidden_size,
                                 const double* W, const double* u, const double* b, const double* x,
                                 double* h, double* workspace,
                                 float zoneout_prob, const double* zoneout_mask, void* stream);
int haste_hip_indrnn_backward_f64(int steps, int batch_size, int input_size, int hidden_size,
                                  const double* W_t, const double* u, const double* b,
                                  const double* x_t, const double* h, const double* dh_new,
                                  double* dx, double* dW, double* du, double* db, double* dh,
                                  double* workspace, const double* zoneout_mask, void* stream);
int haste_hip_layer_norm_indrnn_forward_f64(int training, int steps, int batch_size,
                                            int input_size, int hidden_size,
                                            const double* W, const double* u, const double* b,
                                            const double* x, double* h, double* workspace,
                                            double* act_Wx, const double* gamma1, double* cache1,
                                            float zoneout_prob, const double* zoneout_mask,
                                            void* stream);
int haste_hip_layer_norm_indrnn_backward_f64(int steps, int batch_size, int input_size,
                                             int hidden_size,
                                             const double* W_t, const double* u, const double* b,
                                             const double* x_t, const double* h,
                                             const double* dh_new,
                                             double* dx, double* dW, double* du, double* db, double* dh,
                                             double* workspace,
                                             const double* act_Wx, const double* gamma1,
                                             double* dgamma1,
                                             const double* zoneout_mask, void* stream);

/* ---- half precision (GRU only) ------------------------------------------------------
 * The reference instantiates gru::ForwardPass / BackwardPass for half as well
 * (lib/gru_forward_gpu.cu.cc:373, lib/gru_backward_gpu.cu.cc:411).  Same arguments, shapes and
 * semantics as the GRU *_f32 entry points; every tensor holds IEEE binary16 values and is
 * passed as void* (C has no portable half type).  Products are accumulated in fp32 on the
 * matrix cores and the pointwise math is done in float; results are rounded to half, so
 * accumulated outputs (dh over the steps, dW, dR, dbx, dbr) carry half rounding per update. */
int haste_hip_gemm_f16(int trans_a, int M, int N, int K, const void* A, int lda, const void* B,
                       int ldb, void* C, int ldc, int accumulate, void* stream);
int haste_hip_transpose_f16(int rows, int cols, const void* in, void* out, void* stream);
/* C[M,N] (+)= A[M,K] * Bt[N,K]^T with fp32 accumulation and an fp32 result: the product kernel
 * of the half GRU's passes over more than one step.  Bt holds IEEE binary16 values, A binary16
 * or (a_is_float != 0) fp32 values that are rounded to half as they are read; both have the
 * contraction index contiguous.  K, lda and ldb must be multiples of 8 (4 for an fp32 A) and
 * the operands 16-byte aligned (HASTE_HIP_ERROR_UNSUPPORTED_SIZE otherwise).  No counterpart in
 * the reference (cublasHgemm with a transposition flag); exported for tests and for callers
 * that want the kernel by itself. */
int haste_hip_gemm_half_nt(int a_is_float, int M, int N, int K, const void* A, int lda,
                           const void* Bt, int ldb, float* C, int ldc, int accumulate, void* stream);
int haste_hip_gru_forward_f16(int training, int steps, int batch_size, int input_size,
                              int hidden_size, const void* W, const void* R, const void* bx,
                              const void* br, const void* x, void* h, void* v, void* tmp_Wx,
                              void* tmp_Rh, float zoneout_prob, const void* zoneout_mask,
                              void* stream);
int haste_hip_gru_forward_dropconnect_f16(int training, int steps, int batch_size, int input_size,
                                          int hidden_size, const void* W, const void* R,
                                          const void* bx, const void* br, const void* x, void* h,
                                          void* v, void* tmp_Wx, float zoneout_prob,
                                          const void* zoneout_mask, const void* dropconnect_mask,
                                          float dropconnect_scale, void* stream);
int haste_hip_gru_backward_f16(int steps, int batch_size, int input_size, int hidden_size,
                               const void* W_t, const void* R_t, const void* bx, const void* br,
                               const void* x_t, const void* h, const void* v, const void* dh_new,
                               void* dx, void* dW, void* dR, void* dbx, void* dbr, void* dh, void* dp,
                               void* dq, const void* zoneout_mask, void* stream);
int haste_hip_gru_forward_iterate_f16(int training, int batch_size, int input_size, int hidden_size,
                                      const void* W, const void* R, const void* bx, const void* br,
                                      const void* x, const void* h, void* h_out, void* v,
                                      void* tmp_Wx, void* tmp_Rh, float zoneout_prob,
                                      const void* zoneout_mask, void* stream);
int haste_hip_gru_backward_iterate_f16(int batch_size, int input_size, int hidden_size,
                                       const void* W_t, const void* R_t, const void* bx,
                                       const void* br, const void* x_t, const void* h, const void* v,
                                       const void* dh_new, void* dx, void* dW, void* dR, void* dbx,
                                       void* dbr, void* dh, void* dp, void* dq,
                                       const void* zoneout_mask, void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* HASTE_HIP_H_ */
