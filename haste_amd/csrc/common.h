// Host-side plumbing shared by every translation unit of libhaste_hip.so:
// error codes, argument checks, the per-stream device workspace and the
// internal (non-exported) launch helpers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "../../include/haste_hip.h"

namespace haste_hip {

// Records the text of a failed HIP call for haste_hip_last_runtime_error().
void set_runtime_error(hipError_t err, const char* what);

// Records a plain explanation (a size limit, a refused configuration) for the same query.
void set_error_text(const char* text);

#define HASTE_HIP_TRY(expr)                                   \
  do {                                                        \
    hipError_t err__ = (expr);                                \
    if (err__ != hipSuccess) {                                \
      ::haste_hip::set_runtime_error(err__, #expr);           \
      return HASTE_HIP_ERROR_RUNTIME;                         \
    }                                                         \
  } while (0)

#define HASTE_HIP_REQUIRE(cond)                               \
  do {                                                        \
    if (!(cond)) return HASTE_HIP_ERROR_INVALID_ARGUMENT;     \
  } while (0)

#define HASTE_HIP_PROPAGATE(expr)                             \
  do {                                                        \
    int rc__ = (expr);                                        \
    if (rc__ != HASTE_HIP_OK) return rc__;                    \
  } while (0)

// Layout of the control block of a workspace.  The counters are zero between kernels
// (a kernel that uses one restores it before it exits); the step flags only ever
// grow: each persistent launch is given a fresh range of values (an epoch).
constexpr int kMaxGroups = 64;        // batch tiles a persistent kernel may have
constexpr int kMaxWorkgroups = 2048;  // workgroups a persistent kernel may have
constexpr int kCounterStride = 32;    // uint32 slots between counters (128 B apart)
struct ControlBlock {
  unsigned int step_flags[kMaxWorkgroups];                 // per-workgroup arrival counts
  unsigned int grid_exit_counter[kCounterStride];          // unused (kept for the layout)
  unsigned int tile_counter[4096];                         // arrivals per column block at the end of a launch
  unsigned int xcd_ticket[16 * kCounterStride];            // per-XCD role tickets (only ever grow)
  unsigned int abort_flag[kCounterStride];                 // set when a barrier wait gives up
};

// A block of device memory owned by the library and tied to one (device, stream):
// the control block followed by a scratch area that grows on demand.  Work that
// uses it is ordered by the stream, so one workspace per stream is race free.
struct Workspace {
  ControlBlock* control = nullptr;   // device
  float* scratch = nullptr;          // device
  size_t scratch_bytes = 0;
  size_t scratch_high_water = 0;     // most scratch any call on this stream has asked for
  unsigned int epoch = 0;            // step-flag values handed out so far
  unsigned int ticket_base = 0;      // per-XCD tickets handed out so far
  unsigned int* host_status = nullptr;      // pinned host word the kernels report aborts to
  unsigned int* host_status_dev = nullptr;  // the same word as the device addresses it
  bool self_resetting = false;       // every persistent launch wipes the control block first
                                     // and numbers its flags and tickets from zero (set once a
                                     // launch on this stream has been captured into a graph)
  bool caller_owned = false;         // control and scratch lie in memory the caller lent
                                     // (haste_hip_set_workspace): never freed or grown here
};

// Returns the workspace of (current device, stream) with at least `scratch_bytes`
// of scratch, creating or growing it if needed.  A workspace in memory lent by the caller is
// never grown: HASTE_HIP_ERROR_UNSUPPORTED_SIZE (and the size needed in the error text) when
// it is too small.
int get_workspace(hipStream_t stream, size_t scratch_bytes, Workspace* out);

// While one of these is alive on a host thread, get_workspace() on that thread hands out the
// scratch area behind the first `bytes` bytes (a multiple of 256) of the stream's scratch
// buffer: an entry point that stages tensors of its own there and then calls other entry
// points' implementations keeps its staging area out of their way.  The buffer must already
// be large enough for the prefix and everything asked for behind it (ask get_workspace for
// the sum first): growing replaces the buffer, which would lose what is staged, so with a
// prefix in force get_workspace refuses to grow (HASTE_HIP_ERROR_UNSUPPORTED_SIZE).
class ScratchPrefix {
 public:
  explicit ScratchPrefix(size_t bytes);
  ~ScratchPrefix();
  ScratchPrefix(const ScratchPrefix&) = delete;
  ScratchPrefix& operator=(const ScratchPrefix&) = delete;

 private:
  size_t saved_;
};

// The scratch part of haste_hip_workspace_bytes(T, N, C, H): what a workspace of that size
// offers behind its control block.
size_t workspace_scratch_bound(int T, int N, int C, int H);

// Reserves `count` consecutive step-flag values on the workspace of (current device,
// stream) and returns the value before the first of them.
int reserve_epochs(hipStream_t stream, unsigned int count, unsigned int* base);

// Same for the per-XCD role tickets of a launch that places groups on XCDs.
int reserve_tickets(hipStream_t stream, unsigned int count, unsigned int* base);

// Checks (without synchronizing) whether a persistent kernel launched earlier on
// this workspace reported a barrier time-out; if so re-zeroes the control block and
// returns HASTE_HIP_ERROR_STEP_BARRIER once.
int check_and_clear_abort(hipStream_t stream, Workspace* ws);

int device_cu_count();

// XCDs of the current device on which a launch of one workgroup per CU puts equally many
// workgroups each -- found by running such a launch once per device (a probe kernel that
// records where each workgroup ran) -- or 0 when the placement is not that regular (a
// partition mode or a CU mask the probe does not understand), when HASTE_HIP_XCD_LOCAL=0, or
// after a launch found more workgroups on an XCD than it had been promised: the persistent
// kernels then take the cross-XCD path.  xcc_logical_map: 4 bits per hardware XCC id, its
// index among the XCDs in use.
int device_xcd_count();
unsigned long long device_xcc_logical_map();

// The look at the device's XCD placement allocates, synchronizes the device and launches on the
// null stream: it cannot run while `stream` is being captured into a graph.  HASTE_HIP_OK when
// the device has been looked at (or can be now); HASTE_HIP_ERROR_RUNTIME, with the reason in
// haste_hip_last_runtime_error(), when it has not and `stream` is capturing.
int xcd_layout_ready(hipStream_t stream);

// Keeps the persistent kernels of this process on one device in a single order even when
// they are launched on different streams.  before == true: makes `stream` wait for the
// previous persistent kernel (if it ran on another stream); before == false: records the
// kernel just enqueued on `stream` as the one to wait for.
int order_persistent_launches(hipStream_t stream, bool before);

// Holds the process-wide order of persistent launches from before the wait for the previous
// launch until this launch has been recorded as the last one: two host threads that launch
// on different streams would otherwise both wait for the launch before theirs and then run
// side by side.
class PersistentLaunchOrder {
 public:
  PersistentLaunchOrder();
  ~PersistentLaunchOrder();
  PersistentLaunchOrder(const PersistentLaunchOrder&) = delete;
  PersistentLaunchOrder& operator=(const PersistentLaunchOrder&) = delete;
};

// Polls before a bounded wait of a persistent kernel gives up: 2^24 (seconds), or the value of
// the environment variable HASTE_HIP_SPIN_LIMIT (at least 2^16, a few milliseconds: less only
// together with HASTE_HIP_TEST_HOOKS=1).
unsigned int spin_limit();

// Number of workgroups every group barrier also waits for although no workgroup plays them: 0,
// or -- only when the environment also has HASTE_HIP_TEST_HOOKS=1 -- the value of
// HASTE_HIP_TEST_ABSENT_WORKGROUP.  Only the test of the time-out path sets them, together with
// a small spin limit: the waits then run out, the kernel reports it and every wavefront still
// reaches the end of the kernel.
int test_absent_workgroups();

// False when the environment variable HASTE_HIP_FUSED_INPUT is set to 0: the forward
// recurrences then read x * W from a GEMM launched before them instead of computing it beside
// their waits (for experiments).
bool fused_input_enabled();

// C[M,N] = op(A)*B (+C): fp32 MFMA GEMM on `stream`.  The partial tiles of a split product
// are kept `scratch_offset` bytes (a multiple of 16) into the stream's scratch buffer.
int gemm_f32(hipStream_t stream, bool trans_a, int M, int N, int K,
             const float* A, int lda, const float* B, int ldb,
             float* C, int ldc, bool accumulate, size_t scratch_offset = 0);

// Two products with the same N and K, the second with A stored transposed, in one launch when
// that halves their K pieces (gemm.hip): dW and dR of a backward pass.
int gemm_f32_pair(hipStream_t stream, int M1, int M2, int N, int K, const float* A1, int lda1,
                  const float* B1, int ldb1, float* C1, int ldc1, const float* A2, int lda2,
                  const float* B2, int ldb2, float* C2, int ldc2, bool accumulate);

// The product left as the K pieces of the tile kernel for a consumer that adds them itself;
// *splits == 0 (and nothing launched) when the shape is not cut that way.  See gemm.hip.
int gemm_f32_pieces(hipStream_t stream, int M, int N, int K, const float* A, int lda,
                    const float* B, int ldb, size_t scratch_offset, const float** partial,
                    int* splits, int* bm);

// Bytes of scratch gemm_f32 may use for this shape (0 when nothing is split).
size_t gemm_f32_scratch_bytes(int M, int N, int K);

// The product for M <= 128 with B streamed from HBM straight into the MFMA operands
// (gemm_skinny.hip); gemm_f32 hands such shapes over when the operands are 16-byte aligned.
bool gemm_f32_skinny_shape(bool trans_a, int M, int N, int K);
bool gemm_f32_skinny_applies(bool trans_a, int M, int N, int K, const float* A, int lda,
                             const float* B, int ldb, const float* C, int ldc);
size_t gemm_f32_skinny_scratch_bytes(int M, int N, int K);
int gemm_f32_skinny(hipStream_t stream, int M, int N, int K, const float* A, int lda,
                    const float* B, int ldb, float* C, int ldc, bool accumulate,
                    size_t scratch_offset);
int gemm_f32_skinny_chunks(hipStream_t stream, int M, int N, int K, const float* A, int lda,
                           const float* B, int ldb, size_t scratch_offset, const float** partial,
                           int* chunks);

// The cells in step-wise form, the recurrent matrix streamed from HBM every step (per-step
// GEMM + row-wise norms + pointwise kernels): for hidden sizes whose slices of R do not fit
// on chip.  Arguments as the persistent implementations in lstm.hip / gru.hip /
// layer_norm_lstm.hip / layer_norm_gru.hip.
int lstm_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                          const float* W, const float* R, const float* b, const float* x,
                          const float* h, const float* c, float* h_out, float* c_out, float* v,
                          float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                          float dc_scale);
int lstm_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                           const float* W_t, const float* R_t, const float* x_t,
                           const float* h, const float* c, const float* c_next,
                           const float* dh_next, const float* dc_next,
                           float* dx, float* dW, float* dR, float* db, float* dh, float* dc, float* v,
                           const float* zoneout_mask);
int gru_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                         const float* W, const float* R, const float* bx, const float* br,
                         const float* x, const float* h, float* h_out, float* v, float* tmp_Wx,
                         float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                         float dc_scale);
int gru_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                          const float* W_t, const float* R_t, const float* x_t, const float* h,
                          const float* v, const float* dh_next, float* dx, float* dW, float* dR,
                          float* dbx, float* dbr, float* dh, float* dp, float* dq,
                          const float* zoneout_mask);
int layer_norm_lstm_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                                     const float* W, const float* R, const float* b, const float* x,
                                     float* h, float* c, float* act_Wx, const float* gamma1,
                                     float* cache1, float* act_Wx_norm, float* act_Rh,
                                     const float* gamma2, float* cache2, const float* gamma_h,
                                     const float* beta_h, float* cache3, float* act_c_norm,
                                     float zoneout_prob, const float* zoneout_mask);
int layer_norm_lstm_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                                      const float* W_t, const float* R_t, const float* x_t,
                                      const float* h, const float* c, const float* dh_new,
                                      const float* dc_new, float* dx, float* dW, float* dR, float* db,
                                      float* dh, float* dc, float* act_Wx, const float* gamma1,
                                      float* dgamma1, float* act_Wx_norm, float* act_Rh,
                                      const float* gamma2, float* dgamma2, const float* cache2,
                                      const float* gamma_h, float* dgamma_h, float* dbeta_h,
                                      const float* cache3, float* act_c_norm,
                                      const float* zoneout_mask);
int layer_norm_gru_forward_streamed(hipStream_t stream, int training, int T, int N, int C, int H,
                                    const float* W, const float* R, const float* bx, const float* br,
                                    const float* x, float* h, float* v, float* act_Wx,
                                    const float* gamma1, float* cache1, float* tmp_Wx_norm,
                                    float* act_Rh, const float* gamma2, float* cache2,
                                    float zoneout_prob, const float* zoneout_mask);
int layer_norm_gru_backward_streamed(hipStream_t stream, int T, int N, int C, int H,
                                     const float* W_t, const float* R_t, const float* x_t,
                                     const float* h, const float* v, const float* dh_new, float* dx,
                                     float* dW, float* dR, float* dbx, float* dbr, float* dh,
                                     float* dp, float* dq, const float* act_Wx, const float* gamma1,
                                     float* dgamma1, const float* act_Rh, const float* gamma2,
                                     float* dgamma2, const float* cache2,
                                     const float* zoneout_mask);

// One forward step for a batch of at most 8 rows as a single kernel (single_step.hip): what the
// Iterate entry points and one-step Run calls use.
bool single_step_applies(int N, int C, int H);
int lstm_forward_single_step(hipStream_t stream, int training, int N, int C, int H, const float* W,
                             const float* R, const float* b, const float* x, const float* h,
                             const float* c, float* h_out, float* c_out, float* v,
                             float zoneout_prob, const float* zoneout_mask, const float* dc_mask,
                             float dc_scale);
int gru_forward_single_step(hipStream_t stream, int training, int N, int C, int H, const float* W,
                            const float* R, const float* bx, const float* br, const float* x,
                            const float* h, float* h_out, float* v, float zoneout_prob,
                            const float* zoneout_mask, const float* dc_mask, float dc_scale);
// Half tensors (IEEE binary16), sums and pointwise step in float.
int gru_forward_single_step_half(hipStream_t stream, int training, int N, int C, int H, const void* W,
                                 const void* R, const void* bx, const void* br, const void* x,
                                 const void* h, void* h_out, void* v, float zoneout_prob,
                                 const void* zoneout_mask, const void* dc_mask, float dc_scale);

// The same for rows too wide for layer_norm.hip's row-in-registers kernels (stepwise.hip).
int layer_norm_forward_wide(hipStream_t stream, int rows, int dim, const float* gamma,
                            const float* beta, const float* x, float* y, float* cache);
int layer_norm_backward_wide(hipStream_t stream, int rows, int dim, const float* gamma,
                             const float* x, const float* dy, float* dx, float* dgamma,
                             float* dbeta);

// Row-wise layer norm kernels (rows x dim), used stand-alone and by the LN cells.
int layer_norm_forward(hipStream_t stream, int rows, int dim, const float* gamma,
                       const float* beta, const float* x, float* y, float* cache);
int layer_norm_backward(hipStream_t stream, int rows, int dim, const float* gamma,
                        const float* x, const float* dy, float* dx, float* dgamma,
                        float* dbeta);

// first[c] += sum over b < parts of partial[b][c], second[c] += ... of partial[b][D + c]
// (partial is [parts][2][D]; second may be null), parts added in index order by a small
// parallel kernel: the deterministic finish of column sums parked by many workgroups.
int add_column_partials(hipStream_t stream, int parts, int D, const float* partial, float* first,
                        float* second);

// Brackets the launches made during its lifetime with a pair of events on `stream`
// when profiling has been switched on (haste_hip_profile_enable); otherwise does
// nothing.  `name` must be a string literal.
class ScopedKernelTimer {
 public:
  // `products`: how many launches of `name` the bracket counts as (a fused pair counts 2).
  ScopedKernelTimer(const char* name, hipStream_t stream, int products = 1);
  ~ScopedKernelTimer();
 private:
  hipStream_t stream_;
  int slot_;
};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace haste_hip
