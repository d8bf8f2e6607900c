// Exercises the libhaste-compatible C++ classes (include/haste.h) the way a C++ caller
// of the reference would (cf. reference examples/lstm.cc:72-200): device buffers,
// ForwardPass::Run, host-side transposes, BackwardPass::Run.  Reads one problem from a
// raw float32 file (float64 for "f64:<cell>", which runs the classes instantiated for
// double), writes every output to another; tests/test_gpu_cpp_api.py feeds it
// seeded inputs and checks the outputs against the oracle.
//
// usage: api_check <cell> <T> <N> <C> <H> <zoneout_prob> <in.bin> <out.bin>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "haste.h"

using namespace haste::v0;

#define CHECK_HIP(e)                                                                   \
  do {                                                                                 \
    hipError_t err_ = (e);                                                             \
    if (err_ != hipSuccess) {                                                          \
      std::fprintf(stderr, "%s failed: %s\n", #e, hipGetErrorString(err_));            \
      std::exit(3);                                                                    \
    }                                                                                  \
  } while (0)

template <typename S>
struct DeviceBufT {
  S* p = nullptr;
  size_t n = 0;
  explicit DeviceBufT(size_t count) : n(count) {
    CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&p), (count ? count : 1) * sizeof(S)));
    CHECK_HIP(hipMemset(p, 0, (count ? count : 1) * sizeof(S)));
  }
  DeviceBufT(const std::vector<S>& h) : DeviceBufT(h.size()) {
    if (n) CHECK_HIP(hipMemcpy(p, h.data(), n * sizeof(S), hipMemcpyHostToDevice));
  }
  ~DeviceBufT() { (void)hipFree(p); }
  std::vector<S> host() const {
    std::vector<S> h(n);
    if (n) CHECK_HIP(hipMemcpy(h.data(), p, n * sizeof(S), hipMemcpyDeviceToHost));
    return h;
  }
  DeviceBufT(const DeviceBufT&) = delete;
  DeviceBufT& operator=(const DeviceBufT&) = delete;
};

static FILE* g_in = nullptr;
static FILE* g_out = nullptr;

template <typename S>
static std::vector<S> read_tensor_t(size_t count) {
  std::vector<S> v(count);
  if (count && std::fread(v.data(), sizeof(S), count, g_in) != count) {
    std::fprintf(stderr, "input file too short\n");
    std::exit(4);
  }
  return v;
}

template <typename S>
static void write_tensor(const DeviceBufT<S>& b) {
  const std::vector<S> h = b.host();
  std::fwrite(h.data(), sizeof(S), h.size(), g_out);
}

// [rows, cols] -> [cols, rows]
template <typename S>
static std::vector<S> transpose(const std::vector<S>& a, size_t rows, size_t cols) {
  std::vector<S> t(a.size());
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) t[c * rows + r] = a[r * cols + c];
  return t;
}

static void require_ok(int status, const char* what) {
  if (status != HASTE_HIP_OK) {
    std::fprintf(stderr, "%s: %s [%s]\n", what, haste_hip_error_string(status),
                 haste_hip_last_runtime_error());
    std::exit(5);
  }
}

// The GRU classes also exist for half, as in the reference (lib/gru_forward_gpu.cu.cc:373):
// instantiating every member checks that they bind to the *_f16 entry points.
template class haste::v0::gru::ForwardPass<__half>;
template class haste::v0::gru::BackwardPass<__half>;

// The problem in precision S (the files hold S as well).
template <typename S>
static int run(const std::string& cell, int T, int N, int C, int H, float zoneout) {
  using DeviceBuf = DeviceBufT<S>;


  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  hipblasHandle_t blas = nullptr;  // accepted and ignored by the library
  const size_t TN = (size_t)T * N, NH = (size_t)N * H;

  // HASTE_API_CHECK_LENT_WORKSPACE=1: the library's scratch memory for both streams comes from this
  // caller (the reference's contract: every buffer is the caller's, lib/haste/lstm.h:98-117).
  const char* lend = std::getenv("HASTE_API_CHECK_LENT_WORKSPACE");
  const bool lent = lend != nullptr && lend[0] == '1';
  void* lent_memory[2] = {nullptr, nullptr};
  const bool has_mask = zoneout > 0.f;

  // The *_iterate cells run the same problems one step at a time through Iterate()
  // (cf. reference examples/lstm.cc:252,309), handing each step a second stream as the
  // one the caller works on.
  hipStream_t caller_stream;
  CHECK_HIP(hipStreamCreate(&caller_stream));
  if (lent) {
    const size_t bytes = haste_hip_workspace_bytes(T, N, C, H);
    hipStream_t both[2] = {stream, caller_stream};
    for (int i = 0; i < 2; ++i) {
      CHECK_HIP(hipMalloc(&lent_memory[i], bytes));
      require_ok(haste_hip_set_workspace(both[i], lent_memory[i], bytes), "haste_hip_set_workspace");
    }
  }

  if (cell == "lstm" || cell == "layer_norm_lstm" || cell == "lstm_iterate") {
    const bool ln = cell == "layer_norm_lstm";
    const bool iter = cell == "lstm_iterate";
    const int G = 4;
    std::vector<S> W = read_tensor_t<S>((size_t)C * G * H), R = read_tensor_t<S>((size_t)H * G * H),
                       b = read_tensor_t<S>((size_t)G * H), x = read_tensor_t<S>(TN * C), h0 = read_tensor_t<S>(NH),
                       c0 = read_tensor_t<S>(NH), dh_new = read_tensor_t<S>((T + 1) * NH),
                       dc_new = read_tensor_t<S>((T + 1) * NH);
    std::vector<S> gamma, gamma_h, beta_h;
    if (ln) { gamma = read_tensor_t<S>((size_t)2 * G * H); gamma_h = read_tensor_t<S>(H); beta_h = read_tensor_t<S>(H); }
    std::vector<S> mask = read_tensor_t<S>(has_mask ? TN * H : 0);

    DeviceBuf dW_(W), dR_(R), db_(b), dx_(x), dmask(mask);
    std::vector<S> hinit((T + 1) * NH, 0.f), cinit((T + 1) * NH, 0.f);
    std::memcpy(hinit.data(), h0.data(), NH * sizeof(S));
    std::memcpy(cinit.data(), c0.data(), NH * sizeof(S));
    DeviceBuf h(hinit), c(cinit), v(TN * G * H), tmp_Rh((size_t)N * G * H);
    DeviceBuf act_Wx(ln ? TN * G * H : 0), act_Rh(ln ? TN * G * H : 0), act_c_norm(ln ? TN * H : 0);
    DeviceBuf cache1(ln ? TN * 2 : 0), cache2(ln ? TN * 2 : 0), cache3(ln ? TN * 2 : 0);
    DeviceBuf dgamma(gamma), dgamma_h(gamma_h), dbeta_h(beta_h);
    const S* maskp = has_mask ? dmask.p : nullptr;

    if (iter) {
      lstm::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      for (int t = 0; t < T; ++t) {
        fwd.Iterate(caller_stream, dW_.p, dR_.p, db_.p, dx_.p + (size_t)t * N * C, h.p + t * NH,
                    c.p + t * NH, h.p + (t + 1) * NH, c.p + (t + 1) * NH, v.p + (size_t)t * N * G * H,
                    tmp_Rh.p, zoneout, has_mask ? maskp + t * NH : nullptr);
        require_ok(fwd.last_status(), "lstm forward iterate");
      }
      CHECK_HIP(hipStreamSynchronize(caller_stream));
    } else if (!ln) {
      lstm::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      fwd.Run(T, dW_.p, dR_.p, db_.p, dx_.p, h.p, c.p, v.p, tmp_Rh.p, zoneout, maskp);
      require_ok(fwd.last_status(), "lstm forward");
    } else {
      layer_norm::ForwardPass<S> ln1(T * N, G * H, dgamma.p, nullptr, cache1.p);
      layer_norm::ForwardPass<S> ln2(T * N, G * H, dgamma.p + G * H, nullptr, cache2.p);
      layer_norm::ForwardPass<S> ln3(T * N, H, dgamma_h.p, dbeta_h.p, cache3.p);
      layer_norm_lstm::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      fwd.Run(T, dW_.p, dR_.p, db_.p, dx_.p, h.p, c.p, act_Wx.p, tmp_Rh.p, ln1, v.p, act_Rh.p, ln2,
              ln3, act_c_norm.p, zoneout, maskp);
      require_ok(fwd.last_status(), "layer_norm_lstm forward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(h);
    write_tensor(c);

    DeviceBuf x_t(transpose(x, TN, C)), W_t(transpose(W, C, (size_t)G * H)),
        R_t(transpose(R, H, (size_t)G * H)), ddh_new(dh_new), ddc_new(dc_new);
    DeviceBuf gdx(TN * C), gdW((size_t)C * G * H), gdR((size_t)H * G * H), gdb((size_t)G * H), gdh(NH),
        gdc(NH), gdgamma(ln ? (size_t)2 * G * H : 0), gdgamma_h(ln ? H : 0), gdbeta_h(ln ? H : 0);
    if (iter) {
      // per-step transposes of x: step t is [C,N]
      std::vector<S> xs(TN * C);
      for (int t = 0; t < T; ++t) {
        std::vector<S> one(x.begin() + (size_t)t * N * C, x.begin() + (size_t)(t + 1) * N * C);
        one = transpose(one, N, C);
        std::memcpy(xs.data() + (size_t)t * N * C, one.data(), one.size() * sizeof(S));
      }
      DeviceBuf x_steps(xs);
      lstm::BackwardPass<S> bwd(N, C, H, blas, stream);
      for (int t = T - 1; t >= 0; --t) {
        bwd.Iterate(caller_stream, W_t.p, R_t.p, db_.p, x_steps.p + (size_t)t * N * C, h.p + t * NH,
                    c.p + t * NH, c.p + (t + 1) * NH, ddh_new.p + (t + 1) * NH,
                    ddc_new.p + (t + 1) * NH, gdx.p + (size_t)t * N * C, gdW.p, gdR.p, gdb.p, gdh.p,
                    gdc.p, v.p + (size_t)t * N * G * H, has_mask ? maskp + t * NH : nullptr);
        require_ok(bwd.last_status(), "lstm backward iterate");
      }
      CHECK_HIP(hipStreamSynchronize(caller_stream));
    } else if (!ln) {
      lstm::BackwardPass<S> bwd(N, C, H, blas, stream);
      bwd.Run(T, W_t.p, R_t.p, db_.p, x_t.p, h.p, c.p, ddh_new.p, ddc_new.p, gdx.p, gdW.p, gdR.p,
              gdb.p, gdh.p, gdc.p, v.p, maskp);
      require_ok(bwd.last_status(), "lstm backward");
    } else {
      layer_norm::BackwardPass<S> ln1(T * N, G * H, dgamma.p, nullptr, act_Wx.p, gdgamma.p, nullptr, cache1.p);
      layer_norm::BackwardPass<S> ln2(T * N, G * H, dgamma.p + G * H, nullptr, act_Rh.p,
                                          gdgamma.p + G * H, nullptr, cache2.p);
      layer_norm::BackwardPass<S> ln3(T * N, H, dgamma_h.p, dbeta_h.p, c.p + NH, gdgamma_h.p,
                                          gdbeta_h.p, cache3.p);
      layer_norm_lstm::BackwardPass<S> bwd(N, C, H, blas, stream);
      bwd.Run(T, W_t.p, R_t.p, db_.p, x_t.p, h.p, c.p, ddh_new.p, ddc_new.p, gdx.p, gdW.p, gdR.p,
              gdb.p, gdh.p, gdc.p, act_Wx.p, ln1, v.p, act_Rh.p, ln2, ln3, act_c_norm.p, maskp);
      require_ok(bwd.last_status(), "layer_norm_lstm backward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(gdx); write_tensor(gdW); write_tensor(gdR); write_tensor(gdb);
    write_tensor(gdh); write_tensor(gdc);
    if (ln) { write_tensor(gdgamma); write_tensor(gdgamma_h); write_tensor(gdbeta_h); }
  } else if (cell == "gru" || cell == "layer_norm_gru" || cell == "gru_iterate") {
    const bool ln = cell == "layer_norm_gru";
    const bool iter = cell == "gru_iterate";
    const int G = 3;
    std::vector<S> W = read_tensor_t<S>((size_t)C * G * H), R = read_tensor_t<S>((size_t)H * G * H),
                       bx = read_tensor_t<S>((size_t)G * H), br = read_tensor_t<S>((size_t)G * H),
                       x = read_tensor_t<S>(TN * C), h0 = read_tensor_t<S>(NH), dh_new = read_tensor_t<S>((T + 1) * NH);
    std::vector<S> gamma;
    if (ln) gamma = read_tensor_t<S>((size_t)2 * G * H);
    std::vector<S> mask = read_tensor_t<S>(has_mask ? TN * H : 0);

    DeviceBuf dW_(W), dR_(R), dbx_(bx), dbr_(br), dx_(x), dmask(mask), dgamma(gamma);
    std::vector<S> hinit((T + 1) * NH, 0.f);
    std::memcpy(hinit.data(), h0.data(), NH * sizeof(S));
    DeviceBuf h(hinit), v(TN * 4 * H), tmp_Wx(TN * G * H), tmp_Rh((size_t)N * G * H);
    DeviceBuf act_Wx(ln ? TN * G * H : 0), act_Rh(ln ? TN * G * H : 0), cache1(ln ? TN * 2 : 0),
        cache2(ln ? TN * 2 : 0);
    const S* maskp = has_mask ? dmask.p : nullptr;
    if (iter) {
      gru::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      for (int t = 0; t < T; ++t) {
        fwd.Iterate(dW_.p, dR_.p, dbx_.p, dbr_.p, dx_.p + (size_t)t * N * C, h.p + t * NH,
                    h.p + (t + 1) * NH, v.p + (size_t)t * N * 4 * H, tmp_Wx.p, tmp_Rh.p, zoneout,
                    has_mask ? maskp + t * NH : nullptr);
        require_ok(fwd.last_status(), "gru forward iterate");
      }
    } else if (!ln) {
      gru::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      fwd.Run(T, dW_.p, dR_.p, dbx_.p, dbr_.p, dx_.p, h.p, v.p, tmp_Wx.p, tmp_Rh.p, zoneout, maskp);
      require_ok(fwd.last_status(), "gru forward");
    } else {
      layer_norm::ForwardPass<S> ln1(T * N, G * H, dgamma.p, nullptr, cache1.p);
      layer_norm::ForwardPass<S> ln2(T * N, G * H, dgamma.p + G * H, nullptr, cache2.p);
      layer_norm_gru::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      fwd.Run(T, dW_.p, dR_.p, dbx_.p, dbr_.p, dx_.p, h.p, v.p, act_Wx.p, ln1, tmp_Wx.p, act_Rh.p,
              ln2, tmp_Rh.p, zoneout, maskp);
      require_ok(fwd.last_status(), "layer_norm_gru forward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(h);

    DeviceBuf x_t(transpose(x, TN, C)), W_t(transpose(W, C, (size_t)G * H)),
        R_t(transpose(R, H, (size_t)G * H)), ddh_new(dh_new);
    DeviceBuf gdx(TN * C), gdW((size_t)C * G * H), gdR((size_t)H * G * H), gdbx((size_t)G * H),
        gdbr((size_t)G * H), gdh(NH), dp(TN * G * H), dq(TN * G * H), gdgamma(ln ? (size_t)2 * G * H : 0);
    if (iter) {
      std::vector<S> xs(TN * C);
      for (int t = 0; t < T; ++t) {
        std::vector<S> one(x.begin() + (size_t)t * N * C, x.begin() + (size_t)(t + 1) * N * C);
        one = transpose(one, N, C);
        std::memcpy(xs.data() + (size_t)t * N * C, one.data(), one.size() * sizeof(S));
      }
      DeviceBuf x_steps(xs);
      gru::BackwardPass<S> bwd(N, C, H, blas, stream);
      for (int t = T - 1; t >= 0; --t) {
        bwd.Iterate(W_t.p, R_t.p, dbx_.p, dbr_.p, x_steps.p + (size_t)t * N * C, h.p + t * NH,
                    v.p + (size_t)t * N * 4 * H, ddh_new.p + (t + 1) * NH, gdx.p + (size_t)t * N * C,
                    gdW.p, gdR.p, gdbx.p, gdbr.p, gdh.p, dp.p, dq.p,
                    has_mask ? maskp + t * NH : nullptr);
        require_ok(bwd.last_status(), "gru backward iterate");
      }
    } else if (!ln) {
      gru::BackwardPass<S> bwd(N, C, H, blas, stream);
      bwd.Run(T, W_t.p, R_t.p, dbx_.p, dbr_.p, x_t.p, h.p, v.p, ddh_new.p, gdx.p, gdW.p, gdR.p,
              gdbx.p, gdbr.p, gdh.p, dp.p, dq.p, maskp);
      require_ok(bwd.last_status(), "gru backward");
    } else {
      layer_norm::BackwardPass<S> ln1(T * N, G * H, dgamma.p, nullptr, act_Wx.p, gdgamma.p, nullptr, cache1.p);
      layer_norm::BackwardPass<S> ln2(T * N, G * H, dgamma.p + G * H, nullptr, act_Rh.p,
                                          gdgamma.p + G * H, nullptr, cache2.p);
      layer_norm_gru::BackwardPass<S> bwd(N, C, H, blas, stream);
      bwd.Run(T, W_t.p, R_t.p, dbx_.p, dbr_.p, x_t.p, h.p, v.p, ddh_new.p, gdx.p, gdW.p, gdR.p,
              gdbx.p, gdbr.p, gdh.p, dp.p, dq.p, ln1, ln2, maskp);
      require_ok(bwd.last_status(), "layer_norm_gru backward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(gdx); write_tensor(gdW); write_tensor(gdR); write_tensor(gdbx); write_tensor(gdbr);
    write_tensor(gdh);
    if (ln) write_tensor(gdgamma);
  } else if (cell == "indrnn" || cell == "layer_norm_indrnn") {
    const bool ln = cell == "layer_norm_indrnn";
    std::vector<S> W = read_tensor_t<S>((size_t)C * H), u = read_tensor_t<S>(H), b = read_tensor_t<S>(H),
                       x = read_tensor_t<S>(TN * C), h0 = read_tensor_t<S>(NH), dh_new = read_tensor_t<S>((T + 1) * NH);
    std::vector<S> gamma;
    if (ln) gamma = read_tensor_t<S>((size_t)2 * H);
    std::vector<S> mask = read_tensor_t<S>(has_mask ? TN * H : 0);
    DeviceBuf dW_(W), du_(u), db_(b), dx_(x), dmask(mask), dgamma(gamma);
    std::vector<S> hinit((T + 1) * NH, 0.f);
    std::memcpy(hinit.data(), h0.data(), NH * sizeof(S));
    DeviceBuf h(hinit), workspace(TN * H), act_Wx(ln ? TN * H : 0), cache1(ln ? TN * 2 : 0);
    const S* maskp = has_mask ? dmask.p : nullptr;
    if (!ln) {
      indrnn::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      fwd.Run(T, dW_.p, du_.p, db_.p, dx_.p, h.p, workspace.p, zoneout, maskp);
      require_ok(fwd.last_status(), "indrnn forward");
    } else {
      layer_norm::ForwardPass<S> ln1(T * N, H, dgamma.p, nullptr, cache1.p);
      layer_norm_indrnn::ForwardPass<S> fwd(true, N, C, H, blas, stream);
      fwd.Run(T, dW_.p, du_.p, db_.p, dx_.p, h.p, workspace.p, act_Wx.p, ln1, zoneout, maskp);
      require_ok(fwd.last_status(), "layer_norm_indrnn forward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(h);
    DeviceBuf x_t(transpose(x, TN, C)), W_t(transpose(W, C, H)), ddh_new(dh_new);
    DeviceBuf gdx(TN * C), gdW((size_t)C * H), gdu(H), gdb(H), gdh(NH), ws2(TN * H),
        gdgamma(ln ? (size_t)2 * H : 0);
    if (!ln) {
      indrnn::BackwardPass<S> bwd(N, C, H, blas, stream);
      bwd.Run(T, W_t.p, du_.p, db_.p, x_t.p, h.p, ddh_new.p, gdx.p, gdW.p, gdu.p, gdb.p, gdh.p,
              ws2.p, maskp);
      require_ok(bwd.last_status(), "indrnn backward");
    } else {
      layer_norm::BackwardPass<S> ln1(T * N, H, dgamma.p, nullptr, act_Wx.p, gdgamma.p, nullptr, cache1.p);
      layer_norm_indrnn::BackwardPass<S> bwd(N, C, H, blas, stream);
      bwd.Run(T, W_t.p, du_.p, db_.p, x_t.p, h.p, ddh_new.p, gdx.p, gdW.p, gdu.p, gdb.p, gdh.p,
              ws2.p, ln1, maskp);
      require_ok(bwd.last_status(), "layer_norm_indrnn backward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(gdx); write_tensor(gdW); write_tensor(gdu); write_tensor(gdb); write_tensor(gdh);
    if (ln) write_tensor(gdgamma);
  } else if (cell == "layer_norm") {
    // rows = T*N, dim = H; forward in two partial calls, backward in two partial calls.
    const int rows = T * N;
    std::vector<S> x = read_tensor_t<S>((size_t)rows * H), gamma = read_tensor_t<S>(H), beta = read_tensor_t<S>(H),
                       dy = read_tensor_t<S>((size_t)rows * H);
    DeviceBuf dx_(x), dgamma(gamma), dbeta(beta), ddy(dy), y((size_t)rows * H), cache((size_t)rows * 2),
        gdx((size_t)rows * H), gdgamma(H), gdbeta(H);
    layer_norm::ForwardPass<S> fwd(rows, H, dgamma.p, dbeta.p, cache.p);
    const int first = rows / 2;
    fwd.RunPartial(stream, first, dx_.p, y.p);
    require_ok(fwd.last_status(), "layer_norm forward");
    if (rows - first > 0) {
      fwd.RunPartial(stream, rows - first, dx_.p + (size_t)first * H, y.p + (size_t)first * H);
      require_ok(fwd.last_status(), "layer_norm forward");
    }
    layer_norm::BackwardPass<S> bwd(rows, H, dgamma.p, dbeta.p, dx_.p, gdgamma.p, gdbeta.p, cache.p);
    if (rows - first > 0) {
      bwd.RunPartial(stream, rows - first, ddy.p + (size_t)first * H, gdx.p + (size_t)first * H);
      require_ok(bwd.last_status(), "layer_norm backward");
    }
    if (first > 0) {
      bwd.RunPartial(stream, first, ddy.p, gdx.p);
      require_ok(bwd.last_status(), "layer_norm backward");
    }
    CHECK_HIP(hipStreamSynchronize(stream));
    write_tensor(y); write_tensor(cache); write_tensor(gdx); write_tensor(gdgamma); write_tensor(gdbeta);
  } else {
    std::fprintf(stderr, "unknown cell %s\n", cell.c_str());
    return 2;
  }
  // Everything has been synchronized by now: no kernel of either stream gave up a wait.
  require_ok(haste_hip_stream_status(stream), "haste_hip_stream_status");
  require_ok(haste_hip_stream_status(caller_stream), "haste_hip_stream_status (caller's stream)");
  if (lent) {
    hipStream_t both[2] = {stream, caller_stream};
    for (int i = 0; i < 2; ++i) {
      require_ok(haste_hip_set_workspace(both[i], nullptr, 0), "haste_hip_set_workspace(null)");
      CHECK_HIP(hipFree(lent_memory[i]));
    }
  }
  std::fclose(g_in);
  std::fclose(g_out);
  CHECK_HIP(hipStreamDestroy(stream));
  std::printf("ok\n");
  return 0;
}

int main(int argc, char** argv) {
  if (argc != 9) {
    std::fprintf(stderr, "usage: api_check <cell> T N C H zoneout in.bin out.bin\n");
    return 2;
  }
  const std::string cell = argv[1];
  const int T = std::atoi(argv[2]), N = std::atoi(argv[3]), C = std::atoi(argv[4]), H = std::atoi(argv[5]);
  const float zoneout = (float)std::atof(argv[6]);
  g_in = std::fopen(argv[7], "rb");
  g_out = std::fopen(argv[8], "wb");
  if (!g_in || !g_out) { std::fprintf(stderr, "cannot open files\n"); return 2; }
  // "f64:<cell>" runs the classes instantiated for double.
  if (cell.rfind("f64:", 0) == 0) return run<double>(cell.substr(4), T, N, C, H, zoneout);
  return run<float>(cell, T, N, C, H, zoneout);
}
