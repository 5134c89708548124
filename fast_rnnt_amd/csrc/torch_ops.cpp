// Torch operator module of fast_rnnt_amd: fast_rnnt_amd/_C*.so.
//
// The counterpart of the reference's pybind module (fast_rnnt/python/csrc/fast_rnnt.cu:24,
// fast_rnnt/python/csrc/mutual_information.cu:27-75): plain C++ with no kernels in it.  It
// takes torch tensors, checks them, allocates the outputs with torch, takes the stream from
// c10::hip::getCurrentHIPStream and the device guard from c10::hip, and calls the C
// ABI of libfast_rnnt_amd.so (include/fast_rnnt_amd.h).  Besides the reference's three
// functions it holds the autograd nodes of the loss functions that are called once per
// training step, so that a loss call costs the host a few microseconds of C++ instead of a
// Python autograd Function and a ctypes call each way.  Everything is also registered with
// the dispatcher as torch.ops.fast_rnnt_amd.*.
//
// Built by fast_rnnt_amd/csrc/Makefile (g++ against the installed torch and pybind11
// headers; no hipify pass, no torch.utils.cpp_extension).
#include <torch/extension.h>
#include <torch/library.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <array>
#include <cstring>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "fast_rnnt_amd.h"

namespace {

using at::Tensor;
// PyTorch-ROCm labels the MI355X's tensors with device type "cuda"; this is its device guard
// for them (the counterpart of the reference's DeviceGuard, fast_rnnt/csrc/device_guard.h:31-90)
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

// ---- the C ABI, overloaded on the element type -------------------------------------------
inline int abi_mi_forward(const float *px, const float *py, const int64_t *bnd, float *p,
                          float *ans, int B, int S, int T, int modified, int checks,
                          int32_t *status, void *stream) {
  return frnnt_mi_forward_checked_f32(px, py, bnd, p, ans, B, S, T, modified, checks, status,
                                      stream);
}
inline int abi_mi_forward(const double *px, const double *py, const int64_t *bnd, double *p,
                          double *ans, int B, int S, int T, int modified, int checks,
                          int32_t *status, void *stream) {
  return frnnt_mi_forward_checked_f64(px, py, bnd, p, ans, B, S, T, modified, checks, status,
                                      stream);
}
inline int abi_mi_backward(const float *px, const float *py, const int64_t *bnd, const float *p,
                           float *ans_grad, float *gx, float *gy, int B, int S, int T,
                           int modified, int overwrite, void *stream) {
  return frnnt_mi_backward_f32(px, py, bnd, p, ans_grad, gx, gy, B, S, T, modified, overwrite,
                               stream);
}
inline int abi_mi_backward(const double *px, const double *py, const int64_t *bnd,
                           const double *p, double *ans_grad, double *gx, double *gy, int B,
                           int S, int T, int modified, int overwrite, void *stream) {
  return frnnt_mi_backward_f64(px, py, bnd, p, ans_grad, gx, gy, B, S, T, modified, overwrite,
                               stream);
}
#define FRNNT_BOTH(NAME, PARAMS_F, PARAMS_D, ARGS)                       \
  inline int abi_##NAME PARAMS_F { return frnnt_##NAME##_f32 ARGS; }     \
  inline int abi_##NAME PARAMS_D { return frnnt_##NAME##_f64 ARGS; }

FRNNT_BOTH(simple_logprobs_fwd,
           (const float *lm, const float *am, const int64_t *sym, const int64_t *bnd, float *px,
            float *py, float *lmx, float *amx, float *nr, int B, int S, int T, int C, int term,
            int kind, int window, void *st),
           (const double *lm, const double *am, const int64_t *sym, const int64_t *bnd, double *px,
            double *py, double *lmx, double *amx, double *nr, int B, int S, int T, int C, int term,
            int kind, int window, void *st),
           (lm, am, sym, bnd, px, py, lmx, amx, nr, B, S, T, C, term, kind, window, st))
FRNNT_BOTH(simple_loss_fwd,
           (const float *lm, const float *am, const int64_t *sym, const int64_t *bnd, float *px,
            float *py, float *lmx, float *amx, float *nr, float *p, float *sc, float *gx,
            float *gy, float *loss, int B, int S, int T, int C, int term, int kind, int red,
            int checks, int32_t *status, void *st),
           (const double *lm, const double *am, const int64_t *sym, const int64_t *bnd, double *px,
            double *py, double *lmx, double *amx, double *nr, double *p, double *sc, double *gx,
            double *gy, double *loss, int B, int S, int T, int C, int term, int kind, int red,
            int checks, int32_t *status, void *st),
           (lm, am, sym, bnd, px, py, lmx, amx, nr, p, sc, gx, gy, loss, B, S, T, C, term, kind,
            red, checks, status, st))
FRNNT_BOTH(simple_logprobs_bwd,
           (const float *lm, const float *am, const int64_t *sym, const int64_t *bnd,
            const float *lmx, const float *amx, const float *nr, const float *g, int gstride,
            double gscale, float *gx, float *gy, float *dmat, float *rx, float *ry, float *cy,
            float *lmg, float *amg, int B, int S, int T, int C, int term, int kind, int window,
            void *st),
           (const double *lm, const double *am, const int64_t *sym, const int64_t *bnd,
            const double *lmx, const double *amx, const double *nr, const double *g, int gstride,
            double gscale, double *gx, double *gy, double *dmat, double *rx, double *ry,
            double *cy, double *lmg, double *amg, int B, int S, int T, int C, int term, int kind,
            int window, void *st),
           (lm, am, sym, bnd, lmx, amx, nr, g, gstride, gscale, gx, gy, dmat, rx, ry, cy, lmg, amg,
            B, S, T, C, term, kind, window, st))
FRNNT_BOTH(mi_loss_fwd,
           (const float *px, const float *py, const int64_t *bnd, float *p, float *sc, float *gx,
            float *gy, float *loss, int B, int S, int T, int modified, int red, int checks,
            int32_t *status, void *st),
           (const double *px, const double *py, const int64_t *bnd, double *p, double *sc,
            double *gx, double *gy, double *loss, int B, int S, int T, int modified, int red,
            int checks, int32_t *status, void *st),
           (px, py, bnd, p, sc, gx, gy, loss, B, S, T, modified, red, checks, status, st))
FRNNT_BOTH(mi_scale_grads,
           (float *gx, float *gy, const float *g, int gstride, double gscale, int B, int S, int T,
            int modified, void *st),
           (double *gx, double *gy, const double *g, int gstride, double gscale, int B, int S,
            int T, int modified, void *st),
           (gx, gy, g, gstride, gscale, B, S, T, modified, st))
FRNNT_BOTH(loss_reduce,
           (const float *sc, float *loss, int B, int red, void *st),
           (const double *sc, double *loss, int B, int red, void *st), (sc, loss, B, red, st))
#undef FRNNT_BOTH

void check_rc(int rc, const char *what) {
  TORCH_CHECK(rc == FRNNT_OK, what, " failed (", rc, "): ", frnnt_last_error());
}

template <typename R>
R *ptr(const Tensor &t) {
  return t.defined() ? t.data_ptr<R>() : nullptr;
}
const int64_t *iptr(const Tensor &t) { return t.defined() ? t.data_ptr<int64_t>() : nullptr; }

void *stream_of(const Tensor &t) {
  return static_cast<void *>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

Tensor or_undefined(const std::optional<Tensor> &t) { return t.has_value() ? *t : Tensor(); }

// ---- boundary rows that fail their tests: reported by the device, raised later -----------
// The reference's Python layer asserts every boundary row on the host
// (mutual_information.py:277-288, rnnt_loss.py:25-42) through boundary.tolist(), which makes
// every call wait for the device.  Here the forward kernel of the recursion tests the rows
// (it skips a bad one and makes its score NaN) and stores what failed in two words of pinned
// host memory, one pair per device; the host looks at them on entry to every later call of
// this module and in check_boundaries(), and raises the reference's AssertionError then.
// set_deferred_checks(false) makes the Python layer check on the host before the call, as
// the reference does.
struct BoundaryAssertion : public std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct StatusWords {
  int32_t *host = nullptr;
  int32_t *device = nullptr;
};
std::array<StatusWords, 64> g_status;
std::mutex g_status_mutex;
bool g_deferred = true;

StatusWords status_of(int device) {
  TORCH_CHECK(device >= 0 && device < (int)g_status.size(), "device index out of range");
  std::lock_guard<std::mutex> lock(g_status_mutex);
  StatusWords &w = g_status[device];
  if (w.host == nullptr) {
    void *h = nullptr, *d = nullptr;
    TORCH_CHECK(hipHostMalloc(&h, 64, hipHostMallocDefault) == hipSuccess,
                "hipHostMalloc of the boundary status words failed");
    std::memset(h, 0, 64);
    TORCH_CHECK(hipHostGetDevicePointer(&d, h, 0) == hipSuccess,
                "hipHostGetDevicePointer of the boundary status words failed");
    w.host = static_cast<int32_t *>(h);
    w.device = static_cast<int32_t *>(d);
  }
  return w;
}

std::string describe(int code, int row) {
  std::string what;
  switch (code) {
    case FRNNT_STATUS_WINDOW:
      what = "0 <= s_begin <= s_end <= S and 0 <= t_begin <= t_end <= T";
      break;
    case FRNNT_STATUS_NO_SYMBOLS:
      what = "boundary[:, 2] >= 1";
      break;
    case FRNNT_STATUS_FEW_FRAMES:
      what = "T >= S for the modified transducer (boundary[:, 3] >= boundary[:, 2])";
      break;
    default:
      what = "unknown test " + std::to_string(code);
  }
  return "boundary row " + std::to_string(row) + " of an earlier call violates " + what +
         " (found on the device; that call's loss for the row is nan)";
}

// (code, row) of a failure the device has reported on `device`, or (0, 0); clears it.
std::pair<int, int> take_pending(int device) {
  if (device < 0 || device >= (int)g_status.size()) return {0, 0};
  int32_t *h = g_status[device].host;
  if (h == nullptr) return {0, 0};
  const int code = *reinterpret_cast<volatile int32_t *>(h);
  if (code == 0) return {0, 0};
  const int row = *reinterpret_cast<volatile int32_t *>(h + 1);
  h[0] = 0;
  h[1] = 0;
  return {code, row};
}

void raise_pending(int device) {
  const auto pending = take_pending(device);
  if (pending.first != 0) throw BoundaryAssertion(describe(pending.first, pending.second));
}

// Waits for the device, then raises what it has reported.
void check_boundaries(int64_t device) {
  DeviceGuard guard(static_cast<c10::DeviceIndex>(device));
  TORCH_CHECK(hipDeviceSynchronize() == hipSuccess, "hipDeviceSynchronize failed");
  raise_pending((int)device);
}

int32_t *status_for(const Tensor &like, const Tensor &boundary) {
  if (!g_deferred || !boundary.defined()) return nullptr;
  const int device = like.device().index();
  raise_pending(device);
  return status_of(device).device;
}

// ---- the reference's three operator functions -----------------------------------------
struct Dims {
  int B, S, T, modified;
};

Dims common_checks(const Tensor &px, const Tensor &py, const Tensor &boundary, const Tensor &p) {
  TORCH_CHECK(px.dim() == 3, "px must be 3-dimensional");
  TORCH_CHECK(py.dim() == 3, "py must be 3-dimensional.");
  TORCH_CHECK(p.dim() == 3, "p must be 3-dimensional.");
  TORCH_CHECK(px.is_cuda() && py.is_cuda() && p.is_cuda(),
              "inputs must be GPU tensors: fast_rnnt_amd has no CPU path");
  TORCH_CHECK(px.device() == py.device() && px.device() == p.device(),
              "px, py and p must share one device");
  TORCH_CHECK(px.scalar_type() == py.scalar_type() && px.scalar_type() == p.scalar_type(),
              "px, py and p must share one dtype");
  TORCH_CHECK(px.scalar_type() == at::kFloat || px.scalar_type() == at::kDouble,
              "fast_rnnt_amd supports float32 and float64 tensors here, got ", px.scalar_type());
  const int64_t B = px.size(0), S = px.size(1), T1 = px.size(2), T = py.size(2);
  const bool modified = T1 == T;
  TORCH_CHECK(T1 == (modified ? T : T + 1), "px.size(2) must be T or T + 1");
  TORCH_CHECK(py.size(0) == B && py.size(1) == S + 1, "py must have shape [B][S+1][T]");
  TORCH_CHECK(p.size(0) == B && p.size(1) == S + 1 && p.size(2) == T + 1,
              "p must have shape [B][S+1][T+1]");
  if (boundary.defined()) {
    TORCH_CHECK(boundary.dim() == 2, "boundary must be 2-dimensional.");
    TORCH_CHECK(boundary.size(0) == B && boundary.size(1) == 4, "boundary must have shape [B][4]");
    TORCH_CHECK(boundary.device() == px.device() && boundary.scalar_type() == at::kLong,
                "boundary must be an int64 tensor on the same device");
  }
  return Dims{(int)B, (int)S, (int)T, (int)modified};
}

template <typename R>
Tensor mi_forward_t(const Tensor &px, const Tensor &py, const Tensor &boundary, Tensor &p,
                    const Dims &d) {
  Tensor pxc = px.contiguous(), pyc = py.contiguous();
  Tensor bnd = boundary.defined() ? boundary.contiguous() : Tensor();
  Tensor pc = p.is_contiguous() ? p : at::empty(p.sizes(), p.options());
  Tensor ans = at::empty({d.B}, px.options());
  // a bad row also makes ans[b] NaN; the status words only add the AssertionError later
  int32_t *status = status_for(px, bnd);
  check_rc(abi_mi_forward(ptr<R>(pxc), ptr<R>(pyc), iptr(bnd), ptr<R>(pc), ptr<R>(ans), d.B, d.S,
                          d.T, d.modified, 0, status, stream_of(px)),
           "frnnt_mi_forward");
  if (!pc.is_same(p)) p.copy_(pc);
  return ans;
}

// fast_rnnt/python/csrc/mutual_information.cu:27-45
Tensor mutual_information_forward(const Tensor &px, const Tensor &py,
                                  const std::optional<Tensor> &boundary_, Tensor p) {
  const Tensor boundary = or_undefined(boundary_);
  const Dims d = common_checks(px, py, boundary, p);
  DeviceGuard guard(px.device());
  return px.scalar_type() == at::kFloat ? mi_forward_t<float>(px, py, boundary, p, d)
                                        : mi_forward_t<double>(px, py, boundary, p, d);
}

template <typename R>
std::vector<Tensor> mi_backward_t(const Tensor &px, const Tensor &py, const Tensor &boundary,
                                  const Tensor &p, Tensor &ans_grad, const Dims &d) {
  Tensor pxc = px.contiguous(), pyc = py.contiguous(), pc = p.contiguous();
  Tensor bnd = boundary.defined() ? boundary.contiguous() : Tensor();
  Tensor agc = ans_grad.contiguous();
  Tensor gx = at::empty(pxc.sizes(), pxc.options()), gy = at::empty(pyc.sizes(), pyc.options());
  check_rc(abi_mi_backward(ptr<R>(pxc), ptr<R>(pyc), iptr(bnd), ptr<R>(pc), ptr<R>(agc),
                           ptr<R>(gx), ptr<R>(gy), d.B, d.S, d.T, d.modified, 1, stream_of(px)),
           "frnnt_mi_backward");
  if (!agc.is_same(ans_grad)) ans_grad.copy_(agc);
  return {gx, gy};
}

// fast_rnnt/python/csrc/mutual_information.cu:47-67.  Like the reference's GPU path
// (mutual_information_cuda.cu:667-669) ans_grad is overwritten with the gradient that
// reaches the start of each lattice.
std::vector<Tensor> mutual_information_backward(const Tensor &px, const Tensor &py,
                                                const std::optional<Tensor> &boundary_,
                                                const Tensor &p, Tensor ans_grad) {
  const Tensor boundary = or_undefined(boundary_);
  const Dims d = common_checks(px, py, boundary, p);
  TORCH_CHECK(ans_grad.dim() == 1, "ans_grad must be 1-dimensional.");
  TORCH_CHECK(ans_grad.size(0) == d.B, "ans_grad must have B elements");
  TORCH_CHECK(ans_grad.device() == px.device() && ans_grad.scalar_type() == px.scalar_type(),
              "ans_grad must match px in device and dtype");
  DeviceGuard guard(px.device());
  return px.scalar_type() == at::kFloat ? mi_backward_t<float>(px, py, boundary, p, ans_grad, d)
                                        : mi_backward_t<double>(px, py, boundary, p, ans_grad, d);
}

// fast_rnnt/python/csrc/mutual_information.cu:69-75: PyTorch-ROCm shows the MI355X as
// device type "cuda".
bool with_cuda() { return true; }

// ---- the tail every loss shares: recursion, its eager backward, the reduction ------------
// One autograd node: forward = frnnt_mi_loss_fwd (recursion, its backward with a gradient of
// ones as mutual_information.py:159-168 does whenever gradients will be wanted, and the
// reduction rnnt_loss.py:326-340); backward = frnnt_mi_scale_grads, the in-place scaling of
// the occupation gradients by the gradient of the scores (mutual_information.py:173-181),
// with the reduction's sign and 1/B folded in.
constexpr int kRedNone = 0, kRedMean = 1;

// element offsets of consecutive buffers, each 16-byte aligned for 4- and 8-byte elements
struct Carver {
  int64_t total = 0;
  int64_t take(int64_t n) {
    const int64_t at = total;
    total += (n + 3) & ~int64_t(3);
    return at;
  }
};

struct RecursionLossFn : public torch::autograd::Function<RecursionLossFn> {
  // (an absent boundary travels as an empty optional: the autograd machinery does not take
  // undefined tensors as inputs)
  static variable_list forward(AutogradContext *ctx, const Tensor &px, const Tensor &py,
                               const std::optional<Tensor> &boundary_, bool want_grads,
                               int64_t reduction, int64_t checks, bool need_grad) {
    const Tensor boundary = or_undefined(boundary_);
    return px.scalar_type() == at::kFloat
               ? run<float>(ctx, px, py, boundary, want_grads, reduction, checks, need_grad)
               : run<double>(ctx, px, py, boundary, want_grads, reduction, checks, need_grad);
  }

  template <typename R>
  static variable_list run(AutogradContext *ctx, const Tensor &px_, const Tensor &py_,
                           const Tensor &boundary, bool want_grads, int64_t reduction,
                           int64_t checks, bool need_grad) {
    const Tensor px = px_.contiguous(), py = py_.contiguous();
    const int64_t B = px.size(0), S = px.size(1), T1 = px.size(2), T = py.size(2);
    const Tensor bnd = boundary.defined() ? boundary.contiguous() : Tensor();
    ctx->set_materialize_grads(false);
    DeviceGuard guard(px.device());
    const auto opts = px.options();
    Tensor p = at::empty({B, S + 1, T + 1}, opts), scores = at::empty({B}, opts);
    Tensor gx, gy;
    if (want_grads || need_grad) {
      gx = at::empty({B, S, T1}, opts);
      gy = at::empty({B, S + 1, T}, opts);
    }
    Tensor loss = reduction == kRedNone ? at::empty({B}, opts) : at::empty({}, opts);
    check_rc(abi_mi_loss_fwd(ptr<R>(px), ptr<R>(py), iptr(bnd), ptr<R>(p), ptr<R>(scores),
                             ptr<R>(gx), ptr<R>(gy), ptr<R>(loss), (int)B, (int)S, (int)T,
                             (int)(T1 == T), (int)reduction, (int)checks, status_for(px, bnd),
                             stream_of(px)),
             "frnnt_mi_loss_fwd");
    if (need_grad) {
      ctx->save_for_backward({gx, gy});
      ctx->saved_data["reduction"] = reduction;
    }
    // (undefined tensors cannot be outputs of an autograd node)
    if (!gx.defined()) return {loss};
    ctx->mark_non_differentiable({gx, gy});
    return {loss, gx, gy};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grads) {
    variable_list out(7);
    const Tensor &g_loss = grads[0];
    if (!g_loss.defined()) return out;
    const auto saved = ctx->get_saved_variables();
    Tensor gx = saved[0], gy = saved[1];
    const int64_t reduction = ctx->saved_data["reduction"].toInt();
    const int64_t B = gx.size(0), S = gx.size(1), T1 = gx.size(2), T = gy.size(2);
    DeviceGuard guard(gx.device());
    const Tensor g = g_loss.contiguous();
    const int stride = reduction == kRedNone ? 1 : 0;
    const double scale = reduction == kRedMean ? -1.0 / (double)B : -1.0;
    int rc;
    if (gx.scalar_type() == at::kFloat)
      rc = abi_mi_scale_grads(ptr<float>(gx), ptr<float>(gy), ptr<float>(g), stride, scale,
                              (int)B, (int)S, (int)T, (int)(T1 == T), stream_of(gx));
    else
      rc = abi_mi_scale_grads(ptr<double>(gx), ptr<double>(gy), ptr<double>(g), stride, scale,
                              (int)B, (int)S, (int)T, (int)(T1 == T), stream_of(gx));
    check_rc(rc, "frnnt_mi_scale_grads");
    out[0] = gx;
    out[1] = gy;
    return out;
  }
};

void require_float_gpu(const Tensor &t, const char *name) {
  TORCH_CHECK(t.is_cuda(), "fast_rnnt_amd runs on GPU tensors only (no CPU path): ", name);
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kDouble,
              "fast_rnnt_amd supports float32 and float64 tensors here, got ", t.scalar_type());
}

using LossResult = std::tuple<Tensor, std::optional<Tensor>, std::optional<Tensor>>;

LossResult as_result(const variable_list &out) {
  std::optional<Tensor> gx, gy;
  if (out.size() == 3) {
    gx = out[1];
    gy = out[2];
  }
  return LossResult(out[0], gx, gy);
}

LossResult recursion_loss(const Tensor &px, const Tensor &py,
                          const std::optional<Tensor> &boundary_, bool return_grad,
                          int64_t reduction, int64_t checks) {
  const Tensor boundary = or_undefined(boundary_);
  require_float_gpu(px, "px");
  TORCH_CHECK(px.dim() == 3 && py.dim() == 3, "px and py must be 3-dimensional");
  TORCH_CHECK(py.device() == px.device() && py.scalar_type() == px.scalar_type(),
              "px and py must share device and dtype");
  const int64_t B = px.size(0), S = px.size(1), T1 = px.size(2), T = py.size(2);
  TORCH_CHECK((T1 == T || T1 == T + 1) && py.size(0) == B && py.size(1) == S + 1,
              "px must be [B][S][T or T+1] and py [B][S+1][T]");
  TORCH_CHECK(reduction >= 0 && reduction <= 2, "reduction must be 0 (none), 1 (mean) or 2 (sum)");
  if (boundary.defined())
    TORCH_CHECK(boundary.dim() == 2 && boundary.size(0) == B && boundary.size(1) == 4 &&
                    boundary.scalar_type() == at::kLong && boundary.device() == px.device(),
                "boundary must be an int64 [B][4] tensor on the same device");
  const bool need_grad = at::GradMode::is_enabled() && (px.requires_grad() || py.requires_grad());
  return as_result(
      RecursionLossFn::apply(px, py, boundary_, return_grad, reduction, checks, need_grad));
}

// ---- rnnt_loss_simple behind one autograd node -------------------------------------------
// forward = frnnt_simple_loss_fwd: px / py (row maxima + MFMA contraction,
// rnnt_loss.py:66-227), the recursion, its backward with a gradient of ones
// (mutual_information.py:159-168), the reduction (rnnt_loss.py:326-340);
// backward = frnnt_simple_logprobs_bwd: scales the occupation gradients in place by the
// gradient of the scores (mutual_information.py:173-181) and pushes them through the two
// gradient products to lm.grad and am.grad.
void apply_delay_penalty(Tensor px, const Tensor &boundary, bool regular, double delay_penalty) {
  // px += ((T_b - 1) / 2 - t) * delay_penalty, in the reference's operation order
  // (rnnt_loss.py:309-324)
  const int64_t B = px.size(0), T0 = px.size(2);
  const int64_t T = regular ? T0 - 1 : T0;
  Tensor offset;
  if (boundary.defined())
    offset = at::true_divide(boundary.select(1, 3) - 1, 2);
  else
    offset = at::scalar_tensor((double)(T - 1) / 2, px.options()).expand({B, 1, 1});
  Tensor penalty = offset.reshape({B, 1, 1}) -
                   at::arange(T0, px.options().dtype(at::kLong)).reshape({1, 1, T0});
  penalty = penalty * delay_penalty;
  px += penalty.to(px.scalar_type());
}

struct SimpleLossFn : public torch::autograd::Function<SimpleLossFn> {
  static variable_list forward(AutogradContext *ctx, const Tensor &lm, const Tensor &am,
                               const Tensor &symbols, const std::optional<Tensor> &boundary_,
                               int64_t term, int64_t kind, double delay_penalty, bool want_grads,
                               int64_t reduction, int64_t checks, bool need_lm, bool need_am) {
    const Tensor boundary = or_undefined(boundary_);
    return am.scalar_type() == at::kFloat
               ? run<float>(ctx, lm, am, symbols, boundary, term, kind, delay_penalty, want_grads,
                            reduction, checks, need_lm, need_am)
               : run<double>(ctx, lm, am, symbols, boundary, term, kind, delay_penalty,
                             want_grads, reduction, checks, need_lm, need_am);
  }

  template <typename R>
  static variable_list run(AutogradContext *ctx, const Tensor &lm_, const Tensor &am_,
                           const Tensor &symbols, const Tensor &boundary, int64_t term,
                           int64_t kind, double delay_penalty, bool want_grads, int64_t reduction,
                           int64_t checks, bool need_lm, bool need_am) {
    const Tensor lm = lm_.contiguous(), am = am_.contiguous(), sym = symbols.contiguous();
    const Tensor bnd = boundary.defined() ? boundary.contiguous() : Tensor();
    const int64_t B = am.size(0), T = am.size(1), C = am.size(2), S = lm.size(1) - 1;
    const int64_t T1 = kind == 0 ? T + 1 : T;
    const bool need_grad = need_lm || need_am;
    ctx->set_materialize_grads(false);
    DeviceGuard guard(am.device());
    void *stream = stream_of(am);
    const auto opts = am.options();
    // internal buffers in one allocation: px | py | lm_max | am_max | norm_raw | p | scores
    const int64_t n_px = B * S * T1, n_py = B * (S + 1) * T;
    Carver carve;
    const int64_t o_px = carve.take(n_px), o_py = carve.take(n_py),
                  o_lmx = carve.take(B * (S + 1)), o_amx = carve.take(B * T),
                  o_nr = carve.take(need_grad ? n_py : 0),
                  o_p = carve.take(B * (S + 1) * (T + 1)), o_sc = carve.take(B);
    Tensor work = at::empty({carve.total}, opts);
    R *w = work.data_ptr<R>();
    Tensor gx, gy;
    if (want_grads || need_grad) {
      gx = at::empty({B, S, T1}, opts);
      gy = at::empty({B, S + 1, T}, opts);
    }
    Tensor loss = reduction == kRedNone ? at::empty({B}, opts) : at::empty({}, opts);
    R *nr = need_grad ? w + o_nr : nullptr;
    int32_t *status = status_for(am, bnd);
    if (delay_penalty > 0.0) {
      // the penalty is applied to px between the two stages (rnnt_loss.py:309-326)
      check_rc(abi_simple_logprobs_fwd(ptr<R>(lm), ptr<R>(am), iptr(sym), iptr(bnd), w + o_px,
                                       w + o_py, w + o_lmx, w + o_amx, nr, (int)B, (int)S, (int)T,
                                       (int)C, (int)term, (int)kind, bnd.defined() ? 1 : 0,
                                       stream),
               "frnnt_simple_logprobs_fwd");
      apply_delay_penalty(work.narrow(0, o_px, n_px).view({B, S, T1}), boundary, kind == 0,
                          delay_penalty);
      const int modified = kind != 0;
      check_rc(abi_mi_forward(w + o_px, w + o_py, iptr(bnd), w + o_p, w + o_sc, (int)B, (int)S,
                              (int)T, modified, (int)checks, status, stream),
               "frnnt_mi_forward");
      if (gx.defined())
        check_rc(abi_mi_backward(w + o_px, w + o_py, iptr(bnd), w + o_p, (R *)nullptr, ptr<R>(gx),
                                 ptr<R>(gy), (int)B, (int)S, (int)T, modified, 0, stream),
                 "frnnt_mi_backward");
      check_rc(abi_loss_reduce(w + o_sc, ptr<R>(loss), (int)B, (int)reduction, stream),
               "frnnt_loss_reduce");
    } else {
      check_rc(abi_simple_loss_fwd(ptr<R>(lm), ptr<R>(am), iptr(sym), iptr(bnd), w + o_px,
                                   w + o_py, w + o_lmx, w + o_amx, nr, w + o_p, w + o_sc,
                                   ptr<R>(gx), ptr<R>(gy), ptr<R>(loss), (int)B, (int)S, (int)T,
                                   (int)C, (int)term, (int)kind, (int)reduction, (int)checks,
                                   status, stream),
               "frnnt_simple_loss_fwd");
    }
    if (need_grad) {
      // (an absent boundary is not saved: saved tensors must be defined)
      if (bnd.defined())
        ctx->save_for_backward({lm, am, sym, work, gx, gy, bnd});
      else
        ctx->save_for_backward({lm, am, sym, work, gx, gy});
      ctx->saved_data["term"] = term;
      ctx->saved_data["kind"] = kind;
      ctx->saved_data["reduction"] = reduction;
      ctx->saved_data["o_lmx"] = o_lmx;
      ctx->saved_data["o_amx"] = o_amx;
      ctx->saved_data["o_nr"] = o_nr;
      ctx->saved_data["need_lm"] = need_lm;
      ctx->saved_data["need_am"] = need_am;
    }
    // (undefined tensors cannot be outputs of an autograd node)
    if (!gx.defined()) return {loss};
    ctx->mark_non_differentiable({gx, gy});
    return {loss, gx, gy};
  }

  static variable_list backward(AutogradContext *ctx, variable_list grads) {
    variable_list out(12);
    const Tensor &g_loss = grads[0];
    if (!g_loss.defined()) return out;
    const auto saved = ctx->get_saved_variables();
    const Tensor &am = saved[1];
    if (am.scalar_type() == at::kFloat)
      run_backward<float>(ctx, saved, g_loss, out);
    else
      run_backward<double>(ctx, saved, g_loss, out);
    return out;
  }

  template <typename R>
  static void run_backward(AutogradContext *ctx, const variable_list &saved, const Tensor &g_loss,
                           variable_list &out) {
    const Tensor &lm = saved[0], &am = saved[1], &sym = saved[2], &work = saved[3];
    Tensor gx = saved[4], gy = saved[5];
    const Tensor bnd = saved.size() > 6 ? saved[6] : Tensor();
    const int64_t term = ctx->saved_data["term"].toInt(), kind = ctx->saved_data["kind"].toInt(),
                  reduction = ctx->saved_data["reduction"].toInt(),
                  o_lmx = ctx->saved_data["o_lmx"].toInt(),
                  o_amx = ctx->saved_data["o_amx"].toInt(), o_nr = ctx->saved_data["o_nr"].toInt();
    const bool need_lm = ctx->saved_data["need_lm"].toBool(),
               need_am = ctx->saved_data["need_am"].toBool();
    const int64_t B = am.size(0), T = am.size(1), C = am.size(2), S = lm.size(1) - 1;
    DeviceGuard guard(am.device());
    // d loss / d scores[b] = scale * g_loss[b * stride]
    const Tensor g = g_loss.contiguous();
    const int stride = reduction == kRedNone ? 1 : 0;
    const double scale = reduction == kRedMean ? -1.0 / (double)B : -1.0;
    const int64_t ldd = (T + 3) / 4 * 4;
    // scratch in one allocation: dmat | row_x | row_y | col_y
    Carver carve;
    const int64_t o_d = carve.take(B * (S + 1) * ldd), o_rx = carve.take(B * (S + 1)),
                  o_ry = carve.take(B * (S + 1)), o_cy = carve.take(B * T);
    Tensor scratch = at::empty({carve.total}, am.options());
    R *s = scratch.data_ptr<R>();
    R *w = work.data_ptr<R>();
    Tensor lm_grad = need_lm ? at::empty(lm.sizes(), lm.options()) : Tensor();
    Tensor am_grad = need_am ? at::empty(am.sizes(), am.options()) : Tensor();
    // gx / gy are scaled in place by the scores' gradient, exactly as the recursion's autograd
    // node does to the tensors it handed out
    check_rc(abi_simple_logprobs_bwd(ptr<R>(lm), ptr<R>(am), iptr(sym), iptr(bnd), w + o_lmx,
                                     w + o_amx, w + o_nr, ptr<R>(g), stride, scale, ptr<R>(gx),
                                     ptr<R>(gy), s + o_d, s + o_rx, s + o_ry, s + o_cy,
                                     ptr<R>(lm_grad), ptr<R>(am_grad), (int)B, (int)S, (int)T,
                                     (int)C, (int)term, (int)kind, bnd.defined() ? 1 : 0,
                                     stream_of(am)),
             "frnnt_simple_logprobs_bwd");
    out[0] = lm_grad;
    out[1] = am_grad;
  }
};

LossResult simple_loss(const Tensor &lm, const Tensor &am, const Tensor &symbols,
                       const std::optional<Tensor> &boundary_, int64_t termination_symbol,
                       int64_t rnnt_type, double delay_penalty, bool return_grad,
                       int64_t reduction, int64_t checks) {
  const Tensor boundary = or_undefined(boundary_);
  require_float_gpu(am, "am");
  TORCH_CHECK(lm.dim() == 3 && am.dim() == 3 && symbols.dim() == 2,
              "lm and am must be 3-dimensional, symbols 2-dimensional");
  const int64_t B = am.size(0), S = lm.size(1) - 1;
  TORCH_CHECK(lm.size(0) == B && lm.size(2) == am.size(2) && symbols.size(0) == B &&
                  symbols.size(1) == S,
              "lm must be [B][S+1][C], am [B][T][C], symbols [B][S]");
  TORCH_CHECK(lm.device() == am.device() && symbols.device() == am.device(),
              "all tensors must be on the same device");
  TORCH_CHECK(lm.scalar_type() == am.scalar_type(),
              "floating-point tensors must share one dtype");
  TORCH_CHECK(symbols.scalar_type() == at::kLong, "symbols must be an int64 tensor, got ",
              symbols.scalar_type());
  if (boundary.defined())
    TORCH_CHECK(boundary.dim() == 2 && boundary.size(0) == B && boundary.size(1) == 4 &&
                    boundary.scalar_type() == at::kLong && boundary.device() == am.device(),
                "boundary must be an int64 [B][4] tensor on the same device");
  TORCH_CHECK(rnnt_type >= 0 && rnnt_type <= 2, "rnnt_type must be 0, 1 or 2");
  TORCH_CHECK(reduction >= 0 && reduction <= 2, "reduction must be 0 (none), 1 (mean) or 2 (sum)");
  const bool grad_mode = at::GradMode::is_enabled();
  const bool need_lm = grad_mode && lm.requires_grad(), need_am = grad_mode && am.requires_grad();
  return as_result(SimpleLossFn::apply(lm, am, symbols, boundary_, termination_symbol, rnnt_type,
                                       delay_penalty, return_grad, reduction, checks, need_lm,
                                       need_am));
}

void set_deferred_checks(bool on) { g_deferred = on; }
bool deferred_checks() { return g_deferred; }

}  // namespace

// ---- dispatcher registration: torch.ops.fast_rnnt_amd.* -----------------------------------
TORCH_LIBRARY(fast_rnnt_amd, m) {
  m.def("mutual_information_forward(Tensor px, Tensor py, Tensor? boundary, Tensor(a!) p) -> Tensor");
  m.def(
      "mutual_information_backward(Tensor px, Tensor py, Tensor? boundary, Tensor p, "
      "Tensor(a!) ans_grad) -> Tensor[]");
  m.def(
      "recursion_loss(Tensor px, Tensor py, Tensor? boundary, bool return_grad, int reduction, "
      "int checks) -> (Tensor, Tensor?, Tensor?)");
  m.def(
      "simple_loss(Tensor lm, Tensor am, Tensor symbols, Tensor? boundary, int termination_symbol, "
      "int rnnt_type, float delay_penalty, bool return_grad, int reduction, int checks) -> "
      "(Tensor, Tensor?, Tensor?)");
}
// (PyTorch-ROCm keeps the dispatch key name CUDA for the MI355X)
TORCH_LIBRARY_IMPL(fast_rnnt_amd, CUDA, m) {
  m.impl("mutual_information_forward", &mutual_information_forward);
  m.impl("mutual_information_backward", &mutual_information_backward);
  m.impl("recursion_loss", &recursion_loss);
  m.impl("simple_loss", &simple_loss);
}
// The loss ops carry their own autograd nodes: the same functions serve the Autograd key
// (they call the C ABI themselves and never re-dispatch).
TORCH_LIBRARY_IMPL(fast_rnnt_amd, Autograd, m) {
  m.impl("recursion_loss", &recursion_loss);
  m.impl("simple_loss", &simple_loss);
}

PYBIND11_MODULE(_C, m) {
  m.doc() = "fast_rnnt_amd operator module (torch tensors -> C ABI of libfast_rnnt_amd.so)";
  py::register_exception<BoundaryAssertion>(m, "BoundaryAssertionError", PyExc_AssertionError);
  m.def("mutual_information_forward", &mutual_information_forward, py::arg("px"), py::arg("py"),
        py::arg("boundary"), py::arg("p"));
  m.def("mutual_information_backward", &mutual_information_backward, py::arg("px"),
        py::arg("py"), py::arg("boundary"), py::arg("p"), py::arg("ans_grad"));
  m.def("with_cuda", &with_cuda);
  m.def("recursion_loss", &recursion_loss, py::arg("px"), py::arg("py"), py::arg("boundary"),
        py::arg("return_grad"), py::arg("reduction"), py::arg("checks") = 0);
  m.def("simple_loss", &simple_loss, py::arg("lm"), py::arg("am"), py::arg("symbols"),
        py::arg("boundary"), py::arg("termination_symbol"), py::arg("rnnt_type"),
        py::arg("delay_penalty"), py::arg("return_grad"), py::arg("reduction"),
        py::arg("checks") = 0);
  m.def("set_deferred_checks", &set_deferred_checks, py::arg("on"));
  m.def("deferred_checks", &deferred_checks);
  m.def("check_boundaries", &check_boundaries, py::arg("device"));
  m.def("take_pending", &take_pending, py::arg("device"));
}
