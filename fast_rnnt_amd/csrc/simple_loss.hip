// rnnt_loss_simple's forward pipeline behind one call (rnnt_loss.py:230-340):
// px/py from lm and am, the lattice recursion, optionally its backward with a
// gradient of ones (the occupation probabilities), and the reduction of the scores.
// It only chains the entry points of the other files on one stream; what it saves
// is host time, which matters once a whole call takes ~100 us on the GPU.
#include "common.hip.h"

namespace frnnt {
namespace {

template <typename R, typename Logprobs, typename Forward, typename Backward, typename Reduce>
int simple_loss_fwd(Logprobs logprobs, Forward forward, Backward backward, Reduce reduce,
                    const R *lm, const R *am, const int64_t *symbols, const int64_t *boundary,
                    R *px, R *py, R *lm_max, R *am_max, R *norm_raw, R *p, R *scores, R *px_grad,
                    R *py_grad, R *loss, int B, int S, int T, int C, int term, int rnnt_type,
                    int reduction, int checks, int32_t *status, void *stream) {
  if ((px_grad == nullptr) != (py_grad == nullptr))
    return fail(FRNNT_EINVAL, "simple_loss_fwd: px_grad and py_grad go together");
  // px / py only feed the recursion below, with the same boundary: what lies outside an
  // utterance's window need not be computed
  int rc = logprobs(lm, am, symbols, boundary, px, py, lm_max, am_max, norm_raw, B, S, T, C, term,
                    rnnt_type, boundary != nullptr, stream);
  if (rc != FRNNT_OK) return rc;
  const int modified = rnnt_type != 0;
  rc = forward(px, py, boundary, p, scores, B, S, T, modified, checks, status, stream);
  if (rc != FRNNT_OK) return rc;
  if (px_grad) {
    // with a loss to form, the backward kernel reduces the scores on its way
    if (loss && B > 0)
      return mi_backward_and_loss(px, boundary, p, px_grad, py_grad, scores, loss, B, S, T,
                                  modified, reduction, stream);
    rc = backward(px, py, boundary, p, nullptr, px_grad, py_grad, B, S, T, modified, 0, stream);
    if (rc != FRNNT_OK) return rc;
  }
  if (loss) rc = reduce(scores, loss, B, reduction, stream);
  return rc;
}

// The tail every loss function shares (e.g. rnnt_loss.py:326-340): the recursion, its
// backward with a gradient of ones when the occupation gradients are wanted, the reduction.
template <typename R, typename Forward, typename Backward, typename Reduce>
int mi_loss_fwd(Forward forward, Backward backward, Reduce reduce, const R *px, const R *py,
                const int64_t *boundary, R *p, R *scores, R *px_grad, R *py_grad, R *loss, int B,
                int S, int T, int modified, int reduction, int checks, int32_t *status,
                void *stream) {
  if ((px_grad == nullptr) != (py_grad == nullptr))
    return fail(FRNNT_EINVAL, "mi_loss_fwd: px_grad and py_grad go together");
  int rc = forward(px, py, boundary, p, scores, B, S, T, modified, checks, status, stream);
  if (rc != FRNNT_OK) return rc;
  if (px_grad) {
    // with a loss to form, the backward kernel reduces the scores on its way
    if (loss && B > 0)
      return mi_backward_and_loss(px, boundary, p, px_grad, py_grad, scores, loss, B, S, T,
                                  modified, reduction, stream);
    rc = backward(px, py, boundary, p, nullptr, px_grad, py_grad, B, S, T, modified, 0, stream);
    if (rc != FRNNT_OK) return rc;
  }
  if (loss) rc = reduce(scores, loss, B, reduction, stream);
  return rc;
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_mi_loss_fwd_f32(const float *px, const float *py, const int64_t *boundary, float *p,
                          float *scores, float *px_grad, float *py_grad, float *loss, int B, int S,
                          int T, int modified, int reduction, int checks, int32_t *status,
                          void *stream) {
  return frnnt::mi_loss_fwd<float>(frnnt_mi_forward_checked_f32, frnnt_mi_backward_f32,
                                   frnnt_loss_reduce_f32, px, py, boundary, p, scores, px_grad,
                                   py_grad, loss, B, S, T, modified, reduction, checks, status,
                                   stream);
}
int frnnt_mi_loss_fwd_f64(const double *px, const double *py, const int64_t *boundary, double *p,
                          double *scores, double *px_grad, double *py_grad, double *loss, int B,
                          int S, int T, int modified, int reduction, int checks, int32_t *status,
                          void *stream) {
  return frnnt::mi_loss_fwd<double>(frnnt_mi_forward_checked_f64, frnnt_mi_backward_f64,
                                    frnnt_loss_reduce_f64, px, py, boundary, p, scores, px_grad,
                                    py_grad, loss, B, S, T, modified, reduction, checks, status,
                                    stream);
}

int frnnt_simple_loss_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                              const int64_t *boundary, float *px, float *py, float *lm_max,
                              float *am_max, float *norm_raw, float *p, float *scores,
                              float *px_grad, float *py_grad, float *loss, int B, int S, int T,
                              int C, int termination_symbol, int rnnt_type, int reduction,
                              int checks, int32_t *status, void *stream) {
  return frnnt::simple_loss_fwd<float>(frnnt_simple_logprobs_fwd_f32, frnnt_mi_forward_checked_f32,
                                       frnnt_mi_backward_f32, frnnt_loss_reduce_f32, lm, am,
                                       symbols, boundary, px, py, lm_max, am_max, norm_raw, p,
                                       scores, px_grad, py_grad, loss, B, S, T, C,
                                       termination_symbol, rnnt_type, reduction, checks, status,
                                       stream);
}
int frnnt_simple_loss_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                              const int64_t *boundary, double *px, double *py, double *lm_max,
                              double *am_max, double *norm_raw, double *p, double *scores,
                              double *px_grad, double *py_grad, double *loss, int B, int S, int T,
                              int C, int termination_symbol, int rnnt_type, int reduction,
                              int checks, int32_t *status, void *stream) {
  return frnnt::simple_loss_fwd<double>(frnnt_simple_logprobs_fwd_f64, frnnt_mi_forward_checked_f64,
                                        frnnt_mi_backward_f64, frnnt_loss_reduce_f64, lm, am,
                                        symbols, boundary, px, py, lm_max, am_max, norm_raw, p,
                                        scores, px_grad, py_grad, loss, B, S, T, C,
                                        termination_symbol, rnnt_type, reduction, checks, status,
                                        stream);
}

}  // extern "C"
