/*
 * fast_rnnt_amd -- C ABI of the MI355X (gfx950) library for the fast_rnnt loss
 * hot path.  Shared library: fast_rnnt_amd/csrc/libfast_rnnt_amd.so.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer to a dense, row-major (last axis
 *     fastest) buffer unless stated otherwise; the caller owns and allocates
 *     every buffer, outputs included;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work
 *     is only enqueued, nothing here synchronises or allocates;
 *   - the device the pointers live on must be current when calling;
 *   - return value 0 = enqueued; a negative value is an FRNNT_E* code and
 *     frnnt_last_error() then describes the failure (thread-local text);
 *   - B batch, S symbols, T frames, C vocabulary size; `modified` = 1 when px has
 *     T columns (the "modified"/"constrained" lattices), 0 when it has T+1;
 *   - `boundary` is int64 [B][4] = (s_begin, t_begin, s_end, t_end) or NULL for
 *     (0, 0, S, T) on every row.  A row that violates
 *     0 <= s_begin <= s_end <= S or 0 <= t_begin <= t_end <= T is skipped and its
 *     `ans` is set to NaN (its gradients to 0); nothing is read out of bounds.
 *   - suffix _f32 / _f64 = element type of the floating-point buffers.
 */
#ifndef FAST_RNNT_AMD_H_
#define FAST_RNNT_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FRNNT_OK 0
#define FRNNT_EINVAL (-1)  /* bad argument (null pointer, negative size, ...) */
#define FRNNT_ELAUNCH (-2) /* the HIP runtime refused the launch             */
#define FRNNT_ELIMIT (-3)  /* a size exceeds what the kernels support        */
/*
 * Size limits (FRNNT_ELIMIT): the kernels address one utterance's arrays with 32-bit
 * byte offsets -- the lattice (S+1) x (T+1) of the recursion must stay below 1 GiB per
 * utterance, and for the float32 simple / smoothed loss an utterance's lm ((S+1) x C), am
 * (T x C) and lattice below 2 GiB each; the recursion holds one row of T+1 scores per
 * sweep wave in LDS (T up to a few ten thousand frames); get_rnnt_prune_ranges holds T
 * window starts in LDS (T <= 38400).  The batch size has no limit of its own.
 */

/* Library version, major*100 + minor. */
int frnnt_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char *frnnt_last_error(void);

/*
 * Test hook (no counterpart in the reference).  The recursion kernels synchronise their
 * waves through counters with BOUNDED waits: a wave that polls `polls` times in vain
 * gives up, and the utterance's outputs are marked -- ans[b] = NaN from the forward
 * kernel; NaN at the first cell of the window in px_grad and py_grad (and in ans_grad when
 * it is written back) from the backward kernel -- so a wait that never ends shows as NaN,
 * never as a plausible number, and every kernel still exits.  The default (2^22 polls,
 * seconds) is never reached in normal operation; a tiny value lets a test walk that path.
 * polls <= 0 restores the default.  Process-wide, not synchronised with running launches.
 */
void frnnt_set_spin_limit(int polls);

/*
 * Lattice recursion, forward.  Replaces
 *   _fast_rnnt.mutual_information_forward
 *     (fast_rnnt/python/csrc/mutual_information.cu:27-45), i.e.
 *   MutualInformationCpu / MutualInformationCuda
 *     (fast_rnnt/csrc/mutual_information.h:116-126,
 *      fast_rnnt/csrc/mutual_information_cpu.cu:50-124).
 *   px  [B][S][T+1] (modified: [B][S][T])      in
 *   py  [B][S+1][T]                            in
 *   p   [B][S+1][T+1]                          out: only the boundary window of
 *                                              each row is written
 *   ans [B]                                    out: p[b][s_end][t_end]
 */
int frnnt_mi_forward_f32(const float *px, const float *py, const int64_t *boundary,
                         float *p, float *ans, int B, int S, int T, int modified,
                         void *stream);
int frnnt_mi_forward_f64(const double *px, const double *py, const int64_t *boundary,
                         double *p, double *ans, int B, int S, int T, int modified,
                         void *stream);
/*
 * frnnt_mi_forward_* that also REPORTS a bad boundary row, for callers that do not want to
 * wait for a host copy of the rows before every call (the reference's Python layer checks
 * them through boundary.tolist(), mutual_information.py:277-288, rnnt_loss.py:25-42, which
 * waits for the device).  Every row is tested on the device anyway; a row that fails is
 * skipped (ans[b] = NaN) and, when `status` is given, the kernel stores the failed test in
 * status[0] and the row's index in status[1] (any one of the failing rows).  `status`: two
 * int32 the host can read once the kernel has run, e.g. pinned host memory
 * (hipHostMalloc), zeroed by the caller; it is only ever written on a failure.
 *   checks: FRNNT_CHECK_* bits for the tests of validate_st_lengths on top of the window's
 *           range (which is always tested).
 */
#define FRNNT_CHECK_SYMBOLS 1    /* s_end >= 1                                (rnnt_loss.py:38-39) */
#define FRNNT_CHECK_FRAMES 2     /* t_end >= s_end, non-regular lattices      (rnnt_loss.py:40-42) */
#define FRNNT_STATUS_WINDOW 1    /* not 0 <= s_begin <= s_end <= S, 0 <= t_begin <= t_end <= T */
#define FRNNT_STATUS_NO_SYMBOLS 2
#define FRNNT_STATUS_FEW_FRAMES 3
int frnnt_mi_forward_checked_f32(const float *px, const float *py, const int64_t *boundary,
                                 float *p, float *ans, int B, int S, int T, int modified,
                                 int checks, int32_t *status, void *stream);
int frnnt_mi_forward_checked_f64(const double *px, const double *py, const int64_t *boundary,
                                 double *p, double *ans, int B, int S, int T, int modified,
                                 int checks, int32_t *status, void *stream);

/*
 * Lattice recursion, backward.  Replaces
 *   _fast_rnnt.mutual_information_backward
 *     (fast_rnnt/python/csrc/mutual_information.cu:47-67), i.e.
 *   MutualInformationBackwardCpu / ...Cuda
 *     (fast_rnnt/csrc/mutual_information.h:136-143,
 *      fast_rnnt/csrc/mutual_information_cpu.cu:128-256).
 *   p        [B][S+1][T+1]   in: the table frnnt_mi_forward_* produced
 *   ans_grad [B]             in, or NULL for a gradient of 1 on every row (then
 *                            nothing is written back); if overwrite_ans_grad != 0 it is overwritten
 *                            with the gradient that reaches (s_begin, t_begin),
 *                            which equals the input when the sweep is consistent
 *                            (mutual_information_cuda.cu:667-669)
 *   px_grad  same shape as px, py_grad same shape as py: out.  Every element is
 *            written: the window gets the gradients, the rest exact zeros.
 * The split of a cell's gradient follows the CPU reference: d1 = exp(term1 - p),
 * d2 = 1 - d1, both 0 when d1 is not finite.
 */
int frnnt_mi_backward_f32(const float *px, const float *py, const int64_t *boundary,
                          const float *p, float *ans_grad, float *px_grad,
                          float *py_grad, int B, int S, int T, int modified,
                          int overwrite_ans_grad, void *stream);
int frnnt_mi_backward_f64(const double *px, const double *py, const int64_t *boundary,
                          const double *p, double *ans_grad, double *px_grad,
                          double *py_grad, int B, int S, int T, int modified,
                          int overwrite_ans_grad, void *stream);

/*
 * px / py of the simple (additive-joiner) RNN-T loss.  Replaces the tensor
 * algebra of get_rnnt_logprobs (fast_rnnt/python/fast_rnnt/rnnt_loss.py:66-227):
 * row maxima, the exp(lm) exp(am)^T contraction (fp32 / fp64 MFMA with the
 * exponentials fused into the operand loads), log, and the px / py assembly
 * including the -inf column(s) of the regular lattice and the constrained
 * "px += py[:, 1:]" step.
 *   lm [B][S+1][C], am [B][T][C], symbols int64 [B][S]              in
 *   boundary int64 [B][4] or NULL: only boundary[b][3] is used (regular lattice)
 *   px [B][S][T+1] (rnnt_type 0) or [B][S][T] (1, 2); py [B][S+1][T]   out
 *   lm_max [B][S+1], am_max [B][T]                                  out (row maxima)
 *   norm_raw [B][S+1][T] or NULL  out: log(sum_c exp(lm-lm_max) exp(am-am_max) + tiny),
 *                                 needed by the backward entry point
 *   rnnt_type: 0 regular, 1 modified, 2 constrained
 *   window_only: 0 = every cell is computed.  1 (with a boundary; float32 kernels) = the
 *   caller goes on to the lattice recursion with the same boundary, which only looks at
 *   rows <= s_end and frames <= t_end of utterance b: what lies past them in px, py,
 *   norm_raw and am_max is left undefined (tiles past t_end are not computed at all).
 *   The backward entry point then needs the same flag.
 */
int frnnt_simple_logprobs_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                  const int64_t *boundary, float *px, float *py, float *lm_max,
                                  float *am_max, float *norm_raw, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream);
int frnnt_simple_logprobs_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, double *px, double *py, double *lm_max,
                                  double *am_max, double *norm_raw, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream);

/*
 * Backward of the above: what autograd derives for rnnt_loss.py:174-225, as one
 * elementwise pass plus two MFMA GEMMs.
 *   px_grad, py_grad: dL/dpx, dL/dpy (shapes of px, py)                    in
 *   score_grad or NULL: when given, px_grad[b] and py_grad[b] are first multiplied
 *     IN PLACE by score_grad_scale * score_grad[b * score_grad_stride] -- the scaling
 *     step of the recursion's autograd backward (mutual_information.py:173-181), for
 *     callers that hold the occupation gradients and the gradient of the scores
 *     separately.  score_grad_stride 1: one value per utterance; 0: one scalar for
 *     all (the gradient of a summed or averaged loss, with the sign and the 1/B of
 *     rnnt_loss.py:160-169 in score_grad_scale)
 *   dmat [B][S+1][T rounded up to a multiple of 4], row_x [B][S+1], row_y [B][S+1],
 *   col_y [B][T]                                                           scratch
 *     (what the library keeps there is its own business: besides D and its row and column
 *     sums, the last entry of every row of row_x holds, as an int, the order in which the
 *     utterances are dealt out to the XCDs)
 *   lm_grad [B][S+1][C], am_grad [B][T][C]: out; either may be NULL to skip it
 *   window_only: 1 (with a boundary) = px_grad / py_grad vanish outside each utterance's
 *   boundary window, as the recursion's backward leaves them: nothing outside is read,
 *   the sums stop at s_end / t_end, and am_grad rows of frames >= t_end are stored as
 *   exact zeros without being computed.  Required when the forward ran with window_only.
 */
int frnnt_simple_logprobs_bwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                  const int64_t *boundary, const float *lm_max,
                                  const float *am_max, const float *norm_raw,
                                  const float *score_grad, int score_grad_stride,
                                  double score_grad_scale, float *px_grad, float *py_grad,
                                  float *dmat, float *row_x, float *row_y, float *col_y,
                                  float *lm_grad, float *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream);
int frnnt_simple_logprobs_bwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, const double *lm_max,
                                  const double *am_max, const double *norm_raw,
                                  const double *score_grad, int score_grad_stride,
                                  double score_grad_scale, double *px_grad, double *py_grad,
                                  double *dmat, double *row_x, double *row_y, double *col_y,
                                  double *lm_grad, double *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream);
/*
 * frnnt_simple_logprobs_bwd_f32 for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and results, without the four scratch
 * buffers: dmat, row_x, row_y and col_y live in a 16 MiB array that is part of the
 * library's code object, one copy per GPU, held until the process ends.  The call
 * allocates nothing.  FRNNT_ELIMIT when 4 * (B (S+1) (T rounded up to 4) + 2 B (S+1) + B T)
 * bytes (each part rounded up to 16) exceed 16 MiB.  All calls on one GPU share that
 * array: calls that overlap there (two streams, two threads) race, so issue them one
 * after the other on one stream.  The first call on a device looks the array's address
 * up (hipGetSymbolAddress); make that call outside a stream capture.  The device that
 * holds the buffers must be the calling thread's current device (as for every entry
 * point; here it also selects the array): FRNNT_EINVAL when px_grad lives elsewhere.
 */
int frnnt_simple_logprobs_bwd_noalloc_f32(const float *lm, const float *am, const int64_t *symbols,
                                          const int64_t *boundary, const float *lm_max,
                                          const float *am_max, const float *norm_raw,
                                          const float *score_grad, int score_grad_stride,
                                          double score_grad_scale, float *px_grad,
                                          float *py_grad, float *lm_grad, float *am_grad, int B,
                                          int S, int T, int C, int termination_symbol,
                                          int rnnt_type, int window_only, void *stream);
/*
 * The lm-only / am-only smoothing of get_rnnt_logprobs_smoothed (rnnt_loss.py:1135-1369)
 * applied to joint px / py (px_joint, py_joint: outputs of frnnt_simple_logprobs_fwd
 * without a boundary, regular or modified layout):
 *   px = px_joint * (1 - l - a) + lm_only_px * l + am_only_px * a     (same for py)
 * with l = lm_only_scale, a = am_only_scale, the lm-only model log_softmax(lm) and the
 * am-only model am + log(unigram) normalised per frame, unigram = mean over all
 * (b, s) of softmax(lm[b,s,:]) + tiny.  With a boundary (regular lattice) px[b][:][t_end] is
 * set to -inf after the interpolation (fix_for_boundary, rnnt_loss.py:1364-1365); the
 * backward entry point then takes the same boundary and lets no gradient through those
 * cells, as the reference's scatter_ does (px_grad holds 1 there when the lattice has no
 * path at all; NULL when the caller masks outside); the constrained "px += py[:, 1:]" step is left to the caller.
 *   lm_max, lm_sum [B][S+1], am_max, am_z [B][T], unigram [C]: out, kept for the backward
 *   partial [ceil(B*(S+1)/16)][C] (forward), [ceil(B*T/16)][C] (backward): scratch
 * Backward: px_grad / py_grad are the gradients of px / py; out are the gradients of
 * the joint inputs ((1 - l - a) * px_grad, ...) and the smoothing terms' own
 * contributions to lm_grad [B][S+1][C] and am_grad [B][T][C] (fully written);
 * row_x, row_y [B][S+1], col_y, col_g [B][T], g_unigram [C]: scratch.
 */
int frnnt_smoothed_logprobs_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                    const int64_t *boundary, const float *px_joint, const float *py_joint, float *px,
                                    float *py, float *lm_max, float *lm_sum, float *am_max,
                                    float *am_z, float *unigram, float *partial, int B, int S,
                                    int T, int C, int termination_symbol, int regular,
                                    double lm_only_scale, double am_only_scale, void *stream);
int frnnt_smoothed_logprobs_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                    const int64_t *boundary, const double *px_joint, const double *py_joint, double *px,
                                    double *py, double *lm_max, double *lm_sum, double *am_max,
                                    double *am_z, double *unigram, double *partial, int B, int S,
                                    int T, int C, int termination_symbol, int regular,
                                    double lm_only_scale, double am_only_scale, void *stream);
int frnnt_smoothed_logprobs_bwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                    const int64_t *boundary, const float *lm_max, const float *lm_sum, const float *am_max,
                                    const float *am_z, const float *unigram, const float *px_grad,
                                    const float *py_grad, float *px_joint_grad,
                                    float *py_joint_grad, float *lm_grad, float *am_grad,
                                    float *row_x, float *row_y, float *col_y, float *col_g,
                                    float *g_unigram, float *partial, int B, int S, int T, int C,
                                    int termination_symbol, int regular, double lm_only_scale,
                                    double am_only_scale, void *stream);
int frnnt_smoothed_logprobs_bwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                    const int64_t *boundary, const double *lm_max, const double *lm_sum,
                                    const double *am_max, const double *am_z,
                                    const double *unigram, const double *px_grad,
                                    const double *py_grad, double *px_joint_grad,
                                    double *py_joint_grad, double *lm_grad, double *am_grad,
                                    double *row_x, double *row_y, double *col_y, double *col_g,
                                    double *g_unigram, double *partial, int B, int S, int T, int C,
                                    int termination_symbol, int regular, double lm_only_scale,
                                    double am_only_scale, void *stream);

/*
 * Forward pipeline of rnnt_loss_simple (rnnt_loss.py:230-340) in one call:
 * frnnt_simple_logprobs_fwd, frnnt_mi_forward, then -- when px_grad / py_grad are
 * given -- frnnt_mi_backward with a gradient of ones (what the recursion's autograd
 * wrapper computes eagerly, mutual_information.py:159-168), then -- when loss is
 * given -- frnnt_loss_reduce.  Arguments as in those entry points; p [B][S+1][T+1]
 * and scores [B] are outputs as well; checks / status (may be 0 / NULL) as in
 * frnnt_mi_forward_checked.  It exists to save host time per call.
 */
int frnnt_simple_loss_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                              const int64_t *boundary, float *px, float *py, float *lm_max,
                              float *am_max, float *norm_raw, float *p, float *scores,
                              float *px_grad, float *py_grad, float *loss, int B, int S, int T,
                              int C, int termination_symbol, int rnnt_type, int reduction,
                              int checks, int32_t *status, void *stream);
int frnnt_simple_loss_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                              const int64_t *boundary, double *px, double *py, double *lm_max,
                              double *am_max, double *norm_raw, double *p, double *scores,
                              double *px_grad, double *py_grad, double *loss, int B, int S, int T,
                              int C, int termination_symbol, int rnnt_type, int reduction,
                              int checks, int32_t *status, void *stream);

/*
 * The tail every loss function shares (rnnt_loss.py:326-340, :535-547, :1119-1132, :1481-1494)
 * in one call: frnnt_mi_forward, then -- when px_grad / py_grad are given -- frnnt_mi_backward
 * with a gradient of ones (mutual_information.py:159-168), then -- when loss is given --
 * frnnt_loss_reduce (the backward kernel reduces the scores on its way: no extra launch).
 * p [B][S+1][T+1] and scores [B] are outputs as well; checks / status (may be 0 / NULL) as
 * in frnnt_mi_forward_checked.
 */
int frnnt_mi_loss_fwd_f32(const float *px, const float *py, const int64_t *boundary, float *p,
                          float *scores, float *px_grad, float *py_grad, float *loss, int B, int S,
                          int T, int modified, int reduction, int checks, int32_t *status,
                          void *stream);
int frnnt_mi_loss_fwd_f64(const double *px, const double *py, const int64_t *boundary, double *p,
                          double *scores, double *px_grad, double *py_grad, double *loss, int B,
                          int S, int T, int modified, int reduction, int checks, int32_t *status,
                          void *stream);
/*
 * The backward of that tail: px_grad[b] and py_grad[b] are multiplied IN PLACE by
 * score_grad_scale * score_grad[b * score_grad_stride] -- what the recursion's autograd
 * backward does to the tensors it handed out (mutual_information.py:173-181), with the
 * reduction's sign and 1/B in score_grad_scale (stride 0: one scalar for all utterances).
 */
int frnnt_mi_scale_grads_f32(float *px_grad, float *py_grad, const float *score_grad,
                             int score_grad_stride, double score_grad_scale, int B, int S, int T,
                             int modified, void *stream);
int frnnt_mi_scale_grads_f64(double *px_grad, double *py_grad, const double *score_grad,
                             int score_grad_stride, double score_grad_scale, int B, int S, int T,
                             int modified, void *stream);

/*
 * The reduction at the end of every loss function (rnnt_loss.py:160-169, :330-340):
 * loss = -scores (reduction 0, [B]), -mean(scores) (1, one value) or -sum(scores)
 * (2, one value), summed in a fixed order by one workgroup.
 */
int frnnt_loss_reduce_f32(const float *scores, float *loss, int B, int reduction, void *stream);
int frnnt_loss_reduce_f64(const double *scores, double *loss, int B, int reduction, void *stream);


/*
 * px / py from joiner logits.  Replaces the tensor algebra of
 *   get_rnnt_logprobs_joint  (rnnt_loss.py:343-449)  when ranges == NULL, R == S+1,
 *   get_rnnt_logprobs_pruned (rnnt_loss.py:856-1024) when ranges is given:
 * logsumexp over the vocabulary, the symbol / termination-symbol picks, the -inf
 * padding and per-frame roll that places range row j at lattice row
 * (j + ranges[b][t][0]) mod (S+1), the -inf columns of the regular lattice and
 * the constrained "px += py[:, 1:]" step.
 *   logits [B][T][R][C]; symbols int64 [B][S]; ranges int64 [B][T][R] or NULL   in
 *   boundary int64 [B][4] or NULL (only boundary[b][3] is used, regular lattice)
 *   px [B][S][T+1] (rnnt_type 0) or [B][S][T]; py [B][S+1][T]                   out
 *   norm, xr, yr [B][T][R]: out; norm (the logsumexp) is needed by the backward
 *   entry point, xr / yr are staging buffers
 *   window_only: 0 = every cell of px / py is computed.  1 (needs a boundary) = the caller
 *   goes on to the lattice recursion with the same boundary, which never looks outside
 *   utterance b's window [s_begin, s_end] x [t_begin, t_end): logits rows outside it are
 *   not read and their entries of norm, xr, yr, px, py are left undefined.  The backward
 *   entry point takes the same flag: such rows then get a gradient of exact zeros without
 *   being read (the recursion's px_grad / py_grad vanish there).  This is what rnnt_loss
 *   and rnnt_loss_pruned (rnnt_loss.py:452-547, :1027-1132) use; about a third of the rows
 *   of a ragged batch lie outside.
 */
int frnnt_lattice_logprobs_fwd_f32(const float *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary, float *px,
                                   float *py, float *norm, float *xr, float *yr, int B, int S,
                                   int T, int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream);
int frnnt_lattice_logprobs_fwd_f64(const double *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary, double *px,
                                   double *py, double *norm, double *xr, double *yr, int B, int S,
                                   int T, int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream);

/*
 * Backward of the above (what autograd derives for rnnt_loss.py:418-447 /
 * :940-1022): logits_grad [B][T][R][C] =
 *   -softmax * (gx + gy) + onehot(symbol) * gx + onehot(termination) * gy.
 */
int frnnt_lattice_logprobs_bwd_f32(const float *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary,
                                   const float *norm, const float *px_grad, const float *py_grad,
                                   float *logits_grad, int B, int S, int T, int R, int C,
                                   int termination_symbol, int rnnt_type, int window_only,
                                   void *stream);
int frnnt_lattice_logprobs_bwd_f64(const double *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary,
                                   const double *norm, const double *px_grad,
                                   const double *py_grad, double *logits_grad, int B, int S, int T,
                                   int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream);

/*
 * The two entry points above for 2-byte logits: float16 (_f16) or bfloat16 (_bf16),
 * passed as void*.  The reference has no such form -- its recursion knows float32 and
 * float64 only (mutual_information_cuda.cu:37-38 notes the missing half LogAdd), so
 * half-precision joiner outputs need a float32 copy there.  Here the logits are read as
 * they are (half the bytes of the dominant stream) and everything after the load is
 * float32: norm, xr, yr, px, py and the incoming px_grad / py_grad are float32 buffers of
 * the shapes above, to be used with frnnt_mi_forward_f32 / frnnt_mi_backward_f32; only
 * logits_grad is written in the logits' type (rounded to nearest even).
 */
int frnnt_lattice_logprobs_fwd_f16(const void *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary, float *px,
                                   float *py, float *norm, float *xr, float *yr, int B, int S,
                                   int T, int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream);
int frnnt_lattice_logprobs_fwd_bf16(const void *logits, const int64_t *symbols,
                                    const int64_t *ranges, const int64_t *boundary, float *px,
                                    float *py, float *norm, float *xr, float *yr, int B, int S,
                                    int T, int R, int C, int termination_symbol, int rnnt_type,
                                    int window_only, void *stream);
int frnnt_lattice_logprobs_bwd_f16(const void *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary,
                                   const float *norm, const float *px_grad, const float *py_grad,
                                   void *logits_grad, int B, int S, int T, int R, int C,
                                   int termination_symbol, int rnnt_type, int window_only,
                                   void *stream);
int frnnt_lattice_logprobs_bwd_bf16(const void *logits, const int64_t *symbols,
                                    const int64_t *ranges, const int64_t *boundary,
                                    const float *norm, const float *px_grad, const float *py_grad,
                                    void *logits_grad, int B, int S, int T, int R, int C,
                                    int termination_symbol, int rnnt_type, int window_only,
                                    void *stream);

/*
 * Pruning bounds.  Replaces the device work of get_rnnt_prune_ranges
 * (rnnt_loss.py:726-777 with _adjust_pruning_lower_bound :584-632).  s_range is
 * the FINAL window size: the caller has already raised it to the regular
 * lattice's minimum and capped it at S+1 (rnnt_loss.py:696-724), so
 * 1 <= s_range <= S+1.  The window sums are formed in the input precision and in the
 * order of torch.sum on the CPU (left to right up to 16 rows, stretches of 16 merged
 * upwards beyond), first maximum wins, NaN counts as the maximum: given the same
 * gradients the ranges are those of the reference's CPU run, near-ties included.
 *   px_grad [B][S][T+1] (modified: [B][S][T]), py_grad [B][S+1][T], boundary [B][4]  in
 *   ranges int64 [B][T][s_range]                                                     out
 */
int frnnt_prune_ranges_f32(const float *px_grad, const float *py_grad, const int64_t *boundary,
                           int64_t *ranges, int B, int S, int T, int modified, int s_range,
                           void *stream);
int frnnt_prune_ranges_f64(const double *px_grad, const double *py_grad, const int64_t *boundary,
                           int64_t *ranges, int B, int S, int T, int modified, int s_range,
                           void *stream);

/*
 * Pruning gather and its adjoint.  Replaces the gather of do_rnnt_pruning
 * (rnnt_loss.py:813-817): lm_pruned[b][t][j][:] = lm[b][ranges[b][t][j]][:]
 * (NaN rows for entries outside [0, S]); the adjoint sums the rows of `grad`
 * that were taken from each lm row, in frame order.
 *   lm [B][S+1][C], ranges int64 [B][T][R]; lm_pruned / grad [B][T][R][C]; lm_grad [B][S+1][C]
 */
int frnnt_prune_gather_f32(const float *lm, const int64_t *ranges, float *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream);
int frnnt_prune_gather_f64(const double *lm, const int64_t *ranges, double *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream);
int frnnt_prune_gather_bwd_f32(const float *grad, const int64_t *ranges, float *lm_grad, int B,
                               int S, int T, int R, int C, void *stream);
int frnnt_prune_gather_bwd_f64(const double *grad, const int64_t *ranges, double *lm_grad, int B,
                               int S, int T, int R, int C, void *stream);

/*
 * The same for float16 (_f16) / bfloat16 (_bf16) elements, passed as void*: the reference's
 * do_rnnt_pruning is plain indexing and takes any element type, as half-precision encoder /
 * predictor outputs under autocast need.  The gather copies bit patterns; the adjoint sums in
 * float32 and rounds the result to the element type (to nearest even).
 */
int frnnt_prune_gather_f16(const void *lm, const int64_t *ranges, void *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream);
int frnnt_prune_gather_bf16(const void *lm, const int64_t *ranges, void *lm_pruned, int B, int S,
                            int T, int R, int C, void *stream);
int frnnt_prune_gather_bwd_f16(const void *grad, const int64_t *ranges, void *lm_grad, int B, int S,
                               int T, int R, int C, void *stream);
int frnnt_prune_gather_bwd_bf16(const void *grad, const int64_t *ranges, void *lm_grad, int B,
                                int S, int T, int R, int C, void *stream);

/*
 * The joiner's input straight from the pruning bounds:
 *   out[b][t][j][:] = act(am[b][t][:] + lm[b][ranges[b][t][j]][:])
 * i.e. what a joiner of the usual form computes first from the two tensors of
 * do_rnnt_pruning (rnnt_loss.py:780-818; README.md:193-215: logits =
 * joiner(am_pruned, lm_pruned)), in one pass and without lm_pruned [B][T][R][C] ever
 * existing.  activation: 0 = none (the plain sum), 1 = tanh.  Rows whose range entry lies
 * outside [0, S] are NaN, as in frnnt_prune_gather.
 * Backward: grad is dL/dout, out the forward's result (read for tanh only);
 *   am_grad[b][t][:] = sum_j grad * act'      lm_grad[b][s][:] = sum over the (t, j) with
 * ranges[b][t][j] = s of grad * act', in frame order (deterministic, no atomics); either
 * output may be NULL.
 */
int frnnt_pruned_joiner_fwd_f32(const float *am, const float *lm, const int64_t *ranges, float *out,
                                int B, int S, int T, int R, int C, int activation, void *stream);
int frnnt_pruned_joiner_fwd_f64(const double *am, const double *lm, const int64_t *ranges,
                                double *out, int B, int S, int T, int R, int C, int activation,
                                void *stream);
int frnnt_pruned_joiner_bwd_f32(const float *grad, const float *out, const int64_t *ranges,
                                float *am_grad, float *lm_grad, int B, int S, int T, int R, int C,
                                int activation, void *stream);
int frnnt_pruned_joiner_bwd_f64(const double *grad, const double *out, const int64_t *ranges,
                                double *am_grad, double *lm_grad, int B, int S, int T, int R, int C,
                                int activation, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FAST_RNNT_AMD_H_ */
