/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the mutual-information lattice
 * recursion.  Nothing in the shipped package may link or call this file; it
 * exists so that tests, the smoke check and the benchmark's CPU-baseline leg
 * can compare the HIP kernels against an independent restatement of the
 * reference algorithm.
 *
 * Restates, in plain C99 over dense row-major buffers:
 *   log_add      <- fast_rnnt/csrc/mutual_information.h:36-65        (LogAdd)
 *   mi_forward   <- fast_rnnt/csrc/mutual_information_cpu.cu:50-124
 *   mi_backward  <- fast_rnnt/csrc/mutual_information_cpu.cu:128-256
 *
 * Layouts (all contiguous, last axis fastest):
 *   px  [B][S][T1]   T1 = T+1 (regular) or T (modified)
 *   py  [B][S+1][T]
 *   p   [B][S+1][T+1]
 *   boundary [B][4] int64 = (s_begin, t_begin, s_end, t_end), or NULL for
 *   (0, 0, S, T) on every row.
 *
 * Behaviour kept from the reference CPU path:
 *   - the batch is processed serially on one thread;
 *   - forward writes only the [s_begin..s_end] x [t_begin..t_end] window of p;
 *   - the regular recursion reads the "up" neighbour at column t, the modified
 *     one at column t-1, and the modified first column is -inf below s_begin;
 *   - backward splits the incoming gradient of a cell into d1 = exp(term1 - p)
 *     and d2 = 1 - d1 (not a second exp), zeroing both if d1 is not finite, and
 *     treating a non-finite p[s][t] as 0 inside that exponent;
 *   - with a boundary the gradient outputs are zero outside the window; without
 *     one every cell is written.
 * The return value of the backward functions is the number of batch rows whose
 * gradient arriving at (s_begin, t_begin) differs from ans_grad by more than 1%
 * (the reference prints a warning for those, mutual_information_cpu.cu:242-250).
 *
 * Pinning (see tests/test_oracle_recursion.py): binomial closed forms for
 * px = py = 0, brute-force path enumeration on small lattices with offsets and
 * empty sequences, flow-conservation invariants of the gradients, finite
 * differences, and agreement with the reference's own C++ when oracle/_ref has
 * been built.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CONCAT_(a, b) a##_##b
#define CONCAT(a, b) CONCAT_(a, b)

/* ---- float instantiation ------------------------------------------------ */
#define REAL float
#define SUFFIX f32
#define EXP_FN expf
#define LOG1P_FN log1pf
#define FABS_FN fabsf
#include "mi_oracle_body.inc"
#undef REAL
#undef SUFFIX
#undef EXP_FN
#undef LOG1P_FN
#undef FABS_FN

/* ---- double instantiation ----------------------------------------------- */
#define REAL double
#define SUFFIX f64
#define EXP_FN exp
#define LOG1P_FN log1p
#define FABS_FN fabs
#include "mi_oracle_body.inc"
#undef REAL
#undef SUFFIX
#undef EXP_FN
#undef LOG1P_FN
#undef FABS_FN
