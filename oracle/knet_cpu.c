/*
 * knet_cpu.c -- CPU oracle for the backward-pass gradient kernels.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a plain-C restatement of
 * the formulas of Knet's CPU `Array` path (the reference is Julia and cannot be
 * executed where this is built).  Only the test-suite, the smoke check and the
 * benchmark's `cpu_baseline` leg may load it, and only as the checker or as the
 * timed CPU baseline.  The shipped library never links or calls it.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   - reluback / getents / addents / findindices: closed-form selects and index
 *     arithmetic, checked bit-for-bit against independent numpy expressions and
 *     brute force over IEEE special values.
 *   - sigmback / tanhback / eluback / seluback and the ops21 three-input forms:
 *     checked against the same expression evaluated in higher precision
 *     (<= 2 ulp) and against finite differences of the forward functions.
 *   - selu constants: recomputed from their closed forms
 *     (src/ops20/activation.jl:43-45) with erfc/exp in extended precision.
 *   - reductions: brute force over every dim subset of small arrays, exact
 *     equality on integer-valued inputs, sum(dims=1) then sum(dims=2) == sum(:).
 *   - softmax family: invariants of test/loss.jl:47-56 (softmax == exp(logsoftmax),
 *     columns sum to 1, shift invariance, uniform input -> -log(m)) and fp64
 *     finite differences of the gradients (what test/loss.jl:81-92 asserts).
 *   - nll: the known answer in the reference docstring (src/ops20/loss.jl:22-27,
 *     scores [12.2 0.3; 2.0 21.5; 0.0 -21.0], labels [1,2] -> 2.1657e-5), the
 *     closed form dx = (softmax(x) - onehot)/N, label 0 skipped.
 *   - dropout: deterministic given the uniform buffer; p=0.5 closed form.
 *
 * PARITY UNPINNED (nothing available here can pin them; see also the design notes):
 *   - the exact last-bit rounding of Julia's Base.sum (pairwise/SIMD association)
 *     and of Julia's exp/tanh/erf/log.  The oracle uses correctly rounded wide
 *     accumulation and glibc libm instead; tolerances in the parity tests
 *     (1e-5 relative for reductions/softmax, 2 ulp for forwards measured at the
 *     magnitude of the libm result) absorb the difference.
 *   - AutoGrad's `unbroadcast` (third-party AutoGrad.jl 1.2.4, not vendored in the
 *     reference): restated from its published behaviour in the host mirror and
 *     pinned only indirectly by finite-difference checks of x .+ b.
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off; no other dependencies)
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* selu constants, src/ops20/activation.jl:43-45 (closed forms in the comments there) */
#define KO_LAMBDA01 1.0507009873554805
#define KO_ALPHA01 1.6732632423543778
#define KO_LAMBDAALPHA01 1.7580993408473773
#define KO_SQRT2 1.4142135623730951    /* Julia sqrt(2)   */
#define KO_SQRT2PI 2.5066282746310002  /* Julia sqrt(2pi) */

double ko_const(int which) {
  switch (which) {
    case 0: return KO_LAMBDA01;
    case 1: return KO_ALPHA01;
    case 2: return KO_LAMBDAALPHA01;
  }
  return 0.0;
}

/* findindices(scores,labels;dims)  -- src/ops20/loss.jl:116-140.
 * scores is (y1,y2) column-major.  dims==1: instance j (1-based) with label l>0 maps to
 * linear index (j-1)*y1 + l; dims==2: (l-1)*y1 + j.  Label 0 is skipped.  Returns the
 * number of indices written, or -1 when the label count does not match (the reference
 * throws DimensionMismatch), -2 for dims not in {1,2}. */
long ko_findindices(long y1, long y2, const int *labels, long ninstances, int dims, long *indices) {
  long nind = 0;
  if (dims == 1) {
    if (ninstances != y2) return -1;
    for (long j = 1; j <= ninstances; j++) {
      if (labels[j - 1] == 0) continue;
      indices[nind++] = (j - 1) * y1 + labels[j - 1];
    }
  } else if (dims == 2) {
    if (ninstances != y1) return -1;
    for (long j = 1; j <= ninstances; j++) {
      if (labels[j - 1] == 0) continue;
      indices[nind++] = (long)(labels[j - 1] - 1) * y1 + j;
    }
  } else {
    return -2;
  }
  return nind;
}

#define T float
#define W double
#define S 32
#define EXP expf
#define LOG logf
#define TANH tanhf
#define ERF erff
#define SQRT sqrtf
#include "knet_cpu_body.h"
#undef T
#undef W
#undef S
#undef EXP
#undef LOG
#undef TANH
#undef ERF
#undef SQRT

#define T double
#define W long double
#define S 64
#define EXP exp
#define LOG log
#define TANH tanh
#define ERF erf
#define SQRT sqrt
#include "knet_cpu_body.h"
#undef T
#undef W
#undef S
#undef EXP
#undef LOG
#undef TANH
#undef ERF
#undef SQRT
