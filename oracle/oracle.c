/*
 * CPU oracle for the Gorgonia device-engine hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file.  It is a plain-C restatement of what Gorgonia's CPU engine
 * (StandardEngine{tensor.StdEng} + gonum) computes for the operators the HIP
 * engine replaces; the GPU parity tests, the smoke check and the CPU-baseline
 * leg of the benchmark use it as the checker.
 *
 * Build: see oracle/Makefile (gcc, -ffp-contract=off, no fast-math, no FMA).
 * Every float32 operation below is a single IEEE-754 binary32 operation with
 * one rounding, exactly as Go on amd64 evaluates `float32 op float32`.
 *
 * Pinning status (what, other than retyping the formula, checks each part):
 *   elementwise add/sub/mul/div/pow, cmp   - reference known-answer tables
 *                                            op_math_test.go:23-360,
 *                                            operations_test.go:158-233
 *   relu / leaky relu                      - nn_test.go:538-588 golden
 *   max pool (incl. asymmetric padding)    - nn_test.go:91-138 golden (3072
 *                                            floats), nn_test.go:195-266
 *   conv2d (im2col+gemm+transpose)         - known_issues_test.go:160-240,
 *                                            blas_test.go:426-460, and a
 *                                            float64 brute-force direct conv
 *   gemm / bmm / gemv / outer              - float64 product, integer-exact
 *                                            cases, example_linalg_test.go
 *   batch norm (train step, eval)          - nn_amd64_test.go:25-205 goldens
 *   softmax                                - op_softmax_test.go goldens
 *   sigmoid                                - closed form math_nooptim.go:36-44
 *                                            (float64 exp, one rounding);
 *                                            identities s(x)+s(-x)=1, s(0)=.5
 *   tanh / exp f32                         - PARITY UNPINNED bit-for-bit: the
 *                                            reference routes these through
 *                                            math32 (not vendored).  Oracle is
 *                                            float64 libm rounded once (checked
 *                                            against 200-bit values rounded once);
 *                                            the 2-ulp budget covers the gap.
 *   abs neg square cube ceil floor sqrt    - single IEEE operations: numpy's bits,
 *   inverse invsqrt (f32 and f64)            signed zeros, NaN, infinities, denormals
 *   sin cos exp ln log2 log1p expm1 tanh   - 200-bit mpmath values rounded once
 *   (f32 and f64)                            (<= 1 ulp, f32 equal on > 99.9 %), and
 *                                            known values that tell the codes apart
 *   softplus, float64 sigmoid              - cut-offs of math.go:50-68 and
 *                                            math_nooptim.go:25-34 at their
 *                                            neighbours, where cut-off and formula
 *                                            differ; values as above
 *   sign                                   - numpy sign on non-zero numbers; at +-0
 *                                            and NaN the device kernel's form
 *                                            (elemunaryop.cu:125-131) gives +0.  The
 *                                            CPU engine's tensor.Signer is not
 *                                            vendored: PARITY UNPINNED at +-0 / NaN
 *   pow (general)                          - exact cases (integer powers, square
 *                                            roots of squares, powers of two,
 *                                            C99 / Go special cases), 200-bit
 *                                            values rounded once, exact integers
 *   batch norm backward                    - nn_amd64_test.go ExpectedInputGrad
 *                                            goldens; finite differences of the
 *                                            training forward
 *   solver steps (vanilla, RMSProp, Adam)  - solvers_test.go:100-143 closed form,
 *                                            solvers_test.go:355-437 Adam golden
 *   max-pool backward                      - nn_test.go:140-193 example, brute
 *                                            force on tied inputs, the 3072-float
 *                                            golden's windows
 *   conv2d backward (image, filter)        - the reference's tests are only
 *                                            differential (tape vs lisp machine):
 *                                            pinned by the float64 definition,
 *                                            adjoint identities against the
 *                                            pinned forward pass, finite
 *                                            differences, integer-exact cases
 *   dropout forward / backward             - op_dropout_test.go:14-102 goldens with
 *                                            the injected random sequence
 *   uniform01 (the engine's own generator) - equals gorgonia_amd/synth.py's stream
 *   softmax backward                       - no reference golden: Jacobian and
 *                                            finite differences of the pinned
 *                                            forward pass.  tensor.SoftMaxB
 *                                            itself is not vendored: PARITY
 *                                            UNPINNED bit-for-bit.
 *   float64 twins (forward NN operators,   - each against its pinned float32
 *   conv / max-pool / batch-norm / softmax   counterpart: equal on inputs whose
 *   gradients, dropout, solver steps)        float32 arithmetic is exact, within
 *                                            float32 rounding elsewhere (plus
 *                                            finite differences for batch norm);
 *                                            the reference's float64 goldens where
 *                                            it has them (max pool, softmax)
 *   uniform01 float64                      - its top 24 bits are the float32 stream
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT __attribute__((visibility("default")))

static int g_threads = 1;

EXPORT void oracle_set_threads(int n) {
  g_threads = n < 1 ? 1 : n;
#ifdef _OPENMP
  omp_set_num_threads(g_threads);
#endif
}
EXPORT int oracle_get_threads(void) { return g_threads; }

/* ------------------------------------------------------------------ */
/* Elementwise binary ops.                                             */
/* Semantics: cuda/arith.go:14-64 (in place on a, or on reuse after    */
/* memcpy), kernels "cuda modules/src/elembinop.cu":13-35:             */
/*   vv: A[i] = A[i] op B[i]     vs: A[i] = A[i] op B[0]               */
/*   sv: B[i] = A[0] op B[i]     ss: A[0] = A[0] op B[0]               */
/* CPU twin: operatorPointwise_binary.go:359-426 (tensor.Add ...);     */
/* comparisons return 1/0 in the operand dtype (retSame,               */
/* operatorPointwise_binary.go:305-317).                               */
/* op codes: 0 add 1 sub 2 mul 3 div 4 pow 5 lt 6 lte 7 gt 8 gte 9 eq  */
/*           10 ne   11 mod (Go's math.Mod = C fmod: sign of the dividend) */
/* ------------------------------------------------------------------ */

static inline float binop_f32(int op, float a, float b) {
  switch (op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    case 3: return a / b;
    case 4: return (float)pow((double)a, (double)b); /* math32.Pow stand-in */
    case 5: return a < b ? 1.0f : 0.0f;
    case 6: return a <= b ? 1.0f : 0.0f;
    case 7: return a > b ? 1.0f : 0.0f;
    case 8: return a >= b ? 1.0f : 0.0f;
    case 9: return a == b ? 1.0f : 0.0f;
    case 10: return a != b ? 1.0f : 0.0f;
    case 11: return (float)fmod((double)a, (double)b); /* math32.Mod: math.Mod in float64, exact */
  }
  return NAN;
}

static inline double binop_f64(int op, double a, double b) {
  switch (op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    case 3: return a / b;
    case 4: return pow(a, b);
    case 5: return a < b ? 1.0 : 0.0;
    case 6: return a <= b ? 1.0 : 0.0;
    case 7: return a > b ? 1.0 : 0.0;
    case 8: return a >= b ? 1.0 : 0.0;
    case 9: return a == b ? 1.0 : 0.0;
    case 10: return a != b ? 1.0 : 0.0;
    case 11: return fmod(a, b); /* math.Mod */
  }
  return NAN;
}

/* mode: 0 vv, 1 vs, 2 sv, 3 ss.  Result lands where the device kernel puts it. */
EXPORT void oracle_binop_f32(int op, int mode, float* A, float* B, int64_t n) {
  int64_t i;
  switch (mode) {
    case 0: for (i = 0; i < n; i++) A[i] = binop_f32(op, A[i], B[i]); break;
    case 1: for (i = 0; i < n; i++) A[i] = binop_f32(op, A[i], B[0]); break;
    case 2: for (i = 0; i < n; i++) B[i] = binop_f32(op, A[0], B[i]); break;
    case 3: A[0] = binop_f32(op, A[0], B[0]); break;
  }
}

EXPORT void oracle_binop_f64(int op, int mode, double* A, double* B, int64_t n) {
  int64_t i;
  switch (mode) {
    case 0: for (i = 0; i < n; i++) A[i] = binop_f64(op, A[i], B[i]); break;
    case 1: for (i = 0; i < n; i++) A[i] = binop_f64(op, A[i], B[0]); break;
    case 2: for (i = 0; i < n; i++) B[i] = binop_f64(op, A[0], B[i]); break;
    case 3: A[0] = binop_f64(op, A[0], B[0]); break;
  }
}

/* ------------------------------------------------------------------ */
/* Broadcast binary op: Broadcast (broadcast.go:69-129) materialises   */
/* the small operand with repeatOp (op_tensor.go:354-394) and then     */
/* runs the plain vv op (api_gen.go:129-135).  View every tensor as    */
/* (outer, mid, inner); the small operand has `mid` elements and is    */
/* repeated over outer and inner.  small_left != 0 puts the small      */
/* operand on the left of `op`.                                        */
/* ------------------------------------------------------------------ */
EXPORT void oracle_bcast_binop_f32(int op, int small_left, float* dst, const float* big,
                                   const float* small, int64_t outer, int64_t mid, int64_t inner) {
  int64_t n = outer * mid * inner, i;
  float* rep = (float*)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
  for (i = 0; i < n; i++) rep[i] = small[(i / inner) % mid]; /* tensor.Repeat */
  for (i = 0; i < n; i++)
    dst[i] = small_left ? binop_f32(op, rep[i], big[i]) : binop_f32(op, big[i], rep[i]);
  free(rep);
}

EXPORT void oracle_bcast_binop_f64(int op, int small_left, double* dst, const double* big,
                                   const double* small, int64_t outer, int64_t mid, int64_t inner) {
  int64_t n = outer * mid * inner, i;
  double* rep = (double*)malloc((size_t)(n > 0 ? n : 1) * sizeof(double));
  for (i = 0; i < n; i++) rep[i] = small[(i / inner) % mid]; /* tensor.Repeat */
  for (i = 0; i < n; i++)
    dst[i] = small_left ? binop_f64(op, rep[i], big[i]) : binop_f64(op, big[i], rep[i]);
  free(rep);
}

/* ------------------------------------------------------------------ */
/* Unary ops, in place.  elemunaryop.cu:109-193 names; CPU semantics   */
/* operatorPointwise_unary.go:30-101, math.go:13-68,                   */
/* math_nooptim.go:19-52.                                              */
/* codes: 0 abs 1 sign 2 ceil 3 floor 4 sin 5 cos 6 exp 7 ln 8 log2    */
/*        9 neg 10 square 11 sqrt 12 inverse 13 invsqrt 14 cube        */
/*        15 tanh 16 sigmoid 17 log1p 18 expm1 19 softplus             */
/* ------------------------------------------------------------------ */
static inline float unary_f32(int fn, float x) {
  switch (fn) {
    case 0: return fabsf(x);
    case 1: return (float)((x > 0.0f) - (x < 0.0f)); /* elemunaryop.cu:125-131 */
    case 2: return ceilf(x);
    case 3: return floorf(x);
    case 4: return (float)sin((double)x);
    case 5: return (float)cos((double)x);
    case 6: return (float)exp((double)x);
    case 7: return (float)log((double)x);
    case 8: return (float)log2((double)x);
    case 9: return -x;
    case 10: return x * x;                       /* math.go:27 */
    case 11: return sqrtf(x);
    case 12: return 1.0f / x;                    /* math_nooptim.go:19 */
    case 13: return 1.0f / sqrtf(x);             /* math_nooptim.go:50-52 */
    case 14: return x * x * x;                   /* math.go:30 */
    case 15: return (float)tanh((double)x);      /* math_nooptim.go:22 */
    case 16:                                     /* math_nooptim.go:36-44 */
      if (x < -88.0f) return 0.0f;
      if (x > 15.0f) return 1.0f;
      return (float)(1.0 / (1.0 + exp((double)(-x))));
    case 17: return (float)log1p((double)x);
    case 18: return (float)expm1((double)x);
    case 19:                                     /* math.go:60-68 */
      if (x < -103.0f) return 0.0f;
      if (x > 14.0f) return x;
      return (float)log1p(exp((double)x));
  }
  return NAN;
}

static inline double unary_f64(int fn, double x) {
  switch (fn) {
    case 0: return fabs(x);
    case 1: return (double)((x > 0.0) - (x < 0.0));
    case 2: return ceil(x);
    case 3: return floor(x);
    case 4: return sin(x);
    case 5: return cos(x);
    case 6: return exp(x);
    case 7: return log(x);
    case 8: return log2(x);
    case 9: return -x;
    case 10: return x * x;
    case 11: return sqrt(x);
    case 12: return 1.0 / x;
    case 13: return 1.0 / sqrt(x);
    case 14: return x * x * x;
    case 15: return tanh(x);
    case 16:                                     /* math_nooptim.go:25-34 */
      if (x < -709.0) return 0.0;
      if (x > 19.0) return 1.0;
      return 1.0 / (1.0 + exp(-x));
    case 17: return log1p(x);
    case 18: return expm1(x);
    case 19:                                     /* math.go:50-58 */
      if (x < -708.0) return 0.0;
      if (x > 16.0) return x;
      return log1p(exp(x));
  }
  return NAN;
}

EXPORT void oracle_unary_f32(int fn, float* A, int64_t n) {
  int64_t i;
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (i = 0; i < n; i++) A[i] = unary_f32(fn, A[i]);
}

EXPORT void oracle_unary_f64(int fn, double* A, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) A[i] = unary_f64(fn, A[i]);
}

/* ------------------------------------------------------------------ */
/* ReLU and LeakyReLU as the reference composes them.                  */
/* Rectify: x * float(x >= 0)                 (nn.go:136-163)          */
/* LeakyRelu: x*(x>=0) + (x*(x<0))*alpha      (nn.go:83-131)           */
/* Negative inputs therefore give -0.0 under ReLU, and +-Inf gives NaN */
/* under LeakyRelu (Inf*0).                                            */
/* ------------------------------------------------------------------ */
EXPORT void oracle_relu_f32(float* y, const float* x, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) {
    float m = x[i] >= 0.0f ? 1.0f : 0.0f;
    y[i] = x[i] * m;
  }
}

EXPORT void oracle_leaky_relu_f32(float* y, const float* x, float alpha, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) {
    float ge = x[i] >= 0.0f ? 1.0f : 0.0f;
    float lt = x[i] < 0.0f ? 1.0f : 0.0f;
    float pos = x[i] * ge;
    float neg = x[i] * lt;
    float nega = neg * alpha;
    y[i] = pos + nega;
  }
}

/* ------------------------------------------------------------------ */
/* GEMM, row-major, C = op(A) * op(B), alpha=1 beta=0.                 */
/* The reference CPU path is tensor.MatMul -> gonum Sgemm              */
/* (op_math.go:745-795, blas.go:55-57).  gonum accumulates             */
/* c[i][j] += a[i][l]*b[l][j] over l in ascending order with a rounded */
/* multiply and a rounded add per step (no FMA); the non-transposed    */
/* path below does exactly that.  A and B are the *stored* matrices:   */
/* with transA the stored A is (k x m), with transB the stored B is    */
/* (n x k) (op_math_cuda.go:210-224 sets the same logical transposes). */
/* ------------------------------------------------------------------ */
EXPORT void oracle_gemm_f32(int transA, int transB, int64_t m, int64_t n, int64_t k,
                            const float* A, int64_t lda, const float* B, int64_t ldb,
                            float* C, int64_t ldc) {
  int64_t i;
#pragma omp parallel for if (g_threads > 1) schedule(dynamic, 4)
  for (i = 0; i < m; i++) {
    float* c = C + i * ldc;
    int64_t j, l;
    for (j = 0; j < n; j++) c[j] = 0.0f;
    if (!transB) {
      for (l = 0; l < k; l++) {
        float a = transA ? A[l * lda + i] : A[i * lda + l];
        const float* b = B + l * ldb;
        for (j = 0; j < n; j++) {
          float p = a * b[j];
          c[j] = c[j] + p;
        }
      }
    } else {
      for (j = 0; j < n; j++) {
        const float* b = B + j * ldb;
        float acc = 0.0f;
        for (l = 0; l < k; l++) {
          float a = transA ? A[l * lda + i] : A[i * lda + l];
          float p = a * b[l];
          acc = acc + p;
        }
        c[j] = acc;
      }
    }
  }
}

/* Same contraction with float64 accumulation: the yardstick for the
 * relative-Frobenius tolerance and for pinning oracle_gemm_f32 itself. */
EXPORT void oracle_gemm_f64acc(int transA, int transB, int64_t m, int64_t n, int64_t k,
                               const float* A, int64_t lda, const float* B, int64_t ldb,
                               double* C, int64_t ldc) {
  int64_t i;
#pragma omp parallel for if (g_threads > 1) schedule(dynamic, 4)
  for (i = 0; i < m; i++) {
    int64_t j, l;
    double* c = C + i * ldc;
    for (j = 0; j < n; j++) c[j] = 0.0;
    if (!transB) {
      for (l = 0; l < k; l++) {
        double a = transA ? A[l * lda + i] : A[i * lda + l];
        const float* b = B + l * ldb;
        for (j = 0; j < n; j++) c[j] += a * (double)b[j];
      }
    } else {
      for (j = 0; j < n; j++) {
        const float* b = B + j * ldb;
        double acc = 0.0;
        for (l = 0; l < k; l++) {
          double a = transA ? A[l * lda + i] : A[i * lda + l];
          acc += a * (double)b[l];
        }
        c[j] = acc;
      }
    }
  }
}

/* BatchedMatMul: operatorLinAlg.go:435-502 loops the leading dims and
 * calls MatMul per slice. */
EXPORT void oracle_bmm_f32(int transA, int transB, int64_t batch, int64_t m, int64_t n, int64_t k,
                           const float* A, const float* B, float* C) {
  int64_t b;
  int64_t sa = m * k, sb = k * n, sc = m * n;
  int64_t lda = transA ? m : k, ldb = transB ? k : n;
  for (b = 0; b < batch; b++)
    oracle_gemm_f32(transA, transB, m, n, k, A + b * sa, lda, B + b * sb, ldb, C + b * sc, n);
}

/* MatVecMul y = A x, A row-major (m x n): cuda/linalg.go:47-107; CPU
 * gonum Sgemv: sequential dot per row. trans != 0 computes y = A^T x. */
EXPORT void oracle_gemv_f32(int trans, int64_t m, int64_t n, const float* A, int64_t lda,
                            const float* x, float* y) {
  int64_t i, j;
  if (!trans) {
#pragma omp parallel for if (g_threads > 1) schedule(static)
    for (i = 0; i < m; i++) {
      float acc = 0.0f;
      for (j = 0; j < n; j++) {
        float p = A[i * lda + j] * x[j];
        acc = acc + p;
      }
      y[i] = acc;
    }
  } else {
    for (j = 0; j < n; j++) y[j] = 0.0f;
    for (i = 0; i < m; i++)
      for (j = 0; j < n; j++) {
        float p = A[i * lda + j] * x[i];
        y[j] = y[j] + p;
      }
  }
}

/* Outer product A(m x n) = x y^T (cuda/linalg.go:232-285). */
EXPORT void oracle_outer_f32(int64_t m, int64_t n, const float* x, const float* y, float* A) {
  int64_t i, j;
  for (i = 0; i < m; i++)
    for (j = 0; j < n; j++) A[i * n + j] = x[i] * y[j];
}

/* ------------------------------------------------------------------ */
/* Conv2d the way the CPU graph does it (nn.go:211-305):               */
/*   im2col -> (B*oh*ow, C*kh*kw) x (F, C*kh*kw)^T -> reshape          */
/*   (B,oh,ow,F) -> transpose (0,3,1,2).                               */
/* im2col layout and zero padding: op_nn.go:415-444; output size:      */
/* op_nn.go:311-315.                                                   */
/* ------------------------------------------------------------------ */
EXPORT void oracle_conv_out_hw(int64_t h, int64_t w, int64_t kh, int64_t kw, int64_t padH,
                               int64_t padW, int64_t strideH, int64_t strideW, int64_t dilH,
                               int64_t dilW, int64_t* oh, int64_t* ow) {
  *oh = (h + 2 * padH - (dilH * (kh - 1) + 1)) / strideH + 1;
  *ow = (w + 2 * padW - (dilW * (kw - 1) + 1)) / strideW + 1;
}

EXPORT void oracle_im2col_f32(const float* im, float* col, int64_t B, int64_t C, int64_t H,
                              int64_t W, int64_t kh, int64_t kw, int64_t padH, int64_t padW,
                              int64_t strideH, int64_t strideW, int64_t dilH, int64_t dilW) {
  int64_t oh, ow, b;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
  int64_t K = C * kh * kw;
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (b = 0; b < B; b++) {
    const float* imb = im + b * C * H * W;
    float* colb = col + b * oh * ow * K;
    int64_t idx = 0, orow, ocol, ch, kr, kc;
    for (orow = 0; orow < oh; orow++)
      for (ocol = 0; ocol < ow; ocol++)
        for (ch = 0; ch < C; ch++)
          for (kr = 0; kr < kh; kr++) {
            int64_t ir = -padH + kr * dilH + orow * strideH;
            for (kc = 0; kc < kw; kc++) {
              int64_t ic = -padW + kc * dilW + ocol * strideW;
              if (ir < 0 || ir >= H || ic < 0 || ic >= W) colb[idx] = 0.0f;
              else colb[idx] = imb[ch * H * W + ir * W + ic];
              idx++;
            }
          }
  }
}

EXPORT int oracle_conv2d_f32(const float* x, const float* w, float* y, int64_t B, int64_t C,
                             int64_t H, int64_t W, int64_t F, int64_t kh, int64_t kw, int64_t padH,
                             int64_t padW, int64_t strideH, int64_t strideW, int64_t dilH,
                             int64_t dilW) {
  int64_t oh, ow;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
  int64_t K = C * kh * kw, M = B * oh * ow;
  float* col = (float*)malloc((size_t)M * K * sizeof(float));
  float* out = (float*)malloc((size_t)M * F * sizeof(float));
  if (!col || !out) { free(col); free(out); return -1; }
  oracle_im2col_f32(x, col, B, C, H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW);
  oracle_gemm_f32(0, 1, M, F, K, col, K, w, K, out, F);
  /* (B,oh,ow,F) -> (B,F,oh,ow) */
  int64_t b, f, p, P = oh * ow;
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (b = 0; b < B; b++)
    for (f = 0; f < F; f++)
      for (p = 0; p < P; p++) y[(b * F + f) * P + p] = out[(b * P + p) * F + f];
  free(col);
  free(out);
  return 0;
}

/* Direct NCHW cross-correlation in float64: the brute-force yardstick
 * used to pin oracle_conv2d_f32 (textbook definition, no im2col). */
EXPORT void oracle_conv2d_direct_f64(const float* x, const float* w, double* y, int64_t B,
                                     int64_t C, int64_t H, int64_t W, int64_t F, int64_t kh,
                                     int64_t kw, int64_t padH, int64_t padW, int64_t strideH,
                                     int64_t strideW, int64_t dilH, int64_t dilW) {
  int64_t oh, ow, b;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (b = 0; b < B; b++) {
    int64_t f, r, c, ch, kr, kc;
    for (f = 0; f < F; f++)
      for (r = 0; r < oh; r++)
        for (c = 0; c < ow; c++) {
          double acc = 0.0;
          for (ch = 0; ch < C; ch++)
            for (kr = 0; kr < kh; kr++)
              for (kc = 0; kc < kw; kc++) {
                int64_t ir = r * strideH - padH + kr * dilH;
                int64_t ic = c * strideW - padW + kc * dilW;
                if (ir < 0 || ir >= H || ic < 0 || ic >= W) continue;
                acc += (double)x[((b * C + ch) * H + ir) * W + ic] *
                       (double)w[((f * C + ch) * kh + kr) * kw + kc];
              }
          y[((b * F + f) * oh + r) * ow + c] = acc;
        }
  }
}

/* ------------------------------------------------------------------ */
/* MaxPool2D forward: op_nn.go:860-907, shape op_nn.go:810-816.        */
/* pad4 = {north, south, west, east}.  With explicit (4-value) padding */
/* the reference offsets the window by padSouth/padEast                */
/* (op_nn.go:871-875); with 2-value padding by padNorth/padWest.       */
/* Init -FLT_MAX, strict >, row-major scan of the clipped window.      */
/* ------------------------------------------------------------------ */
EXPORT void oracle_maxpool_out_hw(int64_t h, int64_t w, int64_t kh, int64_t kw,
                                  const int64_t* pad4, int64_t strideH, int64_t strideW,
                                  int64_t* oh, int64_t* ow) {
  *oh = (h + pad4[1] + pad4[0] - (kh - 1) - 1) / strideH + 1;
  *ow = (w + pad4[3] + pad4[2] - (kw - 1) - 1) / strideW + 1;
}

EXPORT void oracle_maxpool2d_f32(const float* x, float* y, int64_t B, int64_t C, int64_t H,
                                 int64_t W, int64_t kh, int64_t kw, const int64_t* pad4,
                                 int explicit_padding, int64_t strideH, int64_t strideW) {
  int64_t oh, ow, bc;
  oracle_maxpool_out_hw(H, W, kh, kw, pad4, strideH, strideW, &oh, &ow);
  int64_t padH = explicit_padding ? pad4[1] : pad4[0];
  int64_t padW = explicit_padding ? pad4[3] : pad4[2];
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (bc = 0; bc < B * C; bc++) {
    const float* in = x + bc * H * W;
    float* out = y + bc * oh * ow;
    int64_t ph, pw, hi, wi;
    for (ph = 0; ph < oh; ph++)
      for (pw = 0; pw < ow; pw++) {
        int64_t hs = ph * strideH - padH, ws = pw * strideW - padW;
        int64_t he = hs + kh < H ? hs + kh : H;
        int64_t we = ws + kw < W ? ws + kw : W;
        if (hs < 0) hs = 0;
        if (ws < 0) ws = 0;
        float best = -FLT_MAX;
        for (hi = hs; hi < he; hi++)
          for (wi = ws; wi < we; wi++)
            if (in[hi * W + wi] > best) best = in[hi * W + wi];
        out[ph * ow + pw] = best;
      }
  }
}

/* ------------------------------------------------------------------ */
/* BatchNorm (per channel; x is (B, C, S) with S = prod of the trailing */
/* dims, or (B, C) with S = 1).                                        */
/* Eval: op_nn.go:1559-1584 + 1610-1631:                               */
/*   a = 1/sqrt(var+eps); b = -mean*a; y = x*a + b  (two roundings)    */
/* then the gamma/beta wrap of nn.go:429-440 as separate broadcast     */
/* mul and add (gamma, beta have C elements here).                     */
/* ------------------------------------------------------------------ */
EXPORT void oracle_bn_alpha_beta_f32(const float* mean, const float* var, float eps, float* alpha,
                                     float* beta, int64_t C) {
  int64_t c;
  for (c = 0; c < C; c++) {
    float v = var[c] + eps;
    float inv = 1.0f / sqrtf(v);
    alpha[c] = inv;
    float nm = -mean[c];
    beta[c] = nm * inv;
  }
}

EXPORT void oracle_bn_infer_f32(const float* x, float* y, const float* run_mean,
                                const float* run_var, const float* gamma, const float* beta_in,
                                float eps, int64_t B, int64_t C, int64_t S) {
  float* a = (float*)malloc((size_t)C * sizeof(float));
  float* b = (float*)malloc((size_t)C * sizeof(float));
  oracle_bn_alpha_beta_f32(run_mean, run_var, eps, a, b, C);
  int64_t bc;
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (bc = 0; bc < B * C; bc++) {
    int64_t c = bc % C, d;
    const float* in = x + bc * S;
    float* out = y + bc * S;
    for (d = 0; d < S; d++) {
      float t = in[d] * a[c];
      t = t + b[c];
      if (gamma) t = gamma[c] * t;
      if (beta_in) t = t + beta_in[c];
      out[d] = t;
    }
  }
  free(a);
  free(b);
}

/* One training-mode forward (op_nn.go:1489-1555, 1559-1584): batch
 * mean, biased variance for normalising, running stats updated with
 * momentum weighting the *new* value and the unbiased variance.  Used
 * only to reproduce the reference's BN goldens (which run one training
 * step before the eval pass). */
EXPORT void oracle_bn_train_f32(const float* x, float* y, float* run_mean, float* run_var,
                                float momentum, float eps, int64_t B, int64_t C, int64_t S) {
  int64_t n = B * S, c;
  for (c = 0; c < C; c++) {
    float mean = 0.0f, var = 0.0f;
    int64_t s, d;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) mean = mean + x[(s * C + c) * S + d];
    mean = mean / (float)n;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        float t = x[(s * C + c) * S + d] - mean;
        float t2 = t * t;
        var = var + t2;
      }
    {
      float m1 = momentum * mean;
      float m2 = (1.0f - momentum) * run_mean[c];
      run_mean[c] = m1 + m2;
      float unb = var / (float)(n - 1);
      float v1 = momentum * unb;
      float v2 = (1.0f - momentum) * run_var[c];
      run_var[c] = v1 + v2;
    }
    float vb = var / (float)n;
    float inv = 1.0f / sqrtf(vb + eps);
    float a = inv;
    float b = -mean * a;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        float t = x[i] * a;
        y[i] = t + b;
      }
  }
}

/* ------------------------------------------------------------------ */
/* SoftMax over the last axis (op_softmax.go:99-128 -> tensor.SoftMax): */
/* max-subtracted exp, sum, divide.                                    */
/* ================================================================== */
/* Backward passes (the reference's diff ops on the CPU engine).       */
/* ================================================================== */

/* MaxPool2D backward: maxPoolDiffOp.f32s (op_nn.go:1067-1093) driven by the
 * argmax mask the forward pass records (op_nn.go:860-907: first element in
 * row-major window order that is strictly greater than everything before,
 * starting from -FLT_MAX; -1 when nothing wins, which contributes nothing
 * here).  dx is zeroed, then every window adds its dy into its argmax in
 * (ph, pw) order. */
EXPORT void oracle_maxpool2d_bwd_f32(const float* x, const float* dy, float* dx, int64_t B,
                                     int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw,
                                     const int64_t* pad4, int explicit_padding, int64_t strideH,
                                     int64_t strideW) {
  int64_t oh, ow, bc;
  oracle_maxpool_out_hw(H, W, kh, kw, pad4, strideH, strideW, &oh, &ow);
  int64_t padH = explicit_padding ? pad4[1] : pad4[0];
  int64_t padW = explicit_padding ? pad4[3] : pad4[2];
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (bc = 0; bc < B * C; bc++) {
    const float* in = x + bc * H * W;
    const float* g = dy + bc * oh * ow;
    float* out = dx + bc * H * W;
    int64_t ph, pw, hi, wi, i;
    for (i = 0; i < H * W; i++) out[i] = 0.0f;
    for (ph = 0; ph < oh; ph++)
      for (pw = 0; pw < ow; pw++) {
        int64_t hs = ph * strideH - padH, ws = pw * strideW - padW;
        int64_t he = hs + kh < H ? hs + kh : H;
        int64_t we = ws + kw < W ? ws + kw : W;
        if (hs < 0) hs = 0;
        if (ws < 0) ws = 0;
        float best = -FLT_MAX;
        int64_t arg = -1;
        for (hi = hs; hi < he; hi++)
          for (wi = ws; wi < we; wi++)
            if (in[hi * W + wi] > best) { best = in[hi * W + wi]; arg = hi * W + wi; }
        if (arg >= 0) out[arg] = out[arg] + g[ph * ow + pw];
      }
  }
}

/* col2im: col2imOp.f32s (op_nn.go:605-640), per image, accumulation in
 * (outputRow, outputCol, channel, kernelRow, kernelCol) order. */
static void col2im_one_f32(const float* col, float* im, int64_t C, int64_t H, int64_t W,
                           int64_t kh, int64_t kw, int64_t padH, int64_t padW, int64_t strideH,
                           int64_t strideW, int64_t dilH, int64_t dilW, int64_t oh, int64_t ow) {
  int64_t i, r, c, ch, kr, kc, idx = 0;
  for (i = 0; i < C * H * W; i++) im[i] = 0.0f;
  for (r = 0; r < oh; r++)
    for (c = 0; c < ow; c++)
      for (ch = 0; ch < C; ch++)
        for (kr = 0; kr < kh; kr++) {
          int64_t ir = -padH + kr * dilH + r * strideH;
          for (kc = 0; kc < kw; kc++) {
            int64_t ic = -padW + kc * dilW + c * strideW;
            if (ir >= 0 && ir < H && ic >= 0 && ic < W) {
              float* t = &im[(ch * H + ir) * W + ic];
              *t = *t + col[idx];
            }
            idx++;
          }
        }
}

/* Conv2d backward as the reference's graph differentiates it (nn.go:211-305):
 * y = transpose(reshape(col . Wflat^T)), so with dY2d = (B*oh*ow, F):
 *   dCol = dY2d . Wflat          (linAlgBinOp diff wrt the first operand)
 *   dX   = col2im(dCol)          (im2colOp.DoDiff, op_nn.go:267-291)
 *   dW   = dY2d^T . col          (diff wrt the second, transposed operand)
 * Either output pointer may be NULL. */
EXPORT int oracle_conv2d_bwd_f32(const float* x, const float* w, const float* dy, float* dx,
                                 float* dw, int64_t B, int64_t C, int64_t H, int64_t W, int64_t F,
                                 int64_t kh, int64_t kw, int64_t padH, int64_t padW,
                                 int64_t strideH, int64_t strideW, int64_t dilH, int64_t dilW) {
  int64_t oh, ow;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
  int64_t K = C * kh * kw, P = oh * ow, M = B * P;
  float* dy2 = (float*)malloc((size_t)M * F * sizeof(float));
  float* col = (float*)malloc((size_t)M * K * sizeof(float));
  if (!dy2 || !col) { free(dy2); free(col); return -1; }
  int64_t b, f, p;
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (b = 0; b < B; b++)
    for (f = 0; f < F; f++)
      for (p = 0; p < P; p++) dy2[(b * P + p) * F + f] = dy[(b * F + f) * P + p];
  if (dw) {
    oracle_im2col_f32(x, col, B, C, H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW);
    oracle_gemm_f32(1, 0, F, K, M, dy2, F, col, K, dw, K);
  }
  if (dx) {
    oracle_gemm_f32(0, 0, M, K, F, dy2, F, w, K, col, K);
#pragma omp parallel for if (g_threads > 1) schedule(static)
    for (b = 0; b < B; b++)
      col2im_one_f32(col + b * P * K, dx + b * C * H * W, C, H, W, kh, kw, padH, padW, strideH,
                     strideW, dilH, dilW, oh, ow);
  }
  free(dy2);
  free(col);
  return 0;
}

/* The same two gradients from the definition, in float64: the yardstick that
 * pins oracle_conv2d_bwd_f32 (every product x*w*dy of the forward sum is
 * attributed to its x and its w). */
EXPORT void oracle_conv2d_bwd_direct_f64(const float* x, const float* w, const float* dy,
                                         double* dx, double* dw, int64_t B, int64_t C, int64_t H,
                                         int64_t W, int64_t F, int64_t kh, int64_t kw,
                                         int64_t padH, int64_t padW, int64_t strideH,
                                         int64_t strideW, int64_t dilH, int64_t dilW) {
  int64_t oh, ow, b, f, r, c, ch, kr, kc, i;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
  for (i = 0; i < B * C * H * W; i++) dx[i] = 0.0;
  for (i = 0; i < F * C * kh * kw; i++) dw[i] = 0.0;
  for (b = 0; b < B; b++)
    for (f = 0; f < F; f++)
      for (r = 0; r < oh; r++)
        for (c = 0; c < ow; c++) {
          const double g = (double)dy[((b * F + f) * oh + r) * ow + c];
          for (ch = 0; ch < C; ch++)
            for (kr = 0; kr < kh; kr++)
              for (kc = 0; kc < kw; kc++) {
                int64_t ir = r * strideH - padH + kr * dilH;
                int64_t ic = c * strideW - padW + kc * dilW;
                if (ir < 0 || ir >= H || ic < 0 || ic >= W) continue;
                int64_t xi = ((b * C + ch) * H + ir) * W + ic;
                int64_t wi = ((f * C + ch) * kh + kr) * kw + kc;
                dx[xi] += g * (double)w[wi];
                dw[wi] += g * (double)x[xi];
              }
        }
}

/* BatchNorm forward in training mode with the saved statistics exposed:
 * updateStatsF32 (op_nn.go:1489-1555) + calculateAlphaAndBetaF32 + the apply
 * loop (op_nn.go:1559-1635).  save_var receives the SUM of squared deviations
 * (the reference divides by n only where it is used). */
EXPORT void oracle_bn_train_stats_f32(const float* x, float* y, float* run_mean, float* run_var,
                                      float* save_mean, float* save_var, float momentum,
                                      float eps, int64_t B, int64_t C, int64_t S) {
  int64_t n = B * S, c;
  for (c = 0; c < C; c++) {
    float mean = 0.0f, var = 0.0f;
    int64_t s, d;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) mean = mean + x[(s * C + c) * S + d];
    mean = mean / (float)n;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        float t = x[(s * C + c) * S + d] - mean;
        float t2 = t * t;
        var = var + t2;
      }
    save_mean[c] = mean;
    save_var[c] = var;
    {
      float m1 = momentum * mean;
      float m2 = (1.0f - momentum) * run_mean[c];
      run_mean[c] = m1 + m2;
      float unb = var / (float)(n - 1);
      float v1 = momentum * unb;
      float v2 = (1.0f - momentum) * run_var[c];
      run_var[c] = v1 + v2;
    }
    float vb = var / (float)n;
    float inv = 1.0f / sqrtf(vb + eps);
    float a = inv;
    float b = -mean * a;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        float t = x[i] * a;
        y[i] = t + b;
      }
  }
}

/* BatchNorm backward, training branch of batchnormDiffOp.f32s for inputs with
 * a spatial extent (op_nn.go:1893-1926; the S == 1 branch, op_nn.go:1850-1878,
 * differs only in how the dot product is written and is followed when S == 1):
 *   sum = SUM dy, dotp = SUM (x*dy - mean*dy), invstd = 1/sqrt(save_var/n + eps),
 *   k = dotp*invstd*invstd/n, gradMean = sum/n,
 *   dx = (dy - gradMean - (x - mean)*k) * invstd.
 * training == 0: dx = dy * invstd (op_nn.go:1928-1936). */
EXPORT void oracle_bn_bwd_f32(const float* x, const float* dy, float* dx, const float* save_mean,
                              const float* save_var, float eps, int training, int64_t B,
                              int64_t C, int64_t S) {
  int64_t n = B * S, c;
  for (c = 0; c < C; c++) {
    float dotp = 0.0f, sum = 0.0f;
    int64_t s, d;
    const float mean = save_mean[c];
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        sum = sum + dy[i];
        float partial;
        if (S == 1) {
          float t = x[i] - mean;
          partial = t * dy[i];
        } else {
          float t1 = x[i] * dy[i];
          float t2 = mean * dy[i];
          partial = t1 - t2;
        }
        dotp = dotp + partial;
      }
    float vb = save_var[c] / (float)n;
    float invstd = 1.0f / sqrtf(vb + eps);
    float kk = dotp * invstd;
    kk = kk * invstd;
    kk = kk / (float)n;
    float gradMean = sum / (float)n;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        if (training) {
          float t = x[i] - mean;
          t = t * kk;
          float u;
          if (S == 1) { u = dy[i] - t; u = u - gradMean; }
          else { u = dy[i] - gradMean; u = u - t; }
          dx[i] = u * invstd;
        } else {
          dx[i] = dy[i] * invstd;
        }
      }
  }
}

/* SoftMax backward over the last axis (softmaxDiffOp -> tensor.SoftMaxB,
 * op_softmax.go:266-279): dx_i = y_i * (dy_i - SUM_j dy_j*y_j). */
EXPORT void oracle_softmax_bwd_f32(const float* y, const float* dy, float* dx, int64_t rows,
                                   int64_t cols) {
  int64_t r, j;
  for (r = 0; r < rows; r++) {
    const float* yy = y + r * cols;
    const float* g = dy + r * cols;
    float dot = 0.0f;
    for (j = 0; j < cols; j++) { float t = g[j] * yy[j]; dot = dot + t; }
    for (j = 0; j < cols; j++) { float t = g[j] - dot; dx[r * cols + j] = yy[j] * t; }
  }
}

/* ================================================================== */
/* Solver steps on float32 tensors: the *tensor.Dense branches of      */
/* VanillaSolver.Step (solvers.go:780-870), RMSPropSolver.Step         */
/* (solvers.go:273-372) and AdamSolver.Step (solvers.go:461-640), one  */
/* element at a time with every tensor op's rounding kept.             */
/* par: 0 eta, 1 eps, 2 l1reg, 3 l2reg, 4 clip, 5 1/batch,             */
/*      6 decay | beta1, 7 1-decay | beta2, 8 1/correction1,           */
/*      9 1/correction2.  use: bit0 l1, bit1 l2, bit2 clip, bit3 batch */
/* The gradient is left as the reference leaves it before g.Zero().    */
/* ================================================================== */
static float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }
static float signf(float v) { return v > 0.0f ? 1.0f : (v < 0.0f ? -1.0f : 0.0f); }

static float prep_grad(float g, float w, int use, const float* par) {
  if (use & 1) { float t = par[2] * signf(w); g = g + t; }
  if (use & 2) { float t = w * par[3]; g = g + t; }
  if (use & 8) g = g * par[5];
  if ((use & 4) && par[4] > 0.0f) g = clampf(g, -par[4], par[4]);
  return g;
}

EXPORT void oracle_solver_step_f32(int kind, float* w, float* g, float* c1, float* c2, int64_t n,
                                   int use, const float* par) {
  int64_t i;
  const float neg_eta = -par[0];
  for (i = 0; i < n; i++) {
    if (kind == 0) {            /* vanilla */
      float gi = prep_grad(g[i], w[i], use, par);
      gi = gi * neg_eta;
      w[i] = w[i] + gi;
      g[i] = gi;
    } else if (kind == 1) {     /* RMSProp */
      float gi = g[i];
      float gt2 = gi * gi;
      float cw = c1[i] * par[6];
      gt2 = gt2 * par[7];
      cw = cw + gt2;
      c1[i] = cw;
      if (use & 4) gi = clampf(gi, -par[4], par[4]);
      float upd = cw + par[1];
      upd = 1.0f / sqrtf(upd);
      gi = gi * neg_eta;
      upd = upd * gi;
      if (use & 2) { float reg = w[i] * par[3]; upd = upd - reg; }
      w[i] = w[i] + upd;
      g[i] = gi;
    } else {                    /* Adam */
      float gi = prep_grad(g[i], w[i], use, par);
      float omb1 = 1.0f - par[6], omb2 = 1.0f - par[7];
      float t1 = gi * omb1;
      float g2 = gi * gi;
      g2 = g2 * omb2;
      float mb = c1[i] * par[6];
      t1 = t1 + mb;
      float vb = c2[i] * par[7];
      g2 = g2 + vb;
      c1[i] = t1;
      c2[i] = g2;
      float mh = t1 * par[8];
      float vh = g2 * par[9];
      vh = sqrtf(vh);
      vh = vh + par[1];
      mh = mh * neg_eta;
      mh = mh / vh;
      w[i] = w[i] + mh;
      g[i] = g2;
    }
  }
}

/* ================================================================== */
/* Dropout: dropoutOp.do (op_dropout.go:107-132) and dropoutDiffOp     */
/* (op_dropout.go:205-238).  r holds the values the op's random source */
/* returns, one per element in order.  Outputs that are not kept stay  */
/* at the zero a fresh tensor holds.  The gradient divides by the DROP */
/* probability, as the reference does.                                 */
/* ================================================================== */
EXPORT void oracle_dropout_f32(const float* x, const float* r, float* y, int64_t n, double prob,
                               int training) {
  int64_t i;
  if (prob == 0.0 || !training) { for (i = 0; i < n; i++) y[i] = x[i]; return; }
  const float keep = (float)(1.0 - prob);
  for (i = 0; i < n; i++) y[i] = r[i] < keep ? x[i] / keep : 0.0f;
}

EXPORT void oracle_dropout_bwd_f32(const float* y, const float* dy, float* dx, int64_t n, double prob) {
  int64_t i;
  const float p = (float)prob;
  for (i = 0; i < n; i++) dx[i] = (prob != 0.0 && y[i] != 0.0f) ? dy[i] / p : 0.0f;
}

/* Counter-based uniform source in [0, 1) with 24 random bits: element i of
 * stream (seed, offset) is SplitMix64's output function applied to
 * seed*0xD1342543DE82EF95 + (offset + i + 1)*0x9E3779B97F4A7C15, top 24 bits.
 * Not the reference's generator (that one is seeded from the wall clock,
 * nn.go:72); this is the engine's own, stated here so the device can be
 * checked bit for bit. */
EXPORT void oracle_uniform01_f32(float* out, int64_t n, uint64_t seed, uint64_t offset) {
  int64_t i;
  for (i = 0; i < n; i++) {
    uint64_t z = seed * 0xD1342543DE82EF95ull + (offset + (uint64_t)i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    out[i] = (float)(z >> 40) * 5.9604644775390625e-08f;
  }
}

/* The float64 form keeps the top 53 bits of the same 64-bit value. */
EXPORT void oracle_uniform01_f64(double* out, int64_t n, uint64_t seed, uint64_t offset) {
  int64_t i;
  for (i = 0; i < n; i++) {
    uint64_t z = seed * 0xD1342543DE82EF95ull + (offset + (uint64_t)i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    out[i] = (double)(z >> 11) * 1.1102230246251565e-16;
  }
}

/* ------------------------------------------------------------------ */
EXPORT void oracle_softmax_f32(const float* x, float* y, int64_t rows, int64_t cols) {
  int64_t r, j;
  for (r = 0; r < rows; r++) {
    const float* in = x + r * cols;
    float* out = y + r * cols;
    float mx = -INFINITY;
    for (j = 0; j < cols; j++) if (in[j] > mx) mx = in[j];
    float sum = 0.0f;
    for (j = 0; j < cols; j++) {
      out[j] = (float)exp((double)(in[j] - mx));
      sum = sum + out[j];
    }
    /* tensor.SoftMax (not vendored) is recalled to scale by the rounded
     * reciprocal of the sum; exp*(1/sum) and exp/sum differ by <= 1 ulp, well
     * inside the softmax tolerance.  PARITY UNPINNED bit-for-bit. */
    float inv = 1.0f / sum;
    for (j = 0; j < cols; j++) out[j] = out[j] * inv;
  }
}

EXPORT void oracle_softmax_f64(const double* x, double* y, int64_t rows, int64_t cols) {
  int64_t r, j;
  for (r = 0; r < rows; r++) {
    const double* in = x + r * cols;
    double* out = y + r * cols;
    double mx = -INFINITY, sum = 0.0;
    for (j = 0; j < cols; j++) if (in[j] > mx) mx = in[j];
    for (j = 0; j < cols; j++) { out[j] = exp(in[j] - mx); sum += out[j]; }
    for (j = 0; j < cols; j++) out[j] /= sum;
  }
}

/* HasNaN / HasInf predicates (cuda/engine.go:144-191, misc.cu:14-56). */
/* ------------------------------------------------------------------ */
/* float64 twins of the forward neural-network operators.  Each is the  */
/* float32 function above with the element type changed (the CPU ops    */
/* switch on the dtype and run the same loops, op_nn.go:909-957,        */
/* 1559-1631; nn.go:83-163): no new algorithm, pinned through the        */
/* float32 instance on data where both are exact, and by the float64    */
/* rows of the reference's batch-norm table.  The convolution sums      */
/* k = (c, kr, kc) in ascending order with a rounded multiply and a     */
/* rounded add per step, like oracle_gemm_f32 does for the im2col form. */
/* ------------------------------------------------------------------ */
EXPORT void oracle_relu_f64(double* y, const double* x, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) {
    double m = x[i] >= 0.0 ? 1.0 : 0.0;
    y[i] = x[i] * m;
  }
}

EXPORT void oracle_leaky_relu_f64(double* y, const double* x, double alpha, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) {
    double ge = x[i] >= 0.0 ? 1.0 : 0.0;
    double lt = x[i] < 0.0 ? 1.0 : 0.0;
    double pos = x[i] * ge;
    double neg = x[i] * lt;
    double nega = neg * alpha;
    y[i] = pos + nega;
  }
}

EXPORT void oracle_conv2d_f64(const double* x, const double* w, double* y, int64_t B, int64_t C,
                              int64_t H, int64_t W, int64_t F, int64_t kh, int64_t kw, int64_t padH,
                              int64_t padW, int64_t strideH, int64_t strideW, int64_t dilH,
                              int64_t dilW) {
  int64_t oh, ow, bf;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (bf = 0; bf < B * F; bf++) {
    int64_t b = bf / F, f = bf % F, orow, ocol, ch, kr, kc;
    for (orow = 0; orow < oh; orow++)
      for (ocol = 0; ocol < ow; ocol++) {
        double acc = 0.0;
        for (ch = 0; ch < C; ch++)
          for (kr = 0; kr < kh; kr++) {
            int64_t ir = -padH + kr * dilH + orow * strideH;
            for (kc = 0; kc < kw; kc++) {
              int64_t ic = -padW + kc * dilW + ocol * strideW;
              double v = (ir < 0 || ir >= H || ic < 0 || ic >= W) ? 0.0 : x[((b * C + ch) * H + ir) * W + ic];
              double p = v * w[((f * C + ch) * kh + kr) * kw + kc];
              acc = acc + p;
            }
          }
        y[(bf * oh + orow) * ow + ocol] = acc;
      }
  }
}

EXPORT void oracle_maxpool2d_f64(const double* x, double* y, int64_t B, int64_t C, int64_t H,
                                 int64_t W, int64_t kh, int64_t kw, const int64_t* pad4,
                                 int explicit_padding, int64_t strideH, int64_t strideW) {
  int64_t oh, ow, bc;
  oracle_maxpool_out_hw(H, W, kh, kw, pad4, strideH, strideW, &oh, &ow);
  int64_t padH = explicit_padding ? pad4[1] : pad4[0];
  int64_t padW = explicit_padding ? pad4[3] : pad4[2];
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (bc = 0; bc < B * C; bc++) {
    const double* in = x + bc * H * W;
    double* out = y + bc * oh * ow;
    int64_t ph, pw, hi, wi;
    for (ph = 0; ph < oh; ph++)
      for (pw = 0; pw < ow; pw++) {
        int64_t hs = ph * strideH - padH, ws = pw * strideW - padW;
        int64_t he = hs + kh < H ? hs + kh : H;
        int64_t we = ws + kw < W ? ws + kw : W;
        if (hs < 0) hs = 0;
        if (ws < 0) ws = 0;
        double best = -DBL_MAX;   /* -maxFloat64, op_nn.go:916 */
        for (hi = hs; hi < he; hi++)
          for (wi = ws; wi < we; wi++)
            if (in[hi * W + wi] > best) best = in[hi * W + wi];
        out[ph * ow + pw] = best;
      }
  }
}

EXPORT void oracle_bn_infer_f64(const double* x, double* y, const double* run_mean,
                                const double* run_var, const double* gamma, const double* beta_in,
                                double eps, int64_t B, int64_t C, int64_t S) {
  int64_t bc;
#pragma omp parallel for if (g_threads > 1) schedule(static)
  for (bc = 0; bc < B * C; bc++) {
    int64_t c = bc % C, d;
    double v = run_var[c] + eps;
    double a = 1.0 / sqrt(v);
    double nm = -run_mean[c];
    double b = nm * a;
    const double* in = x + bc * S;
    double* out = y + bc * S;
    for (d = 0; d < S; d++) {
      double t = in[d] * a;
      t = t + b;
      if (gamma) t = gamma[c] * t;
      if (beta_in) t = t + beta_in[c];
      out[d] = t;
    }
  }
}

/* ================================================================== */
/* float64 twins of the backward operators, dropout and the solver     */
/* steps: the reference's Float64 branches (maxPoolDiffOp.f64s         */
/* op_nn.go:1095-1120, softmaxDiffOp op_softmax.go:266-279, dropout    */
/* op_dropout.go:118-132,215-238, the Float64 cases of the solvers'    */
/* Step solvers.go:299,496,793) - the float32 restatements above with  */
/* every operation in double.                                          */
/* ================================================================== */
EXPORT void oracle_maxpool2d_bwd_f64(const double* x, const double* dy, double* dx, int64_t B,
                                     int64_t C, int64_t H, int64_t W, int64_t kh, int64_t kw,
                                     const int64_t* pad4, int explicit_padding, int64_t strideH,
                                     int64_t strideW) {
  int64_t oh, ow, bc;
  oracle_maxpool_out_hw(H, W, kh, kw, pad4, strideH, strideW, &oh, &ow);
  int64_t padH = explicit_padding ? pad4[1] : pad4[0];
  int64_t padW = explicit_padding ? pad4[3] : pad4[2];
  for (bc = 0; bc < B * C; bc++) {
    const double* in = x + bc * H * W;
    const double* g = dy + bc * oh * ow;
    double* out = dx + bc * H * W;
    int64_t ph, pw, hi, wi, i;
    for (i = 0; i < H * W; i++) out[i] = 0.0;
    for (ph = 0; ph < oh; ph++)
      for (pw = 0; pw < ow; pw++) {
        int64_t hs = ph * strideH - padH, ws = pw * strideW - padW;
        int64_t he = hs + kh < H ? hs + kh : H;
        int64_t we = ws + kw < W ? ws + kw : W;
        if (hs < 0) hs = 0;
        if (ws < 0) ws = 0;
        double best = -DBL_MAX;
        int64_t arg = -1;
        for (hi = hs; hi < he; hi++)
          for (wi = ws; wi < we; wi++)
            if (in[hi * W + wi] > best) { best = in[hi * W + wi]; arg = hi * W + wi; }
        if (arg >= 0) out[arg] = out[arg] + g[ph * ow + pw];
      }
  }
}

EXPORT void oracle_bn_train_stats_f64(const double* x, double* y, double* run_mean, double* run_var,
                                      double* save_mean, double* save_var, double momentum,
                                      double eps, int64_t B, int64_t C, int64_t S) {
  int64_t n = B * S, c;
  for (c = 0; c < C; c++) {
    double mean = 0.0, var = 0.0;
    int64_t s, d;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) mean = mean + x[(s * C + c) * S + d];
    mean = mean / (double)n;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        double t = x[(s * C + c) * S + d] - mean;
        double t2 = t * t;
        var = var + t2;
      }
    save_mean[c] = mean;
    save_var[c] = var;
    {
      double m1 = momentum * mean;
      double m2 = (1.0 - momentum) * run_mean[c];
      run_mean[c] = m1 + m2;
      double unb = var / (double)(n - 1);
      double v1 = momentum * unb;
      double v2 = (1.0 - momentum) * run_var[c];
      run_var[c] = v1 + v2;
    }
    double vb = var / (double)n;
    double a = 1.0 / sqrt(vb + eps);
    double b = -mean * a;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        double t = x[i] * a;
        y[i] = t + b;
      }
  }
}

EXPORT void oracle_bn_bwd_f64(const double* x, const double* dy, double* dx, const double* save_mean,
                              const double* save_var, double eps, int training, int64_t B,
                              int64_t C, int64_t S) {
  int64_t n = B * S, c;
  for (c = 0; c < C; c++) {
    double dotp = 0.0, sum = 0.0;
    int64_t s, d;
    const double mean = save_mean[c];
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        sum = sum + dy[i];
        double partial;
        if (S == 1) {
          double t = x[i] - mean;
          partial = t * dy[i];
        } else {
          double t1 = x[i] * dy[i];
          double t2 = mean * dy[i];
          partial = t1 - t2;
        }
        dotp = dotp + partial;
      }
    double vb = save_var[c] / (double)n;
    double invstd = 1.0 / sqrt(vb + eps);
    double kk = dotp * invstd;
    kk = kk * invstd;
    kk = kk / (double)n;
    double gradMean = sum / (double)n;
    for (s = 0; s < B; s++)
      for (d = 0; d < S; d++) {
        int64_t i = (s * C + c) * S + d;
        if (training) {
          double t = x[i] - mean;
          t = t * kk;
          double u;
          if (S == 1) { u = dy[i] - t; u = u - gradMean; }
          else { u = dy[i] - gradMean; u = u - t; }
          dx[i] = u * invstd;
        } else {
          dx[i] = dy[i] * invstd;
        }
      }
  }
}

/* Conv2d gradients from the definition with float64 operands: the float64 twin
 * of oracle_conv2d_bwd_f32 (same products; float64 sums make the order moot at
 * the conv tolerance, and on integer-valued data every order is exact). */
EXPORT void oracle_conv2d_bwd_f64(const double* x, const double* w, const double* dy, double* dx,
                                  double* dw, int64_t B, int64_t C, int64_t H, int64_t W, int64_t F,
                                  int64_t kh, int64_t kw, int64_t padH, int64_t padW,
                                  int64_t strideH, int64_t strideW, int64_t dilH, int64_t dilW) {
  int64_t oh, ow, b, f, r, c, ch, kr, kc, i;
  oracle_conv_out_hw(H, W, kh, kw, padH, padW, strideH, strideW, dilH, dilW, &oh, &ow);
  for (i = 0; i < B * C * H * W; i++) dx[i] = 0.0;
  for (i = 0; i < F * C * kh * kw; i++) dw[i] = 0.0;
  for (b = 0; b < B; b++)
    for (f = 0; f < F; f++)
      for (r = 0; r < oh; r++)
        for (c = 0; c < ow; c++) {
          const double g = dy[((b * F + f) * oh + r) * ow + c];
          for (ch = 0; ch < C; ch++)
            for (kr = 0; kr < kh; kr++)
              for (kc = 0; kc < kw; kc++) {
                int64_t ir = r * strideH - padH + kr * dilH;
                int64_t ic = c * strideW - padW + kc * dilW;
                if (ir < 0 || ir >= H || ic < 0 || ic >= W) continue;
                int64_t xi = ((b * C + ch) * H + ir) * W + ic;
                int64_t wi = ((f * C + ch) * kh + kr) * kw + kc;
                dx[xi] += g * w[wi];
                dw[wi] += g * x[xi];
              }
        }
}

EXPORT void oracle_softmax_bwd_f64(const double* y, const double* dy, double* dx, int64_t rows,
                                   int64_t cols) {
  int64_t r, j;
  for (r = 0; r < rows; r++) {
    const double* yy = y + r * cols;
    const double* g = dy + r * cols;
    double dot = 0.0;
    for (j = 0; j < cols; j++) { double t = g[j] * yy[j]; dot = dot + t; }
    for (j = 0; j < cols; j++) { double t = g[j] - dot; dx[r * cols + j] = yy[j] * t; }
  }
}

static double clampd(double v, double lo, double hi) { return v < lo ? lo : (v > hi ? hi : v); }
static double signd(double v) { return v > 0.0 ? 1.0 : (v < 0.0 ? -1.0 : 0.0); }

static double prep_grad_f64(double g, double w, int use, const double* par) {
  if (use & 1) { double t = par[2] * signd(w); g = g + t; }
  if (use & 2) { double t = w * par[3]; g = g + t; }
  if (use & 8) g = g * par[5];
  if ((use & 4) && par[4] > 0.0) g = clampd(g, -par[4], par[4]);
  return g;
}

EXPORT void oracle_solver_step_f64(int kind, double* w, double* g, double* c1, double* c2, int64_t n,
                                   int use, const double* par) {
  int64_t i;
  const double neg_eta = -par[0];
  for (i = 0; i < n; i++) {
    if (kind == 0) {            /* vanilla */
      double gi = prep_grad_f64(g[i], w[i], use, par);
      gi = gi * neg_eta;
      w[i] = w[i] + gi;
      g[i] = gi;
    } else if (kind == 1) {     /* RMSProp */
      double gi = g[i];
      double gt2 = gi * gi;
      double cw = c1[i] * par[6];
      gt2 = gt2 * par[7];
      cw = cw + gt2;
      c1[i] = cw;
      if (use & 4) gi = clampd(gi, -par[4], par[4]);
      double upd = cw + par[1];
      upd = 1.0 / sqrt(upd);
      gi = gi * neg_eta;
      upd = upd * gi;
      if (use & 2) { double reg = w[i] * par[3]; upd = upd - reg; }
      w[i] = w[i] + upd;
      g[i] = gi;
    } else {                    /* Adam */
      double gi = prep_grad_f64(g[i], w[i], use, par);
      double omb1 = 1.0 - par[6], omb2 = 1.0 - par[7];
      double t1 = gi * omb1;
      double g2 = gi * gi;
      g2 = g2 * omb2;
      double mb = c1[i] * par[6];
      t1 = t1 + mb;
      double vb = c2[i] * par[7];
      g2 = g2 + vb;
      c1[i] = t1;
      c2[i] = g2;
      double mh = t1 * par[8];
      double vh = g2 * par[9];
      vh = sqrt(vh);
      vh = vh + par[1];
      mh = mh * neg_eta;
      mh = mh / vh;
      w[i] = w[i] + mh;
      g[i] = g2;
    }
  }
}

EXPORT void oracle_dropout_f64(const double* x, const double* r, double* y, int64_t n, double prob,
                               int training) {
  int64_t i;
  if (prob == 0.0 || !training) { for (i = 0; i < n; i++) y[i] = x[i]; return; }
  const double keep = 1.0 - prob;
  for (i = 0; i < n; i++) y[i] = r[i] < keep ? x[i] / keep : 0.0;
}

EXPORT void oracle_dropout_bwd_f64(const double* y, const double* dy, double* dx, int64_t n, double prob) {
  int64_t i;
  for (i = 0; i < n; i++) dx[i] = (prob != 0.0 && y[i] != 0.0) ? dy[i] / prob : 0.0;
}

EXPORT int oracle_has_nan_f32(const float* a, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) if (isnan(a[i])) return 1;
  return 0;
}
EXPORT int oracle_has_inf_f32(const float* a, int64_t n) {
  int64_t i;
  for (i = 0; i < n; i++) if (isinf(a[i])) return 1;
  return 0;
}
