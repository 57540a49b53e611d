// Elementwise kernels for gfx950: binary (vv/vs/sv/ss), unary, fused
// broadcast, ReLU / LeakyReLU, fill and the NaN/Inf predicates.
//
// All of them are HBM-bound.  Each thread moves 16-byte vectors (float4 /
// double2); a workgroup walks whole chunks of kUnroll * 256 vectors in a
// grid-stride loop (16 workgroups per CU), so every wavefront access is a fully
// coalesced 1 KiB segment and a workgroup's accesses stay next to each other.
// Plain (cached) loads and stores while the operands can sit in the 256 MB
// last-level cache (non-temporal accesses lose ~15 % there); operands beyond that
// size stream with non-temporal accesses, which is ~10 % faster from HBM.
//
// Numerics: this file is compiled with -ffp-contract=off, denormals kept and
// IEEE division, so add/sub/mul/div/compare are bit-identical to the CPU
// engine (the reference builds its PTX the same way, cmd/cudagen/main.go:41-43).
// Transcendentals are evaluated in float64 and rounded once, the form the CPU
// engine uses for sigmoid (math_nooptim.go:36-44) and tanh (math_nooptim.go:22).
#include <cstdlib>

#include "gh_internal.h"

namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 2;

template <class T> struct VecOf;
template <> struct VecOf<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };
template <> struct VecOf<double> { typedef double type __attribute__((ext_vector_type(2))); static constexpr int N = 2; };

// ---- scalar functions ------------------------------------------------------

template <int FN, class T>
__device__ __forceinline__ T bin_apply(T a, T b) {
  if constexpr (FN == GH_ADD) return a + b;
  else if constexpr (FN == GH_SUB) return a - b;
  else if constexpr (FN == GH_MUL) return a * b;
  else if constexpr (FN == GH_DIV) return a / b;
  else if constexpr (FN == GH_POW) return (T)pow((double)a, (double)b);
  else if constexpr (FN == GH_LT) return a < b ? (T)1 : (T)0;
  else if constexpr (FN == GH_LTE) return a <= b ? (T)1 : (T)0;
  else if constexpr (FN == GH_GT) return a > b ? (T)1 : (T)0;
  else if constexpr (FN == GH_GTE) return a >= b ? (T)1 : (T)0;
  else if constexpr (FN == GH_EQ) return a == b ? (T)1 : (T)0;
  else if constexpr (FN == GH_MOD) return (T)fmod((double)a, (double)b);   // exact in either width
  else return a != b ? (T)1 : (T)0;
}

// exp in float64 for results that are rounded to float32 afterwards.
// Range reduction x = n ln2 + r with |r| <= ln2/2: n comes from the
// "add 1.5*2^52" trick (the integer sits in the low mantissa bits, so no
// round/convert instructions), exp(r) - 1 from a degree-10 Taylor polynomial
// (relative error below 2^-41, far under half a float32 ulp), and the scaling
// by 2^n is an integer add on the exponent field.  Valid for |x| <= 700;
// callers clamp.  Explicit fma() so the -ffp-contract=off build still gets
// fused steps here.  Conversion, reciprocal and ldexp instructions run at a
// quarter of the FMA rate on this hardware, which is why they are avoided:
// sigmoid/tanh/exp stay memory-bound.
struct ExpParts { double q; int n; };  // exp(x) = (1 + q) * 2^n

// A float64 constant pinned in a scalar register pair.  As a plain literal each
// Horner step costs an extra 64-bit vector move (the compiler materialises the
// coefficient into the accumulator of v_fmac_f64); from a scalar register the
// step is a single v_fma_f64.  The empty asm only hides the value's origin.
__device__ __forceinline__ double sconst(double v) {
  asm("" : "+s"(v));
  return v;
}

__device__ __forceinline__ ExpParts exp_parts(double x) {
  const double kShift = sconst(6755399441055744.0);  // 1.5 * 2^52
  const double t = fma(x, sconst(1.4426950408889634), kShift);
  const double n = t - kShift;
  double r = fma(-n, sconst(0.6931471803691238), x);   // ln2 high part
  r = fma(-n, sconst(1.9082149292705877e-10), r);      // ln2 low part
  double p = sconst(2.7557319223985893e-07);           // 1/10!
  p = fma(p, r, sconst(2.7557319223985888e-06));       // 1/9!
  p = fma(p, r, sconst(2.4801587301587302e-05));       // 1/8!
  p = fma(p, r, sconst(1.9841269841269841e-04));       // 1/7!
  p = fma(p, r, sconst(1.3888888888888889e-03));       // 1/6!
  p = fma(p, r, sconst(8.3333333333333332e-03));       // 1/5!
  p = fma(p, r, sconst(4.1666666666666664e-02));       // 1/4!
  p = fma(p, r, sconst(1.6666666666666666e-01));       // 1/3!
  p = fma(p, r, 0.5);
  p = fma(p, r, 1.0);
  ExpParts e;
  e.q = p * r;
  e.n = (int)(unsigned)__double_as_longlong(t);    // low 32 bits of t hold n
  return e;
}

__device__ __forceinline__ double scale_pow2(double v, int n) {  // v * 2^n, result normal
  return __longlong_as_double(__double_as_longlong(v) + ((long long)n << 52));
}

__device__ __forceinline__ double exp_f64_fast(double x) {
  const ExpParts e = exp_parts(x);
  return scale_pow2(1.0 + e.q, e.n);
}

// 1/s in float64 to ~2^-50: hardware reciprocal estimate plus one Newton step.
__device__ __forceinline__ double rcp_f64_fast(double s) {
  const double r = __builtin_amdgcn_rcp(s);
  return fma(fma(-s, r, 1.0), r, r);
}

// exp(x) for a float32 argument, rounded once from float64.
__device__ __forceinline__ float exp_f32_via_f64(float x) {
  double xd = (double)x;
  xd = xd < -110.0 ? -110.0 : xd;  // beyond the clamps the rounded result is 0 / +inf
  xd = xd > 90.0 ? 90.0 : xd;      // (NaN fails both compares and propagates)
  return (float)exp_f64_fast(xd);
}

// tanh in float64 from one exp, branch free: with a = 2|x|,
// tanh|x| = (e^a - 1)/(e^a + 1) = em1/(em1 + 2).  For n == 0 the polynomial
// yields e^a - 1 directly (no cancellation near zero); otherwise e^a >= sqrt(2)
// and the subtraction is harmless.  Error stays far below half a float32 ulp.
__device__ __forceinline__ double tanh_f64_for_f32(double x) {
  double a = 2.0 * fabs(x);
  a = a > 44.0 ? 44.0 : a;  // tanh rounds to 1 long before; NaN propagates
  const ExpParts e = exp_parts(a);
  const double em1 = e.n == 0 ? e.q : scale_pow2(1.0 + e.q, e.n) - 1.0;
  const double r = em1 * rcp_f64_fast(em1 + 2.0);
  return copysign(r, x);
}

// ---- float32 sigmoid / tanh without float64 ---------------------------------------
// The float64 forms above are within half an ulp but cost two quarter-rate
// conversions, a float64 reciprocal and ~20 half-rate FMAs per element, which
// makes a streaming kernel ALU-bound on this part.  These stay in float32, take
// about twenty instructions each and stay within 2 ulp of the correctly rounded
// result over every float32 input (measured exhaustively; the dense sweep in the
// GPU tests repeats it against the CPU oracle): sigmoid at most 2, tanh at most 1.
// With fewer instructions the kernels stay memory-bound at the clocks a device
// holds after minutes of load as well.
//
// exp(t) = 2^n * (1 + q): n = round(t / ln2) through the 1.5*2^23 shift (the
// integer also sits in the low mantissa bits of `shifted`), Cody-Waite reduction
// with a short-mantissa ln2 high part so that n*ln2_hi is exact, and
// exp(r) - 1 = r + r^2 P(r) with a degree-4 minimax P on |r| <= ln2/2 (relative
// error of exp below 2^-28).
struct ExpF { float q; int shbits; };

constexpr unsigned kShiftBits = 0x4B400000u;   // bits of 1.5 * 2^23

__device__ __forceinline__ ExpF expf_parts(float t) {
  const float kShift = 12582912.0f;  // 1.5 * 2^23
  const float shifted = __builtin_fmaf(t, 1.44269504088896341f, kShift);
  const float nf = shifted - kShift;
  float r = __builtin_fmaf(-nf, 0.693145751953125f, t);
  r = __builtin_fmaf(-nf, 1.428606765330187e-06f, r);
  float p = 0.0013813756f;
  p = __builtin_fmaf(p, r, 0.008369124f);
  p = __builtin_fmaf(p, r, 0.041668426f);
  p = __builtin_fmaf(p, r, 0.16666517f);
  p = __builtin_fmaf(p, r, 0.49999994f);
  ExpF e;
  e.q = __builtin_fmaf(r * r, p, r);
  e.shbits = __float_as_int(shifted);
  return e;
}

// 2^(n + bias) as a float from the shifted sum's bits: one shift-and-add.
template <int BIAS>
__device__ __forceinline__ float pow2_of(int shbits) {
  return __int_as_float((shbits << 23) + (int)(((unsigned)(127 + BIAS) << 23) - (kShiftBits << 23)));
}

// sigmoid with the reference's cut-offs (math_nooptim.go:36-44).  With E = exp(|x|) =
// 2^n (1 + q), r = 1 / (1 + E) is sigmoid(-|x|) and 1 - r is sigmoid(|x|).  The sum
// 1 + E is formed scaled by 2^-64, as (2^(n-64) q + 2^-64) + 2^(n-64): two roundings
// of at most 0.9 ulp together for every n (adding the 1 to 2^n first would lose it
// from n = 24 on), and the scaling keeps the hardware reciprocal's result normal
// where r itself is subnormal (x below -87.3); the final multiply-add by 2^-64
// rounds once.  Beyond the cut-offs r is replaced by 0, which gives exactly 0 and 1.
// NaN fails the compare and propagates through r.
__device__ __forceinline__ float sigmoid_f32_fast(float x) {
  const float a = fabsf(x);
  const ExpF p = expf_parts(a);
  const float s = pow2_of<-64>(p.shbits);
  const float c = 5.421010862427522e-20f;                       // 2^-64
  const float d = __builtin_fmaf(s, p.q, c) + s;
  float rc = __builtin_amdgcn_rcpf(d);                          // 2^64 / (1 + E), within an ulp
  const float cs = copysignf(c, x);
  const float lim = __builtin_fmaf(cs, -36.5f * 18446744073709551616.0f, 51.5f);   // 15 right of zero, 88 left
  const float base = __builtin_fmaf(cs, 0.5f * 18446744073709551616.0f, 0.5f);     // 1 right of zero, 0 left
  rc = a > lim ? 0.0f : rc;
  return __builtin_fmaf(-cs, rc, base);
}

// tanh: below 0.55 an odd polynomial x + x^3 R(x^2) (R fitted on [0, 0.56^2],
// approximation error 0.07 ulp); above it 1 - 2/(e^(2|x|) + 1), where the result
// is at least 0.5 and the quotient's error (the sum's single rounding and the
// hardware reciprocal's ulp) shrinks by the factor 2/(e^(2|x|) + 1) <= 1/2.
// The exponential's argument is clamped (tanh(22) rounds to 1); the clamp drops a
// NaN, so the choice between the two forms is written to fall to the polynomial,
// which keeps it, when the compare fails.
__device__ __forceinline__ float tanh_f32_fast(float x) {
  const float ax = fabsf(x);
  const float s2 = ax * ax;
  float R = 0.0024976127315312624f;
  R = __builtin_fmaf(R, s2, -0.008506525307893753f);
  R = __builtin_fmaf(R, s2, 0.02181374467909336f);
  R = __builtin_fmaf(R, s2, -0.05396425351500511f);
  R = __builtin_fmaf(R, s2, 0.133333221077919f);
  R = __builtin_fmaf(R, s2, -0.3333333432674408f);
  const float small = __builtin_fmaf(ax * s2, R, ax);
  const float ac = fminf(ax, 22.0f);
  const ExpF p = expf_parts(ac + ac);
  const float s = pow2_of<0>(p.shbits);
  const float d = __builtin_fmaf(s, p.q, s + 1.0f);             // e^(2|x|) + 1 in one rounding (n <= 64 / ln2)
  const float rc = __builtin_amdgcn_rcpf(d);
  const float large = __builtin_fmaf(-2.0f, rc, 1.0f);
  return copysignf(ax >= 0.55f ? large : small, x);
}

template <int FN>
__device__ __forceinline__ float unary_apply(float x) {
  if constexpr (FN == GH_ABS) return fabsf(x);
  else if constexpr (FN == GH_SIGN) return (float)((x > 0.0f) - (x < 0.0f));
  else if constexpr (FN == GH_CEIL) return ceilf(x);
  else if constexpr (FN == GH_FLOOR) return floorf(x);
  else if constexpr (FN == GH_SIN) return (float)sin((double)x);
  else if constexpr (FN == GH_COS) return (float)cos((double)x);
  else if constexpr (FN == GH_EXP) return exp_f32_via_f64(x);
  else if constexpr (FN == GH_LN) return (float)log((double)x);
  else if constexpr (FN == GH_LOG2) return (float)log2((double)x);
  else if constexpr (FN == GH_NEG) return -x;
  else if constexpr (FN == GH_SQUARE) return x * x;
  else if constexpr (FN == GH_SQRT) return sqrtf(x);
  else if constexpr (FN == GH_INVERSE) return 1.0f / x;
  else if constexpr (FN == GH_INVSQRT) return 1.0f / sqrtf(x);
  else if constexpr (FN == GH_CUBE) return x * x * x;
  else if constexpr (FN == GH_TANH) return tanh_f32_fast(x);
  else if constexpr (FN == GH_SIGMOID) return sigmoid_f32_fast(x);
  else if constexpr (FN == GH_LOG1P) return (float)log1p((double)x);
  else if constexpr (FN == GH_EXPM1) return (float)expm1((double)x);
  else {  // softplus
    if (x < -103.0f) return 0.0f;
    if (x > 14.0f) return x;
    return (float)log1p(exp((double)x));
  }
}

template <int FN>
__device__ __forceinline__ double unary_apply(double x) {
  if constexpr (FN == GH_ABS) return fabs(x);
  else if constexpr (FN == GH_SIGN) return (double)((x > 0.0) - (x < 0.0));
  else if constexpr (FN == GH_CEIL) return ceil(x);
  else if constexpr (FN == GH_FLOOR) return floor(x);
  else if constexpr (FN == GH_SIN) return sin(x);
  else if constexpr (FN == GH_COS) return cos(x);
  else if constexpr (FN == GH_EXP) return exp(x);
  else if constexpr (FN == GH_LN) return log(x);
  else if constexpr (FN == GH_LOG2) return log2(x);
  else if constexpr (FN == GH_NEG) return -x;
  else if constexpr (FN == GH_SQUARE) return x * x;
  else if constexpr (FN == GH_SQRT) return sqrt(x);
  else if constexpr (FN == GH_INVERSE) return 1.0 / x;
  else if constexpr (FN == GH_INVSQRT) return 1.0 / sqrt(x);
  else if constexpr (FN == GH_CUBE) return x * x * x;
  else if constexpr (FN == GH_TANH) return tanh(x);
  else if constexpr (FN == GH_SIGMOID) {
    if (x < -709.0) return 0.0;
    if (x > 19.0) return 1.0;
    return 1.0 / (1.0 + exp(-x));
  } else if constexpr (FN == GH_LOG1P) return log1p(x);
  else if constexpr (FN == GH_EXPM1) return expm1(x);
  else {
    if (x < -708.0) return 0.0;
    if (x > 16.0) return x;
    return log1p(exp(x));
  }
}

// ---- binary kernels ---------------------------------------------------------
// MODE vv: A[i] = A[i] op B[i]   vs: A[i] = A[i] op B[0]
//      sv: B[i] = A[0] op B[i]   ss: A[0] = A[0] op B[0]   (elembinop.cu:13-35)
// POW2: vs mode only; the exponent was read as 2 by the kernel itself, so
// x*x is used (equal to the correctly rounded pow(x,2)).

// A workgroup walks whole chunks of kUnroll * kBlock vectors (each wavefront touches
// kUnroll runs of 1 KB), grid-strided.  STREAM: operands larger than the last-level cache
// go through non-temporal loads and stores (measured on MI355X, 64 MiB tensors: plain
// accesses run at 8 TB/s when the operands sit in that cache and 5.5 TB/s from HBM;
// non-temporal ones 6.6 and 6.2).
template <class V, bool STREAM>
__device__ __forceinline__ V ld_vec(const V* p) {
  if constexpr (STREAM) return __builtin_nontemporal_load(p);
  else return *p;
}
template <class V, bool STREAM>
__device__ __forceinline__ void st_vec(V* p, V v) {
  if constexpr (STREAM) __builtin_nontemporal_store(v, p);
  else *p = v;
}

template <int FN, class T, int MODE, bool STREAM>
__global__ __launch_bounds__(kBlock) void k_bin_vec(const T* A, const T* B, T* D, int64_t n) {
  using V = typename VecOf<T>::type;
  constexpr int N = VecOf<T>::N;
  const int64_t nv = n / N;
  constexpr int64_t chunk = (int64_t)kBlock * kUnroll;
  const int64_t stride = (int64_t)gridDim.x * chunk;
  T s = (T)0;
  bool pow2 = false;
  if constexpr (MODE == GH_VS) { s = B[0]; if constexpr (FN == GH_POW) pow2 = (s == (T)2); }
  if constexpr (MODE == GH_SV) s = A[0];
  const V* Av = reinterpret_cast<const V*>(A);
  const V* Bv = reinterpret_cast<const V*>(B);
  V* Dv = reinterpret_cast<V*>(D);
  auto apply = [&](V a, V b) {
    V r;
#pragma unroll
    for (int e = 0; e < N; e++) {
      if constexpr (MODE == GH_VV) r[e] = bin_apply<FN, T>(a[e], b[e]);
      else if constexpr (MODE == GH_VS) {
        if constexpr (FN == GH_POW) r[e] = pow2 ? a[e] * a[e] : bin_apply<FN, T>(a[e], s);
        else r[e] = bin_apply<FN, T>(a[e], s);
      } else r[e] = bin_apply<FN, T>(s, b[e]);
    }
    return r;
  };
  for (int64_t i = (int64_t)blockIdx.x * chunk + threadIdx.x; i < nv; i += stride) {
    if (i + (kUnroll - 1) * kBlock < nv) {
      V a[kUnroll], b[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; u++) {
        if constexpr (MODE != GH_SV) a[u] = ld_vec<V, STREAM>(Av + i + u * kBlock);
        if constexpr (MODE != GH_VS) b[u] = ld_vec<V, STREAM>(Bv + i + u * kBlock);
      }
#pragma unroll
      for (int u = 0; u < kUnroll; u++) st_vec<V, STREAM>(Dv + i + u * kBlock, apply(a[u], b[u]));
    } else {
      for (int64_t j = i; j < nv; j += kBlock) {
        V a = V{}, b = V{};
        if constexpr (MODE != GH_SV) a = Av[j];
        if constexpr (MODE != GH_VS) b = Bv[j];
        Dv[j] = apply(a, b);
      }
    }
  }
  // scalar tail (n % N elements)
  const int64_t t = nv * N + (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t < n) {
    if constexpr (MODE == GH_VV) D[t] = bin_apply<FN, T>(A[t], B[t]);
    else if constexpr (MODE == GH_VS) {
      if constexpr (FN == GH_POW) D[t] = pow2 ? A[t] * A[t] : bin_apply<FN, T>(A[t], s);
      else D[t] = bin_apply<FN, T>(A[t], s);
    } else D[t] = bin_apply<FN, T>(s, B[t]);
  }
}

// Unaligned operands, or scalar-scalar: plain one-element-per-thread loop.
template <int FN, class T, int MODE>
__global__ __launch_bounds__(kBlock) void k_bin_scalar(const T* A, const T* B, T* D, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  T s = (T)0;
  if constexpr (MODE == GH_VS) s = B[0];
  if constexpr (MODE == GH_SV || MODE == GH_SS) s = A[0];
  if constexpr (MODE == GH_SS) {
    if (blockIdx.x == 0 && threadIdx.x == 0) D[0] = bin_apply<FN, T>(s, B[0]);
    return;
  }
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    if constexpr (MODE == GH_VV) D[i] = bin_apply<FN, T>(A[i], B[i]);
    else if constexpr (MODE == GH_VS) D[i] = bin_apply<FN, T>(A[i], s);
    else if constexpr (MODE == GH_SV) D[i] = bin_apply<FN, T>(s, B[i]);
  }
}

template <int FN, class T, bool STREAM>
__global__ __launch_bounds__(kBlock) void k_unary_vec(const T* A, T* D, int64_t n) {
  using V = typename VecOf<T>::type;
  constexpr int N = VecOf<T>::N;
  const int64_t nv = n / N;
  constexpr int64_t chunk = (int64_t)kBlock * kUnroll;
  const int64_t stride = (int64_t)gridDim.x * chunk;
  const V* Av = reinterpret_cast<const V*>(A);
  V* Dv = reinterpret_cast<V*>(D);
  auto apply = [&](V a) {
    V r;
#pragma unroll
    for (int e = 0; e < N; e++) r[e] = unary_apply<FN>(a[e]);
    return r;
  };
  for (int64_t i = (int64_t)blockIdx.x * chunk + threadIdx.x; i < nv; i += stride) {
    if (i + (kUnroll - 1) * kBlock < nv) {
      V a[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; u++) a[u] = ld_vec<V, STREAM>(Av + i + u * kBlock);
#pragma unroll
      for (int u = 0; u < kUnroll; u++) st_vec<V, STREAM>(Dv + i + u * kBlock, apply(a[u]));
    } else {
      for (int64_t j = i; j < nv; j += kBlock) Dv[j] = apply(Av[j]);
    }
  }
  const int64_t t = nv * N + (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t < n) D[t] = unary_apply<FN>(A[t]);
}

template <int FN, class T>
__global__ __launch_bounds__(kBlock) void k_unary_scalar(const T* A, T* D, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
    D[i] = unary_apply<FN>(A[i]);
}

// ---- fused broadcast --------------------------------------------------------
// dst[o,m,i] = big[o,m,i] op small[m]  (or small op big with SMALL_LEFT).
// Row form (inner == 1, mid a multiple of the vector width): each thread owns one 128-bit
// column group, keeps its slice of `small` in registers and walks rows.
template <int FN, class T, bool LEFT, bool STREAM>
__global__ __launch_bounds__(kBlock) void k_bcast_row(T* __restrict__ dst,
                                                      const T* __restrict__ big,
                                                      const T* __restrict__ small,
                                                      int64_t rows, int64_t colv) {
  typedef typename VecOf<T>::type V;
  constexpr int N = VecOf<T>::N;
  const int64_t cv = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (cv >= colv) return;
  const V s = reinterpret_cast<const V*>(small)[cv];
  const V* __restrict__ bv = reinterpret_cast<const V*>(big);
  V* __restrict__ dv = reinterpret_cast<V*>(dst);
  auto apply = [&](V a) {
    V o;
#pragma unroll
    for (int e = 0; e < N; e++) o[e] = LEFT ? bin_apply<FN, T>(s[e], a[e]) : bin_apply<FN, T>(a[e], s[e]);
    return o;
  };
  // a workgroup takes kUnroll adjacent rows per step
  const int64_t rs = (int64_t)gridDim.y * kUnroll;
  for (int64_t r = (int64_t)blockIdx.y * kUnroll; r < rows; r += rs) {
    if (r + kUnroll <= rows) {
      V a[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; u++) a[u] = ld_vec<V, STREAM>(bv + (r + u) * colv + cv);
#pragma unroll
      for (int u = 0; u < kUnroll; u++) st_vec<V, STREAM>(dv + (r + u) * colv + cv, apply(a[u]));
    } else {
      for (int64_t q = r; q < rows; q++) dv[q * colv + cv] = apply(bv[q * colv + cv]);
    }
  }
}

// General form: one element per thread, small index = (idx / inner) % mid.
template <int FN, class T, bool LEFT>
__global__ __launch_bounds__(kBlock) void k_bcast_generic(T* dst, const T* big,
                                                          const T* small, int64_t n,
                                                          int64_t mid, int64_t inner) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const T s = small[(i / inner) % mid];
    const T a = big[i];
    dst[i] = LEFT ? bin_apply<FN, T>(s, a) : bin_apply<FN, T>(a, s);
  }
}

// ---- ReLU / LeakyReLU in the reference's arithmetic form --------------------
// Rectify: x * float(x >= 0) (nn.go:136-163) - negative inputs give -0.0.
// LeakyRelu: x*(x>=0) + (x*(x<0))*alpha (nn.go:83-131).
__device__ __forceinline__ float relu_ref(float x) { return x * (x >= 0.0f ? 1.0f : 0.0f); }
__device__ __forceinline__ float leaky_ref(float x, float alpha) {
  const float pos = x * (x >= 0.0f ? 1.0f : 0.0f);
  const float neg = x * (x < 0.0f ? 1.0f : 0.0f);
  const float na = neg * alpha;
  return pos + na;
}

template <bool LEAKY>
__global__ __launch_bounds__(kBlock) void k_relu(const float* __restrict__ x, float* __restrict__ y,
                                                 int64_t n, float alpha, int vec) {
  typedef float V __attribute__((ext_vector_type(4)));
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (vec) {
    const int64_t nv = n / 4;
    const V* xv = reinterpret_cast<const V*>(x);
    V* yv = reinterpret_cast<V*>(y);
    for (; i < nv; i += stride) {
      V a = xv[i], r;
#pragma unroll
      for (int e = 0; e < 4; e++) r[e] = LEAKY ? leaky_ref(a[e], alpha) : relu_ref(a[e]);
      yv[i] = r;
    }
    const int64_t t = nv * 4 + (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n) y[t] = LEAKY ? leaky_ref(x[t], alpha) : relu_ref(x[t]);
  } else {
    for (; i < n; i += stride) y[i] = LEAKY ? leaky_ref(x[i], alpha) : relu_ref(x[i]);
  }
}

// Rectify's gradient as the CPU engine spells it: Gte(x, 0) written as 1.0 / 0.0,
// then HadamardProd with the incoming gradient (one multiplication, so a masked
// element is dy * 0.0 with dy's sign, and a NaN gradient stays NaN).
__global__ __launch_bounds__(kBlock) void k_relu_bwd(const float* __restrict__ x, const float* dy, float* dx,
                                                     int64_t n, int vec) {
  typedef float V __attribute__((ext_vector_type(4)));
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (vec) {
    const int64_t nv = n / 4;
    const V* xv = reinterpret_cast<const V*>(x);
    const V* gv = reinterpret_cast<const V*>(dy);
    V* ov = reinterpret_cast<V*>(dx);
    for (; i < nv; i += stride) {
      const V a = xv[i], g = gv[i];
      V r;
#pragma unroll
      for (int e = 0; e < 4; e++) r[e] = g[e] * (a[e] >= 0.0f ? 1.0f : 0.0f);
      ov[i] = r;
    }
    const int64_t t = nv * 4 + (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n) dx[t] = dy[t] * (x[t] >= 0.0f ? 1.0f : 0.0f);
  } else {
    for (; i < n; i += stride) dx[i] = dy[i] * (x[i] >= 0.0f ? 1.0f : 0.0f);
  }
}

__global__ __launch_bounds__(kBlock) void k_fill(float* A, int64_t n, float v) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) A[i] = v;
}

__global__ void k_set_flag(int* flag, int v) { *flag = v; }

// misc.hasNaN / misc.hasInf (misc.cu:14-56).  The reference increments a
// counter without atomics; here any matching lane stores 1 (a benign race on
// a single value).
template <class T, bool NAN_CHECK>
__device__ __forceinline__ bool has_hit(T v) {
  return NAN_CHECK ? (v != v) : (v == (T)INFINITY || v == -(T)INFINITY);
}
template <class T, bool NAN_CHECK>
__global__ __launch_bounds__(kBlock) void k_has(const T* __restrict__ A, int64_t n, int* flag) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  bool hit = false;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) hit |= has_hit<T, NAN_CHECK>(A[i]);
  if (hit) *flag = 1;
}
// The same search over 16-byte vectors (A aligned to 16 bytes, nv whole vectors), four loads in flight per lane:
// a value this large is a stream out of HBM and nothing else.
template <class T, bool NAN_CHECK>
__global__ __launch_bounds__(kBlock) void k_has_vec(const T* __restrict__ A, int64_t nv, int* flag) {
  typedef typename VecOf<T>::type V;
  constexpr int N = VecOf<T>::N, U = 4;
  const V* Av = reinterpret_cast<const V*>(A);
  const int64_t stride = (int64_t)gridDim.x * kBlock * U;
  bool hit = false;
  for (int64_t i = (int64_t)blockIdx.x * kBlock * U + threadIdx.x; i < nv; i += stride) {
    V v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = Av[min(i + (int64_t)u * kBlock, nv - 1)];   // past the end: the last vector again
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int e = 0; e < N; e++) hit |= has_hit<T, NAN_CHECK>(v[u][e]);
  }
  if (hit) *flag = 1;
}

// ---- launch helpers ---------------------------------------------------------

inline int grid_for(gh_ctx* ctx, int64_t work_items, int per_thread) {
  int64_t blocks = (work_items + (int64_t)kBlock * per_thread - 1) / ((int64_t)kBlock * per_thread);
  const int64_t cap = (int64_t)ctx->cu_count * 64;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

inline bool aligned16(uint64_t p) { return (p & 15u) == 0; }

// Grid of the chunked vector kernels: 16 workgroups per compute unit, fewer when the
// tensor has fewer chunks.
inline int grid_chunks(gh_ctx* ctx, int64_t nvec) {
  int64_t blocks = (nvec + (int64_t)kBlock * kUnroll - 1) / ((int64_t)kBlock * kUnroll);
  const int64_t cap = (int64_t)ctx->cu_count * 16;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

// Operands that cannot all sit in the last-level cache are streamed (non-temporal).
inline bool stream_bytes(int64_t bytes) {
  static const int64_t limit = [] {
    const char* e = getenv("GORGONIA_HIP_EW_STREAM_MIB");   // tuning override
    return (int64_t)(e ? atoll(e) : 256) << 20;
  }();
  return bytes >= limit;
}

// ... and so are operands the cache has lost by now: every tensor the kernel reads was last
// touched more than a cache's worth of traffic ago (or never).  Small launches stay plain.
constexpr uint64_t kWarmWindow = 192ull << 20;
constexpr int64_t kColdMinBytes = 16ll << 20;
inline bool cold_inputs(const gh_ctx* ctx, int64_t bytes, uint64_t a, uint64_t b) {
  static const bool off = getenv("GORGONIA_HIP_EW_NO_RESIDENCY") != nullptr;   // tuning switch: size rule only
  if (off || bytes < kColdMinBytes) return false;
  return !(a && ctx->llc.warm(a, kWarmWindow)) && !(b && ctx->llc.warm(b, kWarmWindow));
}

template <int FN, class T>
int launch_bin_fn(gh_ctx* ctx, const gh_cmd& c) {
  const T* A = (const T*)(uintptr_t)c.ptr[0];
  const T* B = (const T*)(uintptr_t)c.ptr[1];
  const uint32_t mode = gh_mode(c.flags);
  // ptr[2] (optional) is a separate destination; without it the kernel works
  // in place: on A for vv/vs/ss, on B for sv (elembinop.cu:13-35).
  const uint64_t dptr = c.ptr[2] ? c.ptr[2] : (mode == GH_SV ? c.ptr[1] : c.ptr[0]);
  T* Dst = (T*)(uintptr_t)dptr;
  const int64_t n = c.dim[0];
  constexpr int N = VecOf<T>::N;
  if (n == 0) return GH_OK;
  bool vec = n >= N && aligned16(dptr);
  if (mode == GH_VV) vec = vec && aligned16(c.ptr[0]) && aligned16(c.ptr[1]);
  if (mode == GH_VS) vec = vec && aligned16(c.ptr[0]);
  if (mode == GH_SV) vec = vec && aligned16(c.ptr[1]);
  if (mode == GH_SS) vec = false;
  const int gv = grid_chunks(ctx, n / N);
  const int gs = grid_for(ctx, n, 4);
  const int64_t tbytes = (int64_t)sizeof(T) * n;
  const uint64_t va = mode == GH_SV ? 0 : c.ptr[0], vb = mode == GH_VS ? 0 : c.ptr[1];   // the tensor operands
  const bool stream = stream_bytes(tbytes * (mode == GH_VV ? 3 : 2)) ||
                      (mode != GH_SS && cold_inputs(ctx, tbytes * (mode == GH_VV ? 3 : 2), va, vb));
  if (mode != GH_SS) {
    ctx->llc.touch(va, tbytes, true);
    ctx->llc.touch(vb, tbytes, true);
    ctx->llc.touch(dptr, tbytes, dptr != va && dptr != vb);
  }
#define GH_LAUNCH_MODE(M)                                                                   \
  if (vec && stream) hipLaunchKernelGGL((k_bin_vec<FN, T, M, true>), dim3(gv), dim3(kBlock), 0, ctx->stream, A, B, Dst, n); \
  else if (vec) hipLaunchKernelGGL((k_bin_vec<FN, T, M, false>), dim3(gv), dim3(kBlock), 0, ctx->stream, A, B, Dst, n); \
  else hipLaunchKernelGGL((k_bin_scalar<FN, T, M>), dim3(gs), dim3(kBlock), 0, ctx->stream, A, B, Dst, n);
  switch (mode) {
    case GH_VV: GH_LAUNCH_MODE(GH_VV) break;
    case GH_VS: GH_LAUNCH_MODE(GH_VS) break;
    case GH_SV: GH_LAUNCH_MODE(GH_SV) break;
    default:
      hipLaunchKernelGGL((k_bin_scalar<FN, T, GH_SS>), dim3(1), dim3(kBlock), 0, ctx->stream, A, B, Dst, n);
  }
#undef GH_LAUNCH_MODE
  return gh_check_hip(ctx, hipGetLastError(), "elementwise binary launch");
}

template <class T>
int launch_bin(gh_ctx* ctx, const gh_cmd& c) {
  switch (gh_fn(c.flags)) {
    case GH_ADD: return launch_bin_fn<GH_ADD, T>(ctx, c);
    case GH_SUB: return launch_bin_fn<GH_SUB, T>(ctx, c);
    case GH_MUL: return launch_bin_fn<GH_MUL, T>(ctx, c);
    case GH_DIV: return launch_bin_fn<GH_DIV, T>(ctx, c);
    case GH_POW: return launch_bin_fn<GH_POW, T>(ctx, c);
    case GH_LT: return launch_bin_fn<GH_LT, T>(ctx, c);
    case GH_LTE: return launch_bin_fn<GH_LTE, T>(ctx, c);
    case GH_GT: return launch_bin_fn<GH_GT, T>(ctx, c);
    case GH_GTE: return launch_bin_fn<GH_GTE, T>(ctx, c);
    case GH_EQ: return launch_bin_fn<GH_EQ, T>(ctx, c);
    case GH_NE: return launch_bin_fn<GH_NE, T>(ctx, c);
    case GH_MOD: return launch_bin_fn<GH_MOD, T>(ctx, c);
  }
  return gh_fail(ctx, GH_ENOFUNC, "unknown binary function");
}

template <int FN, class T>
int launch_unary_fn(gh_ctx* ctx, const gh_cmd& c) {
  const T* A = (const T*)(uintptr_t)c.ptr[0];
  const uint64_t dptr = c.ptr[1] ? c.ptr[1] : c.ptr[0];  // optional separate destination
  T* Dst = (T*)(uintptr_t)dptr;
  const int64_t n = c.dim[0];
  constexpr int N = VecOf<T>::N;
  if (n == 0) return GH_OK;
  const int64_t tbytes = (int64_t)sizeof(T) * n;
  const bool stream = stream_bytes(tbytes * 2) || cold_inputs(ctx, tbytes * 2, c.ptr[0], 0);
  ctx->llc.touch(c.ptr[0], tbytes, true);
  ctx->llc.touch(dptr, tbytes, dptr != c.ptr[0]);
  if (n >= N && aligned16(c.ptr[0]) && aligned16(dptr)) {
    if (stream)
      hipLaunchKernelGGL((k_unary_vec<FN, T, true>), dim3(grid_chunks(ctx, n / N)), dim3(kBlock), 0, ctx->stream, A, Dst, n);
    else
      hipLaunchKernelGGL((k_unary_vec<FN, T, false>), dim3(grid_chunks(ctx, n / N)), dim3(kBlock), 0, ctx->stream, A, Dst, n);
  } else
    hipLaunchKernelGGL((k_unary_scalar<FN, T>), dim3(grid_for(ctx, n, 4)), dim3(kBlock), 0,
                       ctx->stream, A, Dst, n);
  return gh_check_hip(ctx, hipGetLastError(), "elementwise unary launch");
}

template <class T>
int launch_unary(gh_ctx* ctx, const gh_cmd& c) {
  switch (gh_fn(c.flags)) {
#define GH_U(F) case F: return launch_unary_fn<F, T>(ctx, c);
    GH_U(GH_ABS) GH_U(GH_SIGN) GH_U(GH_CEIL) GH_U(GH_FLOOR) GH_U(GH_SIN) GH_U(GH_COS) GH_U(GH_EXP)
    GH_U(GH_LN) GH_U(GH_LOG2) GH_U(GH_NEG) GH_U(GH_SQUARE) GH_U(GH_SQRT) GH_U(GH_INVERSE)
    GH_U(GH_INVSQRT) GH_U(GH_CUBE) GH_U(GH_TANH) GH_U(GH_SIGMOID) GH_U(GH_LOG1P) GH_U(GH_EXPM1)
    GH_U(GH_SOFTPLUS)
#undef GH_U
  }
  return gh_fail(ctx, GH_ENOFUNC, "unknown unary function");
}

template <int FN, class T>
int launch_bcast_fn(gh_ctx* ctx, const gh_cmd& c) {
  T* dst = (T*)(uintptr_t)c.ptr[0];
  const T* big = (const T*)(uintptr_t)c.ptr[1];
  const T* small = (const T*)(uintptr_t)c.ptr[2];
  constexpr int N = VecOf<T>::N;
  const int64_t outer = c.dim[0], mid = c.dim[1], inner = c.dim[2];
  const int64_t n = outer * mid * inner;
  const int64_t tbytes = (int64_t)sizeof(T) * n;
  const bool left = c.flags & GH_FLAG_SMALL_LEFT;
  if (n == 0) return GH_OK;
  const bool row = inner == 1 && (mid % N) == 0 && aligned16(c.ptr[0]) && aligned16(c.ptr[1]) &&
                   aligned16(c.ptr[2]);
  if (row) {
    const int64_t colv = mid / N;
    const int gx = (int)((colv + kBlock - 1) / kBlock);
    int64_t gy = ((int64_t)ctx->cu_count * 16 + gx - 1) / gx;
    const int64_t need = (outer + kUnroll - 1) / kUnroll;
    if (gy > need) gy = need;
    if (gy < 1) gy = 1;
    if (gy > 65535) gy = 65535;
    const bool stream = stream_bytes(2 * tbytes) || cold_inputs(ctx, 2 * tbytes, c.ptr[1], 0);
    ctx->llc.touch(c.ptr[1], tbytes, true);
    ctx->llc.touch(c.ptr[0], tbytes, c.ptr[0] != c.ptr[1]);
#define GH_BCAST_ROW(L_, S_)                                                                                 \
  hipLaunchKernelGGL((k_bcast_row<FN, T, L_, S_>), dim3(gx, (int)gy), dim3(kBlock), 0, ctx->stream, dst, big, \
                     small, outer, colv)
    if (left) { if (stream) GH_BCAST_ROW(true, true); else GH_BCAST_ROW(true, false); }
    else { if (stream) GH_BCAST_ROW(false, true); else GH_BCAST_ROW(false, false); }
#undef GH_BCAST_ROW
  } else {
    const int g = grid_for(ctx, n, 4);
    if (left)
      hipLaunchKernelGGL((k_bcast_generic<FN, T, true>), dim3(g), dim3(kBlock), 0, ctx->stream, dst, big,
                         small, n, mid, inner);
    else
      hipLaunchKernelGGL((k_bcast_generic<FN, T, false>), dim3(g), dim3(kBlock), 0, ctx->stream, dst, big,
                         small, n, mid, inner);
  }
  return gh_check_hip(ctx, hipGetLastError(), "broadcast launch");
}

template <class T>
int launch_bcast(gh_ctx* ctx, const gh_cmd& c) {
  switch (gh_fn(c.flags)) {
    case GH_ADD: return launch_bcast_fn<GH_ADD, T>(ctx, c);
    case GH_SUB: return launch_bcast_fn<GH_SUB, T>(ctx, c);
    case GH_MUL: return launch_bcast_fn<GH_MUL, T>(ctx, c);
    case GH_DIV: return launch_bcast_fn<GH_DIV, T>(ctx, c);
    case GH_POW: return launch_bcast_fn<GH_POW, T>(ctx, c);
    case GH_LT: return launch_bcast_fn<GH_LT, T>(ctx, c);
    case GH_LTE: return launch_bcast_fn<GH_LTE, T>(ctx, c);
    case GH_GT: return launch_bcast_fn<GH_GT, T>(ctx, c);
    case GH_GTE: return launch_bcast_fn<GH_GTE, T>(ctx, c);
    case GH_EQ: return launch_bcast_fn<GH_EQ, T>(ctx, c);
    case GH_NE: return launch_bcast_fn<GH_NE, T>(ctx, c);
    case GH_MOD: return launch_bcast_fn<GH_MOD, T>(ctx, c);
  }
  return gh_fail(ctx, GH_ENOFUNC, "unknown binary function");
}

}  // namespace

int gh_launch_elem_bin(gh_ctx* ctx, const gh_cmd& c) {
  return gh_dtype_of(c.flags) == GH_F64 ? launch_bin<double>(ctx, c) : launch_bin<float>(ctx, c);
}

int gh_launch_elem_unary(gh_ctx* ctx, const gh_cmd& c) {
  return gh_dtype_of(c.flags) == GH_F64 ? launch_unary<double>(ctx, c) : launch_unary<float>(ctx, c);
}

int gh_launch_bcast_bin(gh_ctx* ctx, const gh_cmd& c) {
  return gh_dtype_of(c.flags) == GH_F64 ? launch_bcast<double>(ctx, c) : launch_bcast<float>(ctx, c);
}

int gh_launch_relu(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_relu_f64(ctx, c, false);
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  const int vec = aligned16(c.ptr[0]) && aligned16(c.ptr[1]) && n >= 4;
  hipLaunchKernelGGL((k_relu<false>), dim3(grid_for(ctx, vec ? n / 4 + 4 : n, 2)), dim3(kBlock), 0,
                     ctx->stream, (const float*)(uintptr_t)c.ptr[0], (float*)(uintptr_t)c.ptr[1], n,
                     0.0f, vec);
  return gh_check_hip(ctx, hipGetLastError(), "relu launch");
}

int gh_launch_relu_bwd(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_relu_bwd_f64(ctx, c);
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  const int vec = aligned16(c.ptr[0]) && aligned16(c.ptr[1]) && aligned16(c.ptr[2]) && n >= 4;
  hipLaunchKernelGGL(k_relu_bwd, dim3(grid_for(ctx, vec ? n / 4 + 4 : n, 2)), dim3(kBlock), 0, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], n, vec);
  return gh_check_hip(ctx, hipGetLastError(), "relu backward launch");
}

int gh_launch_leaky_relu(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_relu_f64(ctx, c, true);
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  const int vec = aligned16(c.ptr[0]) && aligned16(c.ptr[1]) && n >= 4;
  hipLaunchKernelGGL((k_relu<true>), dim3(grid_for(ctx, vec ? n / 4 + 4 : n, 2)), dim3(kBlock), 0,
                     ctx->stream, (const float*)(uintptr_t)c.ptr[0], (float*)(uintptr_t)c.ptr[1], n,
                     c.f[0], vec);
  return gh_check_hip(ctx, hipGetLastError(), "leaky relu launch");
}

int gh_launch_fill(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  hipLaunchKernelGGL(k_fill, dim3(grid_for(ctx, n, 4)), dim3(kBlock), 0, ctx->stream,
                     (float*)(uintptr_t)c.ptr[0], n, c.f[0]);
  return gh_check_hip(ctx, hipGetLastError(), "fill launch");
}

template <class T>
static void launch_has(gh_ctx* ctx, const T* A, int64_t n, int* flag, bool nanc) {
  constexpr int N = VecOf<T>::N;
  // whole 16-byte vectors from the first aligned element on; the few elements in front of them and behind, one by one
  int64_t head = 0;
  while (head < n && (((uintptr_t)(A + head)) & 15u)) head++;
  const int64_t nv = (n - head) / N, tail0 = head + nv * N;
  if (nv >= 4 * kBlock) {
    const int g = grid_for(ctx, nv, 4);
    if (nanc) hipLaunchKernelGGL((k_has_vec<T, true>), dim3(g), dim3(kBlock), 0, ctx->stream, A + head, nv, flag);
    else hipLaunchKernelGGL((k_has_vec<T, false>), dim3(g), dim3(kBlock), 0, ctx->stream, A + head, nv, flag);
    if (head) {
      if (nanc) hipLaunchKernelGGL((k_has<T, true>), dim3(1), dim3(kBlock), 0, ctx->stream, A, head, flag);
      else hipLaunchKernelGGL((k_has<T, false>), dim3(1), dim3(kBlock), 0, ctx->stream, A, head, flag);
    }
    if (tail0 < n) {
      if (nanc) hipLaunchKernelGGL((k_has<T, true>), dim3(1), dim3(kBlock), 0, ctx->stream, A + tail0, n - tail0, flag);
      else hipLaunchKernelGGL((k_has<T, false>), dim3(1), dim3(kBlock), 0, ctx->stream, A + tail0, n - tail0, flag);
    }
    return;
  }
  const int g = grid_for(ctx, n, 8);
  if (nanc) hipLaunchKernelGGL((k_has<T, true>), dim3(g), dim3(kBlock), 0, ctx->stream, A, n, flag);
  else hipLaunchKernelGGL((k_has<T, false>), dim3(g), dim3(kBlock), 0, ctx->stream, A, n, flag);
}

int gh_launch_has_nan_inf(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  int* flag = (int*)(uintptr_t)c.ptr[1];
  hipLaunchKernelGGL(k_set_flag, dim3(1), dim3(1), 0, ctx->stream, flag, 0);
  if (n > 0) {
    const bool nanc = c.opcode == GH_OP_HAS_NAN;
    if (gh_dtype_of(c.flags) == GH_F64) launch_has(ctx, (const double*)(uintptr_t)c.ptr[0], n, flag, nanc);
    else launch_has(ctx, (const float*)(uintptr_t)c.ptr[0], n, flag, nanc);
  }
  return gh_check_hip(ctx, hipGetLastError(), "hasNaN/hasInf launch");
}
