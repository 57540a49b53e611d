// Epilogue arithmetic shared by the convolution kernels (k_gemm.hip, k_conv_small.hip).
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gh_internal.h"

// Epilogue activations in the reference's arithmetic form (nn.go:83-163).
// act 3 is LeakyRelu for a finite alpha >= 0 in four instructions instead of eight, with the
// same bits: for v < 0 the reference's sum is -0 + v alpha = v alpha, for v >= 0 it is v + 0 = v,
// and the v * 0 that fmaf adds is a zero of v's sign (which changes neither) unless v is
// infinite or NaN, where it makes the NaN the reference's inf * 0 makes.
__device__ __forceinline__ float act_apply(float v, int act, float alpha) {
  if (act == 1) return v * (v >= 0.0f ? 1.0f : 0.0f);
  if (act == 3) {
    const float na = v * alpha;
    return __builtin_fmaf(v, 0.0f, v < 0.0f ? na : v);
  }
  if (act == 2) {
    const float pos = v * (v >= 0.0f ? 1.0f : 0.0f);
    const float neg = v * (v < 0.0f ? 1.0f : 0.0f);
    const float na = neg * alpha;
    return pos + na;
  }
  return v;
}

// Operators riding in a convolution's epilogue, applied per stored value in this
// order: BatchNorm in eval mode with BN_INFER's arithmetic (op_nn.go:1559-1584:
// a = 1/sqrt(var+eps), b = -mean*a, y = x*a + b, then gamma*y, then + beta, each
// step rounded), then the activation.  Null mean: no BatchNorm.
struct ConvTail {
  const float* mean; const float* var; const float* gamma; const float* beta;
  float eps; int act; float alpha;
};

__device__ __forceinline__ float tail_apply(const ConvTail& t, int f, float v) {
  if (t.mean) {
    const float a = 1.0f / sqrtf(t.var[f] + t.eps);
    const float b = -t.mean[f] * a;
    v = v * a;
    v = v + b;
    if (t.gamma) v = t.gamma[f] * v;
    if (t.beta) v = v + t.beta[f];
  }
  return act_apply(v, t.act, t.alpha);
}

// The same arithmetic with the per-filter BatchNorm constants taken from a table a
// workgroup fills once (conv_tail_table): a and b are rounded exactly as above, so the
// stored bits are those of tail_apply.  tab = [4][n]: a, b, gamma, beta.
// An absent gamma is stored as 1 and an absent beta as -0: multiplying by 1 and adding -0
// leave every float32 as it is (+0 + -0 = +0, -0 + -0 = -0), so a kernel may apply all four
// steps without asking which exist (tail_apply_fixed) and still store tail_apply's bits.
__device__ __forceinline__ void conv_tail_table(const ConvTail& t, float* tab, int n, int i, int f) {
  if (!t.mean) return;
  const float a = 1.0f / sqrtf(t.var[f] + t.eps);
  tab[i] = a;
  tab[n + i] = -t.mean[f] * a;
  tab[2 * n + i] = t.gamma ? t.gamma[f] : 1.0f;
  tab[3 * n + i] = t.beta ? t.beta[f] : -0.0f;
}
__device__ __forceinline__ float tail_apply_table(const ConvTail& t, const float* tab, int n, int i, float v) {
  if (t.mean) {
    v = v * tab[i];
    v = v + tab[n + i];
    if (t.gamma) v = tab[2 * n + i] * v;
    if (t.beta) v = v + tab[3 * n + i];
  }
  return act_apply(v, t.act, t.alpha);
}

// The epilogue with what it consists of fixed at compile time (BN: BatchNorm from a
// conv_tail_table; ACT: 0 none, 1 Rectify, 2 LeakyRelu, 3 its short form): no branch per stored value.  Scalar
// branches inside an epilogue's value loops were a fifth of a small convolution's run.
template <bool BN, int ACT>
__device__ __forceinline__ float tail_apply_fixed(const float* tab, int n, int i, float v, float alpha) {
  if constexpr (BN) {
    v = v * tab[i];
    v = v + tab[n + i];
    v = tab[2 * n + i] * v;
    v = v + tab[3 * n + i];
  }
  return act_apply(v, ACT, alpha);
}
// Calls body(bool_constant<BN>, integral_constant<int, ACT>) for the tail's combination.
template <class Body>
__device__ __forceinline__ void conv_tail_dispatch(const ConvTail& t, Body&& body) {
  using T = std::true_type; using F = std::false_type;
  using A0 = std::integral_constant<int, 0>; using A1 = std::integral_constant<int, 1>;
  using A2 = std::integral_constant<int, 2>; using A3 = std::integral_constant<int, 3>;
  const bool quick_leaky = t.act == 2 && t.alpha >= 0.0f && t.alpha <= 3.402823466e+38f;
  if (t.mean) {
    if (t.act == 1) body(T{}, A1{}); else if (quick_leaky) body(T{}, A3{}); else if (t.act == 2) body(T{}, A2{}); else body(T{}, A0{});
  } else {
    if (t.act == 1) body(F{}, A1{}); else if (quick_leaky) body(F{}, A3{}); else if (t.act == 2) body(F{}, A2{}); else body(F{}, A0{});
  }
}

inline ConvTail conv_tail(const gh_cmd& c) {
  ConvTail t{};
  if (c.flags & GH_FLAG_CONV_BN) {
    t.mean = (const float*)(uintptr_t)c.ptr[3];
    t.var = (const float*)(uintptr_t)c.ptr[4];
    t.gamma = (c.flags & GH_FLAG_HAS_GAMMA) ? (const float*)(uintptr_t)c.ptr[5] : nullptr;
    t.beta = (c.flags & GH_FLAG_HAS_BETA) ? (const float*)(uintptr_t)c.ptr[6] : nullptr;
    t.eps = c.f[1];
  }
  t.act = (c.flags & GH_FLAG_ACT_RELU) ? 1 : (c.flags & GH_FLAG_ACT_LEAKY) ? 2 : 0;
  t.alpha = c.f[0];
  return t;
}
