// Epilogue arithmetic shared by the convolution kernels (k_gemm.hip, k_conv_small.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "gh_internal.h"

// Epilogue activations in the reference's arithmetic form (nn.go:83-163).
__device__ __forceinline__ float act_apply(float v, int act, float alpha) {
  if (act == 1) return v * (v >= 0.0f ? 1.0f : 0.0f);
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
__device__ __forceinline__ void conv_tail_table(const ConvTail& t, float* tab, int n, int i, int f) {
  if (!t.mean) return;
  const float a = 1.0f / sqrtf(t.var[f] + t.eps);
  tab[i] = a;
  tab[n + i] = -t.mean[f] * a;
  if (t.gamma) tab[2 * n + i] = t.gamma[f];
  if (t.beta) tab[3 * n + i] = t.beta[f];
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
