// MaxPool2D, BatchNorm inference and SoftMax for gfx950.
// Replaces cuDNN PoolingForward (ops/nn/maxpool_cuda.go:109) and
// BatchNormalizationForwardInference (ops/nn/batchnorm_cuda.go:102-110) with
// kernels that reproduce the CPU engine's arithmetic: op_nn.go:860-907 for the
// pool (init -FLT_MAX, strict >, row-major scan of the clipped window) and
// op_nn.go:1559-1631 + nn.go:429-440 for batch norm (per-channel
// a = 1/sqrt(var+eps), b = -mean*a, y = x*a + b in two roundings, then the
// separate gamma multiply and beta add).  All three are HBM-bound.
#include <cfloat>

#include "gh_internal.h"

namespace {

constexpr int kBlock = 256;

struct PoolGeom {
  int H, W, oh, ow, kh, kw, padH, padW, strideH, strideW;
};

// Rectify in the reference's arithmetic (nn.go:136-163), for pooling kernels that take their
// input through it (GH_FLAG_ACT_RELU on MAXPOOL2D: the activation's result is never stored).
__device__ __forceinline__ float relu_of(float v) { return v * (v >= 0.0f ? 1.0f : 0.0f); }

template <bool RELU>
__global__ __launch_bounds__(kBlock) void k_maxpool2d(const float* __restrict__ x,
                                                      float* __restrict__ y, PoolGeom g,
                                                      int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int plane = g.oh * g.ow;
  for (int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += stride) {
    const int64_t bc = idx / plane;
    const int rem = (int)(idx - bc * plane);
    const int ph = rem / g.ow, pw = rem - ph * g.ow;
    int hs = ph * g.strideH - g.padH, ws = pw * g.strideW - g.padW;
    const int he = min(hs + g.kh, g.H), we = min(ws + g.kw, g.W);
    hs = max(hs, 0);
    ws = max(ws, 0);
    const float* in = x + bc * (int64_t)g.H * g.W;
    float best = -FLT_MAX;
    for (int hi = hs; hi < he; hi++)
      for (int wi = ws; wi < we; wi++) {
        float v = in[hi * g.W + wi];
        if (RELU) v = relu_of(v);
        if (v > best) best = v;
      }
    y[idx] = best;
  }
}

// 2x2 / stride 2 / no padding, even W: each thread produces two adjacent
// outputs from two float4 loads (rows hi, hi+1), same compare order as the
// generic kernel: (r0,c0), (r0,c1), (r1,c0), (r1,c1).
template <bool RELU>
__global__ __launch_bounds__(kBlock) void k_maxpool_2x2s2(const float* __restrict__ x,
                                                          float* __restrict__ y, int H, int W,
                                                          int oh, int ow, int64_t pairs) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int owp = ow / 2;  // output pairs per row
  for (int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x; idx < pairs; idx += stride) {
    const int64_t row = idx / owp;  // (bc, ph) flattened
    const int pp = (int)(idx - row * owp);
    const int64_t bc = row / oh;
    const int ph = (int)(row - bc * oh);
    const float* in = x + (bc * H + 2 * ph) * (int64_t)W + 4 * pp;
    f4 r0 = *(reinterpret_cast<const f4*>(in));
    f4 r1 = *(reinterpret_cast<const f4*>(in + W));
    if (RELU) {
#pragma unroll
      for (int j = 0; j < 4; j++) { r0[j] = relu_of(r0[j]); r1[j] = relu_of(r1[j]); }
    }
    f2 o;
#pragma unroll
    for (int e = 0; e < 2; e++) {
      float best = -FLT_MAX;
      if (r0[2 * e] > best) best = r0[2 * e];
      if (r0[2 * e + 1] > best) best = r0[2 * e + 1];
      if (r1[2 * e] > best) best = r1[2 * e];
      if (r1[2 * e + 1] > best) best = r1[2 * e + 1];
      o[e] = best;
    }
    *reinterpret_cast<f2*>(y + (bc * oh + ph) * (int64_t)ow + 2 * pp) = o;
  }
}

// BatchNorm inference.  Grid y walks (b, c) planes, grid x walks the plane.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void k_bn_infer(const float* __restrict__ x,
                                                     float* __restrict__ y,
                                                     const float* __restrict__ mean,
                                                     const float* __restrict__ var,
                                                     const float* __restrict__ gamma,
                                                     const float* __restrict__ beta, float eps,
                                                     int64_t BC, int C, int64_t S) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  for (int64_t bc = blockIdx.y; bc < BC; bc += gridDim.y) {
    const int c = (int)(bc % C);
    const float inv = 1.0f / sqrtf(var[c] + eps);  // op_nn.go:1576
    const float a = inv;
    const float b = -mean[c] * a;                    // op_nn.go:1580
    const bool hg = gamma != nullptr, hb = beta != nullptr;
    const float gm = hg ? gamma[c] : 1.0f, bt = hb ? beta[c] : 0.0f;
    const float* in = x + bc * S;
    float* out = y + bc * S;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    if (VEC) {
      const int64_t sv = S / 4;
      for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < sv; i += stride) {
        f4 v = *(reinterpret_cast<const f4*>(in) + i);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float t = v[e] * a;
          t = t + b;
          if (hg) t = gm * t;
          if (hb) t = t + bt;
          v[e] = t;
        }
        *(reinterpret_cast<f4*>(out) + i) = v;
      }
    } else {
      for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < S; i += stride) {
        float t = in[i] * a;
        t = t + b;
        if (hg) t = gm * t;
        if (hb) t = t + bt;
        out[i] = t;
      }
    }
  }
}

// Row softmax, one wavefront per row: max, exp(x - max) in float64 rounded
// once, sum, scale by the rounded reciprocal.  The sum is taken in column
// order (64 exponentials at a time, added lane by lane through readlane), so
// it carries the same rounding as a sequential CPU loop.
__global__ __launch_bounds__(kBlock) void k_softmax(const float* __restrict__ x,
                                                    float* __restrict__ y, int64_t rows, int cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* in = x + row * cols;
  float* out = y + row * cols;
  float mx = -INFINITY;
  for (int j = lane; j < cols; j += 64) mx = fmaxf(mx, in[j]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  float sum = 0.f;
  float keep = 0.f;  // this lane's exponential when the row fits one chunk
  for (int j0 = 0; j0 < cols; j0 += 64) {
    const int j = j0 + lane;
    float e = 0.f;
    if (j < cols) {
      e = (float)exp((double)(in[j] - mx));
      if (cols > 64) out[j] = e;
    }
    keep = e;
    const int lim = min(64, cols - j0);
    for (int l = 0; l < lim; l++) sum = sum + __shfl(e, l, 64);
  }
  const float inv = 1.0f / sum;
  if (cols <= 64) {
    if (lane < cols) out[lane] = keep * inv;
  } else {
    for (int j = lane; j < cols; j += 64) out[j] = out[j] * inv;
  }
}

inline bool al16(uint64_t p) { return (p & 15u) == 0; }

}  // namespace

int gh_launch_maxpool2d(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_maxpool2d_f64(ctx, c);
  const int64_t B = c.dim[0], C = c.dim[1];
  PoolGeom g;
  g.H = (int)c.dim[2]; g.W = (int)c.dim[3]; g.kh = (int)c.dim[4]; g.kw = (int)c.dim[5];
  const int64_t padN = c.dim[6], padS = c.dim[7], padW = c.dim[8], padE = c.dim[9];
  g.strideH = (int)c.dim[10]; g.strideW = (int)c.dim[11];
  g.oh = (int)gh_pool_out(g.H, g.kh, padN, padS, g.strideH);
  g.ow = (int)gh_pool_out(g.W, g.kw, padW, padE, g.strideW);
  // With explicit 4-value padding the reference shifts the window by the
  // south/east pads (op_nn.go:871-875).
  const bool explicit_pad = c.flags & GH_FLAG_EXPLICIT_PAD;
  g.padH = (int)(explicit_pad ? padS : padN);
  g.padW = (int)(explicit_pad ? padE : padW);
  const int64_t total = B * C * g.oh * g.ow;
  if (total <= 0) return GH_OK;
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  float* y = (float*)(uintptr_t)c.ptr[1];
  const bool relu = c.flags & GH_FLAG_ACT_RELU;   // y = pool(x * (x >= 0))
  const bool fast = g.kh == 2 && g.kw == 2 && g.strideH == 2 && g.strideW == 2 && padN == 0 &&
                    padS == 0 && padW == 0 && padE == 0 && g.W % 4 == 0 && g.H % 2 == 0 &&
                    al16(c.ptr[0]) && (c.ptr[1] & 7u) == 0;
  if (fast) {
    const int64_t pairs = total / 2;
    int64_t blocks = (pairs + kBlock - 1) / kBlock;
    if (blocks > (int64_t)ctx->cu_count * 16) blocks = (int64_t)ctx->cu_count * 16;
    if (relu)
      hipLaunchKernelGGL(k_maxpool_2x2s2<true>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream, x, y, g.H, g.W,
                         g.oh, g.ow, pairs);
    else
      hipLaunchKernelGGL(k_maxpool_2x2s2<false>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream, x, y, g.H, g.W,
                         g.oh, g.ow, pairs);
  } else {
    int64_t blocks = (total + kBlock - 1) / kBlock;
    if (blocks > (int64_t)ctx->cu_count * 16) blocks = (int64_t)ctx->cu_count * 16;
    if (relu) hipLaunchKernelGGL(k_maxpool2d<true>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream, x, y, g, total);
    else hipLaunchKernelGGL(k_maxpool2d<false>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream, x, y, g, total);
  }
  return gh_check_hip(ctx, hipGetLastError(), "maxpool2d launch");
}

int gh_launch_bn_infer(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_bn_infer_f64(ctx, c);
  const int64_t B = c.dim[0], C = c.dim[1], S = c.dim[2];
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  float* y = (float*)(uintptr_t)c.ptr[1];
  const float* mean = (const float*)(uintptr_t)c.ptr[2];
  const float* var = (const float*)(uintptr_t)c.ptr[3];
  const float* gamma = (c.flags & GH_FLAG_HAS_GAMMA) ? (const float*)(uintptr_t)c.ptr[4] : nullptr;
  const float* beta = (c.flags & GH_FLAG_HAS_BETA) ? (const float*)(uintptr_t)c.ptr[5] : nullptr;
  const int64_t BC = B * C;
  const bool vec = S % 4 == 0 && al16(c.ptr[0]) && al16(c.ptr[1]);
  const int64_t per_plane = vec ? S / 4 : S;
  int gx = (int)((per_plane + kBlock * 4 - 1) / (kBlock * 4));
  if (gx < 1) gx = 1;
  if (gx > 1024) gx = 1024;
  int64_t gy = BC;
  if (gy > 65535) gy = 65535;
  if (vec)
    hipLaunchKernelGGL((k_bn_infer<true>), dim3(gx, (int)gy), dim3(kBlock), 0, ctx->stream, x, y, mean,
                       var, gamma, beta, c.f[0], BC, (int)C, S);
  else
    hipLaunchKernelGGL((k_bn_infer<false>), dim3(gx, (int)gy), dim3(kBlock), 0, ctx->stream, x, y, mean,
                       var, gamma, beta, c.f[0], BC, (int)C, S);
  return gh_check_hip(ctx, hipGetLastError(), "batchnorm launch");
}

int gh_launch_softmax(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_softmax_f64(ctx, c);
  const int64_t rows = c.dim[0];
  const int cols = (int)c.dim[1];
  if (rows == 0) return GH_OK;
  const int64_t blocks = (rows + (kBlock / 64) - 1) / (kBlock / 64);
  hipLaunchKernelGGL(k_softmax, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (float*)(uintptr_t)c.ptr[1], rows, cols);
  return gh_check_hip(ctx, hipGetLastError(), "softmax launch");
}
