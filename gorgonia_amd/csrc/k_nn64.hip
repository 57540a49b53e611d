// float64 twins of the forward neural-network operators for gfx950: Conv2d,
// MaxPool2D, BatchNorm (eval), Rectify, LeakyRelu, SoftMax.  The reference's
// CPU operators switch on the dtype and run the same loops for float64
// (op_nn.go:909-957, 1559-1631; nn.go:83-163); its cuDNN path takes the dtype
// from the tensor (ops/nn/convolution_cuda.go:47-60).  These are the plain
// forms - one thread per result, operands read where they lie - with the
// float32 kernels' arithmetic: same operation order, one rounding per step.
// They are not tuned; float64 runs at a quarter of the float32 vector rate
// on this part and the float32 path is the one the benchmarks measure.
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cmath>
#include <cstdint>

#include "gh_internal.h"

namespace {

constexpr int kBlock = 256;

// float64 scalars (LeakyRelu's alpha, BatchNorm's epsilon) travel as the bit
// pattern of a double in a dim slot: gh_cmd.f is float32.
inline double bits_to_double(int64_t bits) {
  double d;
  static_assert(sizeof(d) == sizeof(bits), "double is 64 bits");
  __builtin_memcpy(&d, &bits, sizeof(d));
  return d;
}

__global__ __launch_bounds__(kBlock) void k_relu_f64(const double* __restrict__ x, double* __restrict__ y,
                                                     int64_t n, double alpha, int leaky) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
    const double v = x[i];
    const double pos = v * (v >= 0.0 ? 1.0 : 0.0);
    if (!leaky) { y[i] = pos; continue; }
    const double neg = v * (v < 0.0 ? 1.0 : 0.0);
    const double na = neg * alpha;
    y[i] = pos + na;
  }
}

struct Pool64 {
  int H, W, oh, ow, kh, kw, padH, padW, strideH, strideW;
};

// Reference scan: window clipped to the image, row-major, strict >, start
// value -maxFloat64 (op_nn.go:916-950).  RELU: x is read through Rectify (x * (x >= 0), nn.go:136-163), whose
// result is then never stored.
template <bool RELU>
__global__ __launch_bounds__(kBlock) void k_maxpool2d_f64(const double* __restrict__ x, double* __restrict__ y,
                                                          Pool64 g, int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int plane = g.oh * g.ow;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const int64_t bc = i / plane;
    const int rem = (int)(i - bc * plane);
    const int ph = rem / g.ow, pw = rem - ph * g.ow;
    int hs = ph * g.strideH - g.padH, ws = pw * g.strideW - g.padW;
    const int he = min(hs + g.kh, g.H), we = min(ws + g.kw, g.W);
    hs = max(hs, 0);
    ws = max(ws, 0);
    const double* in = x + bc * (int64_t)g.H * g.W;
    double best = -DBL_MAX;
    for (int hi = hs; hi < he; hi++)
      for (int wi = ws; wi < we; wi++) {
        double v = in[hi * g.W + wi];
        if constexpr (RELU) v = v * (v >= 0.0 ? 1.0 : 0.0);
        if (v > best) best = v;
      }
    y[i] = best;
  }
}

__global__ __launch_bounds__(kBlock) void k_bn_infer_f64(const double* __restrict__ x, double* __restrict__ y,
                                                         const double* __restrict__ mean,
                                                         const double* __restrict__ var,
                                                         const double* __restrict__ gamma,
                                                         const double* __restrict__ beta, double eps,
                                                         int64_t total, int C, int64_t S) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const int c = (int)((i / S) % C);
    const double a = 1.0 / sqrt(var[c] + eps);
    const double b = -mean[c] * a;
    double t = x[i] * a;
    t = t + b;
    if (gamma) t = gamma[c] * t;
    if (beta) t = t + beta[c];
    y[i] = t;
  }
}

// One wavefront per row; the sum is taken in column order like the CPU loop.
__global__ __launch_bounds__(kBlock) void k_softmax_f64(const double* __restrict__ x, double* __restrict__ y,
                                                        int64_t rows, int cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const double* in = x + row * cols;
  double* out = y + row * cols;
  double mx = -INFINITY;
  for (int j = lane; j < cols; j += 64) mx = fmax(mx, in[j]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmax(mx, __shfl_xor(mx, off, 64));
  double sum = 0.0;
  for (int j0 = 0; j0 < cols; j0 += 64) {
    const int j = j0 + lane;
    double e = 0.0;
    if (j < cols) {
      e = exp(in[j] - mx);
      out[j] = e;
    }
    const int lim = min(64, cols - j0);
    for (int l = 0; l < lim; l++) sum = sum + __shfl(e, l, 64);
  }
  for (int j = lane; j < cols; j += 64) out[j] = out[j] / sum;
}

struct Conv64 {
  int B, C, H, W, F, kh, kw, padH, padW, strideH, strideW, dilH, dilW, oh, ow;
};

// One thread per output element; k = (c, kr, kc) ascending, a rounded multiply
// and a rounded add per tap, padding taps contribute 0 * w like the im2col form.
__global__ __launch_bounds__(kBlock) void k_conv2d_f64(const double* __restrict__ x, const double* __restrict__ w,
                                                       double* __restrict__ y, Conv64 g, int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int plane = g.oh * g.ow;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const int64_t bf = i / plane;
    const int rem = (int)(i - bf * plane);
    const int oy = rem / g.ow, ox = rem - oy * g.ow;
    const int b = (int)(bf / g.F), f = (int)(bf - (int64_t)b * g.F);
    const double* xb = x + (int64_t)b * g.C * g.H * g.W;
    const double* wf = w + (int64_t)f * g.C * g.kh * g.kw;
    double acc = 0.0;
    for (int c = 0; c < g.C; c++)
      for (int kr = 0; kr < g.kh; kr++) {
        const int ir = -g.padH + kr * g.dilH + oy * g.strideH;
        for (int kc = 0; kc < g.kw; kc++) {
          const int ic = -g.padW + kc * g.dilW + ox * g.strideW;
          const bool in = ir >= 0 && ir < g.H && ic >= 0 && ic < g.W;
          const double v = in ? xb[((int64_t)c * g.H + ir) * g.W + ic] : 0.0;
          const double p = v * wf[(c * g.kh + kr) * g.kw + kc];
          acc = acc + p;
        }
      }
    y[i] = acc;
  }
}

// Conv2d gradients in float64 (the reference differentiates the im2col form,
// nn.go:211-305, op_nn.go:267-291, 605-640; these sum the same products per
// element): one thread per gradient element, plain loops, not tuned.
// Image gradient: dx[b,c,iy,ix] = sum over f, kr, kc of dy[b,f,oy,ox] * w[f,c,kr,kc]
// where oy*stride - pad + kr*dil = iy (and the same for columns).
__global__ __launch_bounds__(kBlock) void k_conv2d_bwd_data_f64(const double* __restrict__ dy,
                                                                const double* __restrict__ w,
                                                                double* __restrict__ dx, Conv64 g, int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int plane = g.H * g.W;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const int64_t bc = i / plane;
    const int rem = (int)(i - bc * plane);
    const int iy = rem / g.W, ix = rem - iy * g.W;
    const int b = (int)(bc / g.C), c = (int)(bc - (int64_t)b * g.C);
    double acc = 0.0;
    for (int f = 0; f < g.F; f++) {
      const double* gy = dy + ((int64_t)b * g.F + f) * g.oh * g.ow;
      const double* wf = w + ((int64_t)f * g.C + c) * g.kh * g.kw;
      for (int kr = 0; kr < g.kh; kr++) {
        const int ty = iy + g.padH - kr * g.dilH;
        if (ty < 0 || ty % g.strideH) continue;
        const int oy = ty / g.strideH;
        if (oy >= g.oh) continue;
        for (int kc = 0; kc < g.kw; kc++) {
          const int tx = ix + g.padW - kc * g.dilW;
          if (tx < 0 || tx % g.strideW) continue;
          const int ox = tx / g.strideW;
          if (ox >= g.ow) continue;
          const double p = gy[oy * g.ow + ox] * wf[kr * g.kw + kc];
          acc = acc + p;
        }
      }
    }
    dx[i] = acc;
  }
}

// Filter gradient: dw[f,c,kr,kc] = sum over b, oy, ox of dy[b,f,oy,ox] * x[b,c,iy,ix].
__global__ __launch_bounds__(kBlock) void k_conv2d_bwd_filter_f64(const double* __restrict__ x,
                                                                  const double* __restrict__ dy,
                                                                  double* __restrict__ dw, Conv64 g, int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int kk = g.kh * g.kw;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const int64_t fc = i / kk;
    const int tap = (int)(i - fc * kk);
    const int kr = tap / g.kw, kc = tap - kr * g.kw;
    const int f = (int)(fc / g.C), c = (int)(fc - (int64_t)f * g.C);
    double acc = 0.0;
    for (int b = 0; b < g.B; b++) {
      const double* gy = dy + ((int64_t)b * g.F + f) * g.oh * g.ow;
      const double* xc = x + ((int64_t)b * g.C + c) * g.H * g.W;
      for (int oy = 0; oy < g.oh; oy++) {
        const int iy = oy * g.strideH - g.padH + kr * g.dilH;
        if (iy < 0 || iy >= g.H) continue;
        for (int ox = 0; ox < g.ow; ox++) {
          const int ix = ox * g.strideW - g.padW + kc * g.dilW;
          if (ix < 0 || ix >= g.W) continue;
          const double p = gy[oy * g.ow + ox] * xc[iy * g.W + ix];
          acc = acc + p;
        }
      }
    }
    dw[i] = acc;
  }
}

int blocks_for(gh_ctx* ctx, int64_t n) {
  int64_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > (int64_t)ctx->cu_count * 32) blocks = (int64_t)ctx->cu_count * 32;
  return (int)(blocks < 1 ? 1 : blocks);
}

}  // namespace

int gh_launch_relu_f64(gh_ctx* ctx, const gh_cmd& c, bool leaky) {
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  hipLaunchKernelGGL(k_relu_f64, dim3(blocks_for(ctx, n)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (double*)(uintptr_t)c.ptr[1], n,
                     leaky ? bits_to_double(c.dim[1]) : 0.0, leaky ? 1 : 0);
  return gh_check_hip(ctx, hipGetLastError(), "relu launch");
}

int gh_launch_maxpool2d_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t B = c.dim[0], C = c.dim[1];
  Pool64 g;
  g.H = (int)c.dim[2]; g.W = (int)c.dim[3]; g.kh = (int)c.dim[4]; g.kw = (int)c.dim[5];
  const int64_t padN = c.dim[6], padS = c.dim[7], padW = c.dim[8], padE = c.dim[9];
  g.strideH = (int)c.dim[10]; g.strideW = (int)c.dim[11];
  g.oh = (int)gh_pool_out(g.H, g.kh, padN, padS, g.strideH);
  g.ow = (int)gh_pool_out(g.W, g.kw, padW, padE, g.strideW);
  const bool explicit_pad = c.flags & GH_FLAG_EXPLICIT_PAD;   // window shifted by south/east (op_nn.go:871-875)
  g.padH = (int)(explicit_pad ? padS : padN);
  g.padW = (int)(explicit_pad ? padE : padW);
  const int64_t total = B * C * g.oh * g.ow;
  if (total <= 0) return GH_OK;
  if (c.flags & GH_FLAG_ACT_RELU)
    hipLaunchKernelGGL(k_maxpool2d_f64<true>, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                       (const double*)(uintptr_t)c.ptr[0], (double*)(uintptr_t)c.ptr[1], g, total);
  else
    hipLaunchKernelGGL(k_maxpool2d_f64<false>, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                       (const double*)(uintptr_t)c.ptr[0], (double*)(uintptr_t)c.ptr[1], g, total);
  return gh_check_hip(ctx, hipGetLastError(), "maxpool2d launch");
}

int gh_launch_bn_infer_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t B = c.dim[0], C = c.dim[1], S = c.dim[2];
  const int64_t total = B * C * S;
  if (total <= 0) return GH_OK;
  const double* gamma = (c.flags & GH_FLAG_HAS_GAMMA) ? (const double*)(uintptr_t)c.ptr[4] : nullptr;
  const double* beta = (c.flags & GH_FLAG_HAS_BETA) ? (const double*)(uintptr_t)c.ptr[5] : nullptr;
  hipLaunchKernelGGL(k_bn_infer_f64, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (double*)(uintptr_t)c.ptr[1],
                     (const double*)(uintptr_t)c.ptr[2], (const double*)(uintptr_t)c.ptr[3], gamma, beta,
                     bits_to_double(c.dim[3]), total, (int)C, S);
  return gh_check_hip(ctx, hipGetLastError(), "batchnorm launch");
}

int gh_launch_softmax_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t rows = c.dim[0];
  if (rows == 0) return GH_OK;
  const int64_t blocks = (rows + (kBlock / 64) - 1) / (kBlock / 64);
  hipLaunchKernelGGL(k_softmax_f64, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (double*)(uintptr_t)c.ptr[1], rows, (int)c.dim[1]);
  return gh_check_hip(ctx, hipGetLastError(), "softmax launch");
}

static Conv64 conv64_geom(const gh_cmd& c) {
  Conv64 g;
  g.B = (int)c.dim[0]; g.C = (int)c.dim[1]; g.H = (int)c.dim[2]; g.W = (int)c.dim[3]; g.F = (int)c.dim[4];
  g.kh = (int)c.dim[5]; g.kw = (int)c.dim[6]; g.padH = (int)c.dim[7]; g.padW = (int)c.dim[8];
  g.strideH = (int)c.dim[9]; g.strideW = (int)c.dim[10]; g.dilH = (int)c.dim[11]; g.dilW = (int)c.dim[12];
  g.oh = (int)gh_conv_out(g.H, g.kh, g.padH, g.strideH, g.dilH);
  g.ow = (int)gh_conv_out(g.W, g.kw, g.padW, g.strideW, g.dilW);
  return g;
}

int gh_launch_conv2d_bwd_data_f64(gh_ctx* ctx, const gh_cmd& c) {
  const Conv64 g = conv64_geom(c);
  const int64_t total = (int64_t)g.B * g.C * g.H * g.W;
  if (total <= 0) return GH_OK;
  if (gh_try_launch_conv2d_bwd_data_f64_mfma(ctx, c))
    return ctx->err ? ctx->err : gh_check_hip(ctx, hipGetLastError(), "conv2d image gradient launch");
  hipLaunchKernelGGL(k_conv2d_bwd_data_f64, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], g, total);
  return gh_check_hip(ctx, hipGetLastError(), "conv2d image gradient launch");
}

int gh_launch_conv2d_bwd_filter_f64(gh_ctx* ctx, const gh_cmd& c) {
  const Conv64 g = conv64_geom(c);
  const int64_t total = (int64_t)g.F * g.C * g.kh * g.kw;
  if (total <= 0) return GH_OK;
  if (gh_try_launch_conv2d_bwd_filter_f64_mfma(ctx, c))
    return ctx->err ? ctx->err : gh_check_hip(ctx, hipGetLastError(), "conv2d filter gradient launch");
  hipLaunchKernelGGL(k_conv2d_bwd_filter_f64, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], g, total);
  return gh_check_hip(ctx, hipGetLastError(), "conv2d filter gradient launch");
}

int gh_launch_conv2d_f64(gh_ctx* ctx, const gh_cmd& c) {
  const Conv64 g = conv64_geom(c);
  const int64_t total = (int64_t)g.B * g.F * g.oh * g.ow;
  if (total <= 0) return GH_OK;
  if (gh_try_launch_conv2d_f64_mfma(ctx, c)) return ctx->err ? ctx->err : gh_check_hip(ctx, hipGetLastError(), "conv2d launch");
  hipLaunchKernelGGL(k_conv2d_f64, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], g, total);
  return gh_check_hip(ctx, hipGetLastError(), "conv2d launch");
}
