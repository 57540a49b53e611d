// Backward passes of MaxPool2D, BatchNorm and SoftMax, and BatchNorm's
// training-mode forward, for gfx950.  They stand where the reference calls
// cuDNN PoolingBackward (ops/nn/maxpool_cuda.go:177-188),
// BatchNormalizationForwardTraining / Backward (ops/nn/batchnorm_cuda.go:87-100,
// 192-219) and where its CPU engine runs maxPoolDiffOp (op_nn.go:1042-1093),
// BatchNormOp.updateStatsF32 (op_nn.go:1489-1555), batchnormDiffOp.f32s
// (op_nn.go:1834-1943) and softmaxDiffOp (op_softmax.go:266-279); the
// arithmetic follows the CPU engine.  All of them are HBM-bound.
#include <cfloat>
#include <cstring>

#include "gh_internal.h"

namespace {

constexpr int kBlock = 256;

struct PoolGeom {
  int H, W, oh, ow, kh, kw, padH, padW, strideH, strideW;
};

// One thread per input element.  The reference zeroes dx and lets every
// window, in (ph, pw) order, add its dy into the window's argmax (the first
// element in row-major window order that beats everything before it, from
// -FLT_MAX).  Gathering the same contributions per element in the same window
// order gives the same bits without atomics, overlapping windows included.
//
// RELU (GH_FLAG_ACT_RELU): x is the value before a Rectify whose result was pooled.  The windows
// are scanned over x * (x >= 0) and the gathered sum is multiplied by (x >= 0): the gradient
// of MaxPool2D(Rectify(x)) with the bits of MaxPool2DDiff followed by the activation's own
// gradient (dy times the 1.0 / 0.0 of Gte), without the Rectify result or the pooling gradient
// ever being stored.
__device__ __forceinline__ float relu_of(float v) { return v * (v >= 0.0f ? 1.0f : 0.0f); }
__device__ __forceinline__ float relu_mask(float v) { return v >= 0.0f ? 1.0f : 0.0f; }

template <bool RELU>
__global__ __launch_bounds__(kBlock) void k_maxpool2d_bwd(const float* __restrict__ x,
                                                          const float* __restrict__ dy,
                                                          float* __restrict__ dx, PoolGeom g,
                                                          int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int plane = g.H * g.W;
  for (int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += stride) {
    const int64_t bc = idx / plane;
    const int me = (int)(idx - bc * plane);
    const int iy = me / g.W, ix = me - iy * g.W;
    const float* in = x + bc * (int64_t)plane;
    const float* gy = dy + bc * (int64_t)g.oh * g.ow;
    // windows whose extent [p*s - pad, p*s - pad + k) holds this row / column
    const int ny = iy + g.padH - g.kh + 1, nx = ix + g.padW - g.kw + 1;
    const int ph0 = ny > 0 ? (ny + g.strideH - 1) / g.strideH : 0;
    const int pw0 = nx > 0 ? (nx + g.strideW - 1) / g.strideW : 0;
    const int ph1 = min(g.oh - 1, (iy + g.padH) / g.strideH);
    const int pw1 = min(g.ow - 1, (ix + g.padW) / g.strideW);
    float acc = 0.0f;
    for (int ph = ph0; ph <= ph1; ph++)
      for (int pw = pw0; pw <= pw1; pw++) {
        int hs = ph * g.strideH - g.padH, ws = pw * g.strideW - g.padW;
        const int he = min(hs + g.kh, g.H), we = min(ws + g.kw, g.W);
        hs = max(hs, 0);
        ws = max(ws, 0);
        float best = -FLT_MAX;
        int arg = -1;
        for (int hi = hs; hi < he; hi++)
          for (int wi = ws; wi < we; wi++) {
            float v = in[hi * g.W + wi];
            if (RELU) v = relu_of(v);
            if (v > best) { best = v; arg = hi * g.W + wi; }
          }
        if (arg == me) acc = acc + gy[ph * g.ow + pw];
      }
    dx[idx] = RELU ? acc * relu_mask(in[me]) : acc;
  }
}

// 2x2 / stride 2 / no padding with even H and W % 4 == 0: windows do not
// overlap, so one thread owns two adjacent windows - two float4 row loads, one
// float2 of dy, two float4 stores - with the generic kernel's scan order
// (r0c0, r0c1, r1c0, r1c1), strict >, and its "0 + dy" for the winner.
template <bool RELU>
__global__ __launch_bounds__(kBlock) void k_maxpool_2x2s2_bwd(const float* __restrict__ x,
                                                              const float* __restrict__ dy,
                                                              float* __restrict__ dx, int H, int W,
                                                              int64_t pairs) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int oh = H / 2, ow = W / 2, owp = ow / 2;
  for (int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x; idx < pairs; idx += stride) {
    const int64_t row = idx / owp;  // (bc, ph) flattened
    const int pp = (int)(idx - row * owp);
    const int64_t bc = row / oh;
    const int ph = (int)(row - bc * oh);
    const int64_t at = (bc * H + 2 * ph) * (int64_t)W + 4 * pp;
    f4 r0 = *reinterpret_cast<const f4*>(x + at);
    f4 r1 = *reinterpret_cast<const f4*>(x + at + W);
    f4 m0 = {1.f, 1.f, 1.f, 1.f}, m1 = m0;
    if (RELU) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        m0[j] = relu_mask(r0[j]); m1[j] = relu_mask(r1[j]);
        r0[j] = relu_of(r0[j]); r1[j] = relu_of(r1[j]);
      }
    }
    const f2 g = *reinterpret_cast<const f2*>(dy + (bc * oh + ph) * (int64_t)ow + 2 * pp);
    f4 o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 2; e++) {
      float best = -FLT_MAX;
      int arg = -1;
      if (r0[2 * e] > best) { best = r0[2 * e]; arg = 0; }
      if (r0[2 * e + 1] > best) { best = r0[2 * e + 1]; arg = 1; }
      if (r1[2 * e] > best) { best = r1[2 * e]; arg = 2; }
      if (r1[2 * e + 1] > best) { best = r1[2 * e + 1]; arg = 3; }
      const float v = 0.0f + g[e];
      o0[2 * e] = arg == 0 ? v : 0.0f;
      o0[2 * e + 1] = arg == 1 ? v : 0.0f;
      o1[2 * e] = arg == 2 ? v : 0.0f;
      o1[2 * e + 1] = arg == 3 ? v : 0.0f;
    }
    if (RELU) { o0 = o0 * m0; o1 = o1 * m1; }
    *reinterpret_cast<f4*>(dx + at) = o0;
    *reinterpret_cast<f4*>(dx + at + W) = o1;
  }
}

// 2x2 / stride 2 / no padding at any H, W (odd sizes, rows that are no multiple of
// four): one thread per window with scalar accesses; the thread of the last
// window column / row also zeroes the column / row an odd size leaves outside
// every window.  Same scan order, strict > and "0 + dy" as above.
template <bool RELU>
__global__ __launch_bounds__(kBlock) void k_maxpool_2x2s2_bwd_any(const float* __restrict__ x,
                                                                  const float* __restrict__ dy,
                                                                  float* __restrict__ dx, int H, int W,
                                                                  int64_t windows) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int oh = H / 2, ow = W / 2;
  for (int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x; idx < windows; idx += stride) {
    const int pw = (int)(idx % ow);
    const int64_t row = idx / ow;
    const int ph = (int)(row % oh);
    const int64_t bc = row / oh;
    const int64_t at = (bc * H + 2 * ph) * (int64_t)W + 2 * pw;
    float v00 = x[at], v01 = x[at + 1], v10 = x[at + W], v11 = x[at + W + 1];
    float k00 = 1.f, k01 = 1.f, k10 = 1.f, k11 = 1.f;
    if (RELU) {
      k00 = relu_mask(v00); k01 = relu_mask(v01); k10 = relu_mask(v10); k11 = relu_mask(v11);
      v00 = relu_of(v00); v01 = relu_of(v01); v10 = relu_of(v10); v11 = relu_of(v11);
    }
    float best = -FLT_MAX;
    int arg = -1;
    if (v00 > best) { best = v00; arg = 0; }
    if (v01 > best) { best = v01; arg = 1; }
    if (v10 > best) { best = v10; arg = 2; }
    if (v11 > best) { best = v11; arg = 3; }
    const float v = 0.0f + dy[idx];
    dx[at] = (arg == 0 ? v : 0.0f) * k00;   // k.. is 1 without RELU: v * 1 is v
    dx[at + 1] = (arg == 1 ? v : 0.0f) * k01;
    dx[at + W] = (arg == 2 ? v : 0.0f) * k10;
    dx[at + W + 1] = (arg == 3 ? v : 0.0f) * k11;
    if ((W & 1) && pw == ow - 1) { dx[at + 2] = 0.0f; dx[at + W + 2] = 0.0f; }
    if ((H & 1) && ph == oh - 1) {
      dx[at + 2 * (int64_t)W] = 0.0f;
      dx[at + 2 * (int64_t)W + 1] = 0.0f;
      if ((W & 1) && pw == ow - 1) dx[at + 2 * (int64_t)W + 2] = 0.0f;
    }
  }
}

// ---- BatchNorm: per-channel reductions ----------------------------------------------
// A channel's n = B*S values are split over G workgroups; each reduces its share
// with a fixed tree (so results repeat run to run), the consumers add the G
// partial sums in index order.

__device__ __forceinline__ float block_sum(float v, float* sh) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) sh[wave] = v;
  __syncthreads();
  const float r = (sh[0] + sh[1]) + (sh[2] + sh[3]);
  __syncthreads();
  return r;
}

__device__ __forceinline__ float sum_partials(const float* p, int G) {
  float s = 0.0f;
  for (int g = 0; g < G; g++) s = s + p[g];
  return s;
}

// MODE 0: part[c][g] = sum x.  MODE 1: part[c][g] = sum (x - mean)^2 with
// mean = (sum of the MODE 0 partials) / n.
template <int MODE>
__global__ __launch_bounds__(kBlock) void k_bn_reduce(const float* __restrict__ x,
                                                      const float* __restrict__ part_sum,
                                                      float* __restrict__ part, int C, int64_t S,
                                                      int64_t n) {
  __shared__ float sh[4];
  const int c = blockIdx.y, G = gridDim.x;
  float mean = 0.0f;
  if (MODE == 1) mean = sum_partials(part_sum + (int64_t)c * G, G) / (float)n;
  float acc = 0.0f;
  const int64_t B = n / S;
  auto term = [&](float v) {
    if (MODE == 0) return v;
    const float t = v - mean;
    return t * t;
  };
  // A plane is cut into 256-wide strips; workgroup g takes strips g, g + G, ...
  // of every image.  Planes narrower than a strip (dense layers: S == 1) are
  // walked over the batch instead.
  if (S >= kBlock) {
    float a4[4] = {0.f, 0.f, 0.f, 0.f};
    const int64_t img = (int64_t)C * S;
    for (int64_t d = (int64_t)blockIdx.x * kBlock + threadIdx.x; d < S; d += (int64_t)G * kBlock) {
      const float* p = x + (int64_t)c * S + d;
      int64_t b = 0;
      for (; b + 4 <= B; b += 4) {   // four images at a time: four loads in flight
        const float v0 = p[b * img], v1 = p[(b + 1) * img], v2 = p[(b + 2) * img], v3 = p[(b + 3) * img];
        a4[0] = a4[0] + term(v0);
        a4[1] = a4[1] + term(v1);
        a4[2] = a4[2] + term(v2);
        a4[3] = a4[3] + term(v3);
      }
      for (; b < B; b++) a4[0] = a4[0] + term(p[b * img]);
    }
    acc = (a4[0] + a4[1]) + (a4[2] + a4[3]);
  } else {
    for (int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x; b < B; b += (int64_t)G * kBlock) {
      const float* p = x + (b * C + c) * S;
      for (int64_t d = 0; d < S; d++) acc = acc + term(p[d]);
    }
  }
  const float r = block_sum(acc, sh);
  if (threadIdx.x == 0) part[(int64_t)c * G + blockIdx.x] = r;
}

// save_mean, save_var (the SUM of squared deviations, as the reference keeps
// it), the running statistics (momentum weights the NEW value; unbiased
// variance, op_nn.go:1547-1550) and the biased batch variance the apply pass
// normalises with (op_nn.go:1573).
__global__ __launch_bounds__(kBlock) void k_bn_train_finalize(const float* __restrict__ part_sum,
                                                              const float* __restrict__ part_sq,
                                                              float* __restrict__ run_mean,
                                                              float* __restrict__ run_var,
                                                              float* __restrict__ save_mean,
                                                              float* __restrict__ save_var,
                                                              float* __restrict__ batch_var,
                                                              float momentum, int C, int G,
                                                              int64_t n) {
  const int c = blockIdx.x * kBlock + threadIdx.x;
  if (c >= C) return;
  const float mean = sum_partials(part_sum + (int64_t)c * G, G) / (float)n;
  const float var = sum_partials(part_sq + (int64_t)c * G, G);
  save_mean[c] = mean;
  save_var[c] = var;
  const float m1 = momentum * mean, m2 = (1.0f - momentum) * run_mean[c];
  run_mean[c] = m1 + m2;
  const float unb = var / (float)(n - 1);
  const float v1 = momentum * unb, v2 = (1.0f - momentum) * run_var[c];
  run_var[c] = v1 + v2;
  batch_var[c] = var / (float)n;
}

// part[c][g][0] = sum dy, part[c][g][1] = sum (x*dy - mean*dy)  (op_nn.go:1897-1906;
// for S == 1 the reference writes (x - mean)*dy, op_nn.go:1864-1866).
__global__ __launch_bounds__(kBlock) void k_bn_bwd_reduce(const float* __restrict__ x,
                                                          const float* __restrict__ dy,
                                                          const float* __restrict__ save_mean,
                                                          float* __restrict__ part, int C,
                                                          int64_t S, int64_t n) {
  __shared__ float sh[4];
  const int c = blockIdx.y, G = gridDim.x;
  const float mean = save_mean[c];
  float s = 0.0f, dot = 0.0f;
  const int64_t B = n / S;
  auto term2 = [&](float xv, float g) {
    s = s + g;
    float p;
    if (S == 1) {
      const float t = xv - mean;
      p = t * g;
    } else {
      const float t1 = xv * g, t2 = mean * g;
      p = t1 - t2;
    }
    dot = dot + p;
  };
  auto term = [&](int64_t i) {
    const float xv = x[i], g = dy[i];
    s = s + g;
    float p;
    if (S == 1) {
      const float t = xv - mean;
      p = t * g;
    } else {
      const float t1 = xv * g, t2 = mean * g;
      p = t1 - t2;
    }
    dot = dot + p;
  };
  if (S >= kBlock) {
    const int64_t img = (int64_t)C * S;
    for (int64_t d = (int64_t)blockIdx.x * kBlock + threadIdx.x; d < S; d += (int64_t)G * kBlock) {
      const int64_t at = (int64_t)c * S + d;
      int64_t b = 0;
      for (; b + 2 <= B; b += 2) {
        const float x0 = x[at + b * img], g0 = dy[at + b * img];
        const float x1 = x[at + (b + 1) * img], g1 = dy[at + (b + 1) * img];
        term2(x0, g0);
        term2(x1, g1);
      }
      for (; b < B; b++) term2(x[at + b * img], dy[at + b * img]);
    }
  } else {
    for (int64_t b = (int64_t)blockIdx.x * kBlock + threadIdx.x; b < B; b += (int64_t)G * kBlock)
      for (int64_t d = 0; d < S; d++) term((b * C + c) * S + d);
  }
  const float rs = block_sum(s, sh);
  const float rd = block_sum(dot, sh);
  if (threadIdx.x == 0) {
    part[((int64_t)c * G + blockIdx.x) * 2] = rs;
    part[((int64_t)c * G + blockIdx.x) * 2 + 1] = rd;
  }
}

// dx = (dy - gradMean - (x - mean)*k) * invstd in training mode, dy * invstd in
// eval mode (op_nn.go:1908-1936), one (b, c) plane per blockIdx.y.
__global__ __launch_bounds__(kBlock) void k_bn_bwd_apply(const float* __restrict__ x,
                                                         const float* __restrict__ dy,
                                                         float* __restrict__ dx,
                                                         const float* __restrict__ save_mean,
                                                         const float* __restrict__ save_var,
                                                         const float* __restrict__ part, float eps,
                                                         int training, int64_t BC, int C, int64_t S,
                                                         int G, int64_t n, int vec) {
  for (int64_t bc = blockIdx.y; bc < BC; bc += gridDim.y) {
    const int c = (int)(bc % C);
    float s = 0.0f, dot = 0.0f;
    for (int g = 0; g < G; g++) {
      s = s + part[((int64_t)c * G + g) * 2];
      dot = dot + part[((int64_t)c * G + g) * 2 + 1];
    }
    const float mean = save_mean[c];
    const float vb = save_var[c] / (float)n;
    const float invstd = 1.0f / sqrtf(vb + eps);
    float k = dot * invstd;
    k = k * invstd;
    k = k / (float)n;
    const float grad_mean = s / (float)n;
    const float* xi = x + bc * S;
    const float* gi = dy + bc * S;
    float* out = dx + bc * S;
    auto one = [&](float xv, float g) {
      if (!training) return g * invstd;
      float t = xv - mean;
      t = t * k;
      float u;
      if (S == 1) { u = g - t; u = u - grad_mean; }
      else { u = g - grad_mean; u = u - t; }
      return u * invstd;
    };
    if (vec) {
      typedef float f4 __attribute__((ext_vector_type(4)));
      for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < S / 4; i += (int64_t)gridDim.x * kBlock) {
        const f4 xv = *(reinterpret_cast<const f4*>(xi) + i), gv = *(reinterpret_cast<const f4*>(gi) + i);
        f4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = one(xv[e], gv[e]);
        *(reinterpret_cast<f4*>(out) + i) = o;
      }
    } else {
      for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < S; i += (int64_t)gridDim.x * kBlock)
        out[i] = one(xi[i], gi[i]);
    }
  }
}

// SoftMax backward over the last axis, one wavefront per row:
// dx_i = y_i * (dy_i - sum_j dy_j*y_j), the sum taken in column order (lane by
// lane through readlane) like the forward kernel's, so it equals a sequential loop.
__global__ __launch_bounds__(kBlock) void k_softmax_bwd(const float* __restrict__ y,
                                                        const float* __restrict__ dy,
                                                        float* __restrict__ dx, int64_t rows,
                                                        int cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* yy = y + row * cols;
  const float* g = dy + row * cols;
  float dot = 0.0f;
  for (int j0 = 0; j0 < cols; j0 += 64) {
    const int j = j0 + lane;
    const float p = j < cols ? g[j] * yy[j] : 0.0f;
    const int lim = min(64, cols - j0);
    for (int l = 0; l < lim; l++) dot = dot + __shfl(p, l, 64);
  }
  for (int j = lane; j < cols; j += 64) {
    const float t = g[j] - dot;
    dx[row * cols + j] = yy[j] * t;
  }
}

// ---- solver steps ---------------------------------------------------------------------
// One fused pass per tensor instead of the reference's 6-15 tensor ops
// (solvers.go:273-372, 461-640, 780-870); every intermediate is rounded where
// a tensor op of the reference would round it, so the weights and caches get
// the reference's bits.
struct SolverPar { float eta, eps, l1reg, l2reg, clip, one_per_batch, a, b, corr1, corr2; };

__device__ __forceinline__ float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

__device__ __forceinline__ float prep_grad(float g, float w, int use, const SolverPar& p) {
  if (use & 1) { const float t = p.l1reg * (float)((w > 0.0f) - (w < 0.0f)); g = g + t; }
  if (use & 2) { const float t = w * p.l2reg; g = g + t; }
  if (use & 8) g = g * p.one_per_batch;
  if ((use & 4) && p.clip > 0.0f) g = clampf(g, -p.clip, p.clip);
  return g;
}

// Up to kSolverBatch weight tensors per launch: a model's solver steps are many
// small tensors, and one launch per tensor costs more than the arithmetic.
// Tensor t owns workgroups [first[t], first[t + 1]).
constexpr int kSolverBatch = 8;
struct SolverBatch {
  float* w[kSolverBatch]; const float* g[kSolverBatch]; float* c1[kSolverBatch]; float* c2[kSolverBatch];
  int64_t n[kSolverBatch];
  int first[kSolverBatch + 1];
  int count;
};

template <int KIND>
__global__ __launch_bounds__(kBlock) void k_solver_step(SolverBatch sb, int use, SolverPar p,
                                                        const float* __restrict__ corr) {
  // Adam's two bias corrections from device memory when the command names it: they change
  // every step, and as command constants they would make every step a new command
  if (KIND == GH_SOLVER_ADAM && corr) { p.corr1 = corr[0]; p.corr2 = corr[1]; }
  int t = 0;
#pragma unroll
  for (int q = 1; q < kSolverBatch; q++)
    if (q < sb.count && (int)blockIdx.x >= sb.first[q]) t = q;
  float* __restrict__ w = sb.w[t];
  const float* __restrict__ g = sb.g[t];
  float* __restrict__ c1 = sb.c1[t];
  float* __restrict__ c2 = sb.c2[t];
  const int64_t n = sb.n[t];
  const int64_t nblk = sb.first[t + 1] - sb.first[t];
  const float neg_eta = -p.eta;
  for (int64_t i = (int64_t)(blockIdx.x - sb.first[t]) * kBlock + threadIdx.x; i < n; i += nblk * kBlock) {
    if (KIND == GH_SOLVER_VANILLA) {
      float gi = prep_grad(g[i], w[i], use, p);
      gi = gi * neg_eta;
      w[i] = w[i] + gi;
    } else if (KIND == GH_SOLVER_RMSPROP) {
      float gi = g[i];
      float gt2 = gi * gi;
      float cw = c1[i] * p.a;
      gt2 = gt2 * p.b;
      cw = cw + gt2;
      c1[i] = cw;
      if (use & 4) gi = clampf(gi, -p.clip, p.clip);
      float upd = cw + p.eps;
      upd = 1.0f / sqrtf(upd);
      gi = gi * neg_eta;
      upd = upd * gi;
      if (use & 2) { const float reg = w[i] * p.l2reg; upd = upd - reg; }
      w[i] = w[i] + upd;
    } else {
      const float gi = prep_grad(g[i], w[i], use, p);
      const float omb1 = 1.0f - p.a, omb2 = 1.0f - p.b;
      float t1 = gi * omb1;
      float g2 = gi * gi;
      g2 = g2 * omb2;
      const float mb = c1[i] * p.a;
      t1 = t1 + mb;
      const float vb = c2[i] * p.b;
      g2 = g2 + vb;
      c1[i] = t1;
      c2[i] = g2;
      float mh = t1 * p.corr1;
      float vh = g2 * p.corr2;
      vh = sqrtf(vh);
      vh = vh + p.eps;
      mh = mh * neg_eta;
      mh = mh / vh;
      w[i] = w[i] + mh;
    }
  }
}

// ---- dropout and its random source -------------------------------------------------------
// Counter-based: element i is a pure function of (seed, offset + i), so the
// numbers do not depend on the launch shape and a CPU twin can reproduce them.
// T = float: the top 24 bits; T = double: the top 53 bits of the same 64-bit value.
template <class T>
__global__ __launch_bounds__(kBlock) void k_rand_uniform(T* __restrict__ out, int64_t n, uint64_t seed,
                                                         uint64_t offset, const uint64_t* __restrict__ state) {
  if (state) offset = *state;
  const uint64_t base = seed * 0xD1342543DE82EF95ull;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    uint64_t z = base + (offset + (uint64_t)i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    if constexpr (sizeof(T) == 8) out[i] = (double)(z >> 11) * 1.1102230246251565e-16;   // 2^-53
    else out[i] = (float)(uint32_t)(z >> 40) * 5.9604644775390625e-08f;                    // 2^-24
  }
}

__global__ void k_rand_advance(uint64_t* state, uint64_t n) { *state += n; }

__global__ __launch_bounds__(kBlock) void k_dropout(const float* __restrict__ x, const float* __restrict__ r,
                                                    float* __restrict__ y, int64_t n, float keep,
                                                    int identity) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    y[i] = identity ? x[i] : (r[i] < keep ? x[i] / keep : 0.0f);
}

__global__ __launch_bounds__(kBlock) void k_dropout_bwd(const float* __restrict__ y, const float* __restrict__ dy,
                                                        float* __restrict__ dx, int64_t n, float prob) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    dx[i] = (prob != 0.0f && y[i] != 0.0f) ? dy[i] / prob : 0.0f;
}

// how many workgroups share one channel's reduction
int bn_groups(int64_t n, int64_t S) {
  // wide planes: two 256-wide strips of every image per workgroup; else 1024 images per workgroup
  int64_t g = S >= kBlock ? (S + kBlock - 1) / kBlock / 2 : (n / S) / 1024;
  if (g < 1) g = 1;
  if (g > 64) g = 64;
  return (int)g;
}

}  // namespace

int gh_launch_maxpool2d_bwd(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_maxpool2d_bwd_f64(ctx, c);
  const int64_t B = c.dim[0], C = c.dim[1];
  PoolGeom g;
  g.H = (int)c.dim[2]; g.W = (int)c.dim[3]; g.kh = (int)c.dim[4]; g.kw = (int)c.dim[5];
  const int64_t padN = c.dim[6], padS = c.dim[7], padW = c.dim[8], padE = c.dim[9];
  g.strideH = (int)c.dim[10]; g.strideW = (int)c.dim[11];
  g.oh = (int)gh_pool_out(g.H, g.kh, padN, padS, g.strideH);
  g.ow = (int)gh_pool_out(g.W, g.kw, padW, padE, g.strideW);
  const bool explicit_pad = c.flags & GH_FLAG_EXPLICIT_PAD;  // south/east offsets, op_nn.go:871-875
  g.padH = (int)(explicit_pad ? padS : padN);
  g.padW = (int)(explicit_pad ? padE : padW);
  const int64_t total = B * C * g.H * g.W;
  if (total == 0) return GH_OK;
  const bool relu = c.flags & GH_FLAG_ACT_RELU;   // gradient of MaxPool2D(Rectify(x)) with respect to x
  if (g.kh == 2 && g.kw == 2 && g.strideH == 2 && g.strideW == 2 && g.padH == 0 && g.padW == 0 &&
      g.H % 2 == 0 && g.W % 4 == 0 && ((c.ptr[0] | c.ptr[2]) & 15) == 0 && (c.ptr[1] & 7) == 0) {
    const int64_t pairs = total / 8;
    int64_t blocks = (pairs + kBlock - 1) / kBlock;
    if (blocks > (int64_t)ctx->cu_count * 64) blocks = (int64_t)ctx->cu_count * 64;
    if (relu)
      hipLaunchKernelGGL(k_maxpool_2x2s2_bwd<true>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                         (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                         (float*)(uintptr_t)c.ptr[2], g.H, g.W, pairs);
    else
      hipLaunchKernelGGL(k_maxpool_2x2s2_bwd<false>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                         (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                         (float*)(uintptr_t)c.ptr[2], g.H, g.W, pairs);
    return gh_check_hip(ctx, hipGetLastError(), "maxpool backward launch");
  }
  if (g.kh == 2 && g.kw == 2 && g.strideH == 2 && g.strideW == 2 && g.padH == 0 && g.padW == 0 && !explicit_pad &&
      padS == 0 && padE == 0 && g.H >= 2 && g.W >= 2) {
    const int64_t windows = B * C * (int64_t)g.oh * g.ow;
    int64_t blocks = (windows + kBlock - 1) / kBlock;
    if (blocks > (int64_t)ctx->cu_count * 64) blocks = (int64_t)ctx->cu_count * 64;
    if (relu)
      hipLaunchKernelGGL(k_maxpool_2x2s2_bwd_any<true>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                         (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                         (float*)(uintptr_t)c.ptr[2], g.H, g.W, windows);
    else
      hipLaunchKernelGGL(k_maxpool_2x2s2_bwd_any<false>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                         (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                         (float*)(uintptr_t)c.ptr[2], g.H, g.W, windows);
    return gh_check_hip(ctx, hipGetLastError(), "maxpool backward launch");
  }
  int64_t blocks = (total + kBlock - 1) / kBlock;
  if (blocks > (int64_t)ctx->cu_count * 64) blocks = (int64_t)ctx->cu_count * 64;
  if (relu)
    hipLaunchKernelGGL(k_maxpool2d_bwd<true>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                       (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                       (float*)(uintptr_t)c.ptr[2], g, total);
  else
    hipLaunchKernelGGL(k_maxpool2d_bwd<false>, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                       (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                       (float*)(uintptr_t)c.ptr[2], g, total);
  return gh_check_hip(ctx, hipGetLastError(), "maxpool backward launch");
}

int gh_launch_bn_train(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_bn_train_f64(ctx, c);
  const int64_t B = c.dim[0], C = c.dim[1], S = c.dim[2], n = B * S;
  const int G = bn_groups(n, S);
  // scratch: [C][G] sums, [C][G] squared deviations, [C] batch variance
  const int64_t need = (2 * C * G + C) * 4;
  if (need > ctx->workspace_bytes) {
    // under gh_submit_noalloc: the refusal that names the need; there is no smaller plan to fall back to
    if (const int rc = gh_ws_short(ctx, need)) return rc;
    return gh_fail(ctx, GH_ESTATE, "batchnorm: reduction scratch does not fit the workspace");
  }
  float* part_sum = (float*)ctx->workspace;
  float* part_sq = part_sum + C * G;
  float* batch_var = part_sq + C * G;
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  hipLaunchKernelGGL((k_bn_reduce<0>), dim3(G, (int)C), dim3(kBlock), 0, ctx->stream, x, nullptr, part_sum,
                     (int)C, S, n);
  hipLaunchKernelGGL((k_bn_reduce<1>), dim3(G, (int)C), dim3(kBlock), 0, ctx->stream, x, part_sum, part_sq,
                     (int)C, S, n);
  hipLaunchKernelGGL(k_bn_train_finalize, dim3((int)((C + kBlock - 1) / kBlock)), dim3(kBlock), 0, ctx->stream,
                     part_sum, part_sq, (float*)(uintptr_t)c.ptr[2], (float*)(uintptr_t)c.ptr[3],
                     (float*)(uintptr_t)c.ptr[4], (float*)(uintptr_t)c.ptr[5], batch_var, c.f[1], (int)C, G, n);
  int rc = gh_check_hip(ctx, hipGetLastError(), "batchnorm statistics launch");
  if (rc) return rc;
  // y = x*a + b with a = 1/sqrt(batch_var + eps), b = -mean*a: the inference kernel
  gh_cmd a{};
  a.opcode = GH_OP_BN_INFER;
  a.ptr[0] = c.ptr[0]; a.ptr[1] = c.ptr[1]; a.ptr[2] = c.ptr[4]; a.ptr[3] = (uint64_t)(uintptr_t)batch_var;
  a.dim[0] = B; a.dim[1] = C; a.dim[2] = S;
  a.f[0] = c.f[0];
  return gh_launch_bn_infer(ctx, a);
}

int gh_launch_bn_bwd(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_bn_bwd_f64(ctx, c);
  const int64_t B = c.dim[0], C = c.dim[1], S = c.dim[2], n = B * S;
  const int G = bn_groups(n, S);
  if (2 * C * G * 4 > ctx->workspace_bytes) {
    if (const int rc = gh_ws_short(ctx, 2 * C * G * 4)) return rc;
    return gh_fail(ctx, GH_ESTATE, "batchnorm: reduction scratch does not fit the workspace");
  }
  float* part = (float*)ctx->workspace;
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  const float* dy = (const float*)(uintptr_t)c.ptr[1];
  float* dx = (float*)(uintptr_t)c.ptr[2];
  const float* save_mean = (const float*)(uintptr_t)c.ptr[3];
  const float* save_var = (const float*)(uintptr_t)c.ptr[4];
  hipLaunchKernelGGL(k_bn_bwd_reduce, dim3(G, (int)C), dim3(kBlock), 0, ctx->stream, x, dy, save_mean, part,
                     (int)C, S, n);
  const int64_t BC = B * C;
  const int vec = S % 4 == 0 && ((c.ptr[0] | c.ptr[1] | c.ptr[2]) & 15) == 0;
  int gx = (int)(((vec ? S / 4 : S) + kBlock * 4 - 1) / (kBlock * 4));
  if (gx < 1) gx = 1;
  if (gx > 1024) gx = 1024;
  const int64_t gy = BC > 65535 ? 65535 : BC;
  const int training = (c.flags & GH_FLAG_BN_EVAL) ? 0 : 1;
  hipLaunchKernelGGL(k_bn_bwd_apply, dim3(gx, (int)gy), dim3(kBlock), 0, ctx->stream, x, dy, dx, save_mean,
                     save_var, part, c.f[0], training, BC, (int)C, S, G, n, vec);
  return gh_check_hip(ctx, hipGetLastError(), "batchnorm backward launch");
}

int gh_launch_softmax_bwd(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_softmax_bwd_f64(ctx, c);
  const int64_t rows = c.dim[0];
  const int cols = (int)c.dim[1];
  if (rows == 0) return GH_OK;
  const int64_t blocks = (rows + (kBlock / 64) - 1) / (kBlock / 64);
  hipLaunchKernelGGL(k_softmax_bwd, dim3((int)blocks), dim3(kBlock), 0, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], rows, cols);
  return gh_check_hip(ctx, hipGetLastError(), "softmax backward launch");
}

// How many of the commands cmds[0..n) form one solver launch: consecutive
// SOLVER_STEP commands with the same solver, options and hyper-parameters.
int gh_solver_run_length(const gh_cmd* cmds, int n) {
  if (n <= 0 || cmds[0].opcode != GH_OP_SOLVER_STEP) return 0;
  if (gh_dtype_of(cmds[0].flags) == GH_F64) return 1;   // float64 steps go one tensor per launch
  int len = 1;
  while (len < n && len < kSolverBatch && cmds[len].opcode == GH_OP_SOLVER_STEP && cmds[len].flags == cmds[0].flags &&
         cmds[len].ptr[4] == cmds[0].ptr[4] && memcmp(cmds[len].f, cmds[0].f, sizeof(cmds[0].f)) == 0) {
    // a tensor stepped twice keeps its two steps in order: the run ends before the repeat
    bool repeat = false;
    for (int j = 0; j < len; j++) repeat = repeat || cmds[j].ptr[0] == cmds[len].ptr[0];
    if (repeat) break;
    len++;
  }
  return len;
}

// One launch for cmds[0..count) (count from gh_solver_run_length).
int gh_launch_solver_steps(gh_ctx* ctx, const gh_cmd* cmds, int count) {
  const gh_cmd& c = cmds[0];
  const int kind = (int)gh_fn(c.flags), use = (int)gh_mode(c.flags);
  SolverPar p{c.f[0], c.f[1], c.f[2], c.f[3], c.f[4], c.f[5], c.f[6], c.f[7], c.f[8], c.f[9]};
  SolverBatch sb{};
  int nt = 0, blocks_total = 0;
  for (int i = 0; i < count; i++) {
    const int64_t n = cmds[i].dim[0];
    if (n == 0) continue;
    sb.w[nt] = (float*)(uintptr_t)cmds[i].ptr[0];
    sb.g[nt] = (const float*)(uintptr_t)cmds[i].ptr[1];
    sb.c1[nt] = (float*)(uintptr_t)cmds[i].ptr[2];
    sb.c2[nt] = (float*)(uintptr_t)cmds[i].ptr[3];
    sb.n[nt] = n;
    int64_t blocks = (n + kBlock - 1) / kBlock;
    if (blocks > (int64_t)ctx->cu_count * 32) blocks = (int64_t)ctx->cu_count * 32;
    sb.first[nt] = blocks_total;
    blocks_total += (int)blocks;
    nt++;
  }
  if (nt == 0) return GH_OK;
  for (int i = nt; i <= kSolverBatch; i++) sb.first[i] = blocks_total;
  sb.count = nt;
  const dim3 grid(blocks_total), block(kBlock);
  const float* corr = (const float*)(uintptr_t)c.ptr[4];
  if (kind == GH_SOLVER_VANILLA)
    hipLaunchKernelGGL((k_solver_step<GH_SOLVER_VANILLA>), grid, block, 0, ctx->stream, sb, use, p, corr);
  else if (kind == GH_SOLVER_RMSPROP)
    hipLaunchKernelGGL((k_solver_step<GH_SOLVER_RMSPROP>), grid, block, 0, ctx->stream, sb, use, p, corr);
  else
    hipLaunchKernelGGL((k_solver_step<GH_SOLVER_ADAM>), grid, block, 0, ctx->stream, sb, use, p, corr);
  return gh_check_hip(ctx, hipGetLastError(), "solver step launch");
}

int gh_launch_solver_step(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_solver_step_f64(ctx, c);
  return gh_launch_solver_steps(ctx, &c, 1);
}

static int stream_blocks(gh_ctx* ctx, int64_t n) {
  int64_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > (int64_t)ctx->cu_count * 32) blocks = (int64_t)ctx->cu_count * 32;
  return (int)(blocks < 1 ? 1 : blocks);
}

int gh_launch_rand_uniform(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  uint64_t* state = (uint64_t*)(uintptr_t)c.ptr[1];
  if (n > 0 && gh_dtype_of(c.flags) == GH_F64)
    hipLaunchKernelGGL(k_rand_uniform<double>, dim3(stream_blocks(ctx, n)), dim3(kBlock), 0, ctx->stream,
                       (double*)(uintptr_t)c.ptr[0], n, (uint64_t)c.dim[1], (uint64_t)c.dim[2], state);
  else if (n > 0)
    hipLaunchKernelGGL(k_rand_uniform<float>, dim3(stream_blocks(ctx, n)), dim3(kBlock), 0, ctx->stream,
                       (float*)(uintptr_t)c.ptr[0], n, (uint64_t)c.dim[1], (uint64_t)c.dim[2], state);
  if (state && n > 0) hipLaunchKernelGGL(k_rand_advance, dim3(1), dim3(1), 0, ctx->stream, state, (uint64_t)n);
  return gh_check_hip(ctx, hipGetLastError(), "uniform generator launch");
}

int gh_launch_dropout(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_dropout_f64(ctx, c);
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  const int identity = (c.flags & GH_FLAG_BN_EVAL) || c.f[0] == 0.0f;
  const float keep = (float)(1.0 - (double)c.f[0]);
  hipLaunchKernelGGL(k_dropout, dim3(stream_blocks(ctx, n)), dim3(kBlock), 0, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[2],
                     (float*)(uintptr_t)c.ptr[1], n, keep, identity);
  return gh_check_hip(ctx, hipGetLastError(), "dropout launch");
}

int gh_launch_dropout_bwd(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_dropout_bwd_f64(ctx, c);
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  hipLaunchKernelGGL(k_dropout_bwd, dim3(stream_blocks(ctx, n)), dim3(kBlock), 0, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], n, c.f[0]);
  return gh_check_hip(ctx, hipGetLastError(), "dropout backward launch");
}
