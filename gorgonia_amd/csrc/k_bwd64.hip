// float64 twins of the backward operators, dropout and the solver steps for gfx950.
// The reference's CPU engine has a float64 branch beside every float32 one
// (maxPoolDiffOp.f64s op_nn.go:1095-1120, softmaxDiffOp op_softmax.go:266-279,
// dropoutOp / dropoutDiffOp op_dropout.go:107-238, the Float64 cases of
// VanillaSolver / RMSPropSolver / AdamSolver Step solvers.go:273-870); these
// kernels follow the float32 ones of k_bwd.hip and k_elem.hip operation by
// operation in double.  Plain one-thread-per-element kernels, not tuned.
// Scalars ride in dim slots as the bit pattern of a double (gh_cmd.f is float32):
// DROPOUT / DROPOUT_BWD probability in dim[1]; SOLVER_STEP's ten constants in
// dim[1..10]; BN_TRAIN epsilon and momentum in dim[3], dim[4]; BN_BWD epsilon in dim[3].
#include <cfloat>
#include <cstring>

#include "gh_internal.h"

namespace {

constexpr int kBlock = 256;

inline double bits_to_double(int64_t bits) {
  double v;
  memcpy(&v, &bits, sizeof(v));
  return v;
}

int blocks_for(gh_ctx* ctx, int64_t n) {
  int64_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > (int64_t)ctx->cu_count * 32) blocks = (int64_t)ctx->cu_count * 32;
  return (int)(blocks < 1 ? 1 : blocks);
}

// dy * (x >= 0 ? 1 : 0): Gte then HadamardProd
__global__ __launch_bounds__(kBlock) void k_relu_bwd_f64(const double* __restrict__ x, const double* dy, double* dx,
                                                         int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    dx[i] = dy[i] * (x[i] >= 0.0 ? 1.0 : 0.0);
}

__global__ __launch_bounds__(kBlock) void k_dropout_f64(const double* __restrict__ x, const double* __restrict__ r,
                                                        double* __restrict__ y, int64_t n, double keep,
                                                        int identity) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    y[i] = identity ? x[i] : (r[i] < keep ? x[i] / keep : 0.0);
}

__global__ __launch_bounds__(kBlock) void k_dropout_bwd_f64(const double* __restrict__ y,
                                                            const double* __restrict__ dy,
                                                            double* __restrict__ dx, int64_t n, double prob) {
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
    dx[i] = (prob != 0.0 && y[i] != 0.0) ? dy[i] / prob : 0.0;
}

// one thread per row: dot = sum_j dy_j*y_j in column order, dx_j = y_j * (dy_j - dot)
__global__ __launch_bounds__(kBlock) void k_softmax_bwd_f64(const double* __restrict__ y,
                                                            const double* __restrict__ dy,
                                                            double* __restrict__ dx, int64_t rows, int cols) {
  const int64_t row = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (row >= rows) return;
  const double* yy = y + row * cols;
  const double* g = dy + row * cols;
  double dot = 0.0;
  for (int j = 0; j < cols; j++) { const double t = g[j] * yy[j]; dot = dot + t; }
  for (int j = 0; j < cols; j++) { const double t = g[j] - dot; dx[row * cols + j] = yy[j] * t; }
}

struct PoolGeom {
  int H, W, oh, ow, kh, kw, padH, padW, strideH, strideW;
};

// One thread per input element gathers, in (ph, pw) order, the dy of every
// window whose argmax it is (first strict maximum in row-major window order
// from -DBL_MAX): the bits of the reference's zero-then-scatter loop.
__global__ __launch_bounds__(kBlock) void k_maxpool2d_bwd_f64(const double* __restrict__ x,
                                                              const double* __restrict__ dy,
                                                              double* __restrict__ dx, PoolGeom g,
                                                              int64_t total) {
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  const int plane = g.H * g.W;
  for (int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += stride) {
    const int64_t bc = idx / plane;
    const int me = (int)(idx - bc * plane);
    const int iy = me / g.W, ix = me - iy * g.W;
    const double* in = x + bc * (int64_t)plane;
    const double* gy = dy + bc * (int64_t)g.oh * g.ow;
    const int ny = iy + g.padH - g.kh + 1, nx = ix + g.padW - g.kw + 1;
    const int ph0 = ny > 0 ? (ny + g.strideH - 1) / g.strideH : 0;
    const int pw0 = nx > 0 ? (nx + g.strideW - 1) / g.strideW : 0;
    const int ph1 = min(g.oh - 1, (iy + g.padH) / g.strideH);
    const int pw1 = min(g.ow - 1, (ix + g.padW) / g.strideW);
    double acc = 0.0;
    for (int ph = ph0; ph <= ph1; ph++)
      for (int pw = pw0; pw <= pw1; pw++) {
        int hs = ph * g.strideH - g.padH, ws = pw * g.strideW - g.padW;
        const int he = min(hs + g.kh, g.H), we = min(ws + g.kw, g.W);
        hs = max(hs, 0);
        ws = max(ws, 0);
        double best = -DBL_MAX;
        int arg = -1;
        for (int hi = hs; hi < he; hi++)
          for (int wi = ws; wi < we; wi++) {
            const double v = in[hi * g.W + wi];
            if (v > best) { best = v; arg = hi * g.W + wi; }
          }
        if (arg == me) acc = acc + gy[ph * g.ow + pw];
      }
    dx[idx] = acc;
  }
}

// ---- BatchNorm training forward and gradient (op_nn.go:1489-1635, 1834-1943) -------------
// One workgroup per channel: the channel's n = B*S values are summed by a fixed
// tree (thread-strided partial sums, then a tree over the 256 threads), so
// results repeat run to run; against the reference's sequential sums the
// difference is float64 rounding.
__device__ __forceinline__ double block_sum_f64(double v, double* sh) {
  sh[threadIdx.x] = v;
  __syncthreads();
  for (int off = kBlock / 2; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) sh[threadIdx.x] = sh[threadIdx.x] + sh[threadIdx.x + off];
    __syncthreads();
  }
  const double r = sh[0];
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(kBlock) void k_bn_train_f64(const double* __restrict__ x, double* __restrict__ y,
                                                         double* __restrict__ run_mean,
                                                         double* __restrict__ run_var,
                                                         double* __restrict__ save_mean,
                                                         double* __restrict__ save_var, int64_t B, int C,
                                                         int64_t S, double eps, double momentum) {
  __shared__ double sh[kBlock];
  const int c = blockIdx.x;
  const int64_t n = B * S;
  auto at = [&](int64_t e) { return ((e / S) * C + c) * S + e % S; };
  double acc = 0.0;
  for (int64_t e = threadIdx.x; e < n; e += kBlock) acc = acc + x[at(e)];
  const double mean = block_sum_f64(acc, sh) / (double)n;
  acc = 0.0;
  for (int64_t e = threadIdx.x; e < n; e += kBlock) {
    const double t = x[at(e)] - mean;
    const double t2 = t * t;
    acc = acc + t2;
  }
  const double var = block_sum_f64(acc, sh);   // the SUM of squared deviations, as the reference keeps it
  if (threadIdx.x == 0) {
    save_mean[c] = mean;
    save_var[c] = var;
    const double m1 = momentum * mean, m2 = (1.0 - momentum) * run_mean[c];
    run_mean[c] = m1 + m2;
    const double unb = var / (double)(n - 1);
    const double v1 = momentum * unb, v2 = (1.0 - momentum) * run_var[c];
    run_var[c] = v1 + v2;
  }
  const double vb = var / (double)n;
  const double a = 1.0 / sqrt(vb + eps);
  const double b = -mean * a;
  for (int64_t e = threadIdx.x; e < n; e += kBlock) {
    const double t = x[at(e)] * a;
    y[at(e)] = t + b;
  }
}

__global__ __launch_bounds__(kBlock) void k_bn_bwd_f64(const double* __restrict__ x, const double* __restrict__ dy,
                                                       double* __restrict__ dx,
                                                       const double* __restrict__ save_mean,
                                                       const double* __restrict__ save_var, int64_t B, int C,
                                                       int64_t S, double eps, int training) {
  __shared__ double sh[kBlock];
  const int c = blockIdx.x;
  const int64_t n = B * S;
  auto at = [&](int64_t e) { return ((e / S) * C + c) * S + e % S; };
  const double mean = save_mean[c];
  double s = 0.0, dot = 0.0;
  for (int64_t e = threadIdx.x; e < n; e += kBlock) {
    const double xv = x[at(e)], g = dy[at(e)];
    s = s + g;
    double p;
    if (S == 1) {
      const double t = xv - mean;
      p = t * g;
    } else {
      const double t1 = xv * g, t2 = mean * g;
      p = t1 - t2;
    }
    dot = dot + p;
  }
  const double sum = block_sum_f64(s, sh);
  const double dotp = block_sum_f64(dot, sh);
  const double vb = save_var[c] / (double)n;
  const double invstd = 1.0 / sqrt(vb + eps);
  double k = dotp * invstd;
  k = k * invstd;
  k = k / (double)n;
  const double grad_mean = sum / (double)n;
  for (int64_t e = threadIdx.x; e < n; e += kBlock) {
    const double xv = x[at(e)], g = dy[at(e)];
    double out;
    if (!training) {
      out = g * invstd;
    } else {
      double t = xv - mean;
      t = t * k;
      double u;
      if (S == 1) { u = g - t; u = u - grad_mean; }
      else { u = g - grad_mean; u = u - t; }
      out = u * invstd;
    }
    dx[at(e)] = out;
  }
}

struct SolverPar64 { double eta, eps, l1reg, l2reg, clip, one_per_batch, a, b, corr1, corr2; };

__device__ __forceinline__ double clampd(double v, double lo, double hi) { return v < lo ? lo : (v > hi ? hi : v); }

__device__ __forceinline__ double prep_grad(double g, double w, int use, const SolverPar64& p) {
  if (use & 1) { const double t = p.l1reg * (double)((w > 0.0) - (w < 0.0)); g = g + t; }
  if (use & 2) { const double t = w * p.l2reg; g = g + t; }
  if (use & 8) g = g * p.one_per_batch;
  if ((use & 4) && p.clip > 0.0) g = clampd(g, -p.clip, p.clip);
  return g;
}

template <int KIND>
__global__ __launch_bounds__(kBlock) void k_solver_step_f64(double* __restrict__ w, const double* __restrict__ g,
                                                            double* __restrict__ c1, double* __restrict__ c2,
                                                            int64_t n, int use, SolverPar64 p,
                                                            const double* __restrict__ corr) {
  if (KIND == GH_SOLVER_ADAM && corr) { p.corr1 = corr[0]; p.corr2 = corr[1]; }   // see k_solver_step
  const double neg_eta = -p.eta;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    if (KIND == GH_SOLVER_VANILLA) {
      double gi = prep_grad(g[i], w[i], use, p);
      gi = gi * neg_eta;
      w[i] = w[i] + gi;
    } else if (KIND == GH_SOLVER_RMSPROP) {
      double gi = g[i];
      double gt2 = gi * gi;
      double cw = c1[i] * p.a;
      gt2 = gt2 * p.b;
      cw = cw + gt2;
      c1[i] = cw;
      if (use & 4) gi = clampd(gi, -p.clip, p.clip);
      double upd = cw + p.eps;
      upd = 1.0 / sqrt(upd);
      gi = gi * neg_eta;
      upd = upd * gi;
      if (use & 2) { const double reg = w[i] * p.l2reg; upd = upd - reg; }
      w[i] = w[i] + upd;
    } else {
      const double gi = prep_grad(g[i], w[i], use, p);
      const double omb1 = 1.0 - p.a, omb2 = 1.0 - p.b;
      double t1 = gi * omb1;
      double g2 = gi * gi;
      g2 = g2 * omb2;
      const double mb = c1[i] * p.a;
      t1 = t1 + mb;
      const double vb = c2[i] * p.b;
      g2 = g2 + vb;
      c1[i] = t1;
      c2[i] = g2;
      double mh = t1 * p.corr1;
      double vh = g2 * p.corr2;
      vh = sqrt(vh);
      vh = vh + p.eps;
      mh = mh * neg_eta;
      mh = mh / vh;
      w[i] = w[i] + mh;
    }
  }
}

}  // namespace

int gh_launch_relu_bwd_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  hipLaunchKernelGGL(k_relu_bwd_f64, dim3(blocks_for(ctx, n)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], n);
  return gh_check_hip(ctx, hipGetLastError(), "relu backward launch");
}

int gh_launch_dropout_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  const double prob = bits_to_double(c.dim[1]);
  const int identity = (c.flags & GH_FLAG_BN_EVAL) || prob == 0.0;
  hipLaunchKernelGGL(k_dropout_f64, dim3(blocks_for(ctx, n)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[2],
                     (double*)(uintptr_t)c.ptr[1], n, 1.0 - prob, identity);
  return gh_check_hip(ctx, hipGetLastError(), "dropout launch");
}

int gh_launch_dropout_bwd_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  hipLaunchKernelGGL(k_dropout_bwd_f64, dim3(blocks_for(ctx, n)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], n, bits_to_double(c.dim[1]));
  return gh_check_hip(ctx, hipGetLastError(), "dropout backward launch");
}

int gh_launch_softmax_bwd_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t rows = c.dim[0];
  if (rows == 0) return GH_OK;
  hipLaunchKernelGGL(k_softmax_bwd_f64, dim3(blocks_for(ctx, rows)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], rows, (int)c.dim[1]);
  return gh_check_hip(ctx, hipGetLastError(), "softmax backward launch");
}

int gh_launch_maxpool2d_bwd_f64(gh_ctx* ctx, const gh_cmd& c) {
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
  hipLaunchKernelGGL(k_maxpool2d_bwd_f64, dim3(blocks_for(ctx, total)), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], g, total);
  return gh_check_hip(ctx, hipGetLastError(), "maxpool backward launch");
}

int gh_launch_bn_train_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t B = c.dim[0], C = c.dim[1], S = c.dim[2];
  hipLaunchKernelGGL(k_bn_train_f64, dim3((unsigned)C), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], (double*)(uintptr_t)c.ptr[3], (double*)(uintptr_t)c.ptr[4],
                     (double*)(uintptr_t)c.ptr[5], B, (int)C, S, bits_to_double(c.dim[3]), bits_to_double(c.dim[4]));
  return gh_check_hip(ctx, hipGetLastError(), "batchnorm training launch");
}

int gh_launch_bn_bwd_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t B = c.dim[0], C = c.dim[1], S = c.dim[2];
  hipLaunchKernelGGL(k_bn_bwd_f64, dim3((unsigned)C), dim3(kBlock), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                     (double*)(uintptr_t)c.ptr[2], (const double*)(uintptr_t)c.ptr[3],
                     (const double*)(uintptr_t)c.ptr[4], B, (int)C, S, bits_to_double(c.dim[3]),
                     (c.flags & GH_FLAG_BN_EVAL) ? 0 : 1);
  return gh_check_hip(ctx, hipGetLastError(), "batchnorm backward launch");
}

int gh_launch_solver_step_f64(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t n = c.dim[0];
  if (n == 0) return GH_OK;
  const int kind = (int)gh_fn(c.flags), use = (int)gh_mode(c.flags);
  SolverPar64 p{bits_to_double(c.dim[1]), bits_to_double(c.dim[2]), bits_to_double(c.dim[3]),
                bits_to_double(c.dim[4]), bits_to_double(c.dim[5]), bits_to_double(c.dim[6]),
                bits_to_double(c.dim[7]), bits_to_double(c.dim[8]), bits_to_double(c.dim[9]),
                bits_to_double(c.dim[10])};
  double* w = (double*)(uintptr_t)c.ptr[0];
  const double* g = (const double*)(uintptr_t)c.ptr[1];
  double* c1 = (double*)(uintptr_t)c.ptr[2];
  double* c2 = (double*)(uintptr_t)c.ptr[3];
  const dim3 grid(blocks_for(ctx, n)), block(kBlock);
  const double* corr = (const double*)(uintptr_t)c.ptr[4];
  if (kind == GH_SOLVER_VANILLA)
    hipLaunchKernelGGL((k_solver_step_f64<GH_SOLVER_VANILLA>), grid, block, 0, ctx->stream, w, g, c1, c2, n, use, p, corr);
  else if (kind == GH_SOLVER_RMSPROP)
    hipLaunchKernelGGL((k_solver_step_f64<GH_SOLVER_RMSPROP>), grid, block, 0, ctx->stream, w, g, c1, c2, n, use, p, corr);
  else
    hipLaunchKernelGGL((k_solver_step_f64<GH_SOLVER_ADAM>), grid, block, 0, ctx->stream, w, g, c1, c2, n, use, p, corr);
  return gh_check_hip(ctx, hipGetLastError(), "solver step launch");
}
