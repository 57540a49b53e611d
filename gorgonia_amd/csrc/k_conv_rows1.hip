// Conv2d 3x3 / stride 1 of single-channel images (a network's first layer on grey-scale input),
// float32, on the 16x16x4 MFMA with the output pixels on the matrix rows.
//
// Replaces cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117) for C = 1.  K is the nine
// taps padded to twelve, so a 16 x 16 output tile is three MFMAs; what the kernel spends its time on
// is the epilogue and the stores, and the layout is chosen for them: a lane's four accumulator
// registers are one 2x2 pooling window of one filter (gh_conv_rows1.h), so Rectify and a fused
// max-pool never leave the lane.  The same tile function runs inside k_conv3x3_rows when this
// convolution is folded into the one that follows it (GH_FLAG_CONV_PRE), which is why the shapes
// that can be folded run here and not on the vector-ALU kernel: folded or not, a result has one
// summing order.
//
// A workgroup of four wavefronts stages the whole padded image in LDS (a few KB) and the filters in
// MFMA operand order, then takes a run of pixel tiles; a wavefront fetches a tile's pixel operand
// once and walks the filter tiles with it.
#include <cstdlib>

#include "gh_conv_common.h"
#include "gh_conv_rows1.h"
#include "gh_internal.h"

namespace {

using rows1::f32x4;
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads1 = 256;
constexpr int kWaves1 = 4;

inline unsigned magic_of(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
__device__ __forceinline__ int mdiv(int n, unsigned magic) {
  const unsigned q = __umulhi((unsigned)n, magic);
  return (int)(q | ((unsigned)n & (0u - (unsigned)(magic == 0))));
}

struct Rows1Geom {
  int B, H, W, F, pad, oh, ow, ph, pw;
  int RW, ZP;        // padded row pitch; zero floats in front of the image
  int HW, N, PT;     // input pixels, output pixels (4 per window), pixel tiles
  int TPP;           // pixel tiles per workgroup
  int FT;            // filter tiles
  int offW;          // LDS offset of the filter operands, floats
  int y8;            // 1: y is 8-byte aligned (pairs of a window row go out as one store)
  unsigned mW, mPW;
};

// keep: with POOL, where the convolution's own result goes as well (B x F x oh x ow, the values the activation
// and the pool read), or null.
template <bool POOL>
__global__ __launch_bounds__(kThreads1) void k_conv3x3_rows1(const float* __restrict__ x, const float* __restrict__ w,
                                                             float* __restrict__ y, Rows1Geom g, ConvTail tail,
                                                             float* __restrict__ keep) {
  extern __shared__ float lds[];
  float* const Raw = lds;
  float* const Wl = lds + g.offW;   // [FT][3][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lk = lane >> 4;
  const int img = blockIdx.y;
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, g.F * 36, 0x00020000);
  const float* const xi = x + (int64_t)img * g.HW;

  // filters in operand order, the image behind zeroed LDS
  for (int i = tid; i < g.FT * 64; i += kThreads1) {
    float b[3];
    rows1::filter_operand(rw, (i >> 6) * 16 + (i & 15), (i & 63) >> 4, b);
    float* d = Wl + (i >> 6) * 192 + (i & 63);
    d[0] = b[0]; d[64] = b[1]; d[128] = b[2];
  }
  for (int i = tid; i < g.offW; i += kThreads1) Raw[i] = 0.0f;
  __syncthreads();
  for (int e = tid; e < g.HW; e += kThreads1) {
    const int r = mdiv(e, g.mW), c = e - r * g.W;
    Raw[g.ZP + (r + g.pad) * g.RW + c + g.pad] = xi[e];
  }
  __syncthreads();

  const rows1::LaneTaps L = rows1::lane_taps(lk, g.RW);
  const int t_end = min((int)(blockIdx.x + 1) * g.TPP, g.PT);
  const int outplane = POOL ? g.ph * g.pw : g.oh * g.ow;
  float* const yi = y + (int64_t)img * g.F * outplane;
  const float alpha = tail.alpha;
  for (int pt = blockIdx.x * g.TPP + wave; pt < t_end; pt += kWaves1) {
    // the lane's pixel (operand side) ...
    int base = 0;
    {
      const int n = pt * 16 + li;
      if (n < g.N) {
        const int gw = n >> 2, pos = n & 3;
        const int py = mdiv(gw, g.mPW), px = gw - py * g.pw;
        base = g.ZP + (2 * py + (pos >> 1)) * g.RW + 2 * px + (pos & 1);
      }
    }
    float a[3];
    rows1::pixel_operand(Raw, base, L, a);
    // ... and the window its accumulator registers hold (result side)
    const int gwd = pt * 4 + lk;
    const bool wok = gwd < g.ph * g.pw;
    const int pyd = mdiv(gwd, g.mPW), pxd = gwd - pyd * g.pw;
    const int o = POOL ? gwd : 2 * pyd * g.ow + 2 * pxd;
    const int okeep = 2 * pyd * g.ow + 2 * pxd;
    for (int ft = 0; ft < g.FT; ft++) {
      float b[3];
      const float* const wl = Wl + ft * 192 + lane;
      b[0] = wl[0]; b[1] = wl[64]; b[2] = wl[128];
      f32x4 v = rows1::tile(a, b);
      const int col = ft * 16 + li;
      const bool ok = wok && col < g.F;
      const int f = min(col, g.F - 1);
      conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
        constexpr bool BN = decltype(bn_c)::value;
        constexpr int ACT = decltype(act_c)::value;
        if constexpr (BN) {
          // BN_INFER's roundings (op_nn.go:1559-1584), an absent gamma 1 and an absent beta -0
          const float ka = 1.0f / sqrtf(tail.var[f] + tail.eps);
          const float kb = -tail.mean[f] * ka;
          const float kg = tail.gamma ? tail.gamma[f] : 1.0f;
          const float kbeta = tail.beta ? tail.beta[f] : -0.0f;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            float t = v[r] * ka;
            t = t + kb;
            t = kg * t;
            v[r] = t + kbeta;
          }
        }
        if constexpr (POOL) {
          if (keep && ok) {   // the pair stores of the plain command
            float* const kp = keep + ((int64_t)img * g.F + col) * (g.oh * g.ow) + okeep;
            if (g.y8) {
              *reinterpret_cast<f32x2*>(kp) = f32x2{v[0], v[1]};
              *reinterpret_cast<f32x2*>(kp + g.ow) = f32x2{v[2], v[3]};
            } else {
              kp[0] = v[0]; kp[1] = v[1]; kp[g.ow] = v[2]; kp[g.ow + 1] = v[3];
            }
          }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = act_apply(v[r], ACT, alpha);
      });
      float* const yp = yi + (int64_t)col * outplane + o;
      if constexpr (POOL) {
        const float best = rows1::pool_window(v);
        if (ok) *yp = best;
      } else if (ok) {
        if (g.y8) {
          *reinterpret_cast<f32x2*>(yp) = f32x2{v[0], v[1]};
          *reinterpret_cast<f32x2*>(yp + g.ow) = f32x2{v[2], v[3]};
        } else {
          yp[0] = v[0]; yp[1] = v[1]; yp[g.ow] = v[2]; yp[g.ow + 1] = v[3];
        }
      }
    }
  }
}

// Single-channel 3x3 / stride 1 / no dilation, padding 0 or 1 on both axes, even output extents (every
// output pixel lies in a 2x2 window), an image and a filter bank that fit a small LDS budget.
bool rows1_geom(const gh_cmd& c, Rows1Geom* out) {
  if (gh_dtype_of(c.flags) != GH_F32) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4], pad = c.dim[7];
  if (C != 1 || c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 || c.dim[12] != 1 ||
      c.dim[8] != pad || pad < 0 || pad > 1)
    return false;
  if (B < 1 || B > 65535 || F < 16 || F > 256 || H < 2 || W < 2 || H > 64 || W > 64) return false;
  if (getenv("GORGONIA_HIP_CONV_NO_ROWS1")) return false;   // tuning switch: the vector-ALU kernel instead
  Rows1Geom g{};
  g.B = (int)B; g.H = (int)H; g.W = (int)W; g.F = (int)F; g.pad = (int)pad;
  g.oh = g.H + 2 * g.pad - 2; g.ow = g.W + 2 * g.pad - 2;
  if (g.oh < 2 || g.ow < 2 || (g.oh & 1) || (g.ow & 1)) return false;
  g.ph = g.oh / 2; g.pw = g.ow / 2;
  g.RW = g.W + 2 * g.pad;
  g.ZP = (2 * g.RW + 4 + 3) & ~3;
  g.HW = g.H * g.W;
  g.N = g.oh * g.ow;
  g.PT = (g.N + 15) / 16;
  g.FT = (g.F + 15) / 16;
  g.offW = (g.ZP + (g.H + 2 * g.pad) * g.RW + 3) & ~3;
  g.mW = magic_of((unsigned)g.W); g.mPW = magic_of((unsigned)g.pw);
  *out = g;
  return true;
}

}  // namespace

bool gh_conv_rows1_takes(const gh_cmd& c) {
  Rows1Geom g;
  return rows1_geom(c, &g);
}

// Returns -1 when the shape is not one this kernel takes.
int gh_try_launch_conv_rows1(gh_ctx* ctx, const gh_cmd& c) {
  Rows1Geom g;
  if (!rows1_geom(c, &g)) return -1;
  // enough workgroups for a few wavefronts per SIMD, at least four pixel tiles each
  int parts = (int)((4 * (int64_t)ctx->cu_count + g.B - 1) / g.B);
  if (const char* e = getenv("GORGONIA_HIP_CONV_ROWS1_PARTS")) parts = atoi(e);
  if (parts > (g.PT + 3) / 4) parts = (g.PT + 3) / 4;
  if (parts < 1) parts = 1;
  g.TPP = (g.PT + parts - 1) / parts;
  parts = (g.PT + g.TPP - 1) / g.TPP;
  const bool pool = c.flags & GH_FLAG_CONV_POOL2;
  float* const keep = (pool && (c.flags & GH_FLAG_CONV_KEEP)) ? (float*)(uintptr_t)c.ptr[7] : nullptr;
  g.y8 = ((keep ? c.ptr[7] : c.ptr[2]) & 7) == 0;   // of the tensor that gets the unpooled pairs
  const size_t lds = ((size_t)g.offW + (size_t)g.FT * 192) * 4;
  const dim3 grid((unsigned)parts, (unsigned)g.B);
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  const float* w = (const float*)(uintptr_t)c.ptr[1];
  float* y = (float*)(uintptr_t)c.ptr[2];
  if (pool)
    hipLaunchKernelGGL((k_conv3x3_rows1<true>), grid, dim3(kThreads1), lds, ctx->stream, x, w, y, g, conv_tail(c), keep);
  else
    hipLaunchKernelGGL((k_conv3x3_rows1<false>), grid, dim3(kThreads1), lds, ctx->stream, x, w, y, g, conv_tail(c), keep);
  return gh_check_hip(ctx, hipGetLastError(), "conv3x3 rows1 launch");
}
