// Filter gradient of Conv2d 3x3 / stride 1 over small images (up to 16 x 16), float32, on the
// 16x16x4 MFMA.
//
// Replaces cuDNN ConvolutionBackwardFilter (ops/nn/convolution_cuda.go:182-189) for the layers
// whose images are small and many: dW[f][c][kr][kc] = sum over (image, output pixel) of
// dy[image][f][pixel] * x[image][c][pixel + tap].  As a GEMM that is M = filters,
// N = C * 9 in the reference's (c, kr, kc) order, K = B * oh * ow: a small result summed over
// a long K, so K is what gets divided among workgroups.
//
//   * One workgroup of eight wavefronts owns 64 filters x 16 channels (a 64 x 144 tile of dW:
//     wavefront w has filter rows 16 (w & 3) .. + 15, all nine 16-column tiles and one half
//     of every group's k steps; the two halves meet through LDS at the end, second onto
//     first, a fixed order) and a run of images.  Two wavefronts per SIMD: one's LDS and
//     issue latencies run under the other's MFMAs.  It takes the images a few at a time (as many as give about 200 output pixels):
//     their dy rows go to LDS as dyL[filter][k] with k = (image, pixel) and a pitch of 4 mod
//     64, so the 64 lanes of an A fetch hit 64 banks; their x planes go to LDS with a zero
//     halo, rows at a fixed pitch of 18 and planes at a pitch of 4 mod 32.  The tile's 144
//     columns are taken tap-major: MFMA tile t is tap t and lane column c is channel c, so a
//     step's nine B fetches are one address - channel plane + the pixel position a table
//     gives for every k - plus nine compile-time offsets (tap row * 18 + tap column), and
//     the 64 lanes of each land in 64 banks.  Per step of four k: one A read, one table read,
//     one address add and nine B reads feed nine MFMAs.
//   * The tile is accumulated in registers over all of the workgroup's images and stored
//     once, as slab `split` of the workspace; slabs are summed in slab order by the
//     reduction kernel the other filter-gradient kernels use, so results repeat bit for bit.
//     With enough (filter, channel) tiles to fill the device there is one slab and the tile
//     is stored straight into dW.
#include <algorithm>
#include <cstdlib>
#include <mutex>

#include "gh_internal.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));   // a row of dy starts on any float

inline unsigned magic_of(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
// n / d with magic = magic_of(d), exact while n * d < 2^32 (magic 0 stands for d = 1)
__device__ __forceinline__ int mdiv(int n, unsigned magic) {
  const unsigned q = __umulhi((unsigned)n, magic);
  return (int)(q | ((unsigned)n & (0u - (unsigned)(magic == 0))));
}

struct WgGeom {
  int B, C, H, W, F, pad, oh, ow;
  int npx;          // oh * ow
  int nb;           // images staged together
  int K;            // nb * npx
  int KW;           // K rounded up to a multiple of 4
  int DP;           // pitch of a dyL row, = 4 mod 64, >= KW
  int PW, PH, PP;   // padded plane: (W + 2 pad) x (H + 2 pad), PP = PH * PW
  int XP;           // plane pitch in LDS (= 4 mod 32, >= PH * kRowPitch)
  int HW;
  int CKK;          // C * 9
  int ngroups;      // ceil(B / nb)
  int gps;          // image groups per split
  unsigned mNPX, mOW, mPP, mPW, mQIMG;
};

constexpr int kCT = 16;          // channels per workgroup
constexpr int kBM = 64;          // filters per workgroup
constexpr int kThreads = 512;
constexpr int kRowPitch = 18;    // row pitch of a staged plane: the widest padded image (16 + 2)
constexpr int kU = 6;            // loads a thread has in flight while staging

// Held to 128 registers: two workgroups then share a compute unit where their LDS allows (long K, few images).
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) void k_conv3x3_wgrad_small(const float* __restrict__ x,
                                                                  const float* __restrict__ dy,
                                                                  float* __restrict__ out, WgGeom g,
                                                                  int64_t slab) {
  extern __shared__ float lds[];
  float* const dyL = lds;                                  // [64][DP]
  float* const xL = dyL + kBM * g.DP;                      // [nb][16][XP]
  int* const ptab = reinterpret_cast<int*>(xL + g.nb * kCT * g.XP);   // [KW]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mt = wave & 3, khalf = wave >> 2;   // tile row, half of the k steps
  const int li = lane & 15, lk = lane >> 4;
  const int split = blockIdx.x, c0 = blockIdx.y * kCT, f0 = blockIdx.z * kBM;

  // position of every k in the staged planes: image plane block + row + column
  for (int p = tid; p < g.KW; p += kThreads) {
    int pos = 0;
    if (p < g.K) {
      const int img = mdiv(p, g.mNPX), r = p - img * g.npx;
      const int row = mdiv(r, g.mOW), col = r - row * g.ow;
      pos = img * (kCT * g.XP) + row * kRowPitch + col;
    }
    ptab[p] = pos;
  }
  // B column of (tile t, lane li) is (tap t, channel li): the lane's plane, the tile's tap offset
  const int xlane = li * g.XP;
  f32x4 acc[9];
#pragma unroll
  for (int t = 0; t < 9; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int gend = min(g.ngroups, (split + 1) * g.gps);
  for (int grp = split * g.gps; grp < gend; grp++) {
    const int b0 = grp * g.nb;
    // ---- dy rows: element e of the group is (image, filter, pixel), contiguous per image.
    // Loads go out in batches (kU per thread) before any is stored: alone on its SIMD a
    // wavefront that waits for each load in turn spends a memory latency per element.
    const int per_img = kBM * g.npx;
    const int nfv = min(kBM, g.F - f0) * g.npx;     // elements of an image's block that exist
    const int q_img = per_img >> 2;                 // 128-bit pieces per image (64 npx is a multiple of 4)
    for (int base = 0; base < g.nb * q_img; base += kU * kThreads) {
      f32x4 v[kU];
      int dst[kU], left[kU];
#pragma unroll
      for (int u = 0; u < kU; u++) {
        const int q = base + u * kThreads + tid;
        v[u] = f32x4{0.f, 0.f, 0.f, 0.f};
        dst[u] = -1; left[u] = 0;
        if (q < g.nb * q_img) {
          const int img = mdiv(q, g.mQIMG), r = 4 * (q - img * q_img);
          const int f = mdiv(r, g.mNPX), pix = r - f * g.npx;
          dst[u] = f * g.DP + img * g.npx + pix;
          left[u] = g.npx - pix;                    // elements before the piece runs into the next filter row
          if (b0 + img < g.B) {
            const float* const src = dy + ((int64_t)(b0 + img) * g.F + f0) * g.npx + r;
            if (r + 3 < nfv) v[u] = *reinterpret_cast<const f32x4_a4*>(src);
            else
              for (int j = 0; j < 4; j++) if (r + j < nfv) v[u][j] = src[j];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kU; u++) {
        if (dst[u] < 0) continue;
#pragma unroll
        for (int j = 0; j < 4; j++)   // past the row's last pixel: first pixel of the next row
          dyL[dst[u] + j + (j >= left[u] ? g.DP - g.npx : 0)] = v[u][j];
      }
    }
    if (g.KW > g.K)   // the k that pad the last step
      for (int e = tid; e < kBM * (g.KW - g.K); e += kThreads) {
        const int f = e / (g.KW - g.K);
        dyL[f * g.DP + g.K + (e - f * (g.KW - g.K))] = 0.f;
      }
    // ---- x planes with their halo: cell (image, channel, padded row, padded column)
    for (int base = 0; base < g.nb * kCT * g.PP; base += kU * kThreads) {
      float v[kU];
      int dst[kU];
#pragma unroll
      for (int u = 0; u < kU; u++) {
        const int e = base + u * kThreads + tid;
        v[u] = 0.f; dst[u] = -1;
        if (e < g.nb * kCT * g.PP) {
          const int ic = mdiv(e, g.mPP), q = e - ic * g.PP;
          const int py = mdiv(q, g.mPW), px = q - py * g.PW;
          const int img = ic >> 4, c = ic & 15;
          const int iy = py - g.pad, ix = px - g.pad;
          dst[u] = ic * g.XP + py * kRowPitch + px;
          if (b0 + img < g.B && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
            v[u] = x[((int64_t)(b0 + img) * g.C + c0 + c) * g.HW + iy * g.W + ix];
        }
      }
#pragma unroll
      for (int u = 0; u < kU; u++)
        if (dst[u] >= 0) xL[dst[u]] = v[u];
    }
    __syncthreads();
    // ---- MFMA over the group's k: A = dy (filter x k), B = x (k x (channel, tap)).  The
    // operands of step s + 1 and the position of step s + 2 are fetched before the MFMAs of
    // step s: a position leads to nine B reads, two LDS latencies that would otherwise sit
    // between the steps of a wavefront that has its SIMD to itself.
    // this wavefront's half of the group's steps: [kb, ke)
    const int nsteps = g.KW >> 2, half = (nsteps + 1) >> 1;
    const int kb = 4 * (khalf ? half : 0), ke = 4 * (khalf ? nsteps : half);
    const float* const arow = dyL + (16 * mt + li) * g.DP + lk;
    const int* const prow = ptab + lk;
    if (kb < ke) {
      const int klast = ke - 4;
      // two operand sets, used in turn: while one feeds the MFMAs the other is being read.
      // (The fences keep the reads of a set in front of the MFMAs they are meant to run under.)
      float a0 = arow[kb], a1;
      float b0v[9], b1v[9];
      // The k that pad the last step (K..KW) carry dy = 0 and table position 0, so their B operand is
      // real x data; an Inf there would put 0 * Inf = NaN into the sum where the reference has Inf or a
      // number.  Those lanes' B registers are cleared instead, in the one step that has them.
      const int kpad = g.KW > g.K ? g.KW - 4 : -1;
      const bool lane_pad = g.KW - 4 + lk >= g.K;
      auto clear_pad = [&](int ks, float (&bv)[9]) {
        if (ks == kpad && lane_pad) {
#pragma unroll
          for (int t = 0; t < 9; t++) bv[t] = 0.f;
        }
      };
      {
        const float* const xb = xL + xlane + prow[kb];
#pragma unroll
        for (int t = 0; t < 9; t++) b0v[t] = xb[(t / 3) * kRowPitch + t % 3];
        clear_pad(kb, b0v);
      }
      int pn = prow[min(kb + 4, klast)];
      for (int k0 = kb; k0 < ke; k0 += 8) {
        {
          a1 = arow[min(k0 + 4, klast)];
          const float* const xb = xL + xlane + pn;
#pragma unroll
          for (int t = 0; t < 9; t++) b1v[t] = xb[(t / 3) * kRowPitch + t % 3];
          clear_pad(min(k0 + 4, klast), b1v);
          pn = prow[min(k0 + 8, klast)];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 9; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0v[t], acc[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (k0 + 4 >= ke) break;
        {
          a0 = arow[min(k0 + 8, klast)];
          const float* const xb = xL + xlane + pn;
#pragma unroll
          for (int t = 0; t < 9; t++) b0v[t] = xb[(t / 3) * kRowPitch + t % 3];
          clear_pad(min(k0 + 8, klast), b0v);
          pn = prow[min(k0 + 12, klast)];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 9; t++) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b1v[t], acc[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();   // every wavefront is done with the planes before the next group lands
  }

  // ---- the second half's partial tile onto the first's, through LDS (the last barrier of the
  // loop has every wavefront past its reads of dyL): [tile row][t][lane] as 128-bit values
  f32x4* const red = reinterpret_cast<f32x4*>(dyL) + (mt * 9) * 64 + lane;
  if (khalf) {
#pragma unroll
    for (int t = 0; t < 9; t++) red[t * 64] = acc[t];
  }
  __syncthreads();
  if (khalf) return;
#pragma unroll
  for (int t = 0; t < 9; t++) acc[t] = acc[t] + red[t * 64];
  // ---- register v of acc[t] is filter f0 + 16 mt + 4 lk + v, channel c0 + li, tap t: nine
  // consecutive floats of dW per lane and filter
  float* const o = out + (int64_t)split * slab;
#pragma unroll
  for (int v = 0; v < 4; v++) {
    const int f = f0 + 16 * mt + 4 * lk + v;
    if (f >= g.F) continue;
    float* const row = o + (int64_t)f * g.CKK + (c0 + li) * 9;
#pragma unroll
    for (int t = 0; t < 9; t++) row[t] = acc[t][v];
  }
}

struct WgPlan {
  WgGeom g;
  int splits;
  size_t lds;
};

bool wgrad_small_plan(const gh_ctx* ctx, const gh_cmd& c, WgPlan* out) {
  if (gh_dtype_of(c.flags) != GH_F32) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4];
  const int64_t pad = c.dim[7];
  if (c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 || c.dim[12] != 1 ||
      c.dim[8] != pad || pad < 0 || pad > 1)
    return false;
  if (B < 1 || B > (1 << 20) || F < 16 || F > (1 << 16) || C < 16 || C % 16 != 0 || C > 4096 || H < 3 || W < 3 ||
      H > 16 || W > 16)
    return false;
  if (getenv("GORGONIA_HIP_WGRAD_NO_SMALL")) return false;   // tuning switch: the general kernel only
  WgGeom g{};
  g.B = (int)B; g.C = (int)C; g.H = (int)H; g.W = (int)W; g.F = (int)F; g.pad = (int)pad;
  g.oh = g.H + 2 * g.pad - 2; g.ow = g.W + 2 * g.pad - 2;
  if (g.oh <= 0 || g.ow <= 0 || g.oh * g.ow < 4) return false;   // a 128-bit piece of dy spans at most two rows
  g.npx = g.oh * g.ow;
  g.PW = g.W + 2 * g.pad; g.PH = g.H + 2 * g.pad; g.PP = g.PH * g.PW;
  g.XP = g.PH * kRowPitch;
  while (g.XP % 32 != 4) g.XP++;
  // images staged at a time: about 208 output pixels, fewer where their padded planes (tiny images
  // have more halo than pixels) would not fit LDS beside the dy rows
  constexpr size_t kLdsLimit = 150 * 1024;
  g.nb = g.npx >= 208 ? 1 : 208 / g.npx;
  if (g.nb > g.B) g.nb = g.B;
  for (;; g.nb--) {
    g.K = g.nb * g.npx; g.KW = (g.K + 3) & ~3;
    g.DP = g.KW + ((4 - g.KW % 64) + 64) % 64;
    if (g.nb == 1 || ((size_t)kBM * g.DP + (size_t)g.nb * kCT * g.XP + g.KW) * 4 <= kLdsLimit) break;
  }
  g.HW = g.H * g.W; g.CKK = g.C * 9;
  g.ngroups = (g.B + g.nb - 1) / g.nb;
  const int64_t tiles = (C / kCT) * ((F + kBM - 1) / kBM);
  // slabs: enough workgroups for two per compute unit, each with at least one image group
  int64_t splits = (2 * (int64_t)ctx->cu_count + tiles - 1) / tiles;
  if (splits > g.ngroups) splits = g.ngroups;
  if (splits < 1) splits = 1;
  g.gps = (int)((g.ngroups + splits - 1) / splits);
  splits = (g.ngroups + g.gps - 1) / g.gps;
  g.mNPX = magic_of(g.npx); g.mOW = magic_of(g.ow); g.mPP = magic_of(g.PP); g.mPW = magic_of(g.PW);
  g.mQIMG = magic_of(kBM * g.npx / 4);
  out->g = g;
  out->splits = (int)splits;
  out->lds = ((size_t)kBM * g.DP + (size_t)g.nb * kCT * g.XP + g.KW) * 4;
  out->lds = std::max<size_t>(out->lds, (size_t)4 * 9 * 64 * 16);   // the two halves' partial tiles meet in it
  return out->lds <= kLdsLimit;
}

}  // namespace

// Whether the kernel takes the command: a function of its shape alone.
bool gh_conv_wgrad_small_takes(const gh_cmd& c) {
  gh_ctx probe;   // only its compute-unit count is read, for the slab count
  WgPlan p;
  return wgrad_small_plan(&probe, c, &p);
}

// Returns -1 when the shape is not one this kernel takes (or its slabs do not fit the
// workspace); otherwise the partial sums are in the workspace as *splits slabs of F x C*9
// (or, with *splits == 1, dW is complete).
int gh_try_launch_conv_wgrad_small(gh_ctx* ctx, const gh_cmd& c, int* splits) {
  WgPlan p;
  if (!wgrad_small_plan(ctx, c, &p)) return -1;
  const int64_t slab = (int64_t)p.g.F * p.g.CKK;
  if (p.splits > 1 && slab * 4 * p.splits > ctx->workspace_bytes) {
    // fewer, longer runs of images: as many slabs as the workspace holds
    if (int rc = gh_ws_short(ctx, slab * 4 * p.splits)) return rc;
    const int64_t fit = std::max<int64_t>(1, ctx->workspace_bytes / (slab * 4));
    p.g.gps = (int)((p.g.ngroups + fit - 1) / fit);
    p.splits = (p.g.ngroups + p.g.gps - 1) / p.g.gps;
  }
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    attr_rc = hipFuncSetAttribute((const void*)k_conv3x3_wgrad_small, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024);
  });
  if (attr_rc != hipSuccess) return gh_check_hip(ctx, attr_rc, "hipFuncSetAttribute(conv3x3 wgrad small)");
  float* const dst = p.splits > 1 ? (float*)ctx->workspace : (float*)(uintptr_t)c.ptr[2];
  const dim3 grid((unsigned)p.splits, (unsigned)(p.g.C / kCT), (unsigned)((p.g.F + kBM - 1) / kBM));
  hipLaunchKernelGGL(k_conv3x3_wgrad_small, grid, dim3(kThreads), p.lds, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1], dst, p.g, slab);
  *splits = p.splits;
  return gh_check_hip(ctx, hipGetLastError(), "conv3x3 wgrad small launch");
}
