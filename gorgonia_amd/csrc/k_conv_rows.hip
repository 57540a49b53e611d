// Conv2d 3x3 / stride 1 over small images (up to 16 x 16) with 32 or 64 channels, float32, on the
// 16x16x4 MFMA with the output pixels on the matrix rows.
//
// Replaces cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117) for the layers where the
// whole problem is a few microseconds of matrix-core time.  One workgroup of eight wavefronts owns
// 16 or 32 filters and IPB whole images and keeps everything in LDS: the filters already in MFMA
// operand order (one ds_read at lane + constant per step), the images as planes with a zero halo
// (a pixel operand is one ds_read at pixel base + constant).  K = C * 9 runs in the reference's
// (c, kr, kc) order, four channels (one per MFMA k-lane group) and one tap per step
// (op_nn.go:418-437); results go straight into NCHW.
//
//   * The MFMA's A operand is the pixels and its B operand the filters, so a lane's four accumulator
//     registers are four consecutive N entries of one filter.  The N axis enumerates the 2x2 windows
//     of a stride-2 pooling in order, four positions each (and after them, when nothing is pooled,
//     the pixels of an odd last row and column): a fused max-pool is a scan over a lane's own four
//     registers in the pooling kernel's order (op_nn.go:860-907), and the epilogue needs no LDS.
//   * A regular 16-pixel tile is summed by one wavefront over all of K, one accumulator chain per
//     result.  Pixel tiles that do not divide over the wavefronts are "leftover" tiles: each is cut
//     eight ways along K, a wavefront sums its slice, and the eight partial tiles are added through
//     LDS in wavefront order.  Which tiles are leftover depends on the shape of the command alone,
//     and the N order of the window part is the same with and without pooling, so a pooled command
//     stores the bits the plain command followed by the pooling kernel stores.
//   * Every wavefront does the same number of MFMAs; the leftover tiles run first, so the one
//     barrier their sum needs falls where all wavefronts arrive together, and the wavefronts that
//     add them do so while the others already run their regular tiles.
//   * The prologue is kept short (a wavefront's instructions are time the matrix pipe stands idle
//     for all eight): buffer loads whose descriptors' ranges stand for the bounds tests, every
//     staging address a per-lane constant plus an immediate.
#include <cstdio>
#include <cstdlib>
#include <mutex>

#include "gh_conv_common.h"
#include "gh_conv_rows1.h"
#include "gh_internal.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kMaxLoads = 8;            // image load instructions per wavefront
constexpr size_t kLdsBudget = 158 * 1024;

inline unsigned magic_of(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
// n / d with magic = magic_of(d), exact while n * d < 2^32; branch-free (magic 0 stands for d = 1)
__device__ __forceinline__ int mdiv(int n, unsigned magic) {
  const unsigned q = __umulhi((unsigned)n, magic);
  return (int)(q | ((unsigned)n & (0u - (unsigned)(magic == 0))));
}

struct RowsGeom {
  int B, C, H, W, F, pad, oh, ow, ph, pw, Wp;
  int HW, K;
  int IPB;            // images per workgroup
  int PT;             // pixel tiles (16 N entries each) per workgroup
  int PTR;            // regular pixel tiles; the rest are leftover
  int LU, RC;         // leftover units (pixel tile x filter tile); units summed per round through LDS
  int CH, ppl_shift;  // 128-bit chunks per plane; planes per load instruction = 1 << ppl_shift
  int NLD;            // image load instructions per wavefront
  int nplanes;        // IPB * C
  int outplane;       // floats per output plane
  int QP, PP;         // LDS pitch of a channel quad and of a plane (floats, multiples of 4)
  int offW, offP, offTabP, offTabO, offRed;   // LDS offsets in floats
  int nwin, wpart;    // windows per image; N entries of the window part
  int per, er;        // other pixels per image (not pooled), of which in the last row
  unsigned mW, mNWIN, mPW, mPER;
  // GH_FLAG_CONV_PRE: the input is computed in LDS from single-channel images of 2H x 2W (3x3 convolution with
  // C filters and padding 1, Rectify, 2x2 max-pool) instead of being loaded
  int preRW, preRP, preZP;   // padded row pitch, floats per padded image, zero floats in front
  int preOff, preFloats;     // LDS offset and size of the padded images, floats
  int preTab;                // LDS offset of the window tables: [4 prePT] patch offsets, [4 prePT] plane offsets
  // GH_FLAG_CONV_KEEP (the kernel then runs its unpooled form): y gets the pooled result of the window part as
  // well, the convolution's own values go to `keep`
  int keep, offTabO2;        // flag; LDS offset of [4 PT] pooled result offsets per window (-1: none)
  int poolplane;             // floats per pooled plane
  int preHW, preNL, prePT;   // pixels of a single-channel image; loads per thread; 16-pixel tiles of its convolution
  unsigned mHW, mPreHW, mPreW;
};

__device__ __forceinline__ f32x4 bload4(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ float bload1(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}

// The epilogue of one value with a lane's own BatchNorm constants (a lane stores results of one filter):
// k = {a, b, gamma, beta} rounded as BN_INFER rounds them, an absent gamma 1 and an absent beta -0.
template <bool BN, int ACT>
__device__ __forceinline__ float tail_reg(float v, const float (&k)[4], float alpha) {
  if constexpr (BN) {
    v = v * k[0];
    v = v + k[1];
    v = k[2] * v;
    v = v + k[3];
  }
  return act_apply(v, ACT, alpha);
}

// NQ channel quads; A regular pixel tiles per wavefront; TFB filter tiles per workgroup; WPT / QPT: padded
// row and quad pitch as compile-time constants (0: taken from g, then three row pointers per tile advance
// quad by quad); NLDT: image load instructions per wavefront as a constant (0: g.NLD, at most kMaxLoads).
// PRE: x holds single-channel images and w0 the C 3x3 filters that make this convolution's input from them.
// Wavefront w: filter tile w % TFB, regular pixel tiles [(w / TFB) * A, +A).
template <int NQ, int A, int TFB, bool POOL, int WPT, int QPT, int NLDT, bool PRE>
__global__ __launch_bounds__(kThreads) void k_conv3x3_rows(const float* __restrict__ x, const float* __restrict__ w,
                                                           float* __restrict__ y, RowsGeom g, ConvTail tail,
                                                           const float* __restrict__ w0, float* __restrict__ keep) {
  static_assert((TFB * NQ) % kWaves == 0 && NQ % kWaves == 0, "quads divide over the wavefronts");
  constexpr int NFP = TFB * NQ / kWaves;      // filter (tile, quad) pairs staged per wavefront
  constexpr int QW = NQ / kWaves;             // quads of a leftover unit per wavefront
  constexpr bool FIXED = WPT != 0;
  extern __shared__ float lds[];
  float* const Wl = lds + g.offW;             // [TFB][NQ][9][64]: (filter tile, quad, tap) -> lanes in (lk, li) order
  float* const Ps = lds + g.offP;             // image planes with a zero halo
  int* const tabP = reinterpret_cast<int*>(lds + g.offTabP);   // [16 PT] pixel offset of N entry n
  int* const tabO = reinterpret_cast<int*>(lds + g.offTabO);   // pooled: [4 PT] per window; else [16 PT] per pixel
  float* const Red = lds + g.offRed;          // [RC][8][256]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lk = lane >> 4;
  const int m0 = blockIdx.y * 16 * TFB, b0 = blockIdx.x * g.IPB;
  const int nimg = min(g.IPB, g.B - b0);
  const int PP = g.PP;
  const int QPs = FIXED ? QPT : g.QP, Wps = FIXED ? WPT : g.Wp;

  // ---- global loads, all issued before anything waits.  Buffer loads: filter rows past F and planes of
  // images past B lie beyond the descriptors' ranges and read as zero.
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)w, 0, g.F * g.K * 4, 0x00020000);
  const __amdgpu_buffer_rsrc_t rx =
      PRE ? __builtin_amdgcn_make_buffer_rsrc((void*)(x + (int64_t)b0 * g.preHW), 0, nimg * g.preHW * 4, 0x00020000)
          : __builtin_amdgcn_make_buffer_rsrc((void*)(x + (int64_t)b0 * g.C * g.HW), 0, nimg * g.C * g.HW * 4, 0x00020000);
  float wf[NFP][9];
  {
    const int voff = (li * g.K + lk * 9) * 4;
#pragma unroll
    for (int i = 0; i < NFP; i++) {
      const int pi = wave * NFP + i, ft = pi / NQ, q = pi % NQ;
      const int soff = ((m0 + ft * 16) * g.K + 36 * q) * 4;
      const f32x4 a = bload4(rw, voff, soff), b = bload4(rw, voff, soff + 16);
      wf[i][0] = a[0]; wf[i][1] = a[1]; wf[i][2] = a[2]; wf[i][3] = a[3];
      wf[i][4] = b[0]; wf[i][5] = b[1]; wf[i][6] = b[2]; wf[i][7] = b[3];
      wf[i][8] = bload1(rw, voff, soff + 32);
    }
  }
  // image: lane = chunk * planes-per-load + plane in the group; chunk c covers floats [min(4c, HW-4), +4)
  constexpr int NLDMAX = PRE ? 1 : NLDT ? NLDT : kMaxLoads;
  f32x4 xv[NLDMAX];
  const int pl = lane & ((1 << g.ppl_shift) - 1), ch = lane >> g.ppl_shift;
  const bool lane_loads = ch < g.CH;
  const int e0 = min(4 * ch, g.HW - 4);
  // PRE: the single-channel images instead, element tid + 512 i per thread, and the first convolution's
  // filters as this lane's operand of channel tile ct (channels ct * 16 + li)
  constexpr int CT = NQ / 4;
  float rawv[PRE ? kMaxLoads : 1];
  float w0b[PRE ? CT : 1][3];
  if constexpr (PRE) {
#pragma unroll
    for (int i = 0; i < kMaxLoads; i++)
      if (i < g.preNL) rawv[i] = bload1(rx, (tid + kThreads * i) * 4, 0);
    const __amdgpu_buffer_rsrc_t rw0 = __builtin_amdgcn_make_buffer_rsrc((void*)w0, 0, g.C * 36, 0x00020000);
#pragma unroll
    for (int ct = 0; ct < CT; ct++) rows1::filter_operand(rw0, ct * 16 + li, lk, w0b[ct]);
  } else {
    const int voff = lane_loads ? (pl * g.HW + e0) * 4 : 0x7ffffff0;
    const int sstep = (kWaves << g.ppl_shift) * g.HW * 4;
    int soff = (wave << g.ppl_shift) * g.HW * 4;
#pragma unroll
    for (int i = 0; i < NLDMAX; i++, soff += sstep)
      if (NLDT || i < g.NLD) xv[i] = bload4(rx, voff, soff);
  }
  // a lane stores results of filter li of a filter tile: its BatchNorm constants, per filter tile
  float bn[TFB][4];
  if (tail.mean) {
#pragma unroll
    for (int t = 0; t < TFB; t++) {
      const int f = min(m0 + t * 16 + li, g.F - 1);
      const float a = 1.0f / sqrtf(tail.var[f] + tail.eps);
      bn[t][0] = a;
      bn[t][1] = -tail.mean[f] * a;
      bn[t][2] = tail.gamma ? tail.gamma[f] : 1.0f;
      bn[t][3] = tail.beta ? tail.beta[f] : -0.0f;
    }
  }
  // ---- while they fly: zero the planes, the tables of pixel and result offsets
  {
    f32x4* p4 = reinterpret_cast<f32x4*>(Ps);
    const int n4 = g.IPB * NQ * QPs / 4;
    for (int i = tid; i < n4; i += kThreads) p4[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (PRE) {
      f32x4* r4 = reinterpret_cast<f32x4*>(lds + g.preOff);
      for (int i = tid; i < g.preFloats / 4; i += kThreads) r4[i] = f32x4{0.f, 0.f, 0.f, 0.f};
      // per pooling window of the first convolution (= input pixel of this one): where its 4x4 patch starts in
      // the padded single-channel image, and where its result goes in the planes; windows past the workgroup's
      // images read the zeros at offset 0 and store nothing
      int* const tabA = reinterpret_cast<int*>(lds + g.preTab);
      int* const tabD = tabA + 4 * g.prePT;
      for (int gw = tid; gw < 4 * g.prePT; gw += kThreads) {
        const int im = mdiv(gw, g.mHW), wi = gw - im * g.HW;
        const int py = mdiv(wi, g.mW), px = wi - py * g.W;
        const bool ok = gw < g.IPB * g.HW;
        tabA[gw] = ok ? g.preZP + im * g.preRP + 2 * py * g.preRW + 2 * px : 0;
        tabD[gw] = ok ? im * NQ * QPs + (py + g.pad) * Wps + px + g.pad : -1;
      }
    }
  }
  for (int n = tid; n < 16 * g.PT; n += kThreads) {
    // window part: IPB * nwin windows in order, four positions each; then (not pooled) the other pixels
    int img, oy, ox, wi = 0;
    bool valid = true;
    if (POOL || n < g.wpart) {
      const int gw = n >> 2, pos = n & 3;
      img = mdiv(gw, g.mNWIN);
      wi = gw - img * g.nwin;
      const int py = mdiv(wi, g.mPW), px = wi - py * g.pw;
      oy = 2 * py + (pos >> 1); ox = 2 * px + (pos & 1);
    } else {
      const int k = n - g.wpart;
      img = g.per ? mdiv(k, g.mPER) : g.IPB;
      const int r = k - img * g.per;
      if (r < g.er) { oy = g.oh - 1; ox = r; } else { oy = r - g.er; ox = g.ow - 1; }
    }
    if (img >= g.IPB) { valid = false; img = 0; oy = 0; ox = 0; }
    if (img >= nimg) valid = false;
    tabP[n] = img * NQ * QPs + oy * Wps + ox;
    if (!POOL) tabO[n] = valid ? (img * g.F) * g.outplane + oy * g.ow + ox : -1;
    else if ((n & 3) == 0) tabO[n >> 2] = valid ? (img * g.F) * g.outplane + wi : -1;
    if constexpr (!POOL) {
      if (g.keep && (n & 3) == 0)
        reinterpret_cast<int*>(lds + g.offTabO2)[n >> 2] = (valid && n < g.wpart) ? (img * g.F) * g.poolplane + wi : -1;
    }
  }
  __syncthreads();
  // ---- stage: filters (lane order is the MFMA operand order), image interiors
  auto stage_filters = [&]() {
    float* d = Wl + wave * NFP * 9 * 64 + lane;
#pragma unroll
    for (int i = 0; i < NFP; i++)
#pragma unroll
      for (int t = 0; t < 9; t++) d[(i * 9 + t) * 64] = wf[i][t];
  };
  if constexpr (!PRE) stage_filters();
  if constexpr (PRE) {
    // the single-channel images into their zeroed padded frames
    float* const Raw = lds + g.preOff;
#pragma unroll
    for (int i = 0; i < kMaxLoads; i++) {
      const int e = tid + kThreads * i;
      if (i < g.preNL && e < g.IPB * g.preHW) {
        const int im = mdiv(e, g.mPreHW), k = e - im * g.preHW;
        const int r = mdiv(k, g.mPreW), c = k - r * (2 * g.W);
        Raw[g.preZP + im * g.preRP + (r + 1) * g.preRW + c + 1] = rawv[i];
      }
    }
  } else if (lane_loads) {
    // plane p = ((wave + 8 i) << ppl_shift) + pl sits at (p >> 2) * QP + (p & 3) * PP
    const int pw0 = (wave << g.ppl_shift) + pl;
    const int r0 = mdiv(e0, g.mW), c0 = e0 - r0 * g.W;
    float* d[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      int r = r0, c = c0 + e;
      if (c >= g.W) { c -= g.W; r++; }
      if (c >= g.W) { c -= g.W; r++; }
      d[e] = Ps + (pw0 >> 2) * QPs + (pw0 & 3) * PP + (r + g.pad) * Wps + c + g.pad;
    }
    const int istep = ((kWaves << g.ppl_shift) >> 2) * QPs;   // eight groups further: whole quads
#pragma unroll
    for (int i = 0; i < NLDMAX; i++) {
      if ((NLDT || i < g.NLD) && ((wave + kWaves * i) << g.ppl_shift) < g.nplanes) {
#pragma unroll
        for (int e = 0; e < 4; e++) d[e][i * istep] = xv[i][e];
      }
    }
  }
  __syncthreads();
  if constexpr (PRE) {
    // ---- the first convolution, Rectify and the 2x2 pool (gh_conv_rows1.h), straight into the planes: a wavefront
    // takes 16-pixel tiles of the single-channel images in turn and walks the channel tiles with the pixel operand;
    // a lane's four accumulator registers are the pooling window that becomes one input pixel of a channel
    const float* const Raw = lds + g.preOff;
    const rows1::LaneTaps L = rows1::lane_taps(lk, g.preRW);
    int coff[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) coff[ct] = ((ct * 16 + li) >> 2) * QPs + ((ct * 16 + li) & 3) * PP;
    const int* const tabA = reinterpret_cast<const int*>(lds + g.preTab);
    const int* const tabD = tabA + 4 * g.prePT;
    const int posoff = ((li & 3) >> 1) * g.preRW + (li & 1);   // the lane's position in its window, operand side
    for (int pt = wave; pt < g.prePT; pt += kWaves) {
      float a[3];
      rows1::pixel_operand(Raw, tabA[pt * 4 + (li >> 2)] + posoff, L, a);
      const int od = tabD[pt * 4 + lk];
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
        f32x4 v = rows1::tile(a, w0b[ct]);
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = act_apply(v[r], 1, 0.0f);
        const float best = rows1::pool_window(v);
        if (od >= 0) Ps[od + coff[ct]] = best;
      }
    }
    // this convolution's filters have had the first one's time to arrive
    stage_filters();
    __syncthreads();
  }

  const int ft = wave % TFB, pg = wave / TFB;
  const int lkoff = lk * PP;
  // (with `keep` the unpooled values go there and y takes the pooled ones)
  float* const ybase = (!POOL && g.keep ? keep : y) + (int64_t)b0 * g.F * g.outplane;
  float* const pbase = y + (int64_t)b0 * g.F * g.poolplane;
  const int* const tabO2 = reinterpret_cast<const int*>(lds + g.offTabO2);
  const int outplane = g.outplane;
  const float alpha = tail.alpha;
  // the epilogue of one tile: four N entries of filter `fcol` in v
  // (o1: the window's result offset when pooling, read from the table by the caller)
  auto finish = [&](auto bn_c, auto act_c, f32x4 v, int pt, int o1, int fcol, const float (&k)[4]) {
    constexpr bool BN = decltype(bn_c)::value;
    constexpr int ACT = decltype(act_c)::value;
    const bool ok = fcol < g.F;
    if constexpr (!POOL) {
      if (g.keep) {
        // the convolution's own values (after BatchNorm) as the plain command stores them, then the activation
        // and the pooling scan of the window the lane holds
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = tail_reg<BN, 0>(v[r], k, alpha);
        const i32x4 o = *reinterpret_cast<const i32x4*>(tabO + 16 * pt + 4 * lk);
#pragma unroll
        for (int r = 0; r < 4; r++)
          if (ok && o[r] >= 0) ybase[o[r] + fcol * outplane] = v[r];
        const int o2 = tabO2[4 * pt + lk];
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = act_apply(v[r], ACT, alpha);
        float best = -3.402823466e+38f;
#pragma unroll
        for (int r = 0; r < 4; r++) if (v[r] > best) best = v[r];
        if (ok && o2 >= 0) pbase[o2 + fcol * g.poolplane] = best;
        return;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) v[r] = tail_reg<BN, ACT>(v[r], k, alpha);
    if constexpr (POOL) {
      float best = -3.402823466e+38f;
#pragma unroll
      for (int r = 0; r < 4; r++) if (v[r] > best) best = v[r];   // window positions in scan order
      if (ok && o1 >= 0) ybase[o1 + fcol * outplane] = best;
    } else {
      const i32x4 o = *reinterpret_cast<const i32x4*>(tabO + 16 * pt + 4 * lk);
#pragma unroll
      for (int r = 0; r < 4; r++)
        if (ok && o[r] >= 0) ybase[o[r] + fcol * outplane] = v[r];
    }
  };

  // ---- leftover pixel tiles: this wavefront's quads [wave * QW, +QW) of each, for every filter tile of the
  // workgroup (a unit = pixel tile x filter tile); RC units per round: partial tiles to LDS, barrier,
  // wavefront j adds unit j's eight in wavefront order
  if (g.LU > 0) {
    const float* const lf = Wl + wave * QW * 9 * 64 + lane;
    const int tiles_per_round = g.RC / TFB;   // RC is a multiple of TFB
    const int ntiles = g.LU / TFB;
    for (int t0 = 0; t0 < ntiles; t0 += tiles_per_round) {
      const int nt = min(tiles_per_round, ntiles - t0);
      if (t0 > 0) __syncthreads();   // the last round's sums are done with the slots
      for (int j = 0; j < nt; j++) {
        const float* const lp = Ps + tabP[(g.PTR + t0 + j) * 16 + li] + lkoff + wave * QW * QPs;
        f32x4 acc[TFB];
#pragma unroll
        for (int fi = 0; fi < TFB; fi++) acc[fi] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int qq = 0; qq < QW; qq++)
#pragma unroll
          for (int tap = 0; tap < 9; tap++) {
            const float pv = lp[qq * QPs + (tap / 3) * Wps + (tap % 3)];
#pragma unroll
            for (int fi = 0; fi < TFB; fi++)
              acc[fi] = __builtin_amdgcn_mfma_f32_16x16x4f32(pv, lf[((fi * NQ + qq) * 9 + tap) * 64], acc[fi], 0, 0, 0);
          }
#pragma unroll
        for (int fi = 0; fi < TFB; fi++)
          *reinterpret_cast<f32x4*>(Red + ((j * TFB + fi) * kWaves + wave) * 256 + lane * 4) = acc[fi];
      }
      __syncthreads();
      if (wave < nt * TFB) {
        const int t = t0 + wave / TFB, fi = wave % TFB;
        f32x4 s = *reinterpret_cast<const f32x4*>(Red + (wave * kWaves) * 256 + lane * 4);
#pragma unroll
        for (int k = 1; k < kWaves; k++) s = s + *reinterpret_cast<const f32x4*>(Red + (wave * kWaves + k) * 256 + lane * 4);
        const int fcol = m0 + fi * 16 + li;
        const int o1 = POOL ? tabO[4 * (g.PTR + t) + lk] : 0;
        conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
          if (TFB == 1 || fi == 0) finish(bn_c, act_c, s, g.PTR + t, o1, fcol, bn[0]);
          else finish(bn_c, act_c, s, g.PTR + t, o1, fcol, bn[TFB - 1]);
        });
      }
    }
  }

  // ---- regular tiles: step = (channel quad, tap); operands of step s + 2 are fetched while step s runs
  // (three register sets), one LDS read placed after each MFMA
  if constexpr (A > 0) {
    const float* const fbase = Wl + ft * NQ * 9 * 64 + lane;
    const float* pb[A][FIXED ? 1 : 3];
    int otab[A];
#pragma unroll
    for (int t = 0; t < A; t++) {
      otab[t] = POOL ? tabO[4 * (pg * A + t) + lk] : 0;
      const float* p = Ps + tabP[(pg * A + t) * 16 + li] + lkoff;
      pb[t][0] = p;
      if constexpr (!FIXED) { pb[t][1] = p + Wps; pb[t][2] = p + 2 * Wps; }
    }
    f32x4 acc[A];
#pragma unroll
    for (int t = 0; t < A; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float fv[3], pv[3][A];
    // q_rel: quads ahead of the pointers' current quad (the generic form advances them quad by quad)
    auto fetch = [&](int set, int q, int tap, int q_rel) {
      fv[set] = fbase[(q * 9 + tap) * 64];
#pragma unroll
      for (int t = 0; t < A; t++) {
        if constexpr (FIXED) pv[set][t] = pb[t][0][q * QPT + (tap / 3) * WPT + (tap % 3)];
        else pv[set][t] = pb[t][tap / 3][q_rel * QPs + (tap % 3)];
      }
    };
    constexpr int NS = NQ * 9;
    fetch(0, 0, 0, 0);
    fetch(1, 0, 1, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NS; s++) {
      const int tap = s % 9;
      if constexpr (!FIXED) {
        // entering a quad: move the row pointers to it (the fetches below reach at most one quad ahead)
        if (tap == 0 && s > 0) {
#pragma unroll
          for (int t = 0; t < A; t++)
#pragma unroll
            for (int kr = 0; kr < 3; kr++) pb[t][kr] += QPs;
        }
      }
      if (s + 2 < NS) fetch((s + 2) % 3, (s + 2) / 9, (s + 2) % 9, (s + 2) / 9 - s / 9);
#pragma unroll
      for (int t = 0; t < A; t++)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(pv[s % 3][t], fv[s % 3], acc[t], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < A + 1; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // DS read
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    const int fcol = m0 + ft * 16 + li;
    conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
#pragma unroll
      for (int t = 0; t < A; t++) {
        if (TFB == 1 || ft == 0) finish(bn_c, act_c, acc[t], pg * A + t, otab[t], fcol, bn[0]);
        else finish(bn_c, act_c, acc[t], pg * A + t, otab[t], fcol, bn[TFB - 1]);
      }
    });
  }
}

struct RowsPlan {
  RowsGeom g;
  int NQ, A, TFB;
  size_t lds;
};

// Geometry and workgroup shape for one command.  The choice of IPB, TFB, A and of the leftover tiles of
// the window part depends on the command's shape only, not on `pool`: a pooled command and the plain one
// sum every result in the same order.  False when the kernel does not take the shape.
bool rows_plan_compute(const gh_cmd& c, bool pool, RowsPlan* out) {
  if (gh_dtype_of(c.flags) != GH_F32) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4];
  const int64_t pad = c.dim[7];
  if (c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 || c.dim[12] != 1 ||
      c.dim[8] != pad || pad < 0 || pad > 1)
    return false;
  if (B < 1 || F < 1 || (C != 32 && C != 64) || W < 4 || W > 16 || H < 1 || H > 16) return false;
  if (B > (1 << 20) || F > (1 << 16)) return false;
  if (getenv("GORGONIA_HIP_CONV_NO_ROWS")) return false;   // tuning switch: the K-split small-image kernel instead
  RowsGeom g{};
  g.B = (int)B; g.C = (int)C; g.H = (int)H; g.W = (int)W; g.F = (int)F; g.pad = (int)pad;
  g.oh = g.H + 2 * g.pad - 2; g.ow = g.W + 2 * g.pad - 2;
  if (g.oh < 2 || g.ow < 2) return false;
  g.ph = g.oh / 2; g.pw = g.ow / 2; g.Wp = g.W + 2 * g.pad;
  g.HW = g.H * g.W; g.K = g.C * 9;
  if ((int64_t)g.F * g.K * 4 >= (1ll << 31) || B * C * g.HW * 4 >= (1ll << 40)) return false;
  const int NQ = g.C / 4;
  g.nwin = g.ph * g.pw;
  g.er = (g.oh & 1) ? g.ow : 0;
  g.per = g.er + ((g.ow & 1) ? (g.oh - (g.oh & 1)) : 0);
  g.CH = (g.HW + 3) / 4;
  g.ppl_shift = 0;
  while ((2 << g.ppl_shift) * g.CH <= 64 && g.ppl_shift < 4) g.ppl_shift++;
  const int plane = (g.H + 2 * g.pad) * g.Wp;
  // plane pitch, a multiple of 4: the one with the fewest bank conflicts of a pixel fetch (16 N entries
  // x 4 channel planes) over the tiles of one image
  {
    int tp[256];
    int ntp = 0;
    for (int py = 0; py < g.ph; py++)
      for (int px = 0; px < g.pw; px++)
        for (int pos = 0; pos < 4; pos++) tp[ntp++] = (2 * py + (pos >> 1)) * g.Wp + 2 * px + (pos & 1);
    int bestPP = (plane + 3) & ~3;
    long best = -1;
    for (int PP = (plane + 3) & ~3; PP < plane + 68; PP += 4) {
      long tot = 0;
      for (int t = 0; t + 16 <= ntp; t += 16) {
        int cnt[64] = {0}, mx = 0;
        for (int k = 0; k < 4; k++)
          for (int i = 0; i < 16; i++) {
            const int b = (tp[t + i] + k * PP) & 63;
            if (++cnt[b] > mx) mx = cnt[b];
          }
        tot += mx;
      }
      if (best < 0 || tot < best) { best = tot; bestPP = PP; }
    }
    g.PP = bestPP;
    g.QP = 4 * g.PP;
  }
  // Workgroup shape: (filter tiles, images) with the smallest estimated time on 256 compute units - a
  // fixed cost per round of workgroups plus the MFMA time of the window part (microseconds)
  double best = 0;
  int bestTFB = 0, bestIPB = 0;
  for (int TFB = 1; TFB <= 2; TFB++) {
    if (TFB == 2 && F <= 16) continue;
    const int wave_groups = kWaves / TFB;
    for (int IPB = 1; IPB <= 16; IPB *= 2) {
      if (IPB > 1 && IPB / 2 >= B) break;
      const int planes = IPB * g.C;
      if (planes > (kMaxLoads * kWaves << g.ppl_shift)) break;
      const int PTw = (4 * g.nwin * IPB + 15) / 16;
      const int PTu = (4 * g.nwin * IPB + IPB * g.per + 15) / 16;
      const int A = PTw / wave_groups;
      if (A > 4) break;
      const int LUu = (PTu - A * wave_groups) * TFB;
      size_t fl = (size_t)TFB * NQ * 576 + (size_t)IPB * NQ * g.QP + 36 * (size_t)PTu + 4;
      if ((fl + (LUu ? 2048 * TFB : 0)) * 4 > kLdsBudget) break;
      const size_t lds = (fl + (size_t)LUu * 2048) * 4 > kLdsBudget ? kLdsBudget : (fl + (size_t)LUu * 2048) * 4;
      const int64_t blocks = ((F + 16 * TFB - 1) / (16 * TFB)) * ((B + IPB - 1) / IPB);
      const int coresident = lds <= 79 * 1024 ? 2 : 1;
      const int64_t rounds = (blocks + 256 * coresident - 1) / (256 * coresident);
      const double mfma_us = (double)PTw * TFB * NQ * 9 / 4 * 32.0 / 2100.0;
      // what a workgroup does before its first MFMA grows with what it stages (measured on the convnet's
      // layers: 32 filters x 1 image against 16 x 2 at 14 x 14, 16 x 4 against 32 x 2 at 7 x 7)
      const double stage_us = 2.0 + 0.035 * (TFB * NQ * 576 * 4 / 1024.0) + 0.03 * ((double)IPB * NQ * g.QP * 4 / 1024.0);
      const double est = rounds * (stage_us + coresident * mfma_us);
      double score = est;
      if (const char* e = getenv("GORGONIA_HIP_CONV_ROWS_PLAN")) {   // tuning override: "TFB,IPB"
        int ft = 0, ip = 0;
        if (sscanf(e, "%d,%d", &ft, &ip) == 2 && ft == TFB && ip == IPB) score = -1.0;
      }
      if (!bestTFB || score < best) { best = score; bestTFB = TFB; bestIPB = IPB; }
    }
  }
  if (!bestTFB) return false;
  const int TFB = bestTFB;
  const int wave_groups = kWaves / TFB;
  g.IPB = bestIPB;
  g.wpart = 4 * g.nwin * g.IPB;
  const int PTw = (g.wpart + 15) / 16;
  const int PTu = (g.wpart + g.IPB * g.per + 15) / 16;
  const int A = PTw / wave_groups;
  g.PTR = A * wave_groups;
  g.PT = pool ? PTw : PTu;
  g.LU = (g.PT - g.PTR) * TFB;
  g.nplanes = g.IPB * g.C;
  g.NLD = (g.nplanes + (kWaves << g.ppl_shift) - 1) / (kWaves << g.ppl_shift);
  g.outplane = pool ? g.ph * g.pw : g.oh * g.ow;
  int off = 0;
  g.offW = off; off += TFB * NQ * 576;
  g.offP = off; off += g.IPB * NQ * g.QP;
  g.offTabP = off; off += 16 * g.PT;
  g.offTabO = off; off += pool ? 4 * g.PT : 16 * g.PT;
  g.offTabO2 = off; off += pool ? 0 : 4 * g.PT;   // used by GH_FLAG_CONV_KEEP; part of every plain plan, so the flag changes no plan
  g.poolplane = g.ph * g.pw;
  off = (off + 3) & ~3;
  g.offRed = off;
  // as many leftover units per round as the rest of LDS holds
  const int room = (int)((kLdsBudget / 4 - (size_t)off) / 2048);
  g.RC = g.LU < room ? g.LU : room;
  if (g.RC > kWaves) g.RC = kWaves;
  g.RC -= g.RC % TFB;   // whole pixel tiles per round
  if (g.LU > 0 && g.RC < TFB) return false;
  off += g.RC * 2048;
  g.mW = magic_of(g.W); g.mNWIN = magic_of(g.nwin); g.mPW = magic_of(g.pw); g.mPER = magic_of(g.per);
  out->g = g; out->NQ = NQ; out->A = A; out->TFB = TFB; out->lds = (size_t)off * 4;
  return true;
}

// The plan of a command, remembered per shape.
bool rows_plan(const gh_cmd& c, bool pool, RowsPlan* out) {
  return gh_plan_memo(c, pool, out, [&](RowsPlan* p) { return rows_plan_compute(c, pool, p); });
}

// The command of the single-channel convolution a GH_FLAG_CONV_PRE command stands for.
gh_cmd pre_command(const gh_cmd& c) {
  gh_cmd q{};
  q.opcode = GH_OP_CONV2D;
  q.flags = GH_FLAG_DTYPE(GH_F32) | GH_FLAG_ACT_RELU | GH_FLAG_CONV_POOL2;
  q.dim[0] = c.dim[0]; q.dim[1] = 1; q.dim[2] = 2 * c.dim[2]; q.dim[3] = 2 * c.dim[3]; q.dim[4] = c.dim[1];
  q.dim[5] = 3; q.dim[6] = 3; q.dim[7] = 1; q.dim[8] = 1;
  q.dim[9] = 1; q.dim[10] = 1; q.dim[11] = 1; q.dim[12] = 1;
  return q;
}

// Extends a plan by the padded single-channel images of GH_FLAG_CONV_PRE.  False when the fold is not offered:
// 32 channels only, the single-channel convolution must be one k_conv3x3_rows1 takes (so that it sums as it
// would on its own), a workgroup's images at most 8 loads per thread, everything within LDS.
bool rows_pre_plan(const gh_cmd& c, RowsPlan* p) {
  if (p->NQ != 8 || !gh_conv_rows1_takes(pre_command(c))) return false;
  RowsGeom& g = p->g;
  g.preHW = 4 * g.HW;
  if ((int64_t)g.IPB * g.preHW > (int64_t)kMaxLoads * kThreads) return false;
  g.preNL = (g.IPB * g.preHW + kThreads - 1) / kThreads;
  g.preRW = 2 * g.W + 2;
  g.preRP = (2 * g.H + 2) * g.preRW;
  g.preZP = (3 * g.preRW + 8 + 3) & ~3;   // a window past the images reads at its position's offset from 0
  g.preFloats = (g.preZP + g.IPB * g.preRP + 3) & ~3;
  g.preOff = (int)((p->lds / 4 + 3) & ~(size_t)3);
  g.prePT = (g.IPB * g.preHW + 15) / 16;
  g.preTab = g.preOff + g.preFloats;
  g.mHW = magic_of((unsigned)g.HW); g.mPreHW = magic_of((unsigned)g.preHW); g.mPreW = magic_of((unsigned)(2 * g.W));
  p->lds = ((size_t)g.preTab + 8 * (size_t)g.prePT) * 4;
  return p->lds <= kLdsBudget;
}

template <int NQ, int A, int TFB, bool POOL, int WPT, int QPT, int NLDT, bool PRE = false>
int launch_rows(gh_ctx* ctx, const gh_cmd& c, const RowsPlan& p) {
  // more than 64 KB of dynamic LDS has to be allowed per kernel, once
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    attr_rc = hipFuncSetAttribute((const void*)k_conv3x3_rows<NQ, A, TFB, POOL, WPT, QPT, NLDT, PRE>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  if (attr_rc != hipSuccess) return gh_check_hip(ctx, attr_rc, "hipFuncSetAttribute(conv3x3 rows)");
  const dim3 grid((unsigned)((p.g.B + p.g.IPB - 1) / p.g.IPB), (unsigned)((p.g.F + 16 * TFB - 1) / (16 * TFB)));
  hipLaunchKernelGGL((k_conv3x3_rows<NQ, A, TFB, POOL, WPT, QPT, NLDT, PRE>), grid, dim3(kThreads), p.lds, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], p.g, conv_tail(c), PRE ? (const float*)(uintptr_t)c.ptr[7] : nullptr,
                     p.g.keep ? (float*)(uintptr_t)c.ptr[7] : nullptr);
  return gh_check_hip(ctx, hipGetLastError(), "conv3x3 rows launch");
}

template <int NQ, int TFB, bool POOL, bool PRE = false>
int launch_rows_a(gh_ctx* ctx, const gh_cmd& c, const RowsPlan& p) {
  // 16 x 16 and 9 x 9 padded planes (14 x 14 and 7 x 7 images with padding 1) have their pitches compiled in
  if constexpr (NQ == 8 && TFB == 2) {
    if (p.g.Wp == 16 && p.g.QP == 1088 && p.A == 3 && p.g.NLD == 4) return launch_rows<NQ, 3, TFB, POOL, 16, 1088, 4, PRE>(ctx, c, p);
  }
  if constexpr (PRE) {
    switch (p.A) {
      case 0: return launch_rows<NQ, 0, TFB, POOL, 0, 0, 0, true>(ctx, c, p);
      case 1: return launch_rows<NQ, 1, TFB, POOL, 0, 0, 0, true>(ctx, c, p);
      case 2: return launch_rows<NQ, 2, TFB, POOL, 0, 0, 0, true>(ctx, c, p);
      case 3: return launch_rows<NQ, 3, TFB, POOL, 0, 0, 0, true>(ctx, c, p);
      default: return launch_rows<NQ, 4, TFB, POOL, 0, 0, 0, true>(ctx, c, p);
    }
  }
  if constexpr (NQ == 16 && TFB == 1) {
    if (p.g.Wp == 9 && p.g.QP == 336 && p.A == 1 && p.g.NLD == 8) return launch_rows<NQ, 1, TFB, POOL, 9, 336, 8>(ctx, c, p);
    if constexpr (!POOL) {
      if (p.g.Wp == 16 && p.g.QP == 1088 && p.A == 1 && p.g.NLD == 8) return launch_rows<NQ, 1, TFB, POOL, 16, 1088, 8>(ctx, c, p);
    }
  }
  switch (p.A) {
    case 0: return launch_rows<NQ, 0, TFB, POOL, 0, 0, 0>(ctx, c, p);
    case 1: return launch_rows<NQ, 1, TFB, POOL, 0, 0, 0>(ctx, c, p);
    case 2: return launch_rows<NQ, 2, TFB, POOL, 0, 0, 0>(ctx, c, p);
    case 3: return launch_rows<NQ, 3, TFB, POOL, 0, 0, 0>(ctx, c, p);
    default: return launch_rows<NQ, 4, TFB, POOL, 0, 0, 0>(ctx, c, p);
  }
}

int launch_rows_pre(gh_ctx* ctx, const gh_cmd& c, const RowsPlan& p, bool pool) {
  if (p.TFB == 1) return pool ? launch_rows_a<8, 1, true, true>(ctx, c, p) : launch_rows_a<8, 1, false, true>(ctx, c, p);
  return pool ? launch_rows_a<8, 2, true, true>(ctx, c, p) : launch_rows_a<8, 2, false, true>(ctx, c, p);
}

template <int NQ>
int launch_rows_q(gh_ctx* ctx, const gh_cmd& c, const RowsPlan& p, bool pool) {
  if (p.TFB == 1) return pool ? launch_rows_a<NQ, 1, true>(ctx, c, p) : launch_rows_a<NQ, 1, false>(ctx, c, p);
  return pool ? launch_rows_a<NQ, 2, true>(ctx, c, p) : launch_rows_a<NQ, 2, false>(ctx, c, p);
}

}  // namespace

// 1 when this kernel takes the convolution (without fused pooling).
bool gh_conv_rows_takes(const gh_cmd& c) {
  RowsPlan p;
  return rows_plan(c, false, &p);
}

// 1 when it also takes it with the 2x2 pooling in its epilogue.
bool gh_conv_rows_can_pool(const gh_cmd& c) {
  RowsPlan p;
  return rows_plan(c, false, &p) && rows_plan(c, true, &p);
}

// 1 when it takes it with its input computed from single-channel images (GH_FLAG_CONV_PRE), pooled or not.
bool gh_conv_rows_can_pre(const gh_cmd& c) {
  RowsPlan p;
  if (!rows_plan(c, false, &p) || !rows_pre_plan(c, &p)) return false;
  if (gh_conv_rows_can_pool(c)) {
    RowsPlan q;
    if (!rows_plan(c, true, &q) || !rows_pre_plan(c, &q)) return false;
  }
  return true;
}

// Returns -1 when the shape is not one this kernel takes.
int gh_try_launch_conv_rows(gh_ctx* ctx, const gh_cmd& c) {
  RowsPlan p;
  bool pool = c.flags & GH_FLAG_CONV_POOL2;
  // a pooled command only rides here when the plain one would too: both then sum in the same order
  if (!rows_plan(c, false, &p)) return -1;
  if (pool && (c.flags & GH_FLAG_CONV_KEEP)) {
    // the plain command's plan and kernel, which then stores the pooled windows as well
    if (!gh_conv_rows_can_pool(c) || !c.ptr[7] || (c.flags & GH_FLAG_CONV_PRE))
      return gh_fail(ctx, GH_EINVAL, "conv2d: the convolution's own result cannot be kept next to the pooled one here (see gh_conv2d_can_keep)");
    p.g.keep = 1;
    pool = false;
  }
  if (pool && !rows_plan(c, true, &p))
    return gh_fail(ctx, GH_EINVAL, "conv2d: no fused pooling for this shape (see gh_conv2d_can_pool)");
  if (c.flags & GH_FLAG_CONV_PRE) {
    if (!rows_pre_plan(c, &p) || !c.ptr[7])
      return gh_fail(ctx, GH_EINVAL, "conv2d: the single-channel convolution cannot be folded in front of this one (see gh_conv2d_can_pre)");
    return launch_rows_pre(ctx, c, p, pool);
  }
  return p.NQ == 8 ? launch_rows_q<8>(ctx, c, p, pool) : launch_rows_q<16>(ctx, c, p, pool);
}
