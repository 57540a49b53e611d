// Conv2d 3x3 / stride 1 with 64 input channels or more, float32, on the 16x16x4 MFMA:
// one workgroup = 16 or 32 filters x one TH x TW patch of one image, K split over its
// eight wavefronts.
//
// Replaces cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117) for the deep
// layers of a small batch, where output tiles alone are too few to fill the device and
// a tile's K range is long.  Same GEMM view as the other convolution kernels (M =
// filters, N = output pixels, K = C * 9 in the reference's (c, kr, kc) order,
// op_nn.go:418-437), results written straight into NCHW.
//
//   * Wavefront w sums channels [w C/8, (w+1) C/8) for the whole 16 TM x 16 TN tile,
//     four channels (one per MFMA k-lane group) and one tap per step; the eight partial
//     tiles are added through LDS in a fixed order (4..7 onto 0..3, then 0+1+2+3), so
//     results repeat bit for bit and do not depend on the patch shape or on fused pooling.
//   * A wavefront stages its own operands in its own LDS region - 36 filter columns
//     k-major and the four channel planes of the padded patch, halo cells outside the
//     image written as zero - so the main loop has no workgroup barrier (there is one in
//     front of it, behind the shared table of patch cells); the next quad's global loads are
//     in flight while the current one is multiplied.
//   * With GH_FLAG_CONV_POOL2 the patch has even extents and the N axis enumerates
//     (pooled pixel, position in the 2x2 window); the epilogue reads a window as four
//     adjacent columns (scan order and strict > of the pooling kernel, op_nn.go:860-907).
#include <cstdlib>
#include <mutex>

#include "gh_conv_common.h"
#include "gh_internal.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

inline unsigned magic_of(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
// n / d with magic = magic_of(d), exact while n * d < 2^32; branch-free (magic 0 stands for d = 1)
__device__ __forceinline__ int mdiv(int n, unsigned magic) {
  const unsigned q = __umulhi((unsigned)n, magic);
  return (int)(q | ((unsigned)n & (0u - (unsigned)(magic == 0))));
}

struct PatchGeom {
  int B, C, H, W, F, pad, oh, ow, HW, K;
  int TH, TW, tiles_x, tiles_y;   // output patch, patches per image
  int PW, PP, PL;                 // padded patch: row length TW + 2, size (TH + 2) * PW, plane pitch in LDS
  int NQ;                         // channel quads per wavefront: C / 32
  int npix;                       // TH * TW
  int pool, ph, pw, HTW;          // fused 2x2 / stride-2 max-pool: pooled extents of y, TW / 2
  int epi_off;                    // float offset in LDS of the per-filter epilogue table (past every other use)
  unsigned mTXY, mTX, mPP, mPW, mTW, mHTW, mNPIX, mNPOOL;   // magics: tiles_x*tiles_y, tiles_x, PP, PW, TW, HTW, npix, npix/4
  // the launch is one-dimensional: workgroup id -> (patch, filter tile), see the kernel
  int ntiles, ftiles, nwg;        // patches of the batch, filter tiles, their product
  int ft_major;                   // 1: an XCD owns whole filter tiles (all patches of each); 0: whole patches (all filter tiles)
};

constexpr int kWaves = 8;
constexpr int kSlotsX = 15;   // patch cells each lane stages per quad: 4 planes * PP <= 64 * kSlotsX

template <int TM, int TN>
__global__ __launch_bounds__(kWaves * 64) void k_conv3x3_patch(const float* __restrict__ x, const float* __restrict__ w,
                                                               float* __restrict__ y, PatchGeom g, ConvTail tail) {
  constexpr int NTH = kWaves * 64;
  constexpr int BM = 16 * TM;
  constexpr int BMS = TM == 1 ? 4 : 5;   // log2(BM)
  static_assert(TM == 1 || TM == 2, "filter tile of 16 or 32");
  constexpr int SA = BM;                 // k-major filter columns Aw[k][SA]
  constexpr int MP = BM + 4;             // partial sums R[slot][n][MP]: a lane's four rows are one 128-bit access
  constexpr int RW = 16 * TN * MP;       // one slot
  constexpr int QL = 64 >> BMS;          // filter 128-bit columns one load slot covers (lanes / rows)
  constexpr int NWQ = (9 + QL - 1) / QL; // slots for the nine 128-bit columns a quad has per filter row
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lk = lane >> 4;
  const int wsize = 36 * SA + 4 * g.PL;           // floats per wavefront region
  float* const Aw = lds + wave * wsize;           // [36][SA]
  float* const Pw = Aw + 36 * SA;                 // [4][PL]
  int* const tab = reinterpret_cast<int*>(lds + kWaves * wsize);   // [16 TN] cell of N entry n inside the padded patch

  // Workgroup ids are dealt round-robin over the 8 XCDs, each with its own L2.  An XCD gets one contiguous
  // run of the (patch, filter tile) pairs, ordered so that what the run shares is the larger operand:
  // patch-major where the images outweigh the filters (the workgroups of a patch and of its neighbours,
  // whose halos overlap, then meet in one L2), filter-tile-major where the filters do (a filter tile is
  // then fetched from memory by one XCD instead of by every one that holds an image).
  int wpatch, wft;
  {
    const int id = blockIdx.x, xcd = id & 7, per = g.nwg >> 3, extra = g.nwg & 7;
    const int lin = xcd * per + min(xcd, extra) + (id >> 3);
    // (a true division, once per workgroup: the multiply-shift form is exact only while id x divisor < 2^32)
    if (g.ft_major) { wft = (int)((unsigned)lin / (unsigned)g.ntiles); wpatch = lin - wft * g.ntiles; }
    else { wpatch = (int)((unsigned)lin / (unsigned)g.ftiles); wft = lin - wpatch * g.ftiles; }
  }
  const int bimg = mdiv(wpatch, g.mTXY);
  const int trem = wpatch - bimg * (g.tiles_x * g.tiles_y);
  const int tyi = mdiv(trem, g.mTX), txi = trem - tyi * g.tiles_x;
  const int oy0 = tyi * g.TH, ox0 = txi * g.TW;
  const int m0 = wft * BM;
  const int c0 = wave * (4 * g.NQ);
  float* const ftab = lds + g.epi_off;            // [4][BM] BatchNorm constants of this workgroup's filters
  if (tid < BM) conv_tail_table(tail, ftab, BM, tid, min(m0 + tid, g.F - 1));

  // ---- per-lane load slots, the same in every quad: filters (row, 128-bit column), patch cells
  const int wr = lane & (BM - 1), wq0 = lane >> BMS;
  const float* wp = w + (int64_t)min(m0 + wr, g.F - 1) * g.K + c0 * 9;
  int xoff[kSlotsX], xdst[kSlotsX];
  bool xin[kSlotsX];
#pragma unroll
  for (int u = 0; u < kSlotsX; u++) {
    const int id = min(lane + 64 * u, 4 * g.PP - 1);   // slots past the end repeat the last cell
    const int pl = mdiv(id, g.mPP), rem = id - pl * g.PP;
    const int r = mdiv(rem, g.mPW), cc = rem - r * g.PW;
    const int iy = oy0 - g.pad + r, ix = ox0 - g.pad + cc;
    xin[u] = iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
    xoff[u] = pl * g.HW + min(max(iy, 0), g.H - 1) * g.W + min(max(ix, 0), g.W - 1);
    xdst[u] = pl * g.PL + rem;
  }
  const float* xq = x + ((int64_t)bimg * g.C + c0) * g.HW;
  f32x4 wv[NWQ];
  float xv[kSlotsX];
  auto load_quad = [&]() {
#pragma unroll
    for (int u = 0; u < NWQ; u++) wv[u] = *reinterpret_cast<const f32x4_a4*>(wp + 4 * min(wq0 + u * QL, 8));
#pragma unroll
    for (int u = 0; u < kSlotsX; u++) xv[u] = xq[xoff[u]];
    wp += 36;
    xq += 4 * g.HW;
  };
  auto store_quad = [&]() {
#pragma unroll
    for (int u = 0; u < NWQ; u++) {
      const int q = min(wq0 + u * QL, 8);
#pragma unroll
      for (int e = 0; e < 4; e++) Aw[(4 * q + e) * SA + wr] = wv[u][e];
    }
#pragma unroll
    for (int u = 0; u < kSlotsX; u++) Pw[xdst[u]] = xin[u] ? xv[u] : 0.f;
  };
  load_quad();

  // ---- table of patch cells, one entry per thread, then the only barrier in front of the MFMAs
  // (reached with the first quad's loads in flight); operand bases
  static_assert(NTH >= 16 * TN, "one table entry per thread");
  if (tid < 16 * TN) {
    const int n = tid;
    const int nn = n < g.npix ? n : 0;   // idle column: any valid cell
    int ty, tx;
    if (g.pool) {
      const int q = nn >> 2, wpos = nn & 3;
      const int py = mdiv(q, g.mHTW), px = q - py * g.HTW;
      ty = 2 * py + (wpos >> 1);
      tx = 2 * px + (wpos & 1);
    } else {
      ty = mdiv(nn, g.mTW);
      tx = nn - ty * g.TW;
    }
    tab[n] = ty * g.PW + tx;
  }
  __syncthreads();
  int pb[TN][3];   // one base per kernel row, so the column tap is an immediate offset
#pragma unroll
  for (int t = 0; t < TN; t++) {
    const int p = tab[t * 16 + li] + lk * g.PL;
#pragma unroll
    for (int kr = 0; kr < 3; kr++) pb[t][kr] = p + kr * g.PW;
  }
  const float* const abase = Aw + lk * 9 * SA + li;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int t = 0; t < TN; t++) acc[a][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- MFMA: step = (channel quad, tap); lane group lk takes channel 4 quad + lk.  Operands of
  // tap s + 2 are fetched while tap s runs (three register sets), one LDS read after each MFMA.
  float af[3][TM], bf[3][TN];
  auto fetch = [&](int set, int tap) {
    const int kr = tap / 3, kc = tap % 3;
#pragma unroll
    for (int a = 0; a < TM; a++) af[set][a] = abase[tap * SA + a * 16];
#pragma unroll
    for (int t = 0; t < TN; t++) bf[set][t] = Pw[pb[t][kr] + kc];
  };
  for (int qd = 0; qd < g.NQ; qd++) {
    store_quad();                       // this quad: registers to the wavefront's LDS region
    if (qd + 1 < g.NQ) load_quad();     // the next one is in flight during the MFMAs
    fetch(0, 0);
    fetch(1, 1);
#pragma unroll
    for (int tap = 0; tap < 9; tap++) {
      if (tap + 2 < 9) fetch((tap + 2) % 3, tap + 2);
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int t = 0; t < TN; t++)
          acc[a][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[tap % 3][a], bf[tap % 3][t], acc[a][t], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < TM * TN; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // DS read
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  __syncthreads();   // every wavefront is done with its operand region
  // ---- partial tiles to LDS, R[slot][n][MP]: 4..7 write, 0..3 add those to their own and write
  float* const R = lds;
  float* const rt = R + (wave & 3) * RW + li * MP + 4 * lk;
  auto put = [&]() {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int t = 0; t < TN; t++) *reinterpret_cast<f32x4*>(rt + t * 16 * MP + a * 16) = acc[a][t];
  };
  if (wave >= 4) put();
  __syncthreads();
  if (wave < 4) {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int t = 0; t < TN; t++) acc[a][t] = acc[a][t] + *reinterpret_cast<const f32x4*>(rt + t * 16 * MP + a * 16);
    put();
  }
  __syncthreads();

  // ---- sum the four slots in order, epilogue, store: an item is four filters of one result
  // column.  What the epilogue consists of is uniform over the launch, so the item loops are
  // compiled once per combination and the combination chosen once, outside them.
  const float alpha = tail.alpha;
  auto items = [&](auto bn_c, auto act_c, auto all_c) {
    constexpr bool BN = decltype(bn_c)::value;
    constexpr int ACT = decltype(act_c)::value;
    constexpr bool ALL4 = decltype(all_c)::value;   // every item's four filters exist
    if (g.pool) {
      const int npool = g.npix >> 2;
      const int nitems = (BM / 4) * npool;
      const int pplane = g.ph * g.pw;
      for (int it = tid; it < nitems; it += NTH) {
        const int mg = mdiv(it, g.mNPOOL), q = it - mg * npool;
        const int py = mdiv(q, g.mHTW), px = q - py * g.HTW;
        const int oy = (oy0 >> 1) + py, ox = (ox0 >> 1) + px;
        if (oy >= g.ph || ox >= g.pw) continue;
        const int mf = m0 + 4 * mg;
        const float* rp = R + (4 * q) * MP + 4 * mg;
        f32x4 best = {-3.402823466e+38f, -3.402823466e+38f, -3.402823466e+38f, -3.402823466e+38f};
#pragma unroll
        for (int i = 0; i < 4; i++) {   // window positions in scan order
          const f32x4 s0 = *reinterpret_cast<const f32x4*>(rp + i * MP);
          const f32x4 s1 = *reinterpret_cast<const f32x4*>(rp + i * MP + RW);
          const f32x4 s2 = *reinterpret_cast<const f32x4*>(rp + i * MP + 2 * RW);
          const f32x4 s3 = *reinterpret_cast<const f32x4*>(rp + i * MP + 3 * RW);
          const f32x4 s = ((s0 + s1) + s2) + s3;
#pragma unroll
          for (int j = 0; j < 4; j++) {
            // a filter beyond F reads the last filter's table row and is never stored
            const float v = tail_apply_fixed<BN, ACT>(ftab, BM, 4 * mg + j, s[j], alpha);
            if (v > best[j]) best[j] = v;
          }
        }
        float* yp = y + ((int64_t)bimg * g.F + mf) * pplane + oy * g.pw + ox;
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (ALL4 || mf + j < g.F) yp[(int64_t)j * pplane] = best[j];
      }
    } else {
      const int nitems = (BM / 4) * g.npix;
      const int plane = g.oh * g.ow;
      for (int it = tid; it < nitems; it += NTH) {
        const int mg = mdiv(it, g.mNPIX), q = it - mg * g.npix;
        const int ty = mdiv(q, g.mTW), tx = q - ty * g.TW;
        const int oy = oy0 + ty, ox = ox0 + tx;
        if (oy >= g.oh || ox >= g.ow) continue;
        const int mf = m0 + 4 * mg;
        const float* rp = R + q * MP + 4 * mg;
        const f32x4 s0 = *reinterpret_cast<const f32x4*>(rp);
        const f32x4 s1 = *reinterpret_cast<const f32x4*>(rp + RW);
        const f32x4 s2 = *reinterpret_cast<const f32x4*>(rp + 2 * RW);
        const f32x4 s3 = *reinterpret_cast<const f32x4*>(rp + 3 * RW);
        const f32x4 s = ((s0 + s1) + s2) + s3;
        float* yp = y + ((int64_t)bimg * g.F + mf) * plane + oy * g.ow + ox;
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (ALL4 || mf + j < g.F) yp[(int64_t)j * plane] = tail_apply_fixed<BN, ACT>(ftab, BM, 4 * mg + j, s[j], alpha);
      }
    }
  };
  const bool all4 = m0 + BM <= g.F;
  conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
    if (all4) items(bn_c, act_c, std::true_type{}); else items(bn_c, act_c, std::false_type{});
  });
}

struct PatchPlan {
  PatchGeom g;
  int TM, TN;
  size_t lds;
};

constexpr int kTileMenu[] = {4, 7, 9, 11};   // instantiated N extents (in 16-pixel tiles)

// Geometry and workgroup shape for one command, a function of its shape and of `pool`
// only; false when the kernel does not take the shape.
bool patch_plan_compute(const gh_cmd& c, bool pool, PatchPlan* out) {
  if (gh_dtype_of(c.flags) != GH_F32) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4];
  const int64_t pad = c.dim[7];
  if (c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 || c.dim[12] != 1 ||
      c.dim[8] != pad || pad < 0 || pad > 1)
    return false;
  if (B < 1 || F < 16 || C < 64 || C % 32 != 0 || C > 8192 || H < 3 || W < 3 || H > 4096 || W > 4096) return false;
  if (B * C * H * W >= (1ll << 31) || B * F * H * W >= (1ll << 31) || F > (1 << 20)) return false;
  if (getenv("GORGONIA_HIP_CONV_NO_PATCH")) return false;   // tuning switch: the general kernels only
  PatchGeom g{};
  g.B = (int)B; g.C = (int)C; g.H = (int)H; g.W = (int)W; g.F = (int)F; g.pad = (int)pad;
  g.oh = g.H + 2 * g.pad - 2; g.ow = g.W + 2 * g.pad - 2;
  if (g.oh <= 0 || g.ow <= 0) return false;
  g.pool = pool ? 1 : 0; g.ph = g.oh / 2; g.pw = g.ow / 2;
  if (pool && (g.ph == 0 || g.pw == 0)) return false;
  g.HW = g.H * g.W; g.K = g.C * 9; g.NQ = g.C / 32;
  // rows and columns of the convolution result a patch grid has to cover
  const int need_h = pool ? 2 * g.ph : g.oh, need_w = pool ? 2 * g.pw : g.ow;
  // patch shape: the least padded MFMA work, then the smallest halo
  int64_t best_work = 0, best_halo = 0;
  int bTH = 0, bTW = 0, bTN = 0;
  const int step = pool ? 2 : 1;
  for (int TH = step; TH <= 64 && TH <= need_h + step - 1; TH += step)
    for (int TW = step; TW <= 64 && TW <= need_w + step - 1; TW += step) {
      const int npix = TH * TW;
      if (npix > 16 * 11 || 4 * (TH + 2) * (TW + 2) > 64 * kSlotsX) continue;
      int TN = 0;
      for (int m : kTileMenu)
        if (16 * m >= npix) { TN = m; break; }
      const int64_t tiles = (int64_t)((need_h + TH - 1) / TH) * ((need_w + TW - 1) / TW);
      const int64_t work = tiles * 16 * TN, halo = tiles * (TH + 2) * (TW + 2);
      if (!bTN || work < best_work || (work == best_work && halo < best_halo)) {
        best_work = work; best_halo = halo; bTH = TH; bTW = TW; bTN = TN;
      }
    }
  if (!bTN) return false;
  g.TH = bTH; g.TW = bTW; g.HTW = bTW / 2;
  g.tiles_x = (need_w + bTW - 1) / bTW; g.tiles_y = (need_h + bTH - 1) / bTH;
  g.PW = bTW + 2; g.PP = (bTH + 2) * g.PW;
  g.PL = g.PP | 1;   // odd pitch: the four channel planes of a fetch start in different banks
  g.npix = bTH * bTW;
  const int64_t patches = (int64_t)g.B * g.tiles_x * g.tiles_y;
  if (patches > (1ll << 30)) return false;
  // 32 filters per workgroup halve the B-operand reads; 16 when that leaves compute units without one
  const int TM = (F > 16 && patches * ((F + 31) / 32) >= 200) ? 2 : 1;
  g.mTXY = magic_of(g.tiles_x * g.tiles_y); g.mTX = magic_of(g.tiles_x); g.mPP = magic_of(g.PP);
  g.mPW = magic_of(g.PW); g.mTW = magic_of(g.TW); g.mHTW = magic_of(g.HTW); g.mNPIX = magic_of(g.npix);
  g.mNPOOL = magic_of(g.npix / 4);
  const size_t stage = ((size_t)kWaves * (36 * 16 * TM + 4 * g.PL) + 16 * bTN + 8) * 4;
  const size_t red = (size_t)4 * 16 * bTN * (16 * TM + 4) * 4;
  size_t lds = stage > red ? stage : red;
  g.epi_off = (int)(lds / 4);
  lds += (size_t)4 * 16 * TM * 4;
  out->g = g; out->TM = TM; out->TN = bTN; out->lds = lds;
  return lds <= 150 * 1024;
}

// The plan of a command, remembered per shape (the search over patch shapes costs tens of microseconds).
bool patch_plan(const gh_cmd& c, bool pool, PatchPlan* out) {
  return gh_plan_memo(c, pool, out, [&](PatchPlan* p) { return patch_plan_compute(c, pool, p); });
}

template <int TM, int TN>
int launch_patch(gh_ctx* ctx, const gh_cmd& c, const PatchPlan& p) {
  // more than 64 KB of dynamic LDS has to be allowed per kernel, once
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    attr_rc = hipFuncSetAttribute((const void*)k_conv3x3_patch<TM, TN>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024);
  });
  if (attr_rc != hipSuccess) return gh_check_hip(ctx, attr_rc, "hipFuncSetAttribute(conv3x3 patch)");
  PatchGeom g = p.g;
  g.ntiles = g.B * g.tiles_x * g.tiles_y;
  g.ftiles = (g.F + 16 * TM - 1) / (16 * TM);
  const int64_t nwg = (int64_t)g.ntiles * g.ftiles;
  if (nwg >= (1ll << 31)) return gh_fail(ctx, GH_EINVAL, "conv2d: too many workgroups for the patch kernel");
  g.nwg = (int)nwg;
  static const bool no_xcd = getenv("GORGONIA_HIP_CONV_PATCH_ORDER") != nullptr;   // tuning switch: "0" patch-major, "1" filter-tile-major
  g.ft_major = (int64_t)g.F * g.K > (int64_t)g.B * g.C * g.HW ? 1 : 0;
  if (no_xcd) g.ft_major = atoi(getenv("GORGONIA_HIP_CONV_PATCH_ORDER")) != 0;
  hipLaunchKernelGGL((k_conv3x3_patch<TM, TN>), dim3((unsigned)g.nwg), dim3(kWaves * 64), p.lds, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], g, conv_tail(c));
  return gh_check_hip(ctx, hipGetLastError(), "conv3x3 patch launch");
}

}  // namespace

bool gh_conv_patch_takes(const gh_cmd& c) {
  PatchPlan p;
  return patch_plan(c, false, &p);
}

// Pooling rides in the epilogue only where the even-sized patches it needs cost about the
// same matrix work as the best plain patch grid; otherwise the separate pooling kernel is
// cheaper than the extra MFMAs and halo.
bool gh_conv_patch_can_pool(const gh_cmd& c) {
  PatchPlan p, q;
  if (!patch_plan(c, false, &p) || !patch_plan(c, true, &q)) return false;
  const int64_t plain = (int64_t)p.g.tiles_x * p.g.tiles_y * p.TN, pooled = (int64_t)q.g.tiles_x * q.g.tiles_y * q.TN;
  const int64_t plain_cells = (int64_t)p.g.tiles_x * p.g.tiles_y * p.g.PP, pooled_cells = (int64_t)q.g.tiles_x * q.g.tiles_y * q.g.PP;
  return pooled * 100 <= plain * 105 && pooled_cells * 100 <= plain_cells * 110 && q.TM == p.TM;
}

// Returns -1 when the shape is not one this kernel takes.
int gh_try_launch_conv_patch(gh_ctx* ctx, const gh_cmd& c) {
  PatchPlan p;
  const bool pool = c.flags & GH_FLAG_CONV_POOL2;
  // a pooled command only rides here when the plain one would too: both then sum in the same order
  if (!patch_plan(c, false, &p)) return -1;
  if (pool && (!gh_conv_patch_can_pool(c) || !patch_plan(c, true, &p)))
    return gh_fail(ctx, GH_EINVAL, "conv2d: no fused pooling for this shape (see gh_conv2d_can_pool)");
#define GH_PATCH_TN(TM_)                                              \
  switch (p.TN) {                                                     \
    case 4: return launch_patch<TM_, 4>(ctx, c, p);                   \
    case 7: return launch_patch<TM_, 7>(ctx, c, p);                   \
    case 9: return launch_patch<TM_, 9>(ctx, c, p);                   \
    default: return launch_patch<TM_, 11>(ctx, c, p);                 \
  }
  if (p.TM == 1) { GH_PATCH_TN(1) }
  GH_PATCH_TN(2)
#undef GH_PATCH_TN
}
