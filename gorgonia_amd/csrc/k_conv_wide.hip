// Conv2d 3x3 / stride 1 over large images with few input channels (up to 64), float32,
// on the 16x16x4 MFMA: one workgroup = 16 TM filters x one TH x TW patch of one image,
// the patch's pixels split over its eight wavefronts, each of which runs the whole K.
//
// Replaces cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117) for the first
// layers of an image network: many output pixels, a short contraction.  With K = C * 9 of
// a few hundred at most, the whole filter tile and every channel of the padded patch fit
// in LDS at once, so there is one staging phase, one barrier, and then nothing but
// operand fetches and MFMAs; the results leave from the accumulators, no partial sums
// cross wavefronts.  The output pixels are the MFMA's rows and the filters its columns
// (K in the reference's (c, kr, kc) order, op_nn.go:418-437): a lane holds four consecutive
// N entries of one filter, and results are written straight into NCHW.
//
//   * One output is one accumulator chain over K, channel quad by channel quad, tap by
//     tap, whatever the patch shape and whether or not the pooling below is fused: the
//     stored bits depend on the operands only.
//   * A channel count that is not a multiple of four is padded with zero planes and zero
//     filter columns in LDS (a first layer's 3 channels or 1).
//   * With GH_FLAG_CONV_POOL2 the patch has even extents and the N axis enumerates (pooled
//     pixel, position in the 2x2 window), so a window is the four accumulator registers of
//     one lane: the maximum is a scan over them in order with strict > (the pooling kernel's
//     rule, op_nn.go:860-907), no lane waits for another, and every lane stores a result.
//     Without it a lane's four entries are four pixels of a row wherever the patch is a
//     multiple of four wide, and leave as one 128-bit store where the result allows.
#include <algorithm>
#include <cstdio>
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

struct WideGeom {
  int B, C, H, W, F, pad, oh, ow, HW, K;
  int NQ, KP;                     // channel quads ceil(C / 4); padded contraction 36 NQ
  int TH, TW, tiles_x, tiles_y;   // output patch, patches per image
  int PW, PP, PL;                 // padded patch: row length TW + 2, size (TH + 2) * PW, plane pitch in LDS
  int npix;                       // TH * TW
  int pool, ph, pw, HTW;          // fused 2x2 / stride-2 max-pool: pooled extents of y, TW / 2
  unsigned mTXY, mTX, mPP, mPW, mTW, mHTW;   // magics: tiles_x*tiles_y, tiles_x, PP, PW, TW, HTW
  int xcd_walk;                   // workgroups of one XCD walk one contiguous eighth of the tiles
};

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;

// XS: patch cells each thread stages per tile (4 NQ PP <= XS * kThreads); DB: two patch buffers.
// The 12-slot kernels are held to 128 registers so that two workgroups share a compute unit
// where their LDS allows: one's staging, epilogue and barriers then run under the other's MFMAs.
template <int TM, int TN, int XS, bool DB>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(XS == 12 && TM * TN <= 4 ? 4 : 2))) void k_conv3x3_wide(const float* __restrict__ x, const float* __restrict__ w,
                                                           float* __restrict__ y, WideGeom g, ConvTail tail) {
  constexpr int BM = 16 * TM;
  constexpr int NB = kWaves * 16 * TN;   // N entries of the workgroup
  extern __shared__ float lds[];
  const int plane_floats = 4 * g.NQ * g.PL + 8;    // one patch buffer; its last 8 floats take idle slots' writes
  float* const As = lds;                           // [TM][KP][16]: filter tile, k-major, 16 filters a row
  float* const P0 = lds + TM * g.KP * 16;          // [DB ? 2 : 1][4 NQ][PL]: padded patch, one plane per channel
  int* const tab = reinterpret_cast<int*>(P0 + (DB ? 2 : 1) * plane_floats);   // [NB] cell of N entry n in the patch
  float* const ftab = reinterpret_cast<float*>(tab + NB);                      // [4][BM] BatchNorm constants
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lk = lane >> 4;
  const int m0 = blockIdx.y * BM;
  if (tid < BM) conv_tail_table(tail, ftab, BM, tid, min(m0 + tid, g.F - 1));

  // ---- per-thread patch cells, the same for every tile: source offset relative to the patch
  // origin, row and column inside the padded patch, destination in the buffer.  Slots past the
  // last cell and cells of padded channels are flagged: they load nothing that matters and
  // write the spare floats at the end of the buffer; the padded planes are zeroed here, once.
  int xrel[XS], xpk[XS];   // xpk = flag << 31 | row << 24 | column << 16 | destination
  {
    const int cells = 4 * g.NQ * g.PP;
#pragma unroll
    for (int u = 0; u < XS; u++) {
      const int id = tid + u * kThreads;
      const int idc = min(id, cells - 1);
      const int pl = mdiv(idc, g.mPP), rem = idc - pl * g.PP;
      const int r = mdiv(rem, g.mPW), cc = rem - r * g.PW;
      const bool real = id < cells && pl < g.C;
      xrel[u] = min(pl, g.C - 1) * g.HW + r * g.W + cc;
      const int dst = real ? pl * g.PL + rem : 4 * g.NQ * g.PL + (lane & 7);
      xpk[u] = (real ? 0 : (int)0x80000000) | (r << 24) | (cc << 16) | dst;
    }
    const int zero0 = g.C * g.PL, zero1 = 4 * g.NQ * g.PL;
    for (int bsel = 0; bsel < (DB ? 2 : 1); bsel++)
      for (int i = zero0 + tid; i < zero1; i += kThreads) P0[bsel * plane_floats + i] = 0.f;
  }
  float xv[XS];
  // global loads of one tile's patch into registers.  A patch that lies inside the image, halo
  // and all, needs no test: every load is base + per-thread offset.  At the image border each
  // cell is tested and cells outside are zero.
  auto load_patch = [&](int tile) {
    const int bimg = mdiv(tile, g.mTXY);
    const int trem = tile - bimg * (g.tiles_x * g.tiles_y);
    const int tyi = mdiv(trem, g.mTX), txi = trem - tyi * g.tiles_x;
    const int py0 = tyi * g.TH - g.pad, px0 = txi * g.TW - g.pad;
    const float* const xo = x + (int64_t)bimg * g.C * g.HW + py0 * g.W + px0;
    if (py0 >= 0 && px0 >= 0 && py0 + g.TH + 2 <= g.H && px0 + g.TW + 2 <= g.W) {
#pragma unroll
      for (int u = 0; u < XS; u++) xv[u] = xo[xrel[u]];
    } else {
#pragma unroll
      for (int u = 0; u < XS; u++) {
        const int iy = py0 + ((xpk[u] >> 24) & 0x7f), ix = px0 + ((xpk[u] >> 16) & 0xff);
        xv[u] = 0.f;
        if (xpk[u] >= 0 && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W) xv[u] = xo[xrel[u]];
      }
    }
  };
  auto store_patch = [&](float* buf) {
#pragma unroll
    for (int u = 0; u < XS; u++) buf[xpk[u] & 0xffff] = xv[u];
  };

  // Which tiles this workgroup walks.  Workgroup ids are dealt round-robin over the 8 XCDs, each with
  // its own L2: with tiles id, id + G, ... neighbouring patches - which share halo rows and cache
  // lines, and whose results share cache lines - would land on different XCDs, every L2 would fetch
  // nearly the whole input and no L2 would see a whole line of results.  Instead the workgroups of
  // XCD j (ids = j mod 8; the launch has a multiple of 8 in x) share the j-th contiguous eighth
  // of the tiles, whole images where the batch allows.
  const int ntiles = g.B * g.tiles_x * g.tiles_y;
  int tile, tile_end, tile_step;
  if (g.xcd_walk) {
    const int xcd = blockIdx.x & 7;
    tile_end = (int)(((int64_t)ntiles * (xcd + 1)) >> 3);
    tile = (int)(((int64_t)ntiles * xcd) >> 3) + (blockIdx.x >> 3);
    tile_step = gridDim.x >> 3;
  } else {
    tile = blockIdx.x; tile_end = ntiles; tile_step = gridDim.x;
  }
  load_patch(tile);                      // the launch leaves no workgroup without a tile
  // (the first patch is on its way while the filter tile is fetched and the table is filled)
  // ---- the filter tile, once: As[a][k][f] = w[m0 + 16 a + f][k], zero for k >= K
  {
    const int f = tid & (BM - 1), j0 = tid / BM;
    const float* const wrow = w + (int64_t)min(m0 + f, g.F - 1) * g.K;
    float* const ad = As + (f >> 4) * g.KP * 16 + (f & 15);
    constexpr int JS = kThreads / BM;    // 128-bit columns in flight per pass
    const int ncol = g.KP / 4;
    if ((g.K & 3) == 0) {
      // every workgroup reads the same filter rows at the same moment: each starts at a column
      // of its own (and wraps), so that their loads spread over the cache channels
      const int rot = (int)((blockIdx.x * 5u) % (unsigned)ncol);
      for (int j = j0; j < ncol; j += 4 * JS) {
        f32x4 v[4];
        int jj[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int jc = min(j + u * JS, ncol - 1) + rot;   // passes past the end rewrite the last column
          jj[u] = jc >= ncol ? jc - ncol : jc;
          v[u] = *reinterpret_cast<const f32x4_a4*>(wrow + 4 * jj[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
          for (int e = 0; e < 4; e++) ad[(4 * jj[u] + e) * 16] = v[u][e];
        }
      }
    } else {
      for (int k = j0; k < g.KP; k += JS) ad[k * 16] = k < g.K ? wrow[k] : 0.f;
    }
  }
  // ---- table of patch cells of the N entries
  for (int n = tid; n < NB; n += kThreads) {
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

  store_patch(P0);
  __syncthreads();

  const int n0 = wave * 16 * TN;         // this wavefront's first N entry
  int pb[TN][3];   // one base per kernel row, so the column tap is an immediate offset
#pragma unroll
  for (int t = 0; t < TN; t++) {
    const int p = tab[n0 + t * 16 + li] + lk * g.PL;
#pragma unroll
    for (int kr = 0; kr < 3; kr++) pb[t][kr] = p + kr * g.PW;
  }
  int cur = 0;

  for (;;) {
    const int next = tile + tile_step;
    const bool more = next < tile_end;
    if (more) load_patch(next);          // in flight during this tile's MFMAs

    f32x4 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int t = 0; t < TN; t++) acc[a][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- MFMA: step = (channel quad, tap); lane group lk takes channel 4 quad + lk.  Operands
    // of step s + 2 are fetched while step s runs (three register sets), across quad
    // boundaries too; one LDS read is placed after each MFMA.  The fetch stream has its own
    // pointers, moved once per quad just before it enters the next one (taps are immediate
    // offsets), so the loop carries TM + 3 TN vector adds per 9 TM TN MFMAs and no other
    // vector instruction: the SIMD runs vector and matrix instructions one after the other,
    // never at once, so each one outside the matrix pipe is time the matrix pipe stands idle.
    float af[3][TM], bf[3][TN];
    const float* fa[TM];
    const float* fb[TN][3];
#pragma unroll
    for (int a = 0; a < TM; a++) fa[a] = As + a * (g.KP * 16) + lk * 9 * 16 + li;
#pragma unroll
    for (int t = 0; t < TN; t++)
#pragma unroll
      for (int kr = 0; kr < 3; kr++) fb[t][kr] = P0 + cur * plane_floats + pb[t][kr];
    auto fetch = [&](int set, int tap) {
      const int kr = tap / 3, kc = tap % 3;
#pragma unroll
      for (int a = 0; a < TM; a++) af[set][a] = fa[a][tap * 16];
#pragma unroll
      for (int t = 0; t < TN; t++) bf[set][t] = fb[t][kr][kc];
    };
    fetch(0, 0);
    fetch(1, 1);
    for (int qd = 0; qd < g.NQ; qd++) {
      // the last quad's look-ahead fetches repeat its own first taps (unused)
      const int na = qd + 1 < g.NQ ? 36 * 16 : 0, np = qd + 1 < g.NQ ? 4 * g.PL : 0;
#pragma unroll
      for (int tap = 0; tap < 9; tap++) {
        if (tap == 7) {
#pragma unroll
          for (int a = 0; a < TM; a++) fa[a] += na;
#pragma unroll
          for (int t = 0; t < TN; t++)
#pragma unroll
            for (int kr = 0; kr < 3; kr++) fb[t][kr] += np;
        }
        fetch((tap + 2) % 3, (tap + 2) % 9);
#pragma unroll
        for (int a = 0; a < TM; a++)
#pragma unroll
          for (int t = 0; t < TN; t++)
            acc[a][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf[tap % 3][t], af[tap % 3][a], acc[a][t], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < TM * TN; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // DS read
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- epilogue from the accumulators.  The pixels are the MFMA's rows and the filters its columns:
    // register v of acc[a][t] is N entry n0 + 16 t + 4 lk + v of filter m0 + 16 a + li.  With the pool fused
    // the N order is window-major, so those four entries are one 2x2 window and the pool is a scan over
    // the lane's own registers; a lane needs the BatchNorm constants of one filter per filter tile.
    {
      // The lane's coordinates pass through an empty asm here, so that what the epilogue derives
      // from them is computed per tile and does not sit in registers through the MFMA loop.
      int eli = li, elk = lk;
      asm volatile("" : "+v"(eli), "+v"(elk));
      const int bimg = mdiv(tile, g.mTXY);
      const int trem = tile - bimg * (g.tiles_x * g.tiles_y);
      const int tyi = mdiv(trem, g.mTX), txi = trem - tyi * g.tiles_x;
      const int oy0 = tyi * g.TH, ox0 = txi * g.TW;
      const int plane = g.pool ? g.ph * g.pw : g.oh * g.ow;
      // one 64-bit base per tile, 32-bit byte offsets per lane (a filter tile's planes span < 2 GB)
      char* const ytile = reinterpret_cast<char*>(y + ((int64_t)bimg * g.F + m0) * plane);
      const unsigned pbytes = 4u * (unsigned)plane;
      const float alpha = tail.alpha;
      const int nb = n0 + 4 * elk;   // the lane's first N entry of N tile 0
      // What the epilogue consists of is uniform over the launch: the value loops are compiled
      // once per combination and the combination is chosen once per tile, not once per value.
      auto values = [&](auto bn_c, auto act_c, auto pool_c) {
        constexpr bool BN = decltype(bn_c)::value;
        constexpr int ACT = decltype(act_c)::value;
        constexpr bool POOL = decltype(pool_c)::value;
        // where the lane's entries of each N tile go (element offset inside a filter's plane)
        int yoff[TN];        // pooled: the window; else the first of four pixels in a row (row4); -1: nowhere
        int nval[TN];        // row4: how many of the four pixels lie inside the image
        const bool row4 = !POOL && (g.TW & 3) == 0;
#pragma unroll
        for (int t = 0; t < TN; t++) {
          const int n = nb + 16 * t;
          if constexpr (POOL) {
            const int q = n >> 2;
            const int py = mdiv(q, g.mHTW), px = q - py * g.HTW;
            const int oy = (oy0 >> 1) + py, ox = (ox0 >> 1) + px;
            yoff[t] = (n < g.npix && oy < g.ph && ox < g.pw) ? oy * g.pw + ox : -1;
            nval[t] = 0;
          } else {
            const int ty = mdiv(n, g.mTW), tx = n - ty * g.TW;
            const int oy = oy0 + ty, ox = ox0 + tx;
            yoff[t] = (n < g.npix && oy < g.oh && ox < g.ow) ? oy * g.ow + ox : -1;
            nval[t] = min(g.ow - ox, 4);
          }
        }
        const bool vec4 = row4 && (g.ow & 3) == 0 && (plane & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
#pragma unroll
        for (int a = 0; a < TM; a++) {
          const int fl = 16 * a + eli;                 // the lane's filter inside the workgroup's tile
          const bool fok = m0 + fl < g.F;
          const unsigned foff = (unsigned)fl * pbytes;
          float ka = 0.f, kb = 0.f, kg = 0.f, ke = 0.f;
          if constexpr (BN) {   // an absent gamma is 1 and an absent beta -0 in the table, which change no bits
            ka = ftab[fl]; kb = ftab[BM + fl]; kg = ftab[2 * BM + fl]; ke = ftab[3 * BM + fl];
          }
#pragma unroll
          for (int t = 0; t < TN; t++) {
            f32x4 v = acc[a][t];
#pragma unroll
            for (int r = 0; r < 4; r++) {
              if constexpr (BN) {
                v[r] = v[r] * ka;
                v[r] = v[r] + kb;
                v[r] = kg * v[r];
                v[r] = v[r] + ke;
              }
              v[r] = act_apply(v[r], ACT, alpha);
            }
            if constexpr (POOL) {
              // the reference's scan of the window from -FLT_MAX with a strict compare, positions in order
              float best = -3.402823466e+38f;
#pragma unroll
              for (int r = 0; r < 4; r++)
                if (v[r] > best) best = v[r];
              if (fok && yoff[t] >= 0) *reinterpret_cast<float*>(ytile + (foff + 4u * (unsigned)yoff[t])) = best;
            } else if (row4) {
              if (fok && yoff[t] >= 0) {
                char* const yp = ytile + (foff + 4u * (unsigned)yoff[t]);
                if (vec4 && nval[t] >= 4) {
                  *reinterpret_cast<f32x4*>(yp) = v;
                } else {
#pragma unroll
                  for (int r = 0; r < 4; r++)
                    if (r < nval[t]) reinterpret_cast<float*>(yp)[r] = v[r];
                }
              }
            } else {
              // a patch row is no multiple of four pixels: each of the lane's entries has its own row and column
#pragma unroll
              for (int r = 0; r < 4; r++) {
                const int n = nb + 16 * t + r;
                const int ty = mdiv(n, g.mTW), tx = n - ty * g.TW;
                const int oy = oy0 + ty, ox = ox0 + tx;
                if (fok && n < g.npix && oy < g.oh && ox < g.ow)
                  *reinterpret_cast<float*>(ytile + (foff + 4u * (unsigned)(oy * g.ow + ox))) = v[r];
              }
            }
          }
        }
      };
      conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
        if (g.pool) values(bn_c, act_c, std::true_type{}); else values(bn_c, act_c, std::false_type{});
      });
    }
    if (!more) break;
    if constexpr (DB) {
      cur ^= 1;
      store_patch(P0 + cur * plane_floats);   // the buffer nobody reads during this tile
      __syncthreads();
    } else {
      __syncthreads();                        // every wavefront is done reading the patch
      store_patch(P0);
      __syncthreads();
    }
    tile = next;
  }
}

struct WidePlan {
  WideGeom g;
  int TM, TN, XS;
  bool DB;
  size_t lds;
};

constexpr size_t kLdsBudget = 156 * 1024;   // of the 160 KB a workgroup may hold
constexpr int kMaxSlots = 24;               // patch cells per thread the kernel is built for
constexpr int kDeviceCUs = 256;             // the plan is a function of the command alone: MI355X

inline size_t wide_lds(const WideGeom& g, int TM, int TN, int PL, bool db) {
  return ((size_t)TM * g.KP * 16 + (size_t)(db ? 2 : 1) * (4 * g.NQ * PL + 8) + kWaves * 16 * TN + 4 * 16 * TM) * 4;
}

// Geometry and workgroup shape for one command, a function of its shape and of `pool`
// only; false when the kernel does not take the shape.
bool wide_plan_compute(const gh_cmd& c, bool pool, WidePlan* out) {
  if (gh_dtype_of(c.flags) != GH_F32) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4];
  const int64_t pad = c.dim[7];
  if (c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 || c.dim[12] != 1 ||
      c.dim[8] != pad || pad < 0 || pad > 1)
    return false;
  if (B < 1 || F < 1 || C < 3 || C > 64 || H < 3 || W < 3 || H > 8192 || W > 8192) return false;
  if (B * C * H * W >= (1ll << 31) || B * F * H * W >= (1ll << 31) || F > (1 << 20)) return false;
  if (getenv("GORGONIA_HIP_CONV_NO_WIDE")) return false;   // tuning switch: the other kernels only
  WideGeom g{};
  g.B = (int)B; g.C = (int)C; g.H = (int)H; g.W = (int)W; g.F = (int)F; g.pad = (int)pad;
  g.oh = g.H + 2 * g.pad - 2; g.ow = g.W + 2 * g.pad - 2;
  if (g.oh <= 0 || g.ow <= 0 || (int64_t)g.oh * g.ow > (1 << 22)) return false;   // 64 planes of results within 32-bit byte offsets
  g.pool = pool ? 1 : 0; g.ph = g.oh / 2; g.pw = g.ow / 2;
  if (pool && (g.ph == 0 || g.pw == 0)) return false;
  g.HW = g.H * g.W; g.K = g.C * 9; g.NQ = (g.C + 3) / 4; g.KP = 36 * g.NQ;
  // enough pixels that patches alone fill the device: this kernel does not split K
  const int need_h = pool ? 2 * g.ph : g.oh, need_w = pool ? 2 * g.pw : g.ow;
  if ((int64_t)B * need_h * need_w < 128 * 256) return false;
  // Candidates: 16, 32 or 64 filters per workgroup, one or two patch buffers; for each the patch
  // shape with the least padded MFMA work (then the smallest halo) among those whose staging
  // fits the kernel's slots and LDS.  The candidate with the shortest estimated run wins:
  // rounds of tiles over the workgroups the device holds at once (two per compute unit when
  // LDS and registers allow; a lone workgroup's staging and epilogue are not hidden).
  int tm_hi = F > 32 ? 4 : F > 16 ? 2 : 1, tm_lo = 1;
  int menu_lo = 1, menu_hi = 2;
  if (const char* env = getenv("GORGONIA_HIP_CONV_WIDE_PLAN")) {   // tuning override: "TM,TN"
    int tm = 0, tn = 0;
    if (sscanf(env, "%d,%d", &tm, &tn) == 2 && (tm == 1 || tm == 2 || tm == 4) && (tn == 1 || tn == 2)) {
      tm_hi = tm_lo = tm; menu_lo = menu_hi = tn;
    }
  }
  const int step = pool ? 2 : 1;
  double best_est = 0;
  bool found = false;
  for (int TM = tm_hi; TM >= tm_lo; TM >>= 1)
    for (int db = 1; db >= 0; db--)
    for (int TN = menu_lo; TN <= menu_hi; TN++) {
      int64_t best_work = 0, best_halo = 0;
      int bTH = 0, bTW = 0, bTN = 0;
      for (int TH = step; TH <= 64 && TH <= need_h + step - 1; TH += step)
        for (int TW = step; TW <= 128 && TW <= need_w + step - 1; TW += step) {
          const int npix = TH * TW;
          if (npix > kWaves * 16 * TN || npix <= kWaves * 16 * (TN - 1)) continue;
          const int PP = (TH + 2) * (TW + 2);
          if (4 * g.NQ * PP > kMaxSlots * kThreads) continue;
          if (wide_lds(g, TM, TN, PP | 1, db != 0) > kLdsBudget) continue;
          const int64_t tiles = (int64_t)((need_h + TH - 1) / TH) * ((need_w + TW - 1) / TW);
          const int64_t work = tiles * TN, halo = tiles * PP;
          if (!bTN || work < best_work || (work == best_work && halo < best_halo)) {
            best_work = work; best_halo = halo; bTH = TH; bTW = TW; bTN = TN;
          }
        }
      if (!bTN) continue;
      WideGeom h = g;
      h.TH = bTH; h.TW = bTW; h.HTW = bTW / 2;
      h.tiles_x = (need_w + bTW - 1) / bTW; h.tiles_y = (need_h + bTH - 1) / bTH;
      h.PW = bTW + 2; h.PP = (bTH + 2) * h.PW;
      h.PL = h.PP | 1;   // odd pitch: the four channel planes of a fetch start in different banks
      h.npix = bTH * bTW;
      const int64_t ntiles = (int64_t)h.B * h.tiles_x * h.tiles_y;
      if (ntiles > (1ll << 30)) continue;
      const int XS = 4 * h.NQ * h.PP <= 12 * kThreads ? 12 : kMaxSlots;
      const size_t lds = wide_lds(h, TM, bTN, h.PL, db != 0);
      const int occ = (XS == 12 && TM * bTN <= 4 && 2 * lds <= 158 * 1024) ? 2 : 1;
      const int ft = (h.F + 16 * TM - 1) / (16 * TM);
      const int64_t groups = std::max<int64_t>(1, (int64_t)kDeviceCUs * occ / ft);
      const int64_t rounds = (ntiles + groups - 1) / groups;
      // A round costs a workgroup, per 16 pixels of its patch, one unit per 16 filters (MFMAs and
      // epilogue) plus 0.85 of a unit for staging the patch, whatever the filter count: measured
      // on 16 -> 32 channels at 208 x 208 (6.3 us a round for 32 filters, 4.1 for 16).  `occ`
      // workgroups share a compute unit's time; alone, a workgroup's staging is not hidden.
      const double est = (double)rounds * occ * bTN * (TM + 0.85) * (occ == 2 ? 1.0 : db ? 1.35 : 1.45) *
                         (bTN == 2 ? 0.98 : 1.0);
      if (!found || est < best_est) {
        found = true; best_est = est;
        h.mTXY = magic_of(h.tiles_x * h.tiles_y); h.mTX = magic_of(h.tiles_x); h.mPP = magic_of(h.PP);
        h.mPW = magic_of(h.PW); h.mTW = magic_of(h.TW); h.mHTW = magic_of(h.HTW);
        out->g = h; out->TM = TM; out->TN = bTN; out->XS = XS; out->DB = db != 0; out->lds = lds;
      }
    }
  return found;
}

// The plan of a command, remembered per shape (the search over patch shapes costs 60-150 microseconds).
bool wide_plan(const gh_cmd& c, bool pool, WidePlan* out) {
  return gh_plan_memo(c, pool, out, [&](WidePlan* p) { return wide_plan_compute(c, pool, p); });
}

template <int TM, int TN, int XS, bool DB>
int launch_wide(gh_ctx* ctx, const gh_cmd& c, const WidePlan& p) {
  // more than 64 KB of dynamic LDS has to be allowed per kernel, once
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    attr_rc = hipFuncSetAttribute((const void*)k_conv3x3_wide<TM, TN, XS, DB>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  if (attr_rc != hipSuccess) return gh_check_hip(ctx, attr_rc, "hipFuncSetAttribute(conv3x3 wide)");
  // Persistent workgroups: as many as the device holds at once (two per compute unit where
  // their LDS allows), shared among the filter tiles; each walks its tiles id, id + G, ...
  // G is then lowered to the fewest workgroups that need no more rounds.
  const int64_t ntiles = (int64_t)p.g.B * p.g.tiles_x * p.g.tiles_y;
  const int ft = (p.g.F + 16 * TM - 1) / (16 * TM);
  const int per_cu = (XS == 12 && TM * TN <= 4 && 2 * p.lds <= 158 * 1024) ? 2 : 1;
  int64_t G = std::max<int64_t>(1, (int64_t)ctx->cu_count * per_cu / ft);
  if (G > ntiles) G = ntiles;
  WideGeom geom = p.g;
  static const bool no_xcd = getenv("GORGONIA_HIP_CONV_WIDE_NO_XCD") != nullptr;   // tuning switch: tiles id, id + G, ...
  if (ntiles >= 64 && G >= 8 && !no_xcd) {
    // one contiguous eighth of the tiles per XCD (see the kernel): Gx workgroups per XCD, lowered to
    // the fewest that need no more rounds, and never more than the smallest eighth has tiles
    const int64_t t8 = (ntiles + 7) / 8, t8min = ntiles / 8;
    int64_t Gx = std::max<int64_t>(1, G / 8);
    const int64_t rounds = (t8 + Gx - 1) / Gx;
    Gx = std::min((t8 + rounds - 1) / rounds, t8min);
    G = 8 * Gx;
    geom.xcd_walk = 1;
  } else {
    const int64_t rounds = (ntiles + G - 1) / G;
    G = (ntiles + rounds - 1) / rounds;
    geom.xcd_walk = 0;
  }
  const dim3 grid((unsigned)G, (unsigned)ft);
  if (getenv("GORGONIA_HIP_CONV_WIDE_DEBUG"))
    fprintf(stderr, "wide conv: TM=%d TN=%d XS=%d DB=%d patch %dx%d tiles %lld G=%lld ft=%d lds=%zu\n", TM, TN, XS, (int)DB,
            p.g.TH, p.g.TW, (long long)ntiles, (long long)G, ft, p.lds);
  hipLaunchKernelGGL((k_conv3x3_wide<TM, TN, XS, DB>), grid, dim3(kThreads), p.lds, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], geom, conv_tail(c));
  return gh_check_hip(ctx, hipGetLastError(), "conv3x3 wide launch");
}

template <int TM, int TN>
int launch_wide_tile(gh_ctx* ctx, const gh_cmd& c, const WidePlan& p) {
  if (p.XS == 12) return p.DB ? launch_wide<TM, TN, 12, true>(ctx, c, p) : launch_wide<TM, TN, 12, false>(ctx, c, p);
  return p.DB ? launch_wide<TM, TN, kMaxSlots, true>(ctx, c, p) : launch_wide<TM, TN, kMaxSlots, false>(ctx, c, p);
}

}  // namespace

bool gh_conv_wide_takes(const gh_cmd& c) {
  WidePlan p;
  return wide_plan(c, false, &p);
}

// Pooling rides in the epilogue where the even-sized patches it needs cost about the same
// matrix work as the best plain patch grid.
bool gh_conv_wide_can_pool(const gh_cmd& c) {
  WidePlan p, q;
  if (!wide_plan(c, false, &p) || !wide_plan(c, true, &q)) return false;
  auto work = [](const WidePlan& a) {
    return (int64_t)a.g.tiles_x * a.g.tiles_y * a.TN * a.TM * ((a.g.F + 16 * a.TM - 1) / (16 * a.TM));
  };
  return work(q) * 100 <= work(p) * 110;
}

// Returns -1 when the shape is not one this kernel takes.
int gh_try_launch_conv_wide(gh_ctx* ctx, const gh_cmd& c) {
  WidePlan p;
  const bool pool = c.flags & GH_FLAG_CONV_POOL2;
  // a pooled command only rides here when the plain one would too
  if (!wide_plan(c, false, &p)) return -1;
  if (pool && (!gh_conv_wide_can_pool(c) || !wide_plan(c, true, &p)))
    return gh_fail(ctx, GH_EINVAL, "conv2d: no fused pooling for this shape (see gh_conv2d_can_pool)");
#define GH_WIDE_TN(TM_)                                       \
  if (p.TN == 1) return launch_wide_tile<TM_, 1>(ctx, c, p);  \
  return launch_wide_tile<TM_, 2>(ctx, c, p);
  if (p.TM == 1) { GH_WIDE_TN(1) }
  if (p.TM == 2) { GH_WIDE_TN(2) }
  GH_WIDE_TN(4)
#undef GH_WIDE_TN
}
