// Conv2d 3x3 / stride 1 over small images (up to 16 x 16), float32, on the 16x16x4 MFMA.
//
// Replaces cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117) for the layers
// where the whole problem is a few microseconds of matrix-core time, so that what a
// workgroup does around its MFMAs decides the speed.  One workgroup owns 16 or 32 filters
// and IPB whole images and keeps everything it needs in LDS: its filter rows for all of
// K (k-major) and its images, every channel, as planes with a zero halo, so a B-operand
// fetch is one ds_read at (pixel base + tap offset) with no test.  The GEMM view is that
// of the other convolution kernels (M = filters, N = output pixels, K = C * 9 in the
// reference's (c, kr, kc) order, op_nn.go:418-437); the results are written straight into
// NCHW.
//
//   * K is split over the wavefronts of the workgroup: wavefront w sums channels
//     [w C/WV, (w+1) C/WV) for the whole tile, four channels (one per MFMA k-lane group)
//     and one tap per step.  The WV partial tiles are then added through LDS in a fixed
//     order, so results repeat bit for bit and do not depend on the tile shape, on IPB or
//     on whether the pooling below is fused: per output it is always the same WV partial
//     sums, each over the same channels in the same order.
//   * Each wavefront stages only its own channels (filter columns and image planes), so
//     between the start (one barrier, behind the shared table of pixel offsets, with every
//     load already in flight) and that sum nothing needs a workgroup barrier, and the loads
//     of channel quad q + 1 are in flight while quad q is multiplied.
//   * With GH_FLAG_CONV_POOL2 the N axis enumerates (image, pooled pixel, position in the
//     2x2 window): the row and column a 2x2/stride-2 pool discards on an odd extent are
//     never computed, and the epilogue reads a window as four adjacent columns (scan order
//     and strict > of the pooling kernel, op_nn.go:860-907).
//
// A wavefront issues in order, and alone on its SIMD nothing hides an instruction's
// latency, so outside the MFMA loop the instruction count is what costs: every index
// that can be a shift, an immediate offset or a per-thread constant is one.
#include <cstdlib>
#include <mutex>

#include "gh_conv_common.h"
#include "gh_internal.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// n / d with magic = magic_of(d), exact while n * d < 2^32; branch-free (magic 0 stands for d = 1)
inline unsigned magic_of(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
__device__ __forceinline__ int mdiv(int n, unsigned magic) {
  const unsigned q = __umulhi((unsigned)n, magic);
  return (int)(q | ((unsigned)n & (0u - (unsigned)(magic == 0))));
}

struct SmallGeom {
  int B, C, H, W, F, pad;
  int oh, ow;        // convolution output
  int Wp, PL;        // padded row (W + 2 pad); plane pitch in LDS (odd, >= (H + 2 pad) * Wp)
  int HW;
  int IPB;           // images per workgroup
  int K;             // C * 9
  int pool, ph, pw;  // fused 2x2 / stride-2 max-pool and the pooled extents
  int ppi;           // N entries per image: pool ? 4 * ph * pw : oh * ow
  int CW;            // channels per wavefront (C / WV)
  int CH;            // 128-bit chunks per image row: ceil(W / 4)
  int IPP;           // load items per plane: H * CH (<= 64)
  int lpg_shift;     // lanes per plane group = 1 << lpg_shift >= IPP
  int nout;          // result columns per workgroup: pool ? IPB * ph * pw : IPB * oh * ow
  int epi_off;       // float offset in LDS of the per-filter epilogue table (past every other use)
  unsigned mPPI, mOW, mPW, mPQ, mNOUT, mCH;   // magics: ppi, ow, pw, ph*pw, nout, CH
};

constexpr int kSlotsX = 4;   // image load slots per thread and channel quad (IPB <= planes per slot)

template <int WV, int TM, int TN, int NQ>
__global__ __launch_bounds__(WV * 64) void k_conv3x3_small(const float* __restrict__ x, const float* __restrict__ w,
                                                           float* __restrict__ y, SmallGeom g, ConvTail tail) {
  constexpr int NTH = WV * 64;
  constexpr int BM = 16 * TM;
  constexpr int BMS = TM == 1 ? 4 : 5;   // log2(BM)
  static_assert(TM == 1 || TM == 2, "filter tile of 16 or 32");
  static_assert(WV == 4 || WV == 8, "four or eight wavefronts");
  constexpr int SA = BM;                 // k-major filter tile As[k][SA]
  constexpr int MP = BM + 4;             // partial sums R[slot][n][MP]: a lane's four rows are one 128-bit access
  constexpr int RW = 16 * TN * MP;       // one slot
  constexpr int QL = 64 >> BMS;          // filter 128-bit columns one load slot covers (lanes / rows)
  constexpr int NWQ = (9 + QL - 1) / QL; // slots for the nine 128-bit columns a quad has per filter row
  extern __shared__ float lds[];
  float* const As = lds;                 // [K][SA]
  float* const Ps = lds + g.K * SA;      // [IPB * C][PL]: images with a zero halo
  int* const tab = reinterpret_cast<int*>(Ps + g.IPB * g.C * g.PL + 4);   // [16 TN] pixel offset of N entry n
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lk = lane >> 4;
  const int m0 = blockIdx.y * BM, b0 = blockIdx.x * g.IPB;
  const int nimg = min(g.IPB, g.B - b0);
  const int c0 = wave * g.CW;            // this wavefront's first channel
  float* const ftab = lds + g.epi_off;   // [4][BM] BatchNorm constants of this workgroup's filters
  if (tid < BM) conv_tail_table(tail, ftab, BM, tid, min(m0 + tid, g.F - 1));

  // ---- all global loads of this wavefront, quad by quad; slots past the end repeat the last one
  f32x4 wv[NQ][NWQ], xv[NQ][kSlotsX];
  const int wr = lane & (BM - 1), wq0 = lane >> BMS;
  const float* const wrow = w + (int64_t)min(m0 + wr, g.F - 1) * g.K + c0 * 9;
  // image rows, a plane per lane group: item (iy, j) covers columns [min(4j, W-4), +4) of row iy
  const int item = min(lane & ((1 << g.lpg_shift) - 1), g.IPP - 1);
  const int xiy = mdiv(item, g.mCH), xcol = min(4 * (item - xiy * g.CH), g.W - 4);
  const int ppw = 64 >> g.lpg_shift;     // planes per slot
  const float* const xb = x + (int64_t)b0 * g.C * g.HW + c0 * g.HW + xiy * g.W + xcol;
  const int xd0 = c0 * g.PL + (xiy + g.pad) * g.Wp + g.pad + xcol;
  int xpl[kSlotsX];                      // plane of slot u inside quad 0: image * C + channel in quad
#pragma unroll
  for (int u = 0; u < kSlotsX; u++) {
    const int j = min(u * ppw + (lane >> g.lpg_shift), 4 * nimg - 1);   // (image, channel of the quad)
    xpl[u] = (j >> 2) * g.C + (j & 3);
  }
#pragma unroll
  for (int qd = 0; qd < NQ; qd++) {
#pragma unroll
    for (int u = 0; u < NWQ; u++) wv[qd][u] = *reinterpret_cast<const f32x4_a4*>(wrow + qd * 36 + 4 * min(wq0 + u * QL, 8));
#pragma unroll
    for (int u = 0; u < kSlotsX; u++) xv[qd][u] = *reinterpret_cast<const f32x4_a4*>(xb + (xpl[u] + 4 * qd) * g.HW);
  }

  // ---- while they fly: zero this wavefront's planes, table of pixel offsets
  {
    const int per = g.CW * g.PL / 4;     // 128-bit words per image of this wavefront's planes (CW % 4 == 0)
    for (int img = 0; img < g.IPB; img++) {
      f32x4* p4 = reinterpret_cast<f32x4*>(Ps + (img * g.C + c0) * g.PL);
      for (int i = lane; i < per; i += 64) p4[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
  // one entry per thread (the workgroup has more threads than N entries), then the only barrier
  // in front of the MFMAs - every wavefront reaches it with its loads still in flight.  (Each
  // wavefront building the whole table for itself cost 4 x 25 vector instructions per wavefront,
  // and vector instructions are time the matrix pipe stands idle.)
  static_assert(NTH >= 16 * TN, "one table entry per thread");
  if (tid < 16 * TN) {
    const int n = tid;
    int img = mdiv(n, g.mPPI);
    const int r = n - img * g.ppi;
    int oy, ox;
    if (g.pool) {
      const int q = r >> 2, wp = r & 3;
      const int py = mdiv(q, g.mPW), px = q - py * g.pw;
      oy = 2 * py + (wp >> 1);
      ox = 2 * px + (wp & 1);
    } else {
      oy = mdiv(r, g.mOW);
      ox = r - oy * g.ow;
    }
    if (img >= g.IPB) { img = 0; oy = 0; ox = 0; }   // idle column: any valid address
    tab[n] = img * g.C * g.PL + oy * g.Wp + ox;
  }
  __syncthreads();
  // per-lane operand bases: one per kernel row, so the column tap is an immediate offset
  int pb[TN][3];
  {
    const int lanepart = (c0 + lk) * g.PL;
#pragma unroll
    for (int t = 0; t < TN; t++) {
      const int p = tab[t * 16 + li] + lanepart;
#pragma unroll
      for (int kr = 0; kr < 3; kr++) pb[t][kr] = p + kr * g.Wp;
    }
  }
  const float* const abase = As + (c0 + lk) * 9 * SA + li;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int t = 0; t < TN; t++) acc[a][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto stage_quad = [&](int qd) {
    float* const ad = As + (c0 * 9 + qd * 36) * SA + wr;
#pragma unroll
    for (int u = 0; u < NWQ; u++) {
      const int q = min(wq0 + u * QL, 8);
#pragma unroll
      for (int e = 0; e < 4; e++) ad[(4 * q + e) * SA] = wv[qd][u][e];
    }
#pragma unroll
    for (int u = 0; u < kSlotsX; u++) {
      float* const d = Ps + (xpl[u] + 4 * qd) * g.PL + xd0;
#pragma unroll
      for (int e = 0; e < 4; e++) d[e] = xv[qd][u][e];
    }
  };
  stage_quad(0);

  // ---- MFMA: step = (channel quad, tap); lane group lk takes channel 4 quad + lk.
  // Operands of step s + 2 are fetched while step s runs (three register sets), inside a
  // quad; one LDS read is placed after each MFMA (a block of reads in front of a block
  // of MFMAs would delay all of them).
  float af[3][TM], bf[3][TN];
  auto fetch = [&](int set, int qd, int tap) {
    const int kr = tap / 3, kc = tap % 3;
#pragma unroll
    for (int a = 0; a < TM; a++) af[set][a] = abase[(qd * 36 + tap) * SA + a * 16];
#pragma unroll
    for (int t = 0; t < TN; t++) bf[set][t] = Ps[pb[t][kr] + kc];
  };
#pragma unroll
  for (int qd = 0; qd < NQ; qd++) {
    fetch(0, qd, 0);
    fetch(1, qd, 1);
#pragma unroll
    for (int tap = 0; tap < 9; tap++) {
      if (tap + 2 < 9) fetch((tap + 2) % 3, qd, tap + 2);
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
      if (tap == 6 && qd + 1 < NQ) {
        stage_quad(qd + 1);       // its loads have had the whole quad to land
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (qd + 1 < NQ) {
#pragma unroll
      for (int t = 0; t < TN; t++)
#pragma unroll
        for (int kr = 0; kr < 3; kr++) pb[t][kr] += 4 * g.PL;
    }
  }

  __syncthreads();   // every wavefront is done reading the operands
  // ---- partial tiles to LDS, R[slot][n][MP].  Eight wavefronts fold in two rounds:
  // 4..7 write, 0..3 add those to their own and write; the epilogue adds four slots.
  float* const R = lds;
  float* const rt = R + (wave & 3) * RW + li * MP + 4 * lk;
  auto put = [&]() {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int t = 0; t < TN; t++) *reinterpret_cast<f32x4*>(rt + t * 16 * MP + a * 16) = acc[a][t];
  };
  if constexpr (WV == 8) {
    if (wave >= 4) put();
    __syncthreads();
    if (wave < 4) {
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int t = 0; t < TN; t++) acc[a][t] = acc[a][t] + *reinterpret_cast<const f32x4*>(rt + t * 16 * MP + a * 16);
      put();
    }
  } else {
    put();
  }
  __syncthreads();

  // ---- sum the four slots in order, epilogue, store: an item is four filters of one result
  // column.  What the epilogue consists of is uniform over the launch, so the item loop is
  // compiled once per combination and the combination chosen once, outside the loop.
  const int nitems = (BM / 4) * g.nout;
  const float alpha = tail.alpha;
  auto items = [&](auto bn_c, auto act_c, auto all_c) {
    constexpr bool BN = decltype(bn_c)::value;
    constexpr int ACT = decltype(act_c)::value;
    constexpr bool ALL4 = decltype(all_c)::value;   // every item's four filters exist
    for (int it = tid; it < nitems; it += NTH) {
      const int mg = mdiv(it, g.mNOUT), q = it - mg * g.nout;
      const int mf = m0 + 4 * mg;
      const int nf = ALL4 ? 4 : g.F - mf;
      if (g.pool) {
        const int pq = g.ph * g.pw;
        const int img = mdiv(q, g.mPQ), qq = q - img * pq;
        if (img >= nimg) continue;
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
            // a filter beyond F reads a table row of the last filter and is never stored
            const float v = tail_apply_fixed<BN, ACT>(ftab, BM, 4 * mg + j, s[j], alpha);
            if (v > best[j]) best[j] = v;
          }
        }
        float* yp = y + ((int64_t)(b0 + img) * g.F + mf) * pq + qq;
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (ALL4 || j < nf) yp[j * pq] = best[j];
      } else {
        const int plane = g.oh * g.ow;
        const int img = mdiv(q, g.mPPI), r = q - img * plane;
        if (img >= nimg) continue;
        const float* rp = R + q * MP + 4 * mg;
        const f32x4 s0 = *reinterpret_cast<const f32x4*>(rp);
        const f32x4 s1 = *reinterpret_cast<const f32x4*>(rp + RW);
        const f32x4 s2 = *reinterpret_cast<const f32x4*>(rp + 2 * RW);
        const f32x4 s3 = *reinterpret_cast<const f32x4*>(rp + 3 * RW);
        const f32x4 s = ((s0 + s1) + s2) + s3;
        float* yp = y + ((int64_t)(b0 + img) * g.F + mf) * plane + r;
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (ALL4 || j < nf) yp[j * plane] = tail_apply_fixed<BN, ACT>(ftab, BM, 4 * mg + j, s[j], alpha);
      }
    }
  };
  const bool all4 = m0 + BM <= g.F;
  conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
    if (all4) items(bn_c, act_c, std::true_type{}); else items(bn_c, act_c, std::false_type{});
  });
}

struct SmallPlan {
  SmallGeom g;
  int WV, TM, TN, NQ;
  size_t lds;
};

constexpr size_t kLdsBudget = 150 * 1024;        // of the 160 KB a workgroup may hold
constexpr int kTileMenu[] = {4, 7, 9, 13};       // instantiated N extents (in 16-pixel tiles)

// Geometry and workgroup shape for one command, a function of its shape and of
// `pool` only; false when the kernel does not take the shape.
bool small_plan_compute(const gh_cmd& c, bool pool, SmallPlan* out) {
  if (gh_dtype_of(c.flags) != GH_F32) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4];
  const int64_t pad = c.dim[7];
  if (c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 || c.dim[12] != 1 ||
      c.dim[8] != pad || pad < 0 || pad > 1)
    return false;
  if (B < 1 || F < 1 || C < 16 || C % 16 != 0 || C > 1024 || W < 4 || W > 16 || H < 1 || H > 16) return false;
  if (B > (1 << 20) || F > (1 << 20)) return false;
  if (getenv("GORGONIA_HIP_CONV_NO_SMALL")) return false;   // tuning switch: the general kernels only
  SmallGeom g{};
  g.B = (int)B; g.C = (int)C; g.H = (int)H; g.W = (int)W; g.F = (int)F; g.pad = (int)pad;
  g.oh = g.H + 2 * g.pad - 2; g.ow = g.W + 2 * g.pad - 2;
  if (g.oh <= 0 || g.ow <= 0) return false;
  g.pool = pool ? 1 : 0; g.ph = g.oh / 2; g.pw = g.ow / 2;
  if (pool && (g.ph == 0 || g.pw == 0)) return false;
  // the K split, and with it the order of the sum, depends on the channel count alone
  const int WV = C % 32 == 0 ? 8 : 4;
  const int NQ = g.C / (4 * WV);
  if (WV == 8 ? (NQ != 1 && NQ != 2 && NQ != 4) : NQ != 1) return false;   // C = 16, 32, 64 or 128
  g.CW = g.C / WV;
  g.Wp = g.W + 2 * g.pad; g.HW = g.H * g.W; g.K = g.C * 9;
  g.PL = (g.H + 2 * g.pad) * g.Wp;
  if ((g.PL & 1) == 0) g.PL++;   // odd pitch: the four channel planes of a fetch start in different banks
  g.CH = (g.W + 3) / 4;
  g.IPP = g.H * g.CH;
  if (g.IPP > 64) return false;
  g.lpg_shift = 0;
  while ((1 << g.lpg_shift) < g.IPP) g.lpg_shift++;
  const int ppw = 64 >> g.lpg_shift;
  g.ppi = pool ? 4 * g.ph * g.pw : g.oh * g.ow;
  // Workgroup shape: the (filters, images) pair with the smallest estimated time on 256
  // compute units - a fixed cost per workgroup round plus its MFMA time (microseconds).
  double best = 0;
  int bestTM = 0, bestIPB = 0, bestTN = 0;
  size_t best_lds = 0;
  for (int TM = 1; TM <= 2; TM++) {
    if (TM == 2 && F <= 16) continue;
    for (int IPB = 1; IPB <= ppw && IPB <= kSlotsX * ppw / 4 && IPB <= 16; IPB *= 2) {
      if (IPB > 1 && IPB / 2 >= B) break;
      const int tiles = (IPB * g.ppi + 15) / 16;
      int TN = 0;
      for (int m : kTileMenu)
        if (m >= tiles) { TN = m; break; }
      if (!TN) continue;
      const size_t stage = ((size_t)g.K * 16 * TM + (size_t)IPB * g.C * g.PL + 8 + 16 * TN) * 4;
      const size_t red = (size_t)4 * 16 * TN * (16 * TM + 4) * 4;
      const size_t lds = (stage > red ? stage : red) + (size_t)4 * 16 * TM * 4;   // + the epilogue table
      if (lds > kLdsBudget) continue;
      const int64_t blocks = ((F + 16 * TM - 1) / (16 * TM)) * ((B + IPB - 1) / IPB);
      const int coresident = lds <= 75 * 1024 ? 2 : 1;
      const int64_t rounds = (blocks + 256 * coresident - 1) / (256 * coresident);
      const double mfma_us = (WV / 4) * (double)(NQ * 9 * TM * TN) * 32.0 / 2100.0;
      // (two workgroups sharing a compute unit overlap each other's fixed cost only in part)
      const double est = rounds * (4.5 + coresident * mfma_us * 1.1);
      if (!bestTM || est < best) { best = est; bestTM = TM; bestIPB = IPB; bestTN = TN; best_lds = lds; }
    }
  }
  if (!bestTM) return false;
  g.IPB = bestIPB;
  g.epi_off = (int)(best_lds / 4) - 4 * 16 * bestTM;
  g.nout = pool ? g.IPB * g.ph * g.pw : g.IPB * g.oh * g.ow;
  g.mPPI = magic_of(g.ppi); g.mOW = magic_of(g.ow); g.mPW = magic_of(g.pw); g.mPQ = magic_of(g.ph * g.pw);
  g.mNOUT = magic_of(g.nout); g.mCH = magic_of(g.CH);
  // 128 channels and more leave LDS for only 16 filter rows of all of K: half the B-operand reuse.
  // The patch kernel stages K quad by quad and keeps 32 (128 -> 64 at 7 x 7, batch 128: 16.7 us
  // against 21.3 here); where it takes the shape, it has it.
  if (bestTM == 1 && F >= 32 && C >= 128 && gh_conv_patch_takes(c)) return false;
  out->g = g; out->WV = WV; out->TM = bestTM; out->TN = bestTN; out->NQ = NQ; out->lds = best_lds;
  return true;
}

// The plan of a command, remembered per shape.
bool small_plan(const gh_cmd& c, bool pool, SmallPlan* out) {
  return gh_plan_memo(c, pool, out, [&](SmallPlan* p) { return small_plan_compute(c, pool, p); });
}

template <int WV, int TM, int TN, int NQ>
int launch_small(gh_ctx* ctx, const gh_cmd& c, const SmallPlan& p) {
  // more than 64 KB of dynamic LDS has to be allowed per kernel, once
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    attr_rc = hipFuncSetAttribute((const void*)k_conv3x3_small<WV, TM, TN, NQ>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  if (attr_rc != hipSuccess) return gh_check_hip(ctx, attr_rc, "hipFuncSetAttribute(conv3x3 small)");
  const dim3 grid((unsigned)((p.g.B + p.g.IPB - 1) / p.g.IPB), (unsigned)((p.g.F + 16 * TM - 1) / (16 * TM)));
  hipLaunchKernelGGL((k_conv3x3_small<WV, TM, TN, NQ>), grid, dim3(WV * 64), p.lds, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], p.g, conv_tail(c));
  return gh_check_hip(ctx, hipGetLastError(), "conv3x3 small launch");
}

template <int WV, int NQ>
int launch_small_tile(gh_ctx* ctx, const gh_cmd& c, const SmallPlan& p) {
#define GH_SMALL_TN(TM_)                                                        \
  switch (p.TN) {                                                               \
    case 4: return launch_small<WV, TM_, 4, NQ>(ctx, c, p);                     \
    case 7: return launch_small<WV, TM_, 7, NQ>(ctx, c, p);                     \
    case 9: return launch_small<WV, TM_, 9, NQ>(ctx, c, p);                     \
    default: return launch_small<WV, TM_, 13, NQ>(ctx, c, p);                   \
  }
  if (p.TM == 1) { GH_SMALL_TN(1) }
  GH_SMALL_TN(2)
#undef GH_SMALL_TN
}

}  // namespace

// The small-image route is two kernels: 32 and 64 channels go to k_conv3x3_rows (k_conv_rows.hip, pixels
// on the MFMA rows, no K split for regular tiles), the other channel counts to the K-split kernel above.
// Which of the two runs depends on the command's shape alone.

// 1 when the small-image route takes this convolution (without fused pooling).
bool gh_conv_small_takes(const gh_cmd& c) {
  if (gh_conv_rows_takes(c)) return true;
  SmallPlan p;
  return small_plan(c, false, &p);
}

// 1 when it also takes it with the 2x2 pooling in its epilogue.
bool gh_conv_small_can_pool(const gh_cmd& c) {
  if (gh_conv_rows_takes(c)) return gh_conv_rows_can_pool(c);
  SmallPlan p;
  return small_plan(c, false, &p) && small_plan(c, true, &p);
}

// Returns -1 when the shape is not one this route takes.
int gh_try_launch_conv_small(gh_ctx* ctx, const gh_cmd& c) {
  const int rows = gh_try_launch_conv_rows(ctx, c);
  if (rows >= 0) return rows;
  SmallPlan p;
  const bool pool = c.flags & GH_FLAG_CONV_POOL2;
  // a pooled command only rides here when the plain one would too: both then sum in the same order
  if (!small_plan(c, false, &p)) return -1;
  if (pool && !small_plan(c, true, &p))
    return gh_fail(ctx, GH_EINVAL, "conv2d: no fused pooling for this shape (see gh_conv2d_can_pool)");
  if (p.WV == 8) {
    if (p.NQ == 1) return launch_small_tile<8, 1>(ctx, c, p);
    if (p.NQ == 2) return launch_small_tile<8, 2>(ctx, c, p);
    return launch_small_tile<8, 4>(ctx, c, p);
  }
  return launch_small_tile<4, 1>(ctx, c, p);
}
