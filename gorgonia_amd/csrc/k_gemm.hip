// fp32 MFMA contractions for gfx950: SGEMM / strided-batched GEMM and Conv2d
// as implicit GEMM, plus GEMV and the outer product.
//
// Replaces cuBLAS Sgemm/Sgemv/Sger (cuda/linalg.go:102,223,282), the host loop
// of per-slice Sgemm calls behind BatchedMatMul (operatorLinAlg.go:435-502) and
// cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117).
//
// Tiling (one workgroup = 4 wavefronts of 64 lanes):
//   block tile BM x BN, K step BK; LDS holds both operands k-major
//   (As[k][m], Bs[k][n]) so that a v_mfma_f32_32x32x2f32 operand fetch is one
//   conflict-free ds_read_b32 per lane (lane l reads [k0 + l/32][x0 + l%32]);
//   each wavefront owns a (BM/2) x (BN/2) sub-tile = TM x TN MFMA tiles whose
//   accumulators stay in registers for the whole K loop;
//   global->register prefetch of tile k+1 overlaps the MFMAs on tile k, and
//   LDS is double buffered so the loop needs one barrier per K step.
//
// Conv2d uses the same core with M = filters, N = B*oh*ow output pixels,
// K = C*kh*kw: the "B" operand is gathered straight from the NCHW input (no
// im2col buffer) and the result is written straight into NCHW (no transpose
// pass), so lanes run along output pixels for coalesced loads and stores.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "gh_internal.h"
#include "gh_conv_common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
// the same four floats at any 4-byte aligned address (one 128-bit load all the same)
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;

// ---- operand loaders ---------------------------------------------------------
// A loader moves one R x BK (or BK x R) operand tile: load() global->registers,
// store() registers->LDS in k-major order with row stride S.

// What a thread's slots have in common - its row inside the tile, its k offset, the address of
// its first element - is computed once per tile in prep(); a load then costs two compares and
// one 64-bit add of a wavefront-uniform offset per slot.  (Vector instructions in this loop are
// time the matrix pipe stands idle; recomputing row, column, address and LDS index per slot and
// k-tile was 1.9 of them per MFMA.)

// Operand stored [r][k] with k contiguous (A not transposed; B transposed).
template <int R, int BK, bool VEC>
struct LoadKContig {
  static constexpr int S = R + 2;  // S % 32 == 2 keeps the transposing writes conflict-free
  static constexpr int TOTAL = R * BK / 4;  // float4 slots in a tile
  static constexpr int NV = (TOTAL + kThreads - 1) / kThreads;
  static constexpr int RS = kThreads / (BK / 4);   // rows between a thread's slots
  static_assert(kThreads % (BK / 4) == 0, "a thread's slots share their k offset");
  const float* base; int ld; int rmax; int kmax;
  const float* p0;   // first slot's element at k = 0
  int rrel, kq;      // first slot's row (absolute), k offset inside a tile
  f32x4 reg[NV];
  __device__ __forceinline__ void prep(int r0) {
    rrel = r0 + (int)threadIdx.x / (BK / 4);
    kq = ((int)threadIdx.x % (BK / 4)) * 4;
    p0 = base + (int64_t)rrel * ld + kq;
  }
  __device__ __forceinline__ void load(int, int k0) {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if ((TOTAL % kThreads == 0 || (int)threadIdx.x + j * kThreads < TOTAL) && rrel < rmax - j * RS) {
        const float* p = p0 + ((int64_t)(j * RS) * ld + k0);
        if (VEC) {
          if (kq < kmax - k0) v = *reinterpret_cast<const f32x4*>(p);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) if (kq + e < kmax - k0) v[e] = p[e];
        }
      }
      reg[j] = v;
    }
  }
  __device__ __forceinline__ void store(float* lds) const {
    float* const d = lds + kq * S + (int)threadIdx.x / (BK / 4);
#pragma unroll
    for (int j = 0; j < NV; j++) {
      if (TOTAL % kThreads != 0 && (int)threadIdx.x + j * kThreads >= TOTAL) continue;
#pragma unroll
      for (int e = 0; e < 4; e++) d[e * S + j * RS] = reg[j][e];
    }
  }
};

// Operand stored [k][c] with c contiguous (B not transposed; A transposed).
template <int R, int BK, bool VEC>
struct LoadMnContig {
  static constexpr int S = R;
  static constexpr int TOTAL = R * BK / 4;
  static constexpr int NV = (TOTAL + kThreads - 1) / kThreads;
  static constexpr int KS = kThreads / (R / 4);    // k rows between a thread's slots
  static_assert(kThreads % (R / 4) == 0, "a thread's slots share their column");
  const float* base; int ld; int rmax; int kmax;
  const float* p0;   // first slot's element at k0 = 0
  int c, kl;         // the thread's first column (absolute), first slot's k row inside a tile
  f32x4 reg[NV];
  __device__ __forceinline__ void prep(int c0) {
    kl = (int)threadIdx.x / (R / 4);
    c = c0 + ((int)threadIdx.x % (R / 4)) * 4;
    p0 = base + (int64_t)kl * ld + c;
  }
  __device__ __forceinline__ void load(int, int k0) {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if ((TOTAL % kThreads == 0 || (int)threadIdx.x + j * kThreads < TOTAL) && kl < kmax - k0 - j * KS) {
        const float* p = p0 + (int64_t)(k0 + j * KS) * ld;
        if (VEC) {
          if (c < rmax) v = *reinterpret_cast<const f32x4*>(p);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) if (c + e < rmax) v[e] = p[e];
        }
      }
      reg[j] = v;
    }
  }
  __device__ __forceinline__ void store(float* lds) const {
    float* const d = lds + ((int)threadIdx.x / (R / 4)) * S + ((int)threadIdx.x % (R / 4)) * 4;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      if (TOTAL % kThreads != 0 && (int)threadIdx.x + j * kThreads >= TOTAL) continue;
      *reinterpret_cast<f32x4*>(&d[j * KS * S]) = reg[j];
    }
  }
};

// im2col gather for Conv2d: logical operand [k][p], k = (c, kr, kc) in the
// reference's order (op_nn.go:418-437), p = (b, oy, ox).  Each thread keeps
// one output pixel for the whole kernel and walks k.  What depends only on
// the pixel - its base offset and which of the kh*kw taps fall inside the
// image - is computed once; per element only k -> (c, tap) remains.
// KH/KW > 0 are compile-time kernel sizes; 0 means "use the runtime values".
struct ConvGeom {
  int C, H, W, oh, ow, kh, kw, padH, padW, strideH, strideW, dilH, dilW, P /* B*oh*ow */;
};

template <int R, int BK, int KH, int KW>
struct LoadIm2col {
  static constexpr int S = R;
  static constexpr int KSTEP = kThreads / R;  // k distance between a thread's elements
  static constexpr int KPT = BK / KSTEP;      // k values per thread per tile
  const float* x; ConvGeom g; int kmax;
  int pix_off;          // offset of the window's (0,0) tap inside the batch item; may be negative
  int iy0, ix0;
  uint64_t tap_mask;    // bit r set: tap r = kr*kw + kc lies inside the image
  const float* xb;
  float reg[KPT];
  __device__ __forceinline__ void prep(int) {}
  __device__ __forceinline__ void init(int p0) {
    const int kh = KH ? KH : g.kh, kw = KW ? KW : g.kw;
    const int p = p0 + (threadIdx.x % R);
    const bool ok = p < g.P;
    const int pp = ok ? p : 0;
    const int b = pp / (g.oh * g.ow);
    const int rem = pp - b * (g.oh * g.ow);
    const int oy = rem / g.ow, ox = rem - oy * g.ow;
    iy0 = oy * g.strideH - g.padH;
    ix0 = ox * g.strideW - g.padW;
    pix_off = iy0 * g.W + ix0;
    xb = x + (int64_t)b * g.C * g.H * g.W;
    tap_mask = 0;
    if (ok && kh * kw <= 64) {
      for (int kr = 0; kr < kh; kr++)
        for (int kc = 0; kc < kw; kc++) {
          const int iy = iy0 + kr * g.dilH, ix = ix0 + kc * g.dilW;
          if (iy >= 0 && iy < g.H && ix >= 0 && ix < g.W) tap_mask |= 1ull << (kr * kw + kc);
        }
    }
    if (!ok) kmax = 0;  // out-of-range pixel: every element reads as zero
  }
  __device__ __forceinline__ void load(int /*p0*/, int k0) {
    const int kh = KH ? KH : g.kh, kw = KW ? KW : g.kw;
    const int kk = kh * kw;
    const int kb = threadIdx.x / R;
    const int HW = g.H * g.W;
#pragma unroll
    for (int j = 0; j < KPT; j++) {
      const int k = k0 + kb + j * KSTEP;
      float v = 0.f;
      if (k < kmax) {
        const int c = k / kk;
        const int r = k - c * kk;
        const int kr = r / kw, kc = r - kr * kw;
        bool in;
        if (kk <= 64) in = (tap_mask >> r) & 1;
        else {
          const int iy = iy0 + kr * g.dilH, ix = ix0 + kc * g.dilW;
          in = iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
        }
        if (in) v = xb[c * HW + kr * g.dilH * g.W + kc * g.dilW + pix_off];
      }
      reg[j] = v;
    }
  }
  __device__ __forceinline__ void store(float* lds) const {
    const int kb = threadIdx.x / R, pl = threadIdx.x % R;
#pragma unroll
    for (int j = 0; j < KPT; j++) lds[(kb + j * KSTEP) * S + pl] = reg[j];
  }
};

// ---- result writers ------------------------------------------------------------
struct StoreRowMajor {
  float* C; int ldc;
  __device__ __forceinline__ float pre(int, float v) const { return v; }
  __device__ __forceinline__ void put(int i, int j, float v) const { C[(int64_t)i * ldc + j] = v; }
};

// The same with a row vector added to every row of the product before the
// activation (a dense layer's bias).  A type of its own: the tiled kernel is
// tight on registers, and even a never-taken bias branch in its epilogue cost
// 3 % at 4096^3 and 7 % on the batched product.
struct StoreRowMajorBias {
  float* C; int ldc;
  const float* bias;
  __device__ __forceinline__ float pre(int j, float v) const { return v + bias[j]; }
  __device__ __forceinline__ void put(int i, int j, float v) const { C[(int64_t)i * ldc + j] = v; }
};

// Conv result: row i = filter, column j = output pixel (b, oy, ox) -> NCHW.
struct StoreNCHW {
  float* y; int F; int plane /* oh*ow */;
  ConvTail tail;
  __device__ __forceinline__ float pre(int, float v) const { return v; }
  __device__ __forceinline__ void put(int i, int j, float v) const {
    const int b = j / plane, p = j - b * plane;
    y[((int64_t)b * F + i) * plane + p] = tail_apply(tail, i, v);
  }
};

// Split-K partial sums: slab `split` of a [splits][M][N] workspace.
struct StorePartial {
  float* ws; int N;
  __device__ __forceinline__ float pre(int, float v) const { return v; }
  __device__ __forceinline__ void put(int i, int j, float v) const { ws[(int64_t)i * N + j] = v; }
};

// ---- the MFMA core ---------------------------------------------------------------
// WAVES_M x WAVES_N wavefronts (4 in all) tile the BM x BN block; k-tiles
// [kt0, kt1) are accumulated (a split-K slice, or the whole K range).
template <int BM, int BN, int BK, int WAVES_M, class LA, class LB, class SC>
__device__ __forceinline__ void mfma_tile_loop(float* lds, LA& la, LB& lb, const SC& sc, int M, int N,
                                               int kt0, int kt1, int m0, int n0, int act, float alpha) {
  constexpr int WAVES_N = 4 / WAVES_M;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;    // MFMA tiles per wavefront
  static_assert(TM >= 1 && TN >= 1 && WM % 32 == 0 && WN % 32 == 0, "bad wave tiling");
  constexpr int SA = LA::S, SB = LB::S;
  float* const As = lds;                 // two buffers of BK * SA floats
  float* const Bs = lds + 2 * BK * SA;   // two buffers of BK * SB floats

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
  const int lr = lane & 31, lk = lane >> 5;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

  la.prep(m0);
  lb.prep(n0);
  la.load(m0, kt0 * BK);
  lb.load(n0, kt0 * BK);
  la.store(As);
  lb.store(Bs);
  __syncthreads();

  for (int kt = kt0; kt < kt1; kt++) {
    const int cur = (kt - kt0) & 1;
    const bool more = kt + 1 < kt1;
    if (more) {
      la.load(m0, (kt + 1) * BK);
      lb.load(n0, (kt + 1) * BK);
    }
    const float* a_s = As + cur * (BK * SA) + wm + lr;
    const float* b_s = Bs + cur * (BK * SB) + wn + lr;
    // operand fragments are fetched kAhead k-steps ahead of the MFMAs that use
    // them (an LDS read outlasts one MFMA); the scheduling barriers keep the
    // compiler from sinking the reads back to their uses
    constexpr int kSteps = BK / 2, kAhead = (TM * TN >= 4) ? 2 : 4, kRing = 8;
    float af[kRing][TM], bf[kRing][TN];
    auto fetch = [&](int st) {
#pragma unroll
      for (int a = 0; a < TM; a++) af[st % kRing][a] = a_s[(2 * st + lk) * SA + a * 32];
#pragma unroll
      for (int b = 0; b < TN; b++) bf[st % kRing][b] = b_s[(2 * st + lk) * SB + b * 32];
    };
#pragma unroll
    for (int st = 0; st < kAhead && st < kSteps; st++) fetch(st);
#pragma unroll
    for (int st = 0; st < kSteps; st++) {
      if (st + kAhead < kSteps) fetch(st + kAhead);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[st % kRing][a], bf[st % kRing][b], acc[a][b], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) {
      la.store(As + (cur ^ 1) * (BK * SA));
      lb.store(Bs + (cur ^ 1) * (BK * SB));
    }
    __syncthreads();
  }

  // Accumulator layout of v_mfma_f32_32x32x2f32: lane l holds column l%32 and,
  // in register v, row 8*(v/4) + 4*(l/32) + v%4.
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int i = m0 + wm + a * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
#pragma unroll
      for (int b = 0; b < TN; b++) {
        const int j = n0 + wn + b * 32 + lr;
        if (i < M && j < N) sc.put(i, j, act_apply(sc.pre(j, acc[a][b][v]), act, alpha));
      }
    }
}

// k-tile range of split `s` out of `splits` over nk tiles.
__device__ __forceinline__ void split_range(int nk, int splits, int s, int* kt0, int* kt1) {
  const int per = (nk + splits - 1) / splits;
  *kt0 = s * per;
  *kt1 = min(nk, *kt0 + per);
}

// Which output tile a workgroup computes.  Workgroup ids are dealt round-robin
// over the 8 XCDs, each with its own L2, so ids are first regrouped to give
// every XCD one contiguous range of tiles; inside a range, tiles are walked in
// groups of 8 tile-rows so that co-resident workgroups share A rows and B
// columns (a plain row-major walk re-read A and B ~6x from HBM at 4096^3).
// For a batch of products (`batched`: blockIdx.z counts matrices) the regrouping
// runs over the whole launch instead, so that an XCD works through whole
// matrices and each operand tile enters one L2 only; *bz is the matrix.
__device__ __forceinline__ void tile_coords(int* tm, int* tn, int* bz, bool batched) {
  const int gx = gridDim.x, gy = gridDim.y;  // tiles along N, along M
  const int total = gx * gy;
  int id = blockIdx.y * gx + blockIdx.x;
  constexpr int kXcd = 8, kGroup = 8;
  *bz = blockIdx.z;
  if (batched) {
    const int all = total * (int)gridDim.z;
    if (all % kXcd == 0) {
      const int lin = (int)blockIdx.z * total + id;
      const int nid = (lin % kXcd) * (all / kXcd) + lin / kXcd;
      *bz = nid / total;
      id = nid - *bz * total;
    }
  } else if (total % kXcd == 0) {
    id = (id % kXcd) * (total / kXcd) + id / kXcd;
  }
  const int per_group = kGroup * gx;
  const int first_m = (id / per_group) * kGroup;
  const int gsz = min(gy - first_m, kGroup);
  const int in_group = id % per_group;
  *tm = first_m + in_group % gsz;
  *tn = in_group / gsz;
}

// blockIdx.z is the batch index (splits == 1) or the split-K slice (batch == 1).
template <int BM, int BN, int BK, int WAVES_M, bool TA, bool TB, bool VEC, bool BIAS = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(BM == 128 && BN == 128 ? 4 : 1))) void k_sgemm(const float* __restrict__ A,
                                                    const float* __restrict__ B,
                                                    float* __restrict__ C, int M, int N, int K,
                                                    int lda, int ldb, int ldc, int64_t sA,
                                                    int64_t sB, int64_t sC, int act, float alpha,
                                                    int splits, float* __restrict__ ws,
                                                    const float* __restrict__ bias) {
  using LA = typename std::conditional<TA, LoadMnContig<BM, BK, VEC>, LoadKContig<BM, BK, VEC>>::type;
  using LB = typename std::conditional<TB, LoadKContig<BN, BK, VEC>, LoadMnContig<BN, BK, VEC>>::type;
  const int nk = (K + BK - 1) / BK;
  int tile_m, tile_n, bz;
  tile_coords(&tile_m, &tile_n, &bz, splits <= 1 && gridDim.z > 1);

  // one LDS allocation shared by both call sites below (a static array inside
  // the tile loop would be instantiated once per call site)
  __shared__ float lds[2 * BK * (LA::S + LB::S)];
  if (splits > 1) {
    int kt0, kt1;
    split_range(nk, splits, bz, &kt0, &kt1);
    LA la; la.base = A; la.ld = lda; la.rmax = M; la.kmax = K;
    LB lb; lb.base = B; lb.ld = ldb; lb.rmax = N; lb.kmax = K;
    StorePartial sc{ws + (int64_t)bz * M * N, N};
    mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StorePartial>(lds, la, lb, sc, M, N, kt0, kt1,
                                                              tile_m * BM, tile_n * BN, 0, 0.f);
  } else {
    LA la; la.base = A + bz * sA; la.ld = lda; la.rmax = M; la.kmax = K;
    LB lb; lb.base = B + bz * sB; lb.ld = ldb; lb.rmax = N; lb.kmax = K;
    if constexpr (BIAS) {
      StoreRowMajorBias sc{C + bz * sC, ldc, bias};
      mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StoreRowMajorBias>(lds, la, lb, sc, M, N, 0, nk, tile_m * BM,
                                                                     tile_n * BN, act, alpha);
    } else {
      StoreRowMajor sc{C + bz * sC, ldc};
      mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StoreRowMajor>(lds, la, lb, sc, M, N, 0, nk, tile_m * BM,
                                                                 tile_n * BN, act, alpha);
    }
  }
}

template <int BM, int BN, int BK, int WAVES_M, int KH, int KW, bool VEC>
__global__ __launch_bounds__(kThreads) void k_conv2d(const float* __restrict__ x,
                                                     const float* __restrict__ w,
                                                     float* __restrict__ y, ConvGeom g, int F, int K,
                                                     ConvTail tail, int splits,
                                                     float* __restrict__ ws) {
  using LA = LoadKContig<BM, BK, VEC>;
  using LB = LoadIm2col<BN, BK, KH, KW>;
  LA la; la.base = w; la.ld = K; la.rmax = F; la.kmax = K;
  LB lb; lb.x = x; lb.g = g; lb.kmax = K;
  const int n0 = blockIdx.x * BN;
  lb.init(n0);
  const int nk = (K + BK - 1) / BK;
  __shared__ float lds[2 * BK * (LA::S + LB::S)];
  if (splits > 1) {
    int kt0, kt1;
    split_range(nk, splits, blockIdx.z, &kt0, &kt1);
    StorePartial sc{ws + (int64_t)blockIdx.z * F * g.P, g.P};
    mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StorePartial>(lds, la, lb, sc, F, g.P, kt0, kt1,
                                                              blockIdx.y * BM, n0, 0, 0.f);
  } else {
    StoreNCHW sc{y, F, g.oh * g.ow, tail};
    mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StoreNCHW>(lds, la, lb, sc, F, g.P, 0, nk, blockIdx.y * BM,
                                                           n0, 0, 0.f);
  }
}

// Sum the split-K slabs in slab order (deterministic), apply the epilogue and
// write through the same result writer as the unsplit kernel.
template <class SC>
__global__ __launch_bounds__(256) void k_splitk_reduce(const float* __restrict__ ws, int splits, int M,
                                                       int N, SC sc, int act, float alpha) {
  const int64_t total = (int64_t)M * N, stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    float acc = ws[e];
    for (int s = 1; s < splits; s++) acc = acc + ws[(int64_t)s * total + e];
    const int i = (int)(e / N), j = (int)(e - (int64_t)i * N);
    sc.put(i, j, act_apply(sc.pre(j, acc), act, alpha));
  }
}

// Many slabs, few results (filter gradients): L lanes share one result (4, or 16 from 64
// slabs up).  Lane q adds slabs q, q+L, q+2L, ... in that order, then the L sums are
// combined pairwise, neighbours first: (s0 + s1) + (s2 + s3), ... - a fixed order, so
// results repeat.
template <class SC, int L>
__global__ __launch_bounds__(256) void k_splitk_reduce_lanes(const float* __restrict__ ws, int splits, int M,
                                                        int N, SC sc, int act, float alpha) {
  const int64_t total = (int64_t)M * N;
  const int q = threadIdx.x & (L - 1);
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) / L;
  float acc = 0.f;
  if (e < total) {
    const float* p = ws + (int64_t)q * total + e;
    int s = q;
    for (; s + 3 * L < splits; s += 4 * L) {   // four loads in flight
      const float v0 = p[0], v1 = p[(int64_t)L * total], v2 = p[2 * (int64_t)L * total], v3 = p[3 * (int64_t)L * total];
      acc = acc + v0; acc = acc + v1; acc = acc + v2; acc = acc + v3;
      p += 4 * (int64_t)L * total;
    }
    for (; s < splits; s += L) { acc = acc + p[0]; p += (int64_t)L * total; }
  }
  float sum = acc;
#pragma unroll
  for (int d = 1; d < L; d <<= 1) sum = sum + __shfl_xor(sum, d, 64);   // commutative per level: every lane ends with the total
  if (e < total && q == 0) {
    const int i = (int)(e / N), j = (int)(e - (int64_t)i * N);
    sc.put(i, j, act_apply(sc.pre(j, sum), act, alpha));
  }
}

// ---- small-output GEMM: the K range is split across the wavefronts of one block ------
// C(M x N) = A(M x K) B(K x N), both row-major, for products whose output has
// too few 32x32 tiles to fill the chip when each tile walks all of K.  One
// workgroup of WV wavefronts owns one 32x32 tile; wavefront w takes the 16-wide
// k-chunks w, w + WV, ... with operands loaded straight from global memory in
// MFMA lane order (every element is used once per tile, so LDS staging buys
// nothing), then the WV partial tiles are summed through LDS in wavefront order
// - a fixed order, so results repeat bit for bit - and the epilogue is applied.
// (Cutting K across workgroups as well, with the last one to arrive at a
// per-tile counter adding the slices, was measured: the device-wide fences it
// needs cost ~35 us per launch on this part, four times the whole kernel.)
template <int WV, bool VEC, bool VECB>
__global__ __launch_bounds__(WV * 64) void k_gemm_skinny(const float* __restrict__ A,
                                                         const float* __restrict__ B,
                                                         float* __restrict__ C, int M, int N, int K,
                                                         int lda, int ldb, int ldc, int act,
                                                         float alpha, int softmax,
                                                         const float* __restrict__ bias) {
  constexpr int G = 5;                       // k-chunks per group; two groups of loads are in flight
  constexpr int HALF = WV / 2;
  __shared__ float part[HALF * 1024];
  // the wavefront index as a scalar: every branch on chunk numbers below is then
  // a scalar branch, and a load in one arm does not look pending in the other
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 31, h = lane >> 5;
  // VECB (N >= 32): the last column tile is moved left to end at column N, so
  // every tile is whole; the columns it shares with its neighbour get the same
  // bits from both (a column's sum does not depend on the tile it sits in).
  const int m0 = blockIdx.y * 32, n0 = VECB ? min((int)blockIdx.x * 32, N - 32) : blockIdx.x * 32;
  const int m = m0 + r, n = n0 + r;
  const int nchunks = (K + 15) / 16;

  // Lane (r, h) feeds k = 16*chunk + 8*h + t at MFMA step t of a chunk.  B comes
  // in that order straight from memory (32 consecutive columns per k).  A would
  // be one row per lane - 64 cache lines per load instruction - so a chunk of A
  // (32 rows x 16 k) is loaded with k fastest across lanes and turned into MFMA
  // order through a wavefront-private LDS tile just before use.  Loads never
  // branch per lane: rows, columns and k past the matrix are clamped to the
  // last valid one and replaced by zero just before the MFMA, so nothing makes
  // the compiler wait for one load before it issues the next.
  // The texture addresser takes a wavefront's load instruction at four lanes per
  // clock whatever its width, so B read as eight one-float loads per chunk held
  // a compute unit to ~16 bytes per clock; with VECB a chunk of B (16 k x 32
  // columns) is two 128-bit loads per lane (lane = (k row, column quad)) and goes
  // through a second wavefront-private LDS tile into the same MFMA order.
  constexpr int TP = 20;                     // pitch of the transposing tile: rows stay 16-byte aligned
  __shared__ __attribute__((aligned(16))) float tbuf[WV][32 * TP];
  __shared__ float sm_x[32 * 33], sm_e[32 * 33];   // the tile and its exponentials when a softmax follows
  constexpr int TPB = 36;                    // pitch of the B tile: 16-byte aligned rows, conflict-free both ways
  __shared__ __attribute__((aligned(16))) float tbufb[VECB ? WV : 1][16 * TPB];
  float* const T = tbuf[wave];
  float* const TB = tbufb[VECB ? wave : 0];
  const float* const b_vec = B + n0 + (lane & 7) * 4;   // row k0 + (lane >> 3), and 8 rows further down
  const int n_c = min(n, N - 1);
  const float* const a_vec = A + (int64_t)min(m0 + (lane >> 2), M - 1) * lda + (lane & 3) * 4;   // + 16 rows for the second load
  const int64_t a_vec_step = (int64_t)(min(m0 + 16 + (lane >> 2), M - 1) - min(m0 + (lane >> 2), M - 1)) * lda;
  auto load = [&](int chunk, float (&a)[8], float (&b)[8]) {
    if (VEC) {   // 16-byte aligned rows and K a multiple of 16: every chunk is whole
      const f32x4 lo = *reinterpret_cast<const f32x4*>(a_vec + chunk * 16);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(a_vec + a_vec_step + chunk * 16);
#pragma unroll
      for (int t = 0; t < 4; t++) { a[t] = lo[t]; a[4 + t] = hi[t]; }
    } else {
      const int kk = min(chunk * 16 + (lane & 15), K - 1);
#pragma unroll
      for (int t = 0; t < 8; t++) a[t] = A[(int64_t)min(m0 + t * 4 + (lane >> 4), M - 1) * lda + kk];
    }
    if (VECB) {
      const int kr = chunk * 16 + (lane >> 3);
      const f32x4 lo = *reinterpret_cast<const f32x4_a4*>(b_vec + (int64_t)min(kr, K - 1) * ldb);
      const f32x4 hi = *reinterpret_cast<const f32x4_a4*>(b_vec + (int64_t)min(kr + 8, K - 1) * ldb);
#pragma unroll
      for (int t = 0; t < 4; t++) { b[t] = lo[t]; b[4 + t] = hi[t]; }
    } else {
      const int k0 = chunk * 16 + 8 * h;
#pragma unroll
      for (int t = 0; t < 8; t++) b[t] = B[(int64_t)min(k0 + t, K - 1) * ldb + n_c];
    }
  };
  // load order -> MFMA order, in place
  auto transpose_a = [&](int chunk, float (&a)[8]) {
    if (VEC) {
      f32x4 lo = {a[0], a[1], a[2], a[3]}, hi = {a[4], a[5], a[6], a[7]};
      *reinterpret_cast<f32x4*>(T + (lane >> 2) * TP + (lane & 3) * 4) = lo;
      *reinterpret_cast<f32x4*>(T + (16 + (lane >> 2)) * TP + (lane & 3) * 4) = hi;
    } else {
#pragma unroll
      for (int t = 0; t < 8; t++) T[(t * 4 + (lane >> 4)) * TP + (lane & 15)] = a[t];
    }
    const f32x4 lo = *reinterpret_cast<const f32x4*>(T + r * TP + 8 * h);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(T + r * TP + 8 * h + 4);
#pragma unroll
    for (int t = 0; t < 4; t++) { a[t] = lo[t]; a[4 + t] = hi[t]; }
  };
  auto transpose_b = [&](float (&b)[8]) {
    if (!VECB) return;
    f32x4 lo = {b[0], b[1], b[2], b[3]}, hi = {b[4], b[5], b[6], b[7]};
    *reinterpret_cast<f32x4*>(TB + (lane >> 3) * TPB + (lane & 7) * 4) = lo;
    *reinterpret_cast<f32x4*>(TB + (8 + (lane >> 3)) * TPB + (lane & 7) * 4) = hi;
#pragma unroll
    for (int t = 0; t < 8; t++) b[t] = TB[(8 * h + t) * TPB + r];
  };
  // group = chunks c, c + WV, ... (G of them); the chunk order per wavefront is
  // fixed, so the sum is the same whatever the grouping
  auto load_group = [&](int c, float (&a)[G][8], float (&b)[G][8]) {
#pragma unroll
    for (int g = 0; g < G; g++)
      if (c + g * WV < nchunks) load(c + g * WV, a[g], b[g]);
  };
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; v++) acc[v] = 0.f;
  auto mfma_group = [&](int c, float (&a)[G][8], float (&b)[G][8]) {
#pragma unroll
    for (int g = 0; g < G; g++)
      if (c + g * WV < nchunks) {
        transpose_a(c + g * WV, a[g]);
        transpose_b(b[g]);
        const int left = K - ((c + g * WV) * 16 + 8 * h);   // valid k of this lane's eight
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const float av = (m < M && t < left) ? a[g][t] : 0.f;
          const float bv = (n < N && t < left) ? b[g][t] : 0.f;
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
        }
      }
  };

  // The MFMAs of one group form a dependent chain of 8*G*64 cycles; the next
  // group's loads are issued before it so their latency runs underneath.
  float a0[G][8], b0[G][8], a1[G][8], b1[G][8];
  int c0 = wave;
  if (c0 < nchunks) load_group(c0, a0, b0);
  while (c0 < nchunks) {
    const int c1 = c0 + G * WV;
    if (c1 < nchunks) load_group(c1, a1, b1);
    mfma_group(c0, a0, b0);
    if (c1 >= nchunks) break;
    c0 = c1 + G * WV;
    if (c0 < nchunks) load_group(c0, a0, b0);
    mfma_group(c1, a1, b1);
  }
  // upper half of the wavefronts hands its tiles to the lower half, then the
  // HALF sums are added in wavefront order
  if (wave >= HALF) {
#pragma unroll
    for (int v = 0; v < 16; v++) part[((wave - HALF) * 16 + v) * 64 + lane] = acc[v];
  }
  __syncthreads();
  if (wave < HALF) {
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int at = (wave * 16 + v) * 64 + lane;
      part[at] = acc[v] + part[at];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 1024; e += WV * 64) {
    float sum = part[e];
#pragma unroll
    for (int w = 1; w < HALF; w++) sum = sum + part[w * 1024 + e];
    const int v = e >> 6, l = e & 63;
    const int il = 8 * (v / 4) + 4 * (l >> 5) + (v % 4), jl = l & 31;
    const int i = m0 + il, j = n0 + jl;
    if (bias && j < N) sum = sum + bias[j];
    if (softmax) sm_x[il * 33 + jl] = act_apply(sum, act, alpha);
    else if (i < M && j < N) C[(int64_t)i * ldc + j] = act_apply(sum, act, alpha);
  }
  if (!softmax) return;
  // Row softmax of the tile (N <= 32: the tile holds whole rows) with the
  // arithmetic of the softmax kernel: max, exp(x - max) in float64 rounded
  // once, the sum taken in column order, one rounded reciprocal.
  __syncthreads();
  for (int e = threadIdx.x; e < 1024; e += WV * 64) {
    const int il = e >> 5, jl = e & 31;
    float mx = -INFINITY;
    for (int j = 0; j < N; j++) mx = fmaxf(mx, sm_x[il * 33 + j]);
    sm_e[il * 33 + jl] = jl < N ? (float)exp((double)(sm_x[il * 33 + jl] - mx)) : 0.f;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 1024; e += WV * 64) {
    const int il = e >> 5, jl = e & 31;
    float sum = 0.f;
    for (int j = 0; j < N; j++) sum = sum + sm_e[il * 33 + j];
    const float inv = 1.0f / sum;
    if (m0 + il < M && jl < N) C[(int64_t)(m0 + il) * ldc + jl] = sm_e[il * 33 + jl] * inv;
  }
}

// ---- small-output GEMM on 16-row tiles -----------------------------------------------
// A compute unit keeps only so many cache lines in flight, which holds one
// workgroup to ~40 GB/s of operand fill however its loads are written (measured
// on the 32x32 kernel above), so a product whose 32x32 tiles cover a fraction of
// the chip is bounded by the number of compute units it touches.  This kernel
// cuts the output into tiles of 16 rows by 16*NT columns (two to four times as
// many workgroups) on the 16x16x4 MFMA; the K split over the wavefronts of a
// block and the fixed-order sum of their partial tiles are those of
// k_gemm_skinny.  Lane l = (i = l % 16, q = l / 16) owns k = 16*chunk + 4*q + t
// at MFMA step t: its four A values are one 128-bit load of row i, already in
// MFMA order; of B it takes, per k, the NT adjacent columns n0 + NT*i + c (one
// load of NT floats; with NT = 2 sixteen lanes cover one whole 128-byte line)
// and column set c feeds accumulator c.  The last tile in each direction is
// moved back to end at the matrix edge (M >= 16, N >= 16*NT), so no row or
// column is ever masked; k past K is clamped in the address and zeroed before
// the MFMA.
// TA / TB: the operand is a transposed view (A stored k x m, B stored n x k, as
// for k_sgemm); the lane's four k-values are then four loads for A and one
// 128-bit load for B instead of the other way round.  N < 16 (NT = 1 only;
// transposed views alone reach here with so few columns): one column tile,
// column indices clamped in the loads and masked in the store.
template <int WV, int NT, bool TA, bool TB>
__global__ __launch_bounds__(WV * 64) void k_gemm_skinny16(const float* __restrict__ A,
                                                           const float* __restrict__ B,
                                                           float* __restrict__ C, int M, int N, int K,
                                                           int lda, int ldb, int ldc, int act, float alpha,
                                                           const float* __restrict__ bias, int softmax) {
  constexpr int G = NT == 1 ? 5 : 4;
  constexpr int BN = 16 * NT, TILE = 16 * BN;
  typedef float bvec __attribute__((ext_vector_type(NT), aligned(4)));
  __shared__ float part[WV * TILE];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 15, q = lane >> 4;
  const bool ragged_n = N < BN;
  // Workgroup ids are dealt round-robin over the 8 XCDs, each with its own L2.
  // Regroup them so that one XCD gets a contiguous run of ids, and walk a run
  // row-tile fastest: every row tile of a column tile then reads that strip of
  // B (the weights, the big operand of a dense layer) through the same L2, once
  // from memory, instead of once per XCD.
  int tile_x, tile_y;
  {
    const int gx = gridDim.x, gy = gridDim.y, total = gx * gy;
    const int id = blockIdx.y * gx + blockIdx.x;
    const int xcd = id & 7, per = total >> 3, extra = total & 7;
    const int nid = xcd * per + min(xcd, extra) + (id >> 3);
    tile_x = nid / gy;
    tile_y = nid - tile_x * gy;
  }
  const int m0 = min(tile_y * 16, M - 16), n0 = ragged_n ? 0 : min(tile_x * BN, N - BN);
  const int nchunks = (K + 15) / 16;
  int ncol[NT];   // this lane's columns (clamped when the tile is wider than the matrix)
#pragma unroll
  for (int c = 0; c < NT; c++) ncol[c] = min(n0 + NT * i + c, N - 1);
  // k runs along the row of an untransposed A and of a transposed B
  const float* const a_base = TA ? A + m0 + i : A + (int64_t)(m0 + i) * lda;
  // The lane's quad of chunk `chunk` starts at k0 = 16*chunk + 4*q; a quad that
  // would stick out past K starts at K-4 instead, and its elements below k0
  // (which the quad before it already covers) are zeroed before the MFMA.  So
  // element t always stands for k = kb + t with kb = min(k0, K-4): every load is
  // unconditional, k-contiguous operands are one 128-bit load at any 4-byte
  // aligned address, and no loaded value is touched under a branch (which would
  // make each load wait for the one before it).
  auto load_k4 = [&](const float* row, int kb, float (&dst)[4]) {
    const f32x4 v = *reinterpret_cast<const f32x4_a4*>(row + kb);
#pragma unroll
    for (int t = 0; t < 4; t++) dst[t] = v[t];
  };
  auto load = [&](int chunk, float (&a)[4], float (&b)[4][NT]) {
    const int kb = min(chunk * 16 + 4 * q, K - 4);
    if constexpr (TA) {
#pragma unroll
      for (int t = 0; t < 4; t++) a[t] = a_base[(int64_t)(kb + t) * lda];
    } else {
      load_k4(a_base, kb, a);
    }
    if constexpr (TB) {
#pragma unroll
      for (int c = 0; c < NT; c++) {
        float col[4];
        load_k4(B + (int64_t)ncol[c] * ldb, kb, col);
#pragma unroll
        for (int t = 0; t < 4; t++) b[t][c] = col[t];
      }
    } else {
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const float* src = B + (int64_t)(kb + t) * ldb;
        if constexpr (NT == 1) {
          b[t][0] = src[ncol[0]];
        } else {
          const bvec v = *reinterpret_cast<const bvec*>(src + ncol[0]);
#pragma unroll
          for (int c = 0; c < NT; c++) b[t][c] = v[c];
        }
      }
    }
  };
  auto load_group = [&](int c, float (&a)[G][4], float (&b)[G][4][NT]) {
#pragma unroll
    for (int g = 0; g < G; g++)
      if (c + g * WV < nchunks) load(c + g * WV, a[g], b[g]);
  };
  f32x4 acc[NT];
#pragma unroll
  for (int c = 0; c < NT; c++) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto mfma_group = [&](int c, float (&a)[G][4], float (&b)[G][4][NT]) {
#pragma unroll
    for (int g = 0; g < G; g++)
      if (c + g * WV < nchunks) {
        const int k0 = (c + g * WV) * 16 + 4 * q;
        const int first = k0 - min(k0, K - 4);   // elements below this index belong to the quad before
#pragma unroll
        for (int t = 0; t < 4; t++) {
          const float av = t >= first ? a[g][t] : 0.f;
#pragma unroll
          for (int cs = 0; cs < NT; cs++) {
            const float bv = t >= first ? b[g][t][cs] : 0.f;
            acc[cs] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[cs], 0, 0, 0);
          }
        }
      }
  };
  float a0[G][4], b0[G][4][NT], a1[G][4], b1[G][4][NT];
  int c0 = wave;
  if (c0 < nchunks) load_group(c0, a0, b0);
  while (c0 < nchunks) {
    const int c1 = c0 + G * WV;
    if (c1 < nchunks) load_group(c1, a1, b1);
    mfma_group(c0, a0, b0);
    if (c1 >= nchunks) break;
    c0 = c1 + G * WV;
    if (c0 < nchunks) load_group(c0, a0, b0);
    mfma_group(c1, a1, b1);
  }
  // element v of accumulator c in lane (i, q) is C[m0 + 4*q + v][n0 + NT*i + c]
#pragma unroll
  for (int c = 0; c < NT; c++)
#pragma unroll
    for (int v = 0; v < 4; v++) part[wave * TILE + (4 * q + v) * BN + NT * i + c] = acc[c][v];
  __syncthreads();
  if (NT == 1 && softmax) {
    // Row softmax (N <= 16: the one column tile holds whole rows) with the
    // arithmetic of the softmax kernel: max, exp(x - max) in float64 rounded
    // once, the sum taken in column order, one rounded reciprocal.
    __shared__ float sm_x[16 * 17], sm_e[16 * 17];
    const int e = threadIdx.x, row = (e >> 4) & 15, col = e & 15;
    if (e < TILE) {
      float sum = part[e];
#pragma unroll
      for (int w = 1; w < WV; w++) sum = sum + part[w * TILE + e];
      if (bias && col < N) sum = sum + bias[col];
      sm_x[row * 17 + col] = act_apply(sum, act, alpha);
    }
    __syncthreads();
    if (e < TILE) {
      float mx = -INFINITY;
      for (int j = 0; j < N; j++) mx = fmaxf(mx, sm_x[row * 17 + j]);
      sm_e[row * 17 + col] = col < N ? (float)exp((double)(sm_x[row * 17 + col] - mx)) : 0.f;
    }
    __syncthreads();
    if (e < TILE && col < N) {
      float sum = 0.f;
      for (int j = 0; j < N; j++) sum = sum + sm_e[row * 17 + j];
      const float inv = 1.0f / sum;
      C[(int64_t)(m0 + row) * ldc + col] = sm_e[row * 17 + col] * inv;
    }
    return;
  }
  for (int e = threadIdx.x; e < TILE; e += WV * 64) {
    float sum = part[e];
#pragma unroll
    for (int w = 1; w < WV; w++) sum = sum + part[w * TILE + e];
    const int col = n0 + e % BN;
    if (col >= N) continue;
    if (bias) sum = sum + bias[col];
    C[(int64_t)(m0 + e / BN) * ldc + col] = act_apply(sum, act, alpha);
  }
}

// ---- Conv2d 3x3 / stride 1 with the input staged in LDS -----------------------------
// Same GEMM view as k_conv2d (M = filters, N = B*oh*ow output pixels in
// flattened order, K = C*9), but the B operand is not gathered element by
// element.  Per chunk of CC input channels the block copies into LDS
//   - the weights of its BM filters for those channels, k-major, and
//   - every input row its BN pixels touch, as rows of a zero-padded image:
//     image b contributes H+2p padded rows of W+2p padded columns, stacked over
//     b, so padded row b*(H+2p) + oy + kr, column ox + kc is tap (kr, kc) of
//     output pixel (b, oy, ox) and the zero halo needs no test in the hot loop.
// A lane then fetches its B value with one ds_read at (pixel base + tap offset);
// the two lane halves of a 32x32x2 MFMA take channels c and c + CC/2 of the same
// tap, which keeps both operands' offsets lane-constant plus a uniform term.
// One barrier pair per chunk (CC*9 = 72 k-values) instead of one per 16.
struct Conv3Geom {
  int C, H, W, F, oh, ow, pad, P /* B*oh*ow */, B;
  int Hp, PW;      // padded image height, padded row pitch (W + 2 pad)
  int R;           // patch rows held in LDS (upper bound over all blocks)
  int CP;          // floats per channel plane of the patch (R * PW)
  int K;           // C * 9
  int nchunks;     // ceil(C / CC)
  // Wide images: a block's BN pixels are a TH x TW rectangle of one image
  // instead of BN consecutive flattened pixels, and the patch is the
  // (TH+2) x (TW+2) window under it (PW, R, CP then describe that window).
  // TW == 0: the row-stacked layout above.
  int TH, TW, tiles_x, tiles_y;
  // ceil(2^32 / d) for d = CP, PW, Hp: the staging decode divides by them once
  // per element (see div_magic)
  unsigned mCP, mPW, mHp;
  // Row-stacked layout: a block owns BNU <= BN consecutive pixels (BNU = BN
  // unless the tile is cut to whole output rows for the fused pooling).
  int BNU;
  // Fused 2x2/stride-2 max-pool: pool != 0, y has the pooled shape (ph x pw per
  // plane) and every block's pixels form whole pooling windows - row-stacked: a
  // multiple of two rows starting on an even row (oh even) or whole images (oh
  // odd); tiled: TH and TW even.  NPR = pooled rows a block produces.
  int pool, ph, pw, NPR;
  int vsplits;   // pool only: K slices of the unfused launch of this layer (see conv3_tile)
};

// n / d through one high multiply, exact while n * d < 2^32; magic 0 stands for d = 1.
__host__ __device__ __forceinline__ unsigned div_magic_of(unsigned d) {
  return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d);
}
__device__ __forceinline__ int div_magic(int n, unsigned magic) {
  return magic ? (int)__umulhi((unsigned)n, magic) : n;
}

template <int BM, int BN, int CC, int WAVES_M, int PMAX, bool VEC, class SC>
__device__ __forceinline__ void conv3_tile(const float* __restrict__ x, const float* __restrict__ w,
                                           const SC& sc, const Conv3Geom& g, int chunk0, int chunk1,
                                           int m0, int n0, int act, float alpha) {
  constexpr int WAVES_N = 4 / WAVES_M;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int KC = CC * 9;          // k-values per chunk
  constexpr int KHALF = KC / 2;       // MFMA steps per chunk
  constexpr int SA = BM + 2;          // (BM + 2) % 32 == 2: conflict-free transposing writes
  constexpr int QPR = KC / 4;         // float4 slots per filter row
  constexpr int QG = (QPR + 3) / 4;   // groups of four slots
  constexpr int WTOTAL = BM * QG * 4; // weight float4 slots per chunk (some past QPR)
  constexpr int NW = (WTOTAL + kThreads - 1) / kThreads;
  static_assert(CC % 2 == 0 && BM % 32 == 0 && TM >= 1 && TN >= 1, "bad conv tile");
  extern __shared__ float lds[];
  float* const As = lds;                       // [KC][SA]
  float* const Ps = lds + KC * SA;             // [CC][CP]

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
  const int lr = lane & 31, lk = lane >> 5;
  const int plane = g.oh * g.ow;
  const int HW = g.H * g.W;

  // patch rows: the padded-row window of this block's pixels (row r of the patch
  // is padded row gp_lo + r of the stacked images), or in the tiled layout the
  // TH+2 input rows under the tile
  const bool tiled = g.TW > 0;
  int tb = 0, oy0 = 0, ox0 = 0;   // tiled: image, first output row / column of the tile
  if (tiled) {
    const int t = blockIdx.x;
    const int tx = t % g.tiles_x, ty = (t / g.tiles_x) % g.tiles_y;
    tb = t / (g.tiles_x * g.tiles_y);
    oy0 = ty * g.TH;
    ox0 = tx * g.TW;
  }
  const int b_lo = n0 / plane;
  const int gp_lo = b_lo * g.Hp + (n0 - b_lo * plane) / g.ow;

  // What each thread copies per chunk never changes except for the channel
  // base, so it is decoded once: patch element e = tid + j*256 of the
  // [CC][R][PW] patch comes from x[c0*HW + psrc[j]] (or is a halo zero), and
  // weight slot f = tid + j*256 from w[wsrc[j] + c0*9].
  const int patch_total = CC * g.CP;
  int psrc[PMAX];
#pragma unroll
  for (int j = 0; j < PMAX; j++) {
    const int e = threadIdx.x + j * kThreads;
    int src = -1;
    if (e < patch_total) {
      const int c = div_magic(e, g.mCP);
      const int rem = e - c * g.CP;
      const int r = div_magic(rem, g.mPW);
      const int ix = ox0 + rem - r * g.PW - g.pad;
      int b = tb, iy = oy0 + r - g.pad;
      if (!tiled) {
        const int gpr = gp_lo + r;
        b = div_magic(gpr, g.mHp);
        iy = gpr - b * g.Hp - g.pad;
      }
      if (b < g.B && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W) src = c * HW + (b * g.C * g.H + iy) * g.W + ix;
    }
    psrc[j] = src;
  }
  int wsrc[NW];   // element offset into w at c0 = 0, -1 = nothing to copy
  int wdst[NW];   // LDS offset of the slot's first element
#pragma unroll
  for (int j = 0; j < NW; j++) {
    const int f = threadIdx.x + j * kThreads;
    const int q_lo = f & 3;
    const int row = (f >> 2) % BM;
    const int q = ((f >> 2) / BM) * 4 + q_lo;
    const bool ok = f < WTOTAL && q < QPR && m0 + row < g.F;
    wsrc[j] = ok ? (m0 + row) * g.K + q * 4 : -1;
    wdst[j] = (q * 4) * SA + row;
  }

  // per-lane pixel bases inside the patch (one per MFMA column group) and the
  // flattened index of that pixel in y (-1: outside the image)
  int pbase[TN], jout[TN];
#pragma unroll
  for (int t = 0; t < TN; t++) {
    if (tiled) {
      const int n = wn + t * 32 + lr;
      const int ty = n / g.TW, tx = n - ty * g.TW;
      const int oy = oy0 + ty, ox = ox0 + tx;
      jout[t] = (oy < g.oh && ox < g.ow) ? tb * plane + oy * g.ow + ox : -1;
      pbase[t] = ty * g.PW + tx + lk * (CC / 2) * g.CP;
    } else {
      const int nl = wn + t * 32 + lr;
      int j = n0 + nl;
      const bool ok = nl < g.BNU && j < g.P;
      jout[t] = ok ? j : -1;
      j = ok ? j : n0;   // idle lanes read the block's first pixel
      const int b = j / plane;
      const int rem = j - b * plane;
      const int oy = rem / g.ow, ox = rem - oy * g.ow;
      pbase[t] = (b * g.Hp + oy - gp_lo) * g.PW + ox + lk * (CC / 2) * g.CP;
    }
  }
  const int abase = lk * KHALF * SA + wm + lr;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

  float preg[PMAX];
  f32x4 wreg[NW];
  // Variants of this staging that were measured and not kept (MI355X, the 3x3
  // layers of the benchmark configurations): a second register set so loads get
  // two chunks to land (185 registers instead of 87, large layers 30 % slower);
  // branch-free loads with the zero chosen at the LDS write, and loads spread
  // between the MFMAs (a few percent slower); eight wavefronts per block with
  // the k-steps of a chunk split between two quads (MFMA phase at its ideal
  // length, but the wait for the next chunk's loads grows by as much; large
  // layers 8-25 % slower); a per-block rotation of the chunk order (no change);
  // a kernel of its own in which global_load_lds copies the operands straight
  // into a ring of four LDS stages of four channels (filter rows as they lie in
  // memory, pitch 36 floats, A fragments read along k; every thread issuing the
  // same six copies per chunk so that "chunk landed" is s_waitcnt vmcnt(12), a
  // bare s_barrier per chunk, copies written as asm because the compiler waits
  // for every tracked LDS copy at each loop merge): bit-correct, loads three
  // phases ahead and no LDS stores, yet 4-13 % slower on every layer it took -
  // so load latency is not what holds this kernel back.
  auto stage_load = [&](int chunk) {
    const int c0 = chunk * CC;
    const float* xc = x + (int64_t)c0 * HW;
    const float* wc = w + c0 * 9;
#pragma unroll
    for (int j = 0; j < PMAX; j++) preg[j] = psrc[j] >= 0 ? xc[psrc[j]] : 0.f;
#pragma unroll
    for (int j = 0; j < NW; j++) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (wsrc[j] >= 0) {
        const float* src = wc + wsrc[j];
        if (VEC) v = *reinterpret_cast<const f32x4*>(src);
        else { v[0] = src[0]; v[1] = src[1]; v[2] = src[2]; v[3] = src[3]; }
      }
      wreg[j] = v;
    }
  };
  auto stage_store = [&]() {
#pragma unroll
    for (int j = 0; j < PMAX; j++) {
      const int e = threadIdx.x + j * kThreads;
      if (e < patch_total) Ps[e] = preg[j];
    }
#pragma unroll
    for (int j = 0; j < NW; j++) {
      const int f = threadIdx.x + j * kThreads;
      const int q = ((f >> 2) / BM) * 4 + (f & 3);
      if (f < WTOTAL && q < QPR) {
#pragma unroll
        for (int e = 0; e < 4; e++) As[wdst[j] + e * SA] = wreg[j][e];
      }
    }
  };

  // With fused pooling the whole K range is summed here, but in the slices a
  // split-K launch of the same layer would use (vsplits of them, added in slab
  // order), so the stored bits do not depend on whether the pool was fused.
  const int vsplits = (g.pool && g.vsplits > 1) ? g.vsplits : 1;
  const int vper = (chunk1 - chunk0 + vsplits - 1) / vsplits;
  f32x16 tot[TM][TN];
  for (int vz = 0; vz < vsplits; vz++) {
  const int vc0 = chunk0 + vz * vper, vc1 = min(chunk1, vc0 + vper);
  if (vz > 0) {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++) {
        if (vz == 1) tot[a][b] = acc[a][b];
        else tot[a][b] = tot[a][b] + acc[a][b];
#pragma unroll
        for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;
      }
  }
  if (vc0 < vc1) stage_load(vc0);
  for (int chunk = vc0; chunk < vc1; chunk++) {
    __syncthreads();           // the previous chunk's LDS reads are done
    stage_store();
    __syncthreads();
    if (chunk + 1 < vc1) stage_load(chunk + 1);  // in flight during the MFMAs below
    // ---- MFMA over the chunk: step s pairs k = s (channel s/9) with k = s + KHALF
    // Operand fragments run kAhead steps ahead of the MFMAs that use them: an LDS
    // read takes longer than one 32x32x2 MFMA, so a distance of one left the
    // matrix pipe idle about 40 % of the time (measured MFMA-busy 59 %).
    constexpr int kAhead = 4, kRing = 8;
    float af[kRing][TM], bf[kRing][TN];
    auto fetch = [&](int s1) {
      const int cs = s1 / 9, tap = s1 % 9, kr = tap / 3, kc = tap % 3;
      const int boff = cs * g.CP + kr * g.PW + kc;
#pragma unroll
      for (int a = 0; a < TM; a++) af[s1 % kRing][a] = As[abase + s1 * SA + a * 32];
#pragma unroll
      for (int t = 0; t < TN; t++) bf[s1 % kRing][t] = Ps[pbase[t] + boff];
    };
#pragma unroll
    for (int s = 0; s < kAhead && s < KHALF; s++) fetch(s);
#pragma unroll
    for (int s = 0; s < KHALF; s++) {
      if (s + kAhead < KHALF) fetch(s + kAhead);
      // keep the compiler from sinking the reads back to just before their use
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int t = 0; t < TN; t++)
          acc[a][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s % kRing][a], bf[s % kRing][t], acc[a][t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  }
  if (vsplits > 1) {
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int b = 0; b < TN; b++) acc[a][b] = tot[a][b] + acc[a][b];
  }

  if constexpr (std::is_same<SC, StoreNCHW>::value) {
    if (g.pool) {
      // The block's results (after BatchNorm / activation) go to LDS as
      // S[filter][pixel]; then each thread owns one pooled pixel and walks
      // filters: window scan order and strict > of the pooling kernel.
      constexpr int SP = BN + 1;
      constexpr int QL = BN / 4;            // pooled pixels per block, at most
      constexpr int FSTEP = kThreads / QL;  // filters advance by this per thread
      float* const S = lds;
      __syncthreads();                      // operand reads of the last chunk are done
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int il = wm + a * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
          if (m0 + il < g.F) {
#pragma unroll
            for (int t = 0; t < TN; t++) S[il * SP + wn + t * 32 + lr] = tail_apply(sc.tail, m0 + il, acc[a][t][v]);
          }
        }
      __syncthreads();
      const int q = threadIdx.x % QL;
      int nl, rowstep, b;
      int64_t obase;   // offset of the pooled pixel inside its (b, f) plane
      bool ok;
      if (tiled) {
        const int hw = g.TW / 2;
        const int pr = q / hw, pc = q - pr * hw;
        ok = pr < g.NPR && oy0 + 2 * pr + 1 < g.oh && ox0 + 2 * pc + 1 < g.ow;
        nl = 2 * pr * g.TW + 2 * pc;
        rowstep = g.TW;
        b = tb;
        obase = (int64_t)(oy0 / 2 + pr) * g.pw + ox0 / 2 + pc;
      } else {
        const int pr = q / g.pw, pc = q - pr * g.pw;
        int rr = 2 * pr;   // local row of the window's top
        if (g.oh & 1) { const int k = pr / g.ph; rr = k * g.oh + 2 * (pr - k * g.ph); }
        const int gr = n0 / g.ow + rr;   // stacked output row
        b = gr / g.oh;
        const int oy = gr - b * g.oh;
        ok = pr < g.NPR && b < g.B;
        nl = rr * g.ow + 2 * pc;
        rowstep = g.ow;
        obase = (int64_t)(oy / 2) * g.pw + pc;
      }
      if (ok) {
        const int64_t pplane = (int64_t)g.ph * g.pw;
        for (int il = threadIdx.x / QL; il < BM && m0 + il < g.F; il += FSTEP) {
          const float* s0 = S + il * SP + nl;
          float out = -3.402823466e+38f;
          if (s0[0] > out) out = s0[0];
          if (s0[1] > out) out = s0[1];
          if (s0[rowstep] > out) out = s0[rowstep];
          if (s0[rowstep + 1] > out) out = s0[rowstep + 1];
          sc.y[((int64_t)b * g.F + m0 + il) * pplane + obase] = out;
        }
      }
      return;
    }
  }
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int i = m0 + wm + a * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
#pragma unroll
      for (int t = 0; t < TN; t++)
        if (i < g.F && jout[t] >= 0) sc.put(i, jout[t], act_apply(acc[a][t][v], act, alpha));
    }
}

template <int BM, int BN, int CC, int WAVES_M, int PMAX, bool VEC>
__global__ __launch_bounds__(kThreads) void k_conv3x3_lds(const float* __restrict__ x,
                                                          const float* __restrict__ w,
                                                          float* __restrict__ y, Conv3Geom g,
                                                          ConvTail tail, int splits,
                                                          float* __restrict__ ws) {
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * g.BNU;
  if (splits > 1) {
    const int per = (g.nchunks + splits - 1) / splits;
    const int c0 = blockIdx.z * per, c1 = min(g.nchunks, c0 + per);
    StorePartial sc{ws + (int64_t)blockIdx.z * g.F * g.P, g.P};
    conv3_tile<BM, BN, CC, WAVES_M, PMAX, VEC, StorePartial>(x, w, sc, g, c0, c1, m0, n0, 0, 0.f);
  } else {
    StoreNCHW sc{y, g.F, g.oh * g.ow, tail};
    conv3_tile<BM, BN, CC, WAVES_M, PMAX, VEC, StoreNCHW>(x, w, sc, g, 0, g.nchunks, m0, n0, 0, 0.f);
  }
}

// ---- Conv2d 3x3 / stride 1 over a few input channels, on the vector ALUs ------------
// With C*9 <= 36 the contraction is too short for the matrix cores to pay, and
// the layer is bound by writing y.  One thread owns one stored pixel: it holds
// the input patch in registers, walks this workgroup's filters (weights are
// uniform across the wavefront, so they come through scalar loads) and applies
// the epilogue.  With WS == 2 the stored pixel is the 2x2/stride-2 max-pool
// window of four convolution results (scan order and strict > of the pooling
// kernel), which cuts the bytes written by four.
// (The same shapes on the 16x16x4 MFMA - one wavefront per 16 stored pixels,
// each lane fetching its own tap per step from x - were measured slower: 59 us
// against 41 on 8x3x416x416 -> 16; the per-tap address arithmetic and bounds
// tests cost more than the matrix cores save at K = 27.)
template <int C, int WS>
__global__ __launch_bounds__(256) void k_conv3x3_direct(const float* __restrict__ x,
                                                        const float* __restrict__ w,
                                                        float* __restrict__ y, int B, int H, int W,
                                                        int F, int pad, int yh, int yw, int fper,
                                                        ConvTail tail) {
  constexpr int PS = WS + 2;
  // gridDim.z > 1: one image per z, the x blocks walk that image's stored pixels (one 32-bit division
  // per thread; the 64-bit divisions of the flat numbering were a quarter of a small layer's run).
  // gridDim.z == 1: stored pixels numbered over the whole batch (more images than z can count).
  int px, py, b;
  if (gridDim.z > 1 || B == 1) {
    const unsigned t = blockIdx.x * 256u + threadIdx.x;
    if (t >= (unsigned)(yh * yw)) return;
    py = (int)(t / (unsigned)yw); px = (int)(t - (unsigned)py * (unsigned)yw); b = blockIdx.z;
  } else {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= (int64_t)B * yh * yw) return;
    px = (int)(t % yw); py = (int)((t / yw) % yh); b = (int)(t / ((int64_t)yw * yh));
  }
  const int iy0 = py * WS - pad, ix0 = px * WS - pad;
  float patch[C][PS][PS];
#pragma unroll
  for (int c = 0; c < C; c++)
#pragma unroll
    for (int r = 0; r < PS; r++)
#pragma unroll
      for (int q = 0; q < PS; q++) {
        const int iy = iy0 + r, ix = ix0 + q;
        const bool in = iy >= 0 && iy < H && ix >= 0 && ix < W;
        patch[c][r][q] = in ? x[(((int64_t)b * C + c) * H + iy) * W + ix] : 0.f;
      }
  const int f0 = blockIdx.y * fper, f1 = min(F, f0 + fper);
  for (int f = f0; f < f1; f++) {
    const float* wf = w + (int64_t)f * (C * 9);
    float acc[WS][WS];
#pragma unroll
    for (int dy = 0; dy < WS; dy++)
#pragma unroll
      for (int dx = 0; dx < WS; dx++) acc[dy][dx] = 0.f;
#pragma unroll
    for (int c = 0; c < C; c++)
#pragma unroll
      for (int kr = 0; kr < 3; kr++)
#pragma unroll
        for (int kc = 0; kc < 3; kc++) {
          const float wv = wf[(c * 3 + kr) * 3 + kc];
#pragma unroll
          for (int dy = 0; dy < WS; dy++)
#pragma unroll
            for (int dx = 0; dx < WS; dx++)
              acc[dy][dx] = __builtin_fmaf(patch[c][dy + kr][dx + kc], wv, acc[dy][dx]);
        }
    float out;
    if (WS == 2) {
      out = -3.402823466e+38f;
#pragma unroll
      for (int dy = 0; dy < WS; dy++)
#pragma unroll
        for (int dx = 0; dx < WS; dx++) {
          const float v = tail_apply(tail, f, acc[dy][dx]);
          if (v > out) out = v;
        }
    } else {
      out = tail_apply(tail, f, acc[0][0]);
    }
    y[(((int64_t)b * F + f) * yh + py) * yw + px] = out;
  }
}

// ---- float64 GEMM -----------------------------------------------------------------
// C = op(A) op(B) in float64 on the matrix cores (v_mfma_f64_16x16x4f64: lane l
// feeds A[l%16][l/16] and B[l/16][l%16]; accumulator register v of lane l is
// C[4*v + l/16][l%16]), any transpose, extents and leading dimensions.
// Global loads are pairs of doubles along the operand's contiguous axis: VEC
// when every pair is whole and 16-byte aligned (even extents, leading
// dimensions and batch strides, aligned bases), otherwise 8-byte aligned pairs
// with a single at an odd end (the extra tests cost about 9 % at 2048^3).  LDS tiles are
// k-pair-major: element (r, k) of a tile sits at (k/2)*S2 + 2*r + (k&1).  The
// four k-rows a 16x16x4 MFMA reads are then two pair rows: lanes 0-31 of a
// ds_read_b64 (k and k+1 of rows r..r+15) cover 32 consecutive doubles, lanes
// 32-63 the next pair row - no bank conflict for any S2 - and an operand whose
// k axis is contiguous in memory goes to LDS with one 16-byte store per pair
// (S2*8 = 64 mod 256 keeps the k-pairs of a row apart).  BM x BN block, 2x2
// wavefronts of (BM/2) x (BN/2), register-staged double buffering with one
// barrier per k-tile.
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x2_a8 __attribute__((ext_vector_type(2), aligned(8)));

// Operand stored [r][k] with k contiguous (A not transposed; B transposed).
template <int R, int BK, bool VEC>
struct LoadKContig64 {
  static constexpr int S2 = 2 * R + 8;
  static constexpr int SIZE = (BK / 2) * S2;
  static constexpr int TOTAL = R * BK / 2;   // pairs per tile
  static constexpr int NV = (TOTAL + kThreads - 1) / kThreads;
  const double* base; int ld; int rmax; int kmax;
  f64x2 reg[NV];
  __device__ __forceinline__ void load(int r0, int k0) {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int f = threadIdx.x + j * kThreads;
      const int r = r0 + f / (BK / 2);
      const int k = k0 + (f % (BK / 2)) * 2;
      f64x2 v = {0.0, 0.0};
      if ((TOTAL % kThreads == 0 || f < TOTAL) && r < rmax) {
        const double* p = base + (int64_t)r * ld + k;
        if (VEC) {
          if (k < kmax) v = *reinterpret_cast<const f64x2*>(p);
        } else {
          if (k + 1 < kmax) v = *reinterpret_cast<const f64x2_a8*>(p);
          else if (k < kmax) v[0] = p[0];
        }
      }
      reg[j] = v;
    }
  }
  __device__ __forceinline__ void store(double* lds) const {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int f = threadIdx.x + j * kThreads;
      if (TOTAL % kThreads != 0 && f >= TOTAL) continue;
      *reinterpret_cast<f64x2*>(&lds[(f % (BK / 2)) * S2 + 2 * (f / (BK / 2))]) = reg[j];
    }
  }
};

// Operand stored [k][c] with c contiguous (B not transposed; A transposed): a
// thread takes columns c, c+1 of rows k, k+1 and writes the two k-pairs.
template <int R, int BK, bool VEC>
struct LoadMnContig64 {
  static constexpr int S2 = 2 * R + 8;
  static constexpr int SIZE = (BK / 2) * S2;
  static constexpr int TOTAL = (R / 2) * (BK / 2);   // 2x2 cells per tile
  static constexpr int NV = (TOTAL + kThreads - 1) / kThreads;
  const double* base; int ld; int rmax; int kmax;
  f64x2 reg[NV][2];
  __device__ __forceinline__ void load(int c0, int k0) {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int f = threadIdx.x + j * kThreads;
      const int c = c0 + (f % (R / 2)) * 2;
      const int k = k0 + (f / (R / 2)) * 2;
      f64x2 v0 = {0.0, 0.0}, v1 = {0.0, 0.0};
      if ((TOTAL % kThreads == 0 || f < TOTAL) && c < rmax) {
        const double* p = base + (int64_t)k * ld + c;
        if (VEC) {
          if (k < kmax) v0 = *reinterpret_cast<const f64x2*>(p);
          if (k + 1 < kmax) v1 = *reinterpret_cast<const f64x2*>(p + ld);
        } else if (c + 1 < rmax) {
          if (k < kmax) v0 = *reinterpret_cast<const f64x2_a8*>(p);
          if (k + 1 < kmax) v1 = *reinterpret_cast<const f64x2_a8*>(p + ld);
        } else {
          if (k < kmax) v0[0] = p[0];
          if (k + 1 < kmax) v1[0] = p[ld];
        }
      }
      reg[j][0] = v0;
      reg[j][1] = v1;
    }
  }
  __device__ __forceinline__ void store(double* lds) const {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int f = threadIdx.x + j * kThreads;
      if (TOTAL % kThreads != 0 && f >= TOTAL) continue;
      double* d = &lds[(f / (R / 2)) * S2 + 4 * (f % (R / 2))];
      *reinterpret_cast<f64x2*>(d) = f64x2{reg[j][0][0], reg[j][1][0]};
      *reinterpret_cast<f64x2*>(d + 2) = f64x2{reg[j][0][1], reg[j][1][1]};
    }
  }
};

// The float64 MFMA core: 2x2 wavefronts over a BM x BN block, k-tiles [kt0, kt1).
template <int BM, int BN, int BK, class LA, class LB>
__device__ __forceinline__ void dmfma_tile_loop(double* lds, LA& la, LB& lb, int m0, int n0, int kt0, int kt1,
                                                f64x4 (&acc)[BM / 32][BN / 32]) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
  static_assert(TM >= 1 && TN >= 1 && WM % 16 == 0 && WN % 16 == 0, "bad wave tiling");
  double* const As = lds;
  double* const Bs = lds + 2 * LA::SIZE;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
  const int lr = lane & 15, lk = lane >> 4;
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) acc[a][b] = f64x4{0.0, 0.0, 0.0, 0.0};

  la.load(m0, kt0 * BK);
  lb.load(n0, kt0 * BK);
  la.store(As);
  lb.store(Bs);
  __syncthreads();
  // this lane's element of MFMA k-step 0: pair row lk/2, parity lk&1
  const int a_off = (lk >> 1) * LA::S2 + 2 * (wm + lr) + (lk & 1);
  const int b_off = (lk >> 1) * LB::S2 + 2 * (wn + lr) + (lk & 1);
  for (int kt = kt0; kt < kt1; kt++) {
    const int cur = (kt - kt0) & 1;
    const bool more = kt + 1 < kt1;
    if (more) {
      la.load(m0, (kt + 1) * BK);
      lb.load(n0, (kt + 1) * BK);
    }
    const double* a_s = As + cur * LA::SIZE + a_off;
    const double* b_s = Bs + cur * LB::SIZE + b_off;
    double af[BK / 4][TM], bf[BK / 4][TN];
#pragma unroll
    for (int st = 0; st < BK / 4; st++) {
#pragma unroll
      for (int a = 0; a < TM; a++) af[st][a] = a_s[st * 2 * LA::S2 + a * 32];
#pragma unroll
      for (int b = 0; b < TN; b++) bf[st][b] = b_s[st * 2 * LB::S2 + b * 32];
    }
#pragma unroll
    for (int st = 0; st < BK / 4; st++)
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
          acc[a][b] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[st][a], bf[st][b], acc[a][b], 0, 0, 0);
    if (more) {
      la.store(As + (cur ^ 1) * LA::SIZE);
      lb.store(Bs + (cur ^ 1) * LB::SIZE);
    }
    __syncthreads();
  }
}

// A barrier that orders LDS traffic only: __syncthreads() also waits for every
// global load in flight, which would cancel a prefetch that spans two k-tiles.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The same loop with the global loads two k-tiles ahead (two register sets,
// i.e. two copies of each loader): for the small tiles, whose MFMA phase is
// shorter than a memory round trip.  Loads and LDS stores are unconditional -
// past the end the last tile is fetched again and stored into the buffer nobody
// reads - so the loop body is straight-line code and the wait in front of a
// store counts only the younger set's loads.
template <int BM, int BN, int BK, class LA, class LB>
__device__ __forceinline__ void dmfma_tile_loop_deep(double* lds, LA& la0, LB& lb0, int m0, int n0, int kt0,
                                                     int kt1, f64x4 (&acc)[BM / 32][BN / 32]) {
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
  static_assert(TM >= 1 && TN >= 1 && WM % 16 == 0 && WN % 16 == 0, "bad wave tiling");
  double* const As = lds;
  double* const Bs = lds + 2 * LA::SIZE;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
  const int lr = lane & 15, lk = lane >> 4;
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) acc[a][b] = f64x4{0.0, 0.0, 0.0, 0.0};

  LA la1 = la0;
  LB lb1 = lb0;
  const int last = max(kt1 - 1, kt0);
  la0.load(m0, kt0 * BK);
  lb0.load(n0, kt0 * BK);
  la1.load(m0, min(kt0 + 1, last) * BK);
  lb1.load(n0, min(kt0 + 1, last) * BK);
  la0.store(As);
  lb0.store(Bs);
  lds_barrier();
  const int a_off = (lk >> 1) * LA::S2 + 2 * (wm + lr) + (lk & 1);
  const int b_off = (lk >> 1) * LB::S2 + 2 * (wn + lr) + (lk & 1);
  // lc/lbc hold tile kt+1; ln/lbn are free and fetch tile kt+2
  auto step = [&](int kt, LA& lc, LB& lbc, LA& ln, LB& lbn) {
    const int cur = (kt - kt0) & 1;
    ln.load(m0, min(kt + 2, last) * BK);
    lbn.load(n0, min(kt + 2, last) * BK);
    const double* a_s = As + cur * LA::SIZE + a_off;
    const double* b_s = Bs + cur * LB::SIZE + b_off;
    double af[BK / 4][TM], bf[BK / 4][TN];
#pragma unroll
    for (int st = 0; st < BK / 4; st++) {
#pragma unroll
      for (int a = 0; a < TM; a++) af[st][a] = a_s[st * 2 * LA::S2 + a * 32];
#pragma unroll
      for (int b = 0; b < TN; b++) bf[st][b] = b_s[st * 2 * LB::S2 + b * 32];
    }
#pragma unroll
    for (int st = 0; st < BK / 4; st++)
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
          acc[a][b] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[st][a], bf[st][b], acc[a][b], 0, 0, 0);
    lc.store(As + (cur ^ 1) * LA::SIZE);
    lbc.store(Bs + (cur ^ 1) * LB::SIZE);
    lds_barrier();
  };
  for (int kt = kt0; kt < kt1; kt += 2) {
    step(kt, la1, lb1, la0, lb0);
    if (kt + 1 < kt1) step(kt + 1, la0, lb0, la1, lb1);
  }
}

// Which loop a forward kernel runs: the small tiles take the deep prefetch once
// there are at least three k-tiles (measured on the float64 convnet's layers:
// 13-21 % faster on 32x64 tiles, 3-7 % on 64x64 and 32x128); with one or two
// k-tiles the second register set only fetches a tile twice (a 9-tap first layer
// ran 30 % slower), and the 128x128 tiles lose with the second set (2048^3
// product 358 -> 399 us): their MFMA phase already covers one tile in flight.
// The filter-gradient kernel keeps the plain loop: its gathers gained nothing
// from the second set.
template <int BM, int BN, int BK, class LA, class LB>
__device__ __forceinline__ void dmfma_tile_loop_auto(double* lds, LA& la, LB& lb, int m0, int n0, int nkt,
                                                     f64x4 (&acc)[BM / 32][BN / 32]) {
  if constexpr (BM <= 64) {
    if (nkt >= 3) {
      dmfma_tile_loop_deep<BM, BN, BK, LA, LB>(lds, la, lb, m0, n0, 0, nkt, acc);
      return;
    }
  }
  dmfma_tile_loop<BM, BN, BK, LA, LB>(lds, la, lb, m0, n0, 0, nkt, acc);
}

template <int BM, int BN, int BK, bool TA, bool TB, bool VEC>
__global__ __launch_bounds__(kThreads) void k_dgemm(const double* __restrict__ A,
                                                    const double* __restrict__ B,
                                                    double* __restrict__ C, int M, int N, int K,
                                                    int lda, int ldb, int ldc, int64_t sA,
                                                    int64_t sB, int64_t sC) {
  using LA = typename std::conditional<TA, LoadMnContig64<BM, BK, VEC>, LoadKContig64<BM, BK, VEC>>::type;
  using LB = typename std::conditional<TB, LoadKContig64<BN, BK, VEC>, LoadMnContig64<BN, BK, VEC>>::type;
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
  __shared__ double lds[2 * (LA::SIZE + LB::SIZE)];
  int tile_m, tile_n, bz;
  tile_coords(&tile_m, &tile_n, &bz, gridDim.z > 1);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  LA la; la.base = A + bz * sA; la.ld = lda; la.rmax = M; la.kmax = K;
  LB lb; lb.base = B + bz * sB; lb.ld = ldb; lb.rmax = N; lb.kmax = K;
  C += bz * sC;
  f64x4 acc[TM][TN];
  dmfma_tile_loop_auto<BM, BN, BK, LA, LB>(lds, la, lb, m0, n0, (K + BK - 1) / BK, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
  const int lr = lane & 15, lk = lane >> 4;
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int i = m0 + wm + a * 16 + 4 * v + lk, j = n0 + wn + b * 16 + lr;
        if (i < M && j < N) C[(int64_t)i * ldc + j] = acc[a][b][v];
      }
}

// Float64 product with a small result (a dense layer on a batch: too few 64x64
// tiles to occupy the device, and a k loop of a thousand steps behind each).
// One workgroup per 16x16 tile of C, its WV wavefronts each summing a slice of
// K straight from global memory into one MFMA accumulator (element (i, k) of
// op(A) at A[i*sai + k*sak], (k, j) of op(B) at B[k*sbk + j*sbj], so every
// transpose is the same code); loads are unconditional at clamped addresses and
// masked afterwards, so they all stay in flight.  The slices are added in LDS in
// wavefront order: the result does not depend on scheduling.
template <int WV, bool AV, bool BV>
__global__ __launch_bounds__(WV * 64) void k_dgemm_skinny(const double* __restrict__ A,
                                                          const double* __restrict__ B,
                                                          double* __restrict__ C, int M, int N, int K,
                                                          int64_t sai, int64_t sak, int64_t sbk,
                                                          int64_t sbj, int ldc) {
  __shared__ double part[WV][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lk = lane >> 4;
  const int m0 = blockIdx.y * 16, n0 = blockIdx.x * 16;
  const double* ap = A + (int64_t)min(m0 + lr, M - 1) * sai;
  const double* bp = B + (int64_t)min(n0 + lr, N - 1) * sbj;
  const int kper = (((K + WV - 1) / WV) + 7) & ~7;
  const int k0 = wave * kper, k1 = min(K, k0 + kper);
  f64x4 acc = {0.0, 0.0, 0.0, 0.0};
  if constexpr (AV || BV) {
    // An operand that is k-contiguous: a lane fetches two consecutive k of its row or column in one load (the
    // sixteen k of a step are then two 64-byte pieces instead of sixteen 8-byte ones; 8-byte alignment is all
    // the load needs); which k a lane group multiplies in which MFMA is the same for both operands -
    // k0 + 8 u + 2 lk + e.  The pair that would start at the last k of an odd K starts one earlier and is
    // shifted into place.
    for (int k = k0; k < k1; k += 16) {
      f64x2 a[2], b[2];
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const int kk = k + 8 * u + 2 * lk;
        const bool last = kk > K - 2;   // kk == K - 1 (its second k does not exist), or past the end (masked below)
        if constexpr (AV) {
          const f64x2 v = *reinterpret_cast<const f64x2_a8*>(ap + min(kk, K - 2));
          a[u] = last ? f64x2{v[1], 0.0} : v;
        }
        if constexpr (BV) {
          const f64x2 v = *reinterpret_cast<const f64x2_a8*>(bp + min(kk, K - 2));
          b[u] = last ? f64x2{v[1], 0.0} : v;
        }
#pragma unroll
        for (int e = 0; e < 2; e++) {
          if constexpr (!AV) a[u][e] = ap[(int64_t)min(kk + e, K - 1) * sak];
          if constexpr (!BV) b[u][e] = bp[(int64_t)min(kk + e, K - 1) * sbk];
        }
      }
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int e = 0; e < 2; e++) {
          const bool ok = k + 8 * u + 2 * lk + e < k1;
          const double av = ok ? a[u][e] : 0.0, bv = ok ? b[u][e] : 0.0;
          acc = __builtin_amdgcn_mfma_f64_16x16x4f64(av, bv, acc, 0, 0, 0);
        }
    }
  } else {
    for (int k = k0; k < k1; k += 16) {
      double a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int kc = min(k + 4 * u + lk, K - 1);
        a[u] = ap[kc * sak];
        b[u] = bp[kc * sbk];
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const bool ok = k + 4 * u + lk < k1;
        a[u] = ok ? a[u] : 0.0;
        b[u] = ok ? b[u] : 0.0;
      }
#pragma unroll
      for (int u = 0; u < 4; u++) acc = __builtin_amdgcn_mfma_f64_16x16x4f64(a[u], b[u], acc, 0, 0, 0);
    }
  }
#pragma unroll
  for (int v = 0; v < 4; v++) part[wave][v * 64 + lane] = acc[v];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int v = 0; v < 4; v++) {
      double sum = part[0][v * 64 + lane];
      for (int w = 1; w < WV; w++) sum = sum + part[w][v * 64 + lane];
      const int i = m0 + 4 * v + lk, j = n0 + lr;
      if (i < M && j < N) C[(int64_t)i * ldc + j] = sum;
    }
  }
}

// ---- float64 Conv2d as an implicit GEMM on the matrix cores ---------------------------
// y(F x P) = w(F x C*kh*kw) . col(C*kh*kw x P), P = B*oh*ow, with the same tile
// loop as the float64 product.  The filter matrix is the k-contiguous operand;
// the col operand is gathered from NCHW x: a thread keeps one output pixel for
// the whole kernel (its image offset and first input row / column are decoded
// once) and fetches pairs of consecutive k = (c, kr, kc) for it, padding taps as
// zeros.  Any kernel size, stride, dilation and padding.
struct ConvGeom64 {
  int C, H, W, F, oh, ow, kh, kw, padH, padW, strideH, strideW, dilH, dilW;
  int P, K;           // B*oh*ow, C*kh*kw
  unsigned mKK, mkw;  // division magics for kh*kw and kw (see div_magic)
};

template <int R, int BK>
struct LoadIm2col64 {
  static constexpr int S2 = 2 * R + 8;
  static constexpr int SIZE = (BK / 2) * S2;
  static constexpr int KP_STEP = kThreads / R;            // k-pairs covered per pass
  static constexpr int NV = (BK / 2 + KP_STEP - 1) / KP_STEP;
  static_assert(kThreads % R == 0, "pixel columns must divide the block");
  const double* xp;   // x at (image, first input row, first input column) of this thread's pixel
  const ConvGeom64* g;
  int iy0, ix0;
  int safe;           // offset from xp of an element that is always readable (the image's first)
  bool pvalid;
  f64x2 reg[NV];
  __device__ __forceinline__ void init(const double* x, const ConvGeom64* geom, int n0) {
    g = geom;
    const int p = n0 + (int)(threadIdx.x % R);
    pvalid = p < g->P;
    const int plane = g->oh * g->ow;
    const int pp = pvalid ? p : 0;
    const int b = pp / plane, rem = pp - b * plane;
    const int oy = rem / g->ow, ox = rem - oy * g->ow;
    iy0 = oy * g->strideH - g->padH;
    ix0 = ox * g->strideW - g->padW;
    xp = x + ((int64_t)b * g->C * g->H + iy0) * g->W + ix0;
    safe = -(iy0 * g->W + ix0);
  }
  // Every load is issued, at a clamped address (the image base for a padding tap
  // or a k past the end), and masked afterwards: a load inside a branch would make
  // the wavefront wait for it before the next one is issued.
  __device__ __forceinline__ void load(int, int k0) {
    const int KK = g->kh * g->kw;
    unsigned okbits = 0;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int kp = (int)(threadIdx.x / R) + j * KP_STEP;
#pragma unroll
      for (int e = 0; e < 2; e++) {
        const int k = k0 + 2 * kp + e;
        const int kk = min(k, g->K - 1);
        const int c = div_magic(kk, g->mKK), tap = kk - c * KK;
        const int kr = div_magic(tap, g->mkw), kc = tap - kr * g->kw;
        const int dy = kr * g->dilH, dx = kc * g->dilW;
        const int iy = iy0 + dy, ix = ix0 + dx;
        const bool ok = pvalid && k < g->K && iy >= 0 && iy < g->H && ix >= 0 && ix < g->W;
        const int off = ok ? (c * g->H + dy) * g->W + dx : safe;
        reg[j][e] = xp[off];
        okbits |= (ok ? 1u : 0u) << (2 * j + e);
      }
    }
#pragma unroll
    for (int j = 0; j < NV; j++)
#pragma unroll
      for (int e = 0; e < 2; e++) reg[j][e] = ((okbits >> (2 * j + e)) & 1u) ? reg[j][e] : 0.0;
  }
  __device__ __forceinline__ void store(double* lds) const {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int kp = (int)(threadIdx.x / R) + j * KP_STEP;
      if ((BK / 2) % KP_STEP != 0 && kp >= BK / 2) continue;
      *reinterpret_cast<f64x2*>(&lds[kp * S2 + 2 * (int)(threadIdx.x % R)]) = reg[j];
    }
  }
};

template <int BM, int BN, int BK, bool VEC>
__global__ __launch_bounds__(kThreads) void k_conv2d_f64_mfma(const double* __restrict__ x,
                                                              const double* __restrict__ w,
                                                              double* __restrict__ y, ConvGeom64 g) {
  using LA = LoadKContig64<BM, BK, VEC>;
  using LB = LoadIm2col64<BN, BK>;
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
  __shared__ double lds[2 * (LA::SIZE + LB::SIZE)];
  int tile_m, tile_n, bz_unused;
  tile_coords(&tile_m, &tile_n, &bz_unused, false);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  LA la; la.base = w; la.ld = g.K; la.rmax = g.F; la.kmax = g.K;
  LB lb; lb.init(x, &g, n0);
  f64x4 acc[TM][TN];
  dmfma_tile_loop_auto<BM, BN, BK, LA, LB>(lds, la, lb, m0, n0, (g.K + BK - 1) / BK, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
  const int lr = lane & 15, lk = lane >> 4;
  const int plane = g.oh * g.ow;
#pragma unroll
  for (int b = 0; b < TN; b++) {
    const int j = n0 + wn + b * 16 + lr;
    if (j >= g.P) continue;
    const int bb = j / plane, pix = j - bb * plane;
    double* yb = y + (int64_t)bb * g.F * plane + pix;
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int i = m0 + wm + a * 16 + 4 * v + lk;
        if (i < g.F) yb[(int64_t)i * plane] = acc[a][b][v];
      }
  }
}

// ---- float64 Conv2d filter gradient on the matrix cores ------------------------------
// dW(F x C*kh*kw) = sum over pixels p = (b, oy, ox) of dy[b][f][oy][ox] * col[k][p]
// (the reference's dY2d^T . col, op_nn.go:267-291): the same tile loop with the
// pixel axis as the contraction, cut into slices (blockIdx.z) whose partial
// sums are added in slice order by k_splitk_reduce_f64.  Both operands are
// gathered; every load is issued at a clamped address and masked afterwards.

// A operand: row f, k = pixel, from NCHW dy.
template <int R, int BK>
struct LoadDyRows64 {
  static constexpr int S2 = 2 * R + 8;
  static constexpr int SIZE = (BK / 2) * S2;
  static constexpr int TOTAL = R * BK / 2;
  static constexpr int NV = TOTAL / kThreads;
  static_assert(TOTAL % kThreads == 0, "tile must divide over the block");
  const double* dy; int F, plane, P;
  f64x2 reg[NV];
  __device__ __forceinline__ void load(int r0, int k0) {
    unsigned okbits = 0;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int f = threadIdx.x + j * kThreads;
      const int r = r0 + f / (BK / 2);
      const int rc = min(r, F - 1);
#pragma unroll
      for (int e = 0; e < 2; e++) {
        const int p = k0 + (f % (BK / 2)) * 2 + e;
        const unsigned pc = (unsigned)min(p, P - 1);
        const unsigned b = pc / (unsigned)plane, pix = pc - b * (unsigned)plane;
        reg[j][e] = dy[((int64_t)b * F + rc) * plane + pix];
        okbits |= ((r < F && p < P) ? 1u : 0u) << (2 * j + e);
      }
    }
#pragma unroll
    for (int j = 0; j < NV; j++)
#pragma unroll
      for (int e = 0; e < 2; e++) reg[j][e] = ((okbits >> (2 * j + e)) & 1u) ? reg[j][e] : 0.0;
  }
  __device__ __forceinline__ void store(double* lds) const {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int f = threadIdx.x + j * kThreads;
      *reinterpret_cast<f64x2*>(&lds[(f % (BK / 2)) * S2 + 2 * (f / (BK / 2))]) = reg[j];
    }
  }
};

// B operand: column n = (c, kr, kc) kept by the thread, k = pixel, gathered from NCHW x.
template <int R, int BK>
struct LoadColT64 {
  static constexpr int S2 = 2 * R + 8;
  static constexpr int SIZE = (BK / 2) * S2;
  static constexpr int KP_STEP = kThreads / R;
  static constexpr int NV = (BK / 2) / KP_STEP;
  static_assert(kThreads % R == 0 && (BK / 2) % KP_STEP == 0, "columns and k-pairs must divide the block");
  const double* xc;   // x at channel c of image 0
  const ConvGeom64* g;
  int dy0, dx0;       // input row / column of output pixel (0, 0) for this tap
  bool nvalid;
  f64x2 reg[NV];
  __device__ __forceinline__ void init(const double* x, const ConvGeom64* geom, int n0) {
    g = geom;
    const int n = n0 + (int)(threadIdx.x % R);
    nvalid = n < g->K;
    const int nn = nvalid ? n : 0;
    const int KK = g->kh * g->kw;
    const int c = nn / KK, tap = nn - c * KK;
    const int kr = tap / g->kw, kc = tap - kr * g->kw;
    dy0 = kr * g->dilH - g->padH;
    dx0 = kc * g->dilW - g->padW;
    xc = x + (int64_t)c * g->H * g->W;
  }
  __device__ __forceinline__ void load(int, int k0) {
    const unsigned plane = (unsigned)(g->oh * g->ow);
    unsigned okbits = 0;
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int kp = (int)(threadIdx.x / R) + j * KP_STEP;
#pragma unroll
      for (int e = 0; e < 2; e++) {
        const int p = k0 + 2 * kp + e;
        const unsigned pc = (unsigned)min(p, g->P - 1);
        const unsigned b = pc / plane, rem = pc - b * plane;
        const unsigned oy = rem / (unsigned)g->ow, ox = rem - oy * (unsigned)g->ow;
        const int iy = (int)oy * g->strideH + dy0, ix = (int)ox * g->strideW + dx0;
        const bool ok = nvalid && p < g->P && iy >= 0 && iy < g->H && ix >= 0 && ix < g->W;
        const int64_t off = ok ? ((int64_t)b * g->C * g->H + iy) * g->W + ix : 0;
        reg[j][e] = xc[off];
        okbits |= (ok ? 1u : 0u) << (2 * j + e);
      }
    }
#pragma unroll
    for (int j = 0; j < NV; j++)
#pragma unroll
      for (int e = 0; e < 2; e++) reg[j][e] = ((okbits >> (2 * j + e)) & 1u) ? reg[j][e] : 0.0;
  }
  __device__ __forceinline__ void store(double* lds) const {
#pragma unroll
    for (int j = 0; j < NV; j++) {
      const int kp = (int)(threadIdx.x / R) + j * KP_STEP;
      *reinterpret_cast<f64x2*>(&lds[kp * S2 + 2 * (int)(threadIdx.x % R)]) = reg[j];
    }
  }
};

template <int BM, int BN, int BK>
__global__ __launch_bounds__(kThreads) void k_conv2d_wgrad_f64(const double* __restrict__ x,
                                                               const double* __restrict__ dy,
                                                               double* __restrict__ dw, ConvGeom64 g,
                                                               int splits, double* __restrict__ ws) {
  using LA = LoadDyRows64<BM, BK>;
  using LB = LoadColT64<BN, BK>;
  constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
  __shared__ double lds[2 * (LA::SIZE + LB::SIZE)];
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int nk = (g.P + BK - 1) / BK;
  const int per = (nk + splits - 1) / splits;
  const int kt0 = blockIdx.z * per, kt1 = min(nk, kt0 + per);
  LA la; la.dy = dy; la.F = g.F; la.plane = g.oh * g.ow; la.P = g.P;
  LB lb; lb.init(x, &g, n0);
  f64x4 acc[TM][TN];
  dmfma_tile_loop<BM, BN, BK, LA, LB>(lds, la, lb, m0, n0, kt0, kt1, acc);
  double* out = splits > 1 ? ws + (int64_t)blockIdx.z * g.F * g.K : dw;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
  const int lr = lane & 15, lk = lane >> 4;
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int i = m0 + wm + a * 16 + 4 * v + lk, j = n0 + wn + b * 16 + lr;
        if (i < g.F && j < g.K) out[(int64_t)i * g.K + j] = acc[a][b][v];
      }
}

__global__ __launch_bounds__(256) void k_splitk_reduce_f64(const double* __restrict__ ws, int splits,
                                                           int64_t total, double* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    // slices are added in order; eight loads are issued before their adds so the
    // chain of additions does not wait for one memory round trip per slice
    double s = 0.0;
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
      double v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = ws[(int64_t)(z + u) * total + i];
#pragma unroll
      for (int u = 0; u < 8; u++) s = s + v[u];
    }
    for (; z < splits; z++) s = s + ws[(int64_t)z * total + i];
    out[i] = s;
  }
}

// ---- Conv2d backward ---------------------------------------------------------------
// The reference differentiates Conv2d through its im2col + MatMul graph
// (nn.go:211-305): dW = dY2d^T . col and dX = col2im(dY2d . Wflat)
// (op_nn.go:267-291, 605-640).  Here both are implicit GEMMs on the matrix
// cores with no col buffer.
//
// Filter gradient: dW(F x CKK) = sum over pixels j = (b, oy, ox) of
// dy[b][f][oy][ox] * x[b][c][oy*s - p + kr*d][ox*s - p + kc*d]: M = F, N = C*kh*kw,
// K = B*oh*ow, split over K.

// A operand: row f, k = pixel index across the batch, from NCHW dy.  The tile
// loop asks for consecutive k-tiles, so after the first call the (image, pixel)
// position is advanced by carries instead of being divided out again.
template <int R, int BK>
struct LoadDyRows {
  static constexpr int S = R + 2;
  static constexpr int RSTEP = kThreads / BK;   // row distance between a thread's elements
  static constexpr int RPT = R / RSTEP;
  const float* dy; int F; int plane; int kmax /* B*plane */;
  int next_k = -1, b = 0, p = 0;
  float reg[RPT];
  __device__ __forceinline__ void prep(int) {}
  __device__ __forceinline__ void load(int r0, int k0) {
    const int kk = threadIdx.x % BK, rb = threadIdx.x / BK;
    const int j = k0 + kk;
    if (k0 != next_k) {
      b = j / plane;
      p = j - b * plane;
    }
    next_k = k0 + BK;
    const bool ok = j < kmax;
    const float* base = dy + (int64_t)b * F * plane + p;
#pragma unroll
    for (int i = 0; i < RPT; i++) {
      const int f = r0 + rb + i * RSTEP;
      reg[i] = (ok && f < F) ? base[(int64_t)f * plane] : 0.f;
    }
    p += BK;
    while (p >= plane) { p -= plane; b++; }
  }
  __device__ __forceinline__ void store(float* lds) const {
    const int kk = threadIdx.x % BK, rb = threadIdx.x / BK;
#pragma unroll
    for (int i = 0; i < RPT; i++) lds[kk * S + rb + i * RSTEP] = reg[i];
  }
};

// B operand: column n = (c, kr, kc), k = pixel index: the im2col gather read the
// other way round.  What depends only on the column is computed once; the
// pixel position (image, oy, ox) is carried from tile to tile.
template <int R, int BK>
struct LoadIm2colT {
  static constexpr int S = R + 2;
  static constexpr int RSTEP = kThreads / BK;
  static constexpr int RPT = R / RSTEP;
  const float* x; ConvGeom g; int nmax /* C*kh*kw */; int kmax /* B*oh*ow */;
  int coff[RPT];   // c*H*W + kr*dilH*W + kc*dilW, or -1 for a column past the end
  int dyo[RPT], dxo[RPT];
  int next_k = -1, b = 0, oy = 0, ox = 0;
  float reg[RPT];
  __device__ __forceinline__ void prep(int) {}
  __device__ __forceinline__ void init(int n0) {
    const int rb = threadIdx.x / BK;
    const int kk = g.kh * g.kw;
#pragma unroll
    for (int i = 0; i < RPT; i++) {
      const int n = n0 + rb + i * RSTEP;
      const bool okn = n < nmax;
      const int nn = okn ? n : 0;
      const int c = nn / kk, r = nn - c * kk;
      const int kr = r / g.kw, kc = r - kr * g.kw;
      dyo[i] = kr * g.dilH;
      dxo[i] = kc * g.dilW;
      coff[i] = okn ? c * g.H * g.W + dyo[i] * g.W + dxo[i] : -1;
    }
  }
  __device__ __forceinline__ void load(int /*n0*/, int k0) {
    const int j = k0 + threadIdx.x % BK;
    if (k0 != next_k) {
      const int plane = g.oh * g.ow;
      b = j / plane;
      const int rem = j - b * plane;
      oy = rem / g.ow;
      ox = rem - oy * g.ow;
    }
    next_k = k0 + BK;
    const bool ok = j < kmax;
    const int iy0 = oy * g.strideH - g.padH, ix0 = ox * g.strideW - g.padW;
    const float* xb = x + (int64_t)b * g.C * g.H * g.W + iy0 * g.W + ix0;
#pragma unroll
    for (int i = 0; i < RPT; i++) {
      const int iy = iy0 + dyo[i], ix = ix0 + dxo[i];
      const bool in = ok && coff[i] >= 0 && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
      reg[i] = in ? xb[coff[i]] : 0.f;
    }
    ox += BK;
    while (ox >= g.ow) { ox -= g.ow; oy++; }
    while (oy >= g.oh) { oy -= g.oh; b++; }
  }
  __device__ __forceinline__ void store(float* lds) const {
    const int kk = threadIdx.x % BK, rb = threadIdx.x / BK;
#pragma unroll
    for (int i = 0; i < RPT; i++) lds[kk * S + rb + i * RSTEP] = reg[i];
  }
};

template <int BM, int BN, int BK, int WAVES_M>
__global__ __launch_bounds__(kThreads) void k_conv2d_wgrad(const float* __restrict__ x,
                                                           const float* __restrict__ dy,
                                                           float* __restrict__ dw, ConvGeom g,
                                                           int F, int CKK, int splits,
                                                           float* __restrict__ ws) {
  using LA = LoadDyRows<BM, BK>;
  using LB = LoadIm2colT<BN, BK>;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  LA la; la.dy = dy; la.F = F; la.plane = g.oh * g.ow; la.kmax = g.P;
  LB lb; lb.x = x; lb.g = g; lb.nmax = CKK; lb.kmax = g.P;
  lb.init(n0);
  const int nk = (g.P + BK - 1) / BK;
  __shared__ float lds[2 * BK * (LA::S + LB::S)];
  if (splits > 1) {
    int kt0, kt1;
    split_range(nk, splits, blockIdx.z, &kt0, &kt1);
    StorePartial sc{ws + (int64_t)blockIdx.z * F * CKK, CKK};
    mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StorePartial>(lds, la, lb, sc, F, CKK, kt0, kt1, m0, n0, 0, 0.f);
  } else {
    StoreRowMajor sc{dw, CKK};
    mfma_tile_loop<BM, BN, BK, WAVES_M, LA, LB, StoreRowMajor>(lds, la, lb, sc, F, CKK, 0, nk, m0, n0, 0, 0.f);
  }
}

// Filter gradient for the direct kernel's shapes (3x3, stride 1, at most four
// input channels): only F*C*9 results, each a sum over all output pixels, so
// this is a reduction on the vector ALUs.  Workgroup (g, fb) walks every G-th
// image for FB filters at once: a thread gathers the C*9 patch values of a pixel once
// (the gathers with their bounds tests, not the multiply-adds, are what the kernel
// spends its time on) and adds dy * patch into FB x C*9 accumulators, the workgroup
// folds them with a fixed tree, and slab g of the [G][F][C*9] workspace gets the
// partials; the split-K reduce kernel adds the slabs in order.
template <int C, int FB>
__global__ __launch_bounds__(256) void k_conv3x3_wgrad_direct(const float* __restrict__ x,
                                                              const float* __restrict__ dy,
                                                              float* __restrict__ ws, int B, int H,
                                                              int W, int F, int pad, int oh, int ow) {
  constexpr int Q = C * 9;
  __shared__ float sh[4][FB * Q];
  const int f0 = blockIdx.y * FB, G = gridDim.x;
  const int plane = oh * ow;
  float acc[FB][Q];
#pragma unroll
  for (int j = 0; j < FB; j++)
#pragma unroll
    for (int q = 0; q < Q; q++) acc[j][q] = 0.f;
  for (int b = blockIdx.x; b < B; b += G) {
    const float* gy = dy + ((int64_t)b * F + f0) * plane;
    const float* xb = x + (int64_t)b * C * H * W;
    for (int p = threadIdx.x; p < plane; p += 256) {
      const int oy = p / ow, ox = p - oy * ow;
      float xv[Q];
#pragma unroll
      for (int c = 0; c < C; c++)
#pragma unroll
        for (int kr = 0; kr < 3; kr++)
#pragma unroll
          for (int kc = 0; kc < 3; kc++) {
            const int iy = oy - pad + kr, ix = ox - pad + kc;
            const bool in = iy >= 0 && iy < H && ix >= 0 && ix < W;
            xv[(c * 3 + kr) * 3 + kc] = in ? xb[(c * H + iy) * W + ix] : 0.f;
          }
#pragma unroll
      for (int j = 0; j < FB; j++) {
        const float g = f0 + j < F ? gy[(int64_t)j * plane + p] : 0.f;
#pragma unroll
        for (int q = 0; q < Q; q++) acc[j][q] = __builtin_fmaf(g, xv[q], acc[j][q]);
      }
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int j = 0; j < FB; j++)
#pragma unroll
    for (int q = 0; q < Q; q++) {
      float v = acc[j][q];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
      if (lane == 0) sh[wave][j * Q + q] = v;
    }
  __syncthreads();
  for (int i = threadIdx.x; i < FB * Q; i += 256) {
    const int j = i / Q, q = i - j * Q;
    if (f0 + j < F) ws[((int64_t)blockIdx.x * F + f0 + j) * Q + q] = (sh[0][i] + sh[1][i]) + (sh[2][i] + sh[3][i]);
  }
}

// The same reduction for a single input channel (a network's first layer): the padded image sits in LDS
// with a zero halo, so a pixel's nine taps are nine reads at fixed offsets and no bounds test; a wavefront owns
// one filter and walks the pixels 64 at a time (one coalesced read of dy), nine accumulators per lane; four
// filters per workgroup, workgroup (g, fb) takes every G-th image.  Slab g of the [G][F][9] workspace gets the
// lanes' sums folded by a fixed tree; the split-K reduce kernel adds the slabs in order.
__global__ __launch_bounds__(256) void k_conv3x3_wgrad_c1(const float* __restrict__ x, const float* __restrict__ dy,
                                                          float* __restrict__ ws, int B, int H, int W, int F, int pad,
                                                          int oh, int ow, unsigned m_ow, unsigned m_pw) {
  extern __shared__ float img[];   // (H + 2 pad) rows of W + 2 pad
  const int PW = W + 2 * pad, PH = H + 2 * pad;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int f = blockIdx.y * 4 + wave;
  const bool fok = f < F;
  const int plane = oh * ow;
  float acc[9];
#pragma unroll
  for (int q = 0; q < 9; q++) acc[q] = 0.f;
  for (int b = blockIdx.x; b < B; b += gridDim.x) {
    __syncthreads();   // every wavefront is done with the image before
    const float* xb = x + (int64_t)b * H * W;
    for (int i = threadIdx.x; i < PH * PW; i += 256) {
      const int r = (int)__umulhi((unsigned)i, m_pw), c = i - r * PW;
      const int iy = r - pad, ix = c - pad;
      img[i] = (iy >= 0 && iy < H && ix >= 0 && ix < W) ? xb[iy * W + ix] : 0.f;
    }
    __syncthreads();
    const float* gy = dy + ((int64_t)b * F + (fok ? f : F - 1)) * plane;
    // eight pixels per lane at a time: their dy loads are all in flight before the first is used
    for (int p0 = lane; p0 < plane; p0 += 8 * 64) {
      float g[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int p = p0 + 64 * u;
        g[u] = (fok && p < plane) ? gy[p] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int p = min(p0 + 64 * u, plane - 1);   // (a pixel past the end multiplies a zero)
        const int oy = (int)__umulhi((unsigned)p, m_ow), ox = p - oy * ow;
        const float* ip = img + oy * PW + ox;
#pragma unroll
        for (int kr = 0; kr < 3; kr++)
#pragma unroll
          for (int kc = 0; kc < 3; kc++) acc[kr * 3 + kc] = __builtin_fmaf(g[u], ip[kr * PW + kc], acc[kr * 3 + kc]);
      }
    }
  }
#pragma unroll
  for (int q = 0; q < 9; q++) {
    float v = acc[q];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (lane == 0 && fok) ws[((int64_t)blockIdx.x * F + f) * 9 + q] = v;
  }
}

// Input gradient, stride 1: dX is the forward convolution of dy with the
// filters mirrored and their channel axes swapped, under padding
// dil*(k-1) - pad, so the forward kernels compute it.  This writes those filters:
// wt[c][f][kr][kc] = w[f][c][kh-1-kr][kw-1-kc].
template <class T>
__global__ __launch_bounds__(256) void k_flip_filters(const T* __restrict__ w, T* __restrict__ wt, int F,
                                                      int C, int kh, int kw) {
  const int64_t total = (int64_t)F * C * kh * kw;
  const int kk = kh * kw;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int r = (int)(i % kk);
    const int64_t cf = i / kk;
    const int f = (int)(cf % F), c = (int)(cf / F);
    wt[i] = w[((int64_t)f * C + c) * kk + (kk - 1 - r)];
  }
}

// Input gradient for any stride: one thread per dx element gathers the
// (f, kr, kc) terms whose window position divides evenly.  Not on the matrix
// cores; strided convolutions are rare on this path.
__global__ __launch_bounds__(256) void k_conv2d_dgrad_gather(const float* __restrict__ dy,
                                                             const float* __restrict__ w,
                                                             float* __restrict__ dx, ConvGeom g,
                                                             int B, int F) {
  const int64_t total = (int64_t)B * g.C * g.H * g.W;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int ix = (int)(i % g.W), iy = (int)((i / g.W) % g.H);
    const int c = (int)((i / ((int64_t)g.W * g.H)) % g.C), b = (int)(i / ((int64_t)g.W * g.H * g.C));
    float acc = 0.f;
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
        for (int f = 0; f < F; f++)
          acc = __builtin_fmaf(dy[(((int64_t)b * F + f) * g.oh + oy) * g.ow + ox],
                               w[(((int64_t)f * g.C + c) * g.kh + kr) * g.kw + kc], acc);
      }
    }
    dx[i] = acc;
  }
}

// ---- GEMV / outer ------------------------------------------------------------------
// y(m) = A(m x n) x: one wavefront per row, float4 loads when the row is
// 16-byte aligned, butterfly reduction across the 64 lanes.
__global__ __launch_bounds__(256) void k_gemv_n(const float* __restrict__ A,
                                                const float* __restrict__ x, float* __restrict__ y,
                                                int m, int n, int lda, int vec) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= m) return;
  const float* a = A + (int64_t)row * lda;
  float acc = 0.f;
  if (vec) {
    const f32x4* av = reinterpret_cast<const f32x4*>(a);
    const f32x4* xv = reinterpret_cast<const f32x4*>(x);
    const int nv = n / 4;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    for (int i = lane; i < nv; i += 64) {
      const f32x4 p = av[i] * xv[i];
      s += p;
    }
    acc = (s[0] + s[1]) + (s[2] + s[3]);
    for (int i = nv * 4 + lane; i < n; i += 64) acc += a[i] * x[i];
  } else {
    for (int i = lane; i < n; i += 64) acc += a[i] * x[i];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) y[row] = acc;
}

// y(n) = A(m x n)^T x.  A workgroup takes 256*V*J adjacent columns and a range
// of rows and walks the rows in order, RU rows in flight; a thread owns J groups
// of V adjacent columns 256*V apart, so one load instruction of the workgroup
// reads 1024*V contiguous bytes of a row and J of them a contiguous run.  No
// thread shares a sum with another.  With more than one row range the partial
// rows go to `out` = [chunks][n] scratch and k_gemv_t_sum adds them in a fixed
// order, so the result does not depend on timing.  (Measured at 8192 x 8192: V=4,
// J=2, RU=8 with half as many workgroups as compute units streams at 6.7 TB/s;
// more, smaller workgroups scatter the row streams and lose a quarter of that.)
template <int V, int J, int RU>
__global__ __launch_bounds__(256) void k_gemv_t(const float* __restrict__ A, const float* __restrict__ x,
                                                float* __restrict__ out, int m, int n, int lda,
                                                int rows_per_chunk) {
  typedef float vec __attribute__((ext_vector_type(V), aligned(4 * V)));
  constexpr int GS = 256 * V;  // columns between a thread's groups
  const int cb = blockIdx.x * GS * J + threadIdx.x * V;
  const int r0 = blockIdx.y * rows_per_chunk, r1 = min(m, r0 + rows_per_chunk);
  // a group past the last column reads its neighbour to the left instead (same
  // rows, valid memory) and is not stored
  int col[J];
#pragma unroll
  for (int j = 0; j < J; j++) col[j] = min(cb + j * GS, n - V);
  if (col[0] < 0) return;  // n < V cannot happen for V = 1; for V = 4 the caller guarantees n >= 4
  const float* a = A + (int64_t)r0 * lda;
  vec acc[J];
#pragma unroll
  for (int j = 0; j < J; j++) acc[j] = vec{};
  int r = r0;
  for (; r + RU <= r1; r += RU) {
    vec v[RU][J];
    float xv[RU];
#pragma unroll
    for (int i = 0; i < RU; i++)
#pragma unroll
      for (int j = 0; j < J; j++) v[i][j] = *reinterpret_cast<const vec*>(a + (int64_t)i * lda + col[j]);
#pragma unroll
    for (int i = 0; i < RU; i++) xv[i] = x[r + i];
#pragma unroll
    for (int i = 0; i < RU; i++)
#pragma unroll
      for (int j = 0; j < J; j++) acc[j] += v[i][j] * xv[i];
    a += (int64_t)RU * lda;
  }
  for (; r < r1; r++, a += lda) {
    const float xr = x[r];
#pragma unroll
    for (int j = 0; j < J; j++) acc[j] += *reinterpret_cast<const vec*>(a + col[j]) * xr;
  }
#pragma unroll
  for (int j = 0; j < J; j++)
    if (cb + j * GS < n) *reinterpret_cast<vec*>(out + (int64_t)blockIdx.y * n + cb + j * GS) = acc[j];
}

// y[c] = sum over chunks of part[k][c].  Four threads share a column: thread q
// adds chunks q, q+4, q+8, ... in that order (eight loads in flight), then the
// four sums are added as (s0 + s1) + (s2 + s3).
__global__ __launch_bounds__(256) void k_gemv_t_sum(const float* __restrict__ part, float* __restrict__ y,
                                                    int chunks, int n) {
  __shared__ float sh[4][64];
  const int cg = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + cg;
  float acc = 0.f;
  if (c < n) {
    int k = q;
    for (; k + 28 < chunks; k += 32) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = part[(int64_t)(k + 4 * i) * n + c];
#pragma unroll
      for (int i = 0; i < 8; i++) acc += v[i];
    }
    for (; k < chunks; k += 4) acc += part[(int64_t)k * n + c];
  }
  sh[q][cg] = acc;
  __syncthreads();
  if (q == 0 && c < n) y[c] = (sh[0][cg] + sh[1][cg]) + (sh[2][cg] + sh[3][cg]);
}

__global__ __launch_bounds__(256) void k_outer(const float* __restrict__ x,
                                               const float* __restrict__ y, float* __restrict__ A,
                                               int64_t m, int64_t n) {
  const int64_t total = m * n, stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
    A[i] = x[i / n] * y[i % n];
}

// float64 twins (Dgemv / Dger, cuda/linalg.go:94-159): same shapes, plain loads.
__global__ __launch_bounds__(256) void k_dgemv_n(const double* __restrict__ A, const double* __restrict__ x,
                                                 double* __restrict__ y, int m, int n, int lda) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= m) return;
  const double* a = A + (int64_t)row * lda;
  double acc = 0.0;
  for (int i = lane; i < n; i += 64) acc += a[i] * x[i];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) y[row] = acc;
}

__global__ __launch_bounds__(256) void k_dgemv_t(const double* __restrict__ A, const double* __restrict__ x,
                                                 double* __restrict__ y, int m, int n, int lda) {
  const int col = blockIdx.x * 256 + threadIdx.x;
  if (col >= n) return;
  double acc = 0.0;
  for (int r = 0; r < m; r++) acc += A[(int64_t)r * lda + col] * x[r];
  y[col] = acc;
}

__global__ __launch_bounds__(256) void k_douter(const double* __restrict__ x, const double* __restrict__ y,
                                                double* __restrict__ A, int64_t m, int64_t n) {
  const int64_t total = m * n, stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
    A[i] = x[i / n] * y[i % n];
}

inline bool al16(uint64_t p) { return (p & 15u) == 0; }

// ---- tile plan -------------------------------------------------------------------
// Three block shapes: 128x128 (each wavefront 64x64: the throughput shape),
// 64x64 (each wavefront 32x32: more, smaller blocks for problems that would
// leave CUs idle) and 32x256 (all four wavefronts along N: few filters, many
// pixels).  When even the small shape yields too few blocks, K is split across
// grid.z and a second kernel sums the slabs.
enum { kTile128 = 0, kTile64 = 1, kTile32x256 = 2, kTile128x64 = 3 };
struct TilePlan { int tile; int splits; };

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Largest split count whose [splits][M][N] slabs fit the context workspace.
inline int clamp_splits(gh_ctx* ctx, int64_t splits, int64_t M, int64_t N, int64_t K, int64_t batch) {
  if (batch > 1 || splits < 1) return 1;
  const int64_t nk = cdiv(K, 16);
  if (splits > nk) splits = nk;
  if (splits > 64) splits = 64;
  const int64_t slab = M * N * 4;
  if (slab <= 0 || !ctx->workspace) return 1;
  const int64_t fit = ctx->workspace_bytes / slab;
  if (splits > fit) {
    if (gh_ws_short(ctx, splits * slab)) return 1;   // the caller returns ctx->err
    splits = fit;
  }
  return splits < 1 ? 1 : (int)splits;
}

TilePlan plan_tiles(gh_ctx* ctx, int64_t M, int64_t N, int64_t K, int64_t batch, bool allow_32x256) {
  TilePlan p{kTile128, 1};
  if (const char* env = getenv("GORGONIA_HIP_GEMM_PLAN")) {  // tuning override: "tile,splits"
    int t = 0, sp = 1;
    if (sscanf(env, "%d,%d", &t, &sp) == 2 && t >= 0 && t <= 3 && sp >= 1) {
      p.tile = (t == kTile32x256 && !allow_32x256) ? kTile64 : t;
      p.splits = clamp_splits(ctx, sp, M, N, K, batch);
      return p;
    }
  }
  const int64_t cus = ctx->cu_count;
  const int64_t big = cdiv(M, 128) * cdiv(N, 128) * batch;
  if (big >= cus && M > 64) return p;
  if (allow_32x256 && M <= 32) p.tile = kTile32x256;
  else p.tile = kTile64;
  const int64_t blocks = p.tile == kTile64 ? cdiv(M, 64) * cdiv(N, 64) * batch : cdiv(M, 32) * cdiv(N, 256);
  if (batch == 1 && blocks < 2 * cus) {
    const int64_t nk = cdiv(K, 16);
    int64_t sp = 1;
    if (!allow_32x256) {
      // matrix product on 64x64 tiles: a compute unit works through its workgroups' k-tiles at about
      // 0.8 us each however many share it, and a second launch to add the slabs costs 3.5 us plus
      // 1 us per slab and million results (1152 x 625 results, K = 128 ... 2048: this picks the
      // measured best count, one slice up to K = 256 and four from 512 on, where
      // cdiv(2 cus, blocks) = 3 lost 8-25 %)
      double best = 0;
      const double slab_us = (double)M * (double)N * 1e-6;
      for (int64_t s = 1; s <= 16 && (s == 1 || 2 * s <= nk); s++) {
        const double est = (double)(cdiv(blocks * s, cus) * cdiv(nk, s)) * 0.8 + (s > 1 ? 3.5 + slab_us * (double)s : 0.0);
        if (s == 1 || est < best) { best = est; sp = s; }
      }
    } else {
      sp = cdiv(2 * cus, blocks);
      const int64_t max_sp = nk / 4 > 0 ? nk / 4 : 1;  // at least 4 k-tiles per slice
      if (sp > max_sp) sp = max_sp;
    }
    p.splits = clamp_splits(ctx, sp, M, N, K, batch);
  }
  return p;
}

template <int BM, int BN, int WAVES_M>
int launch_sgemm_cfg(gh_ctx* ctx, const gh_cmd& c, int splits) {
  constexpr int BK = 16;
  const int M = (int)c.dim[0], N = (int)c.dim[1], K = (int)c.dim[2];
  const int lda = (int)c.dim[3], ldb = (int)c.dim[4], ldc = (int)c.dim[5];
  const int batch = c.dim[6] <= 0 ? 1 : (int)c.dim[6];
  const bool ta = c.flags & GH_FLAG_TRANS_A, tb = c.flags & GH_FLAG_TRANS_B;
  const float* A = (const float*)(uintptr_t)c.ptr[0];
  const float* B = (const float*)(uintptr_t)c.ptr[1];
  float* C = (float*)(uintptr_t)c.ptr[2];
  const int64_t sA = batch > 1 ? c.dim[7] : 0, sB = batch > 1 ? c.dim[8] : 0, sC = batch > 1 ? c.dim[9] : 0;
  // 16-byte vector loads need aligned bases, leading dimensions and batch
  // strides, and a contiguous extent that is a multiple of four.
  const bool vec = al16(c.ptr[0]) && al16(c.ptr[1]) && lda % 4 == 0 && ldb % 4 == 0 &&
                   sA % 4 == 0 && sB % 4 == 0 && (ta ? M % 4 == 0 : K % 4 == 0) &&
                   (tb ? K % 4 == 0 : N % 4 == 0);
  const int act = (c.flags & GH_FLAG_ACT_RELU) ? 1 : (c.flags & GH_FLAG_ACT_LEAKY) ? 2 : 0;
  const float* bias = (c.flags & GH_FLAG_GEMM_BIAS) ? (const float*)(uintptr_t)c.ptr[3] : nullptr;
  float* ws = (float*)ctx->workspace;
  if (splits > 1 && (batch > 1 || (int64_t)splits * M * N * 4 > ctx->workspace_bytes))
    return gh_fail(ctx, GH_ESTATE, "sgemm: split-K slabs do not fit the workspace");
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM, splits > 1 ? splits : batch);
#define GH_GEMM_LAUNCH(TA_, TB_, V_)                                                                 \
  hipLaunchKernelGGL((k_sgemm<BM, BN, BK, WAVES_M, TA_, TB_, V_>), grid, dim3(kThreads), 0, ctx->stream, \
                     A, B, C, M, N, K, lda, ldb, ldc, sA, sB, sC, act, c.f[0], splits, ws, bias)
  if (bias && splits <= 1) {   // untransposed only (the command is validated that way)
    if (vec)
      hipLaunchKernelGGL((k_sgemm<BM, BN, BK, WAVES_M, false, false, true, true>), grid, dim3(kThreads), 0, ctx->stream,
                         A, B, C, M, N, K, lda, ldb, ldc, sA, sB, sC, act, c.f[0], splits, ws, bias);
    else
      hipLaunchKernelGGL((k_sgemm<BM, BN, BK, WAVES_M, false, false, false, true>), grid, dim3(kThreads), 0, ctx->stream,
                         A, B, C, M, N, K, lda, ldb, ldc, sA, sB, sC, act, c.f[0], splits, ws, bias);
  } else if (vec) {
    if (!ta && !tb) GH_GEMM_LAUNCH(false, false, true);
    else if (!ta && tb) GH_GEMM_LAUNCH(false, true, true);
    else if (ta && !tb) GH_GEMM_LAUNCH(true, false, true);
    else GH_GEMM_LAUNCH(true, true, true);
  } else {
    if (!ta && !tb) GH_GEMM_LAUNCH(false, false, false);
    else if (!ta && tb) GH_GEMM_LAUNCH(false, true, false);
    else if (ta && !tb) GH_GEMM_LAUNCH(true, false, false);
    else GH_GEMM_LAUNCH(true, true, false);
  }
#undef GH_GEMM_LAUNCH
  int rc = gh_check_hip(ctx, hipGetLastError(), "sgemm launch");
  if (rc || splits <= 1) return rc;
  const int64_t total = (int64_t)M * N;
  int64_t blocks = cdiv(total, 256);
  if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
  if (bias)
    hipLaunchKernelGGL((k_splitk_reduce<StoreRowMajorBias>), dim3((int)blocks), dim3(256), 0, ctx->stream, ws,
                       splits, M, N, StoreRowMajorBias{C, ldc, bias}, act, c.f[0]);
  else
    hipLaunchKernelGGL((k_splitk_reduce<StoreRowMajor>), dim3((int)blocks), dim3(256), 0, ctx->stream, ws,
                       splits, M, N, StoreRowMajor{C, ldc}, act, c.f[0]);
  return gh_check_hip(ctx, hipGetLastError(), "split-K reduce launch");
}

template <int BM, int BN, int WAVES_M, int KH, int KW>
int launch_conv_cfg(gh_ctx* ctx, const gh_cmd& c, const ConvGeom& g, int F, int K, int splits) {
  constexpr int BK = 16;
  const bool vec = al16(c.ptr[1]) && K % 4 == 0;
  const ConvTail tail = conv_tail(c);
  const dim3 grid((g.P + BN - 1) / BN, (F + BM - 1) / BM, splits);
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  const float* w = (const float*)(uintptr_t)c.ptr[1];
  float* y = (float*)(uintptr_t)c.ptr[2];
  float* ws = (float*)ctx->workspace;
  if (splits > 1 && (int64_t)splits * F * g.P * 4 > ctx->workspace_bytes)
    return gh_fail(ctx, GH_ESTATE, "conv2d: split-K slabs do not fit the workspace");
  if (vec)
    hipLaunchKernelGGL((k_conv2d<BM, BN, BK, WAVES_M, KH, KW, true>), grid, dim3(kThreads), 0,
                       ctx->stream, x, w, y, g, F, K, tail, splits, ws);
  else
    hipLaunchKernelGGL((k_conv2d<BM, BN, BK, WAVES_M, KH, KW, false>), grid, dim3(kThreads), 0,
                       ctx->stream, x, w, y, g, F, K, tail, splits, ws);
  int rc = gh_check_hip(ctx, hipGetLastError(), "conv2d launch");
  if (rc || splits <= 1) return rc;
  const int64_t total = (int64_t)F * g.P;
  int64_t blocks = cdiv(total, 256);
  if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
  hipLaunchKernelGGL((k_splitk_reduce<StoreNCHW>), dim3((int)blocks), dim3(256), 0, ctx->stream, ws,
                     splits, F, g.P, StoreNCHW{y, F, g.oh * g.ow, tail}, 0, 0.f);
  return gh_check_hip(ctx, hipGetLastError(), "split-K reduce launch");
}

template <int BM, int BN, int WAVES_M>
int launch_conv_k(gh_ctx* ctx, const gh_cmd& c, const ConvGeom& g, int F, int K, int splits) {
  if (g.kh == 3 && g.kw == 3) return launch_conv_cfg<BM, BN, WAVES_M, 3, 3>(ctx, c, g, F, K, splits);
  if (g.kh == 1 && g.kw == 1) return launch_conv_cfg<BM, BN, WAVES_M, 1, 1>(ctx, c, g, F, K, splits);
  return launch_conv_cfg<BM, BN, WAVES_M, 0, 0>(ctx, c, g, F, K, splits);
}

// Exact number of padded rows the widest block window needs.
int conv3_patch_rows(const Conv3Geom& g, int BNU) {
  const int plane = g.oh * g.ow;
  int best = 0;
  for (int n0 = 0; n0 < g.P; n0 += BNU) {
    const int pl = (n0 + BNU < g.P ? n0 + BNU : g.P) - 1;
    const int b0 = n0 / plane, b1 = pl / plane;
    const int gp0 = b0 * g.Hp + (n0 - b0 * plane) / g.ow;
    const int gp1 = b1 * g.Hp + (pl - b1 * plane) / g.ow;
    const int need = gp1 - gp0 + 3;
    if (need > best) best = need;
  }
  return best;
}

template <int BM, int BN, int CC, int WAVES_M, int PMAX>
int launch_conv3_cfg(gh_ctx* ctx, const gh_cmd& c, Conv3Geom g, int splits, size_t lds_bytes) {
  const bool vec = al16(c.ptr[1]) && g.K % 4 == 0;
  const ConvTail tail = conv_tail(c);
  const unsigned pixel_tiles = g.TW > 0 ? (unsigned)(g.B * g.tiles_y * g.tiles_x) : (unsigned)((g.P + g.BNU - 1) / g.BNU);
  const dim3 grid(pixel_tiles, (g.F + BM - 1) / BM, splits);
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  const float* w = (const float*)(uintptr_t)c.ptr[1];
  float* y = (float*)(uintptr_t)c.ptr[2];
  float* ws = (float*)ctx->workspace;
  if (splits > 1 && (int64_t)splits * g.F * g.P * 4 > ctx->workspace_bytes)
    return gh_fail(ctx, GH_ESTATE, "conv2d: split-K slabs do not fit the workspace");
  if (vec)
    hipLaunchKernelGGL((k_conv3x3_lds<BM, BN, CC, WAVES_M, PMAX, true>), grid, dim3(kThreads), lds_bytes,
                       ctx->stream, x, w, y, g, tail, splits, ws);
  else
    hipLaunchKernelGGL((k_conv3x3_lds<BM, BN, CC, WAVES_M, PMAX, false>), grid, dim3(kThreads), lds_bytes,
                       ctx->stream, x, w, y, g, tail, splits, ws);
  int rc = gh_check_hip(ctx, hipGetLastError(), "conv3x3 launch");
  if (rc || splits <= 1) return rc;
  const int64_t total = (int64_t)g.F * g.P;
  int64_t blocks = cdiv(total, 256);
  if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
  hipLaunchKernelGGL((k_splitk_reduce<StoreNCHW>), dim3((int)blocks), dim3(256), 0, ctx->stream, ws,
                     splits, g.F, g.P, StoreNCHW{y, g.F, g.oh * g.ow, tail}, 0, 0.f);
  return gh_check_hip(ctx, hipGetLastError(), "split-K reduce launch");
}

// Geometry, tile shape and LDS need of the LDS-staged kernel for one command;
// false when the shape is not one it takes (or, with `pool`, when the result
// cannot be cut into blocks of whole pooling windows).
template <int CC>
bool conv3_plan(const gh_cmd& c, bool pool, Conv3Geom* gout, int* BMo, int* BNo, size_t* lds_out, int* per_thread_out) {
  const int B = (int)c.dim[0], C = (int)c.dim[1], H = (int)c.dim[2], W = (int)c.dim[3], F = (int)c.dim[4];
  const int pad = (int)c.dim[7];
  if (c.dim[5] != 3 || c.dim[6] != 3 || c.dim[9] != 1 || c.dim[10] != 1 || c.dim[11] != 1 ||
      c.dim[12] != 1 || c.dim[8] != pad || pad > 1 || C < CC || C % CC != 0)
    return false;
  if (getenv("GORGONIA_HIP_CONV_GATHER")) return false;  // tuning switch: force the gather kernel
  Conv3Geom g{};
  g.B = B; g.C = C; g.H = H; g.W = W; g.F = F; g.pad = pad;
  g.oh = H + 2 * pad - 2; g.ow = W + 2 * pad - 2;
  if (g.oh <= 0 || g.ow <= 0) return false;
  if (pool && (g.oh < 2 || g.ow < 2)) return false;
  g.P = B * g.oh * g.ow;
  g.Hp = H + 2 * pad; g.PW = W + 2 * pad;
  g.K = C * 9;
  g.nchunks = (C + CC - 1) / CC;
  g.pool = pool ? 1 : 0; g.ph = g.oh / 2; g.pw = g.ow / 2;
  // Tile choice: 64x64 blocks measured fastest on every 3x3 layer of the
  // benchmark configurations (more, smaller blocks hide the staging latency
  // better than 128-wide ones).
  int BM = 64, BN = 64;
  const char* tile_env = getenv("GORGONIA_HIP_CONV_TILE");  // tuning override: 0 = 128 wide, 1 = 64x64, 2 = 128x64
  if (tile_env && !pool) {
    if (atoi(tile_env) == 0) { BM = F > 64 ? 128 : 64; BN = 128; }
    if (atoi(tile_env) == 2 && F > 64) { BM = 128; BN = 64; }
  }
  g.BNU = BN;
  if (g.ow >= 64 && !getenv("GORGONIA_HIP_CONV_GATHER_WIDE") && (!tile_env || pool)) {
    // Wide rows: BN consecutive pixels touch only one or two image rows, and the
    // row-stacked patch would hold whole rows for them.  Cut the image into
    // TH x TW rectangles instead (the shape that wastes the fewest pixels on
    // partial tiles, then the smallest patch) and stage the window under each.
    if (F <= 32) { BM = 32; BN = 128; }
    int best_th = 0, best_tw = 0;
    int64_t best_tiles = 0, best_patch = 0;
    for (int tw = 4; tw <= BN; tw *= 2) {
      const int th = BN / tw;
      if (pool && th < 2) continue;   // a block must hold whole 2x2 windows
      const int64_t tiles = cdiv(g.oh, th) * cdiv(g.ow, tw);
      const int64_t patch = (int64_t)(th + 2) * (tw + 2);
      if (!best_tw || tiles < best_tiles || (tiles == best_tiles && patch < best_patch)) {
        best_th = th; best_tw = tw; best_tiles = tiles; best_patch = patch;
      }
    }
    g.TH = best_th; g.TW = best_tw;
    g.tiles_x = (int)cdiv(g.ow, g.TW); g.tiles_y = (int)cdiv(g.oh, g.TH);
    g.PW = g.TW + 2; g.R = g.TH + 2; g.CP = g.R * g.PW;
    g.BNU = BN;
    g.NPR = g.TH / 2;
  } else {
    if (pool) {
      // rows per block: an even count when oh is even (stacked rows then pair
      // up inside every image), whole images when it is odd
      const int unit = (g.oh & 1) ? g.oh : 2;
      int rt = (BN / g.ow) / unit * unit;
      if (rt == 0) { BN = 128; rt = (BN / g.ow) / unit * unit; }
      if (rt == 0) return false;
      g.BNU = rt * g.ow;
      g.NPR = (g.oh & 1) ? (rt / g.oh) * g.ph : rt / 2;
    }
    g.R = conv3_patch_rows(g, g.BNU);
    g.CP = g.R * g.PW;
  }
  size_t lds = ((size_t)CC * 9 * (BM + 2) + (size_t)CC * g.CP) * 4;
  if (pool && lds < (size_t)BM * (BN + 1) * 4) lds = (size_t)BM * (BN + 1) * 4;
  if (lds > 64 * 1024) return false;
  // the staging decode's multiply-high divisions are exact below 2^32
  if ((int64_t)CC * g.CP * g.CP >= (1ll << 32) || ((int64_t)B * g.Hp + g.R) * g.Hp >= (1ll << 32)) return false;
  g.mCP = div_magic_of((unsigned)g.CP); g.mPW = div_magic_of((unsigned)g.PW); g.mHp = div_magic_of((unsigned)g.Hp);
  const int per_thread = (CC * g.CP + kThreads - 1) / kThreads;  // patch elements each thread stages
  if (per_thread > 16) return false;  // the gather kernel does better
  *gout = g; *BMo = BM; *BNo = BN; *lds_out = lds; *per_thread_out = per_thread;
  return true;
}

// Returns -1 when the shape is not one the LDS-staged kernel takes.
template <int CC>
int try_launch_conv3_cc(gh_ctx* ctx, const gh_cmd& c) {
  Conv3Geom g;
  int BM, BN, per_thread;
  size_t lds;
  const bool pool = c.flags & GH_FLAG_CONV_POOL2;
  if (!conv3_plan<CC>(c, pool, &g, &BM, &BN, &lds, &per_thread)) return -1;
  const int F = g.F;
  const int64_t cus = ctx->cu_count;
  const int64_t pixel_tiles = g.TW > 0 ? (int64_t)g.B * g.tiles_x * g.tiles_y : cdiv(g.P, g.BNU);
  // the channel chunks are split across grid.z when the tiles alone leave the
  // chip under-filled (never with fused pooling: the pooled epilogue needs the
  // finished sums)
  const int64_t blocks = cdiv(F, BM) * pixel_tiles;
  int splits = 1;
  if (const char* env = getenv("GORGONIA_HIP_CONV_SPLITS")) splits = atoi(env);
  else {
    splits = (int)((5 * cus / 2 + blocks / 2) / blocks);       // aim at ~2.5 blocks per CU
    if (splits > g.nchunks / 4) splits = g.nchunks / 4;        // at least 4 chunks per slice
  }
  if (splits > g.nchunks) splits = g.nchunks;
  if (splits < 1) splits = 1;
  if (pool) {
    // the K slices the same layer gets without the pool (its own block count)
    Conv3Geom g0;
    int BM0, BN0, pt0;
    size_t lds0;
    int vs = 1;
    if (conv3_plan<CC>(c, false, &g0, &BM0, &BN0, &lds0, &pt0)) {
      const int64_t tiles0 = g0.TW > 0 ? (int64_t)g0.B * g0.tiles_x * g0.tiles_y : cdiv(g0.P, g0.BNU);
      const int64_t blocks0 = cdiv(F, BM0) * tiles0;
      if (const char* env = getenv("GORGONIA_HIP_CONV_SPLITS")) vs = atoi(env);
      else {
        vs = (int)((5 * cus / 2 + blocks0 / 2) / blocks0);
        if (vs > g.nchunks / 4) vs = g.nchunks / 4;
      }
      if (vs > g.nchunks) vs = g.nchunks;
      if (vs < 1) vs = 1;
      if (vs > 1 && (int64_t)vs * F * g.P * 4 > ctx->workspace_bytes) {
        if (int rc = gh_ws_short(ctx, (int64_t)vs * F * g.P * 4)) return rc;
        while (vs > 1 && (int64_t)vs * F * g.P * 4 > ctx->workspace_bytes) vs--;
      }
    }
    g.vsplits = vs;
    splits = 1;
  }
  if (splits > 1 && (int64_t)splits * F * g.P * 4 > ctx->workspace_bytes) {
    if (int rc = gh_ws_short(ctx, (int64_t)splits * F * g.P * 4)) return rc;
    while (splits > 1 && (int64_t)splits * F * g.P * 4 > ctx->workspace_bytes) splits--;
  }
#define GH_CONV3(BM_, BN_)                                                                        \
  (per_thread <= 8 ? launch_conv3_cfg<BM_, BN_, CC, 2, 8>(ctx, c, g, splits, lds)                 \
                   : launch_conv3_cfg<BM_, BN_, CC, 2, 16>(ctx, c, g, splits, lds))
  if (BM == 32)
    return per_thread <= 8 ? launch_conv3_cfg<32, 128, CC, 1, 8>(ctx, c, g, splits, lds)
                           : launch_conv3_cfg<32, 128, CC, 1, 16>(ctx, c, g, splits, lds);
  if (BN == 64 && BM == 128) return GH_CONV3(128, 64);
  if (BN == 64) return GH_CONV3(64, 64);
  if (BM == 128) return GH_CONV3(128, 128);
  return GH_CONV3(64, 128);
#undef GH_CONV3
}

// Eight channels per chunk: sixteen measured within 3 % either way on the
// benchmark layers and doubles the LDS footprint.
int try_launch_conv3(gh_ctx* ctx, const gh_cmd& c) { return try_launch_conv3_cc<8>(ctx, c); }

}  // namespace

// GORGONIA_HIP_SKINNY_TILE = "32", "16x32" or "16x16" pins the small-output kernel (measurements).
static const char* force_tile() { return getenv("GORGONIA_HIP_SKINNY_TILE"); }

// (A kernel with one wavefront per output row for N <= 16 - lane l taking
// k = l, l + 64, ... and a butterfly sum - was measured at 13 us on 128x625x10
// against 7 us for the 32x32 tile: every B load touches 64 different lines.)
// Small-output products (dense layers of a small batch): returns -1 when the
// shape belongs to the tiled kernel.
// Whether the small-output kernels take a product, on a device of `cus` compute units: the one test
// behind the launcher and the route query.
static bool gemm_skinny_takes(const gh_cmd& c, int cus) {
  const int64_t batch = c.dim[6] <= 0 ? 1 : c.dim[6];
  const bool ta = c.flags & GH_FLAG_TRANS_A, tb = c.flags & GH_FLAG_TRANS_B;
  if (batch != 1 || (ta && tb)) return false;
  if (cdiv(c.dim[0], 32) * cdiv(c.dim[1], 32) > cus || c.dim[2] < 32) return false;
  if (getenv("GORGONIA_HIP_GEMM_PLAN")) return false;  // a forced tile plan means the tiled kernel
  // transposed views only have the 16-row kernel, which wants 16 rows and has no softmax for them
  if ((ta || tb) && (c.dim[0] < 16 || (c.flags & GH_FLAG_GEMM_SOFTMAX))) return false;
  return true;
}

static int try_launch_gemm_skinny(gh_ctx* ctx, const gh_cmd& c) {
  if (!gemm_skinny_takes(c, ctx->cu_count)) return -1;
  const bool ta = c.flags & GH_FLAG_TRANS_A, tb = c.flags & GH_FLAG_TRANS_B;
  const int M = (int)c.dim[0], N = (int)c.dim[1], K = (int)c.dim[2];
  const int64_t tiles = cdiv(M, 32) * cdiv(N, 32);
  const int lda = (int)c.dim[3], ldb = (int)c.dim[4], ldc = (int)c.dim[5];
  const int act = (c.flags & GH_FLAG_ACT_RELU) ? 1 : (c.flags & GH_FLAG_ACT_LEAKY) ? 2 : 0;
  constexpr int WV = 8;  // 512 threads leave each wavefront 256 registers for the grouped loads
  const int softmax = (c.flags & GH_FLAG_GEMM_SOFTMAX) ? 1 : 0;
  const float* A = (const float*)(uintptr_t)c.ptr[0];
  const float* B = (const float*)(uintptr_t)c.ptr[1];
  float* C = (float*)(uintptr_t)c.ptr[2];
  const float* bias = (c.flags & GH_FLAG_GEMM_BIAS) ? (const float*)(uintptr_t)c.ptr[3] : nullptr;
  // Few 32x32 tiles: 16-row tiles reach two to four times as many compute units.
  // Which kernel takes a product depends on its shape only, never on the
  // softmax flag, so the fused and the separate softmax see the same product
  // bits: N <= 16 goes to the 16x16 tiles (softmax in their epilogue), 16 < N <=
  // 32 stays on the 32x32 tile.  Transposed views (the weight and input
  // gradients of a dense layer) only have the 16-row kernel.
  const char* force = force_tile();
  const bool transposed = ta || tb;
  const bool tiles16 = N <= 16 || (N > 32 && tiles * 2 <= ctx->cu_count);
  if (transposed || (M >= 16 && tiles16 && !(force && !strcmp(force, "32")))) {
    // 16x32 tiles read whole 128-byte lines of B; when even those leave half the
    // chip without a tile, 16x16 (measured on MI355X, 8 wavefronts per block:
    // 128x625x1152 11.0 us on 32x32, 8.4 on 16x32, 9.8 on 16x16; 64x1000x4096
    // 33 / 21.8 / 19.5 us)
    const int64_t blocks_wide = cdiv(M, 16) * cdiv(N, 32);
    const bool narrow = N < 32 || (force ? !strcmp(force, "16x16") : blocks_wide * 2 <= ctx->cu_count);
    auto launch16 = [&](auto kernel, int bn) {
      hipLaunchKernelGGL(kernel, dim3((N + bn - 1) / bn, (M + 15) / 16), dim3(WV * 64), 0, ctx->stream, A, B, C, M,
                         N, K, lda, ldb, ldc, act, c.f[0], bias, softmax);
    };
    // Sixteen wavefronts share the K of a long contraction (a function of the shape alone, like the tile): each
    // wavefront's chain of grouped loads is half as long (measured: 128x1152x625 7.8 -> 7.2 us, 256x784x300
    // 5.8 -> 5.3, 128x625x10 4.3 -> 4.1; nothing below K = 512, where a wavefront has four chunks or fewer).
    static const bool no16 = getenv("GORGONIA_HIP_SKINNY_WAVES8") != nullptr;   // tuning switch
    const bool wide16 = K >= 512 && !no16;
    auto launch16w = [&](auto kernel, int bn) {
      hipLaunchKernelGGL(kernel, dim3((N + bn - 1) / bn, (M + 15) / 16), dim3(16 * 64), 0, ctx->stream, A, B, C, M,
                         N, K, lda, ldb, ldc, act, c.f[0], bias, softmax);
    };
#define GH_SKINNY16(TA_, TB_)                                                               \
  do {                                                                                      \
    if (wide16 && !narrow) launch16w(k_gemm_skinny16<16, 2, TA_, TB_>, 32);                 \
    else if (wide16) launch16w(k_gemm_skinny16<16, 1, TA_, TB_>, 16);                       \
    else if (narrow) launch16(k_gemm_skinny16<WV, 1, TA_, TB_>, 16);                        \
    else launch16(k_gemm_skinny16<WV, 2, TA_, TB_>, 32);                                    \
  } while (0)
    if (ta) GH_SKINNY16(true, false);
    else if (tb) GH_SKINNY16(false, true);
    else GH_SKINNY16(false, false);
#undef GH_SKINNY16
    return gh_check_hip(ctx, hipGetLastError(), "skinny gemm launch");
  }
  const bool vec_a = al16(c.ptr[0]) && lda % 4 == 0 && K % 16 == 0;
  const dim3 grid((N + 31) / 32, (M + 31) / 32);
  const bool vec_b = N >= 32;   // whole column tiles (the last one moved left)
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(WV * 64), 0, ctx->stream, A, B, C, M, N, K, lda, ldb, ldc, act, c.f[0],
                       softmax, bias);
  };
  if (vec_a && vec_b) launch(k_gemm_skinny<WV, true, true>);
  else if (vec_a) launch(k_gemm_skinny<WV, true, false>);
  else if (vec_b) launch(k_gemm_skinny<WV, false, true>);
  else launch(k_gemm_skinny<WV, false, false>);
  return gh_check_hip(ctx, hipGetLastError(), "skinny gemm launch");
}

template <int BM, int BN, int BK>
static void launch_conv64_cfg(gh_ctx* ctx, const gh_cmd& c, const ConvGeom64& g) {
  const dim3 grid((g.P + BN - 1) / BN, (g.F + BM - 1) / BM, 1);
  const double* x = (const double*)(uintptr_t)c.ptr[0];
  const double* w = (const double*)(uintptr_t)c.ptr[1];
  double* y = (double*)(uintptr_t)c.ptr[2];
  if ((g.K & 1) == 0 && (c.ptr[1] & 15) == 0)
    hipLaunchKernelGGL((k_conv2d_f64_mfma<BM, BN, BK, true>), grid, dim3(kThreads), 0, ctx->stream, x, w, y, g);
  else
    hipLaunchKernelGGL((k_conv2d_f64_mfma<BM, BN, BK, false>), grid, dim3(kThreads), 0, ctx->stream, x, w, y, g);
}

// Geometry of a float64 convolution command; false when an extent leaves the
// 32-bit index arithmetic of the matrix-core kernels.
static bool conv64_fill(const gh_cmd& c, ConvGeom64* out) {
  ConvGeom64& g = *out;
  const int64_t B = c.dim[0];
  g.C = (int)c.dim[1]; g.H = (int)c.dim[2]; g.W = (int)c.dim[3]; g.F = (int)c.dim[4];
  g.kh = (int)c.dim[5]; g.kw = (int)c.dim[6]; g.padH = (int)c.dim[7]; g.padW = (int)c.dim[8];
  g.strideH = (int)c.dim[9]; g.strideW = (int)c.dim[10]; g.dilH = (int)c.dim[11]; g.dilW = (int)c.dim[12];
  g.oh = (int)gh_conv_out(g.H, g.kh, g.padH, g.strideH, g.dilH);
  g.ow = (int)gh_conv_out(g.W, g.kw, g.padW, g.strideW, g.dilW);
  const int64_t P = B * g.oh * g.ow, K = (int64_t)g.C * g.kh * g.kw;
  if (P <= 0 || K <= 0 || P > 0x7fffffff || K * (int64_t)(g.kh * g.kw) >= ((int64_t)1 << 32)) return false;
  if ((int64_t)g.C * g.H * g.W + (int64_t)(g.padH + 1) * g.W + g.padW >= 0x7fffffff) return false;  // 32-bit offsets inside an image
  g.P = (int)P;
  g.K = (int)K;
  g.mKK = div_magic_of((unsigned)(g.kh * g.kw));
  g.mkw = div_magic_of((unsigned)g.kw);
  return true;
}

// Float64 Conv2d on the matrix cores; false = not taken (few filters or a tiny
// problem: the one-thread-per-result kernel stays).
bool gh_try_launch_conv2d_f64_mfma(gh_ctx* ctx, const gh_cmd& c) {
  ConvGeom64 g;
  if (!conv64_fill(c, &g)) return false;
  const int64_t P = g.P, K = g.K;
  if (g.F < 16 || P < 256 || K < 8 || P * g.F * K < (int64_t)1 << 22) return false;
  const int64_t tiles128 = (int64_t)((g.F + 127) / 128) * ((P + 127) / 128);
  // the smaller tiles do less per k-tile, so they take twice the k range per barrier
  const int64_t tiles64 = (int64_t)((g.F + 63) / 64) * ((P + 63) / 64);
  if (const char* e = getenv("GORGONIA_HIP_CONV64_TILE")) {   // tuning override: 0 32x128, 1 128x128, 2 64x64, 3 32x64
    switch (atoi(e)) {
      case 0: launch_conv64_cfg<32, 128, 16>(ctx, c, g); return true;
      case 1: launch_conv64_cfg<128, 128, 8>(ctx, c, g); return true;
      case 2: launch_conv64_cfg<64, 64, 16>(ctx, c, g); return true;
      default: launch_conv64_cfg<32, 64, 16>(ctx, c, g); return true;
    }
  }
  if (g.F <= 32) launch_conv64_cfg<32, 128, 16>(ctx, c, g);
  else if (tiles128 >= ctx->cu_count) launch_conv64_cfg<128, 128, 8>(ctx, c, g);
  else if (tiles64 >= ctx->cu_count) launch_conv64_cfg<64, 64, 16>(ctx, c, g);
  else launch_conv64_cfg<32, 64, 16>(ctx, c, g);   // too few 64x64 tiles for the device (measured: 97 against 108 us on
                                                   // 128x128x7x7 -> 64 filters, no gain once every CU has a 64x64 tile)
  return true;
}

// Float64 image gradient of a stride-1 convolution: the forward kernel over dy
// with mirrored, transposed filters (held at the top of the workspace).
bool gh_try_launch_conv2d_bwd_data_f64_mfma(gh_ctx* ctx, const gh_cmd& c) {
  ConvGeom64 g;
  if (!conv64_fill(c, &g)) return false;
  const int padH = g.dilH * (g.kh - 1) - g.padH, padW = g.dilW * (g.kw - 1) - g.padW;
  const int64_t wcount = (int64_t)g.F * g.K;
  const int64_t wbytes = (wcount * 8 + 255) / 256 * 256;
  if (g.strideH != 1 || g.strideW != 1 || padH < 0 || padW < 0) return false;
  if (wbytes > ctx->workspace_bytes) return gh_ws_short(ctx, wbytes) != GH_OK;   // true: the caller returns ctx->err
  gh_cmd f{};
  f.opcode = GH_OP_CONV2D;
  f.flags = c.flags;
  double* wt = (double*)((char*)ctx->workspace + ctx->workspace_bytes - wbytes);
  f.ptr[0] = c.ptr[0]; f.ptr[1] = (uint64_t)(uintptr_t)wt; f.ptr[2] = c.ptr[2];
  f.dim[0] = c.dim[0]; f.dim[1] = g.F; f.dim[2] = g.oh; f.dim[3] = g.ow; f.dim[4] = g.C;
  f.dim[5] = g.kh; f.dim[6] = g.kw; f.dim[7] = padH; f.dim[8] = padW;
  f.dim[9] = 1; f.dim[10] = 1; f.dim[11] = g.dilH; f.dim[12] = g.dilW;
  // decide before mirroring whether the forward kernel takes the shape (same tests as above)
  ConvGeom64 gf;
  if (!conv64_fill(f, &gf)) return false;
  if (gf.F < 16 || gf.P < 256 || gf.K < 8 || (int64_t)gf.P * gf.F * gf.K < (int64_t)1 << 22) return false;
  int64_t blocks = cdiv(wcount, 256);
  if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
  hipLaunchKernelGGL(k_flip_filters<double>, dim3((int)blocks), dim3(256), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[1], wt, g.F, g.C, g.kh, g.kw);
  return gh_try_launch_conv2d_f64_mfma(ctx, f);
}

// Float64 filter gradient on the matrix cores, pixel axis cut into slices.
bool gh_try_launch_conv2d_bwd_filter_f64_mfma(gh_ctx* ctx, const gh_cmd& c) {
  ConvGeom64 g;
  if (!conv64_fill(c, &g)) return false;
  if ((int64_t)g.P * g.F * g.K < (int64_t)1 << 22 || g.P < 64) return false;
  constexpr int BM = 64, BN = 64, BK = 16;
  const int64_t tiles = cdiv(g.F, BM) * cdiv(g.K, BN);
  const int64_t nk = cdiv(g.P, BK);
  int64_t splits = cdiv(5 * (int64_t)ctx->cu_count / 2, tiles);   // ~2.5 workgroups per CU
  if (splits > nk / 4) splits = nk / 4;
  if (splits > 512) splits = 512;
  const int64_t slab = (int64_t)g.F * g.K * 8;
  if (splits > 1 && ctx->workspace_bytes / slab < splits) {
    if (gh_ws_short(ctx, splits * slab)) return true;   // the caller returns ctx->err
    splits = ctx->workspace_bytes / slab;
  }
  if (splits < 1) splits = 1;
  double* dw = (double*)(uintptr_t)c.ptr[2];
  const dim3 grid((unsigned)cdiv(g.K, BN), (unsigned)cdiv(g.F, BM), (unsigned)splits);
  hipLaunchKernelGGL((k_conv2d_wgrad_f64<BM, BN, BK>), grid, dim3(kThreads), 0, ctx->stream,
                     (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1], dw, g, (int)splits,
                     (double*)ctx->workspace);
  if (splits > 1) {
    const int64_t total = (int64_t)g.F * g.K;
    int64_t blocks = cdiv(total, 256);
    if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
    hipLaunchKernelGGL(k_splitk_reduce_f64, dim3((int)blocks), dim3(256), 0, ctx->stream,
                       (const double*)ctx->workspace, (int)splits, total, dw);
  }
  return true;
}

template <int BM, int BN, int BK>
static void launch_dgemm_cfg(gh_ctx* ctx, const gh_cmd& c, int M, int N, int K, int64_t batch) {
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM, (unsigned)batch);
  const double* A = (const double*)(uintptr_t)c.ptr[0];
  const double* B = (const double*)(uintptr_t)c.ptr[1];
  double* C = (double*)(uintptr_t)c.ptr[2];
  const int lda = (int)c.dim[3], ldb = (int)c.dim[4], ldc = (int)c.dim[5];
  const int64_t sA = batch > 1 ? c.dim[7] : 0, sB = batch > 1 ? c.dim[8] : 0, sC = batch > 1 ? c.dim[9] : 0;
  const bool ta = c.flags & GH_FLAG_TRANS_A, tb = c.flags & GH_FLAG_TRANS_B;
  const auto even = [](int64_t v) { return (v & 1) == 0; };
  const bool vec = even(M) && even(N) && even(K) && even(lda) && even(ldb) && even(sA) && even(sB) &&
                   ((c.ptr[0] | c.ptr[1]) & 15) == 0;
#define GH_DGEMM_GO(TA, TB)                                                                                    \
  do {                                                                                                         \
    if (vec)                                                                                                   \
      hipLaunchKernelGGL((k_dgemm<BM, BN, BK, TA, TB, true>), grid, dim3(kThreads), 0, ctx->stream, A, B, C, M, \
                         N, K, lda, ldb, ldc, sA, sB, sC);                                                     \
    else                                                                                                       \
      hipLaunchKernelGGL((k_dgemm<BM, BN, BK, TA, TB, false>), grid, dim3(kThreads), 0, ctx->stream, A, B, C,  \
                         M, N, K, lda, ldb, ldc, sA, sB, sC);                                                  \
  } while (0)
  if (ta && tb) GH_DGEMM_GO(true, true);
  else if (ta) GH_DGEMM_GO(true, false);
  else if (tb) GH_DGEMM_GO(false, true);
  else GH_DGEMM_GO(false, false);
#undef GH_DGEMM_GO
}

int gh_launch_gemm(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) {
    const int M = (int)c.dim[0], N = (int)c.dim[1], K = (int)c.dim[2];
    const int64_t batch = c.dim[6] <= 0 ? 1 : c.dim[6];
    const int64_t tiles64 = (int64_t)((M + 63) / 64) * ((N + 63) / 64);
    if (batch == 1 && K >= 64 && tiles64 * 4 <= ctx->cu_count && M >= 1 && N >= 1) {
      const bool ta = c.flags & GH_FLAG_TRANS_A, tb = c.flags & GH_FLAG_TRANS_B;
      const int64_t lda = c.dim[3], ldb = c.dim[4];
      const dim3 grid((N + 15) / 16, (M + 15) / 16, 1);
      const double* A = (const double*)(uintptr_t)c.ptr[0];
      const double* B = (const double*)(uintptr_t)c.ptr[1];
      double* C = (double*)(uintptr_t)c.ptr[2];
      // (which wavefront sums which k, and with AV which k shares an MFMA, depends on the shape and the operands'
      // layout only: a product's bits repeat from run to run)
      const bool pairs = K >= 2 && !getenv("GORGONIA_HIP_DGEMM_SKINNY_SCALAR");   // (tuning switch)
      const bool av = pairs && !ta, bv = pairs && tb;
#define GH_DSK(WV_, AV_, BV_)                                                                                          \
  hipLaunchKernelGGL((k_dgemm_skinny<WV_, AV_, BV_>), grid, dim3(WV_ * 64), 0, ctx->stream, A, B, C, M, N, K,           \
                     ta ? 1 : lda, ta ? lda : 1, tb ? 1 : ldb, tb ? ldb : 1, (int)c.dim[5])
#define GH_DSK_W(WV_)                                            \
  do {                                                           \
    if (av && bv) GH_DSK(WV_, true, true);                       \
    else if (av) GH_DSK(WV_, true, false);                       \
    else if (bv) GH_DSK(WV_, false, true);                       \
    else GH_DSK(WV_, false, false);                              \
  } while (0)
      if (K >= 256) GH_DSK_W(8);   // (sixteen wavefronts, as the float32 kernel has them from K = 512, are slower here: 15.7 us against 14.4)
      else GH_DSK_W(4);
#undef GH_DSK_W
#undef GH_DSK
      return gh_check_hip(ctx, hipGetLastError(), "dgemm launch");
    }
    // 128x128 tiles once they fill the device, 64x64 with a longer k-tile below that
    const int64_t tiles128 = (int64_t)((M + 127) / 128) * ((N + 127) / 128) * batch;
    if (tiles128 >= ctx->cu_count) launch_dgemm_cfg<128, 128, 8>(ctx, c, M, N, K, batch);
    else launch_dgemm_cfg<64, 64, 16>(ctx, c, M, N, K, batch);
    return gh_check_hip(ctx, hipGetLastError(), "dgemm launch");
  }
  const int rs = try_launch_gemm_skinny(ctx, c);
  if (rs >= 0) return rs;
  if (c.flags & GH_FLAG_GEMM_SOFTMAX)
    return gh_fail(ctx, GH_EINVAL, "gemm: no fused softmax for this shape (see gh_gemm_can_softmax)");
  const int64_t batch = c.dim[6] <= 0 ? 1 : c.dim[6];
  const TilePlan p = plan_tiles(ctx, c.dim[0], c.dim[1], c.dim[2], batch, false);
  if (ctx->err) return ctx->err;
  if (p.tile == kTile128) return launch_sgemm_cfg<128, 128, 2>(ctx, c, p.splits);
  if (p.tile == kTile128x64) return launch_sgemm_cfg<128, 64, 2>(ctx, c, p.splits);
  return launch_sgemm_cfg<64, 64, 2>(ctx, c, p.splits);
}

// The choices of gh_launch_gemm for a float32 product, asked without launching (MI355X's
// compute-unit count, a workspace of the default size).
extern "C" int gh_gemm_route(const gh_cmd* c, int* splits) {
  if (splits) *splits = 1;
  if (!c || c->opcode != GH_OP_GEMM) return -1;
  if (gh_dtype_of(c->flags) == GH_F64) return GH_GEMM_ROUTE_F64;
  const int64_t batch = c->dim[6] <= 0 ? 1 : c->dim[6];
  gh_ctx probe;
  probe.workspace = &probe;   // never dereferenced: only "there is one" and its size are read
  probe.workspace_bytes = 64ll << 20;
  if (gemm_skinny_takes(*c, probe.cu_count)) return GH_GEMM_ROUTE_SMALL_OUTPUT;
  const TilePlan p = plan_tiles(&probe, c->dim[0], c->dim[1], c->dim[2], batch, false);
  if (splits) *splits = p.splits;
  return p.tile == kTile128 ? GH_GEMM_ROUTE_TILE128 : p.tile == kTile128x64 ? GH_GEMM_ROUTE_TILE128X64 : GH_GEMM_ROUTE_TILE64;
}

// The direct kernel's shapes: 3x3, stride 1, no dilation, square padding, at
// most four input channels.
static bool conv_direct_shape(const gh_cmd& c) {
  return c.dim[5] == 3 && c.dim[6] == 3 && c.dim[9] == 1 && c.dim[10] == 1 && c.dim[11] == 1 &&
         c.dim[12] == 1 && c.dim[7] == c.dim[8] && c.dim[1] >= 1 && c.dim[1] <= 4;
}

// The direct kernel's shapes, less those the wide-image kernel runs quicker: three or four
// channels fill most of a quad of its K steps, and on images with enough pixels its matrix
// cores then beat the vector units (3 -> 16 at 416 x 416: 42 us against 53).  Only where it can
// also pool, so that a shape's plain and pooled commands stay with one kernel and one summing
// order.
static bool conv_direct_takes(const gh_cmd& c) {
  if (!conv_direct_shape(c) || getenv("GORGONIA_HIP_CONV_NO_DIRECT")) return false;
  if (c.dim[1] >= 3 && gh_conv_wide_takes(c) && gh_conv_wide_can_pool(c)) return false;
  return true;
}

static int launch_conv_direct(gh_ctx* ctx, const gh_cmd& c) {
  const int B = (int)c.dim[0], C = (int)c.dim[1], H = (int)c.dim[2], W = (int)c.dim[3], F = (int)c.dim[4];
  const int pad = (int)c.dim[7];
  const int oh = H + 2 * pad - 2, ow = W + 2 * pad - 2;
  const bool pool = c.flags & GH_FLAG_CONV_POOL2;
  const int yh = pool ? oh / 2 : oh, yw = pool ? ow / 2 : ow;
  const int64_t pix = (int64_t)B * yh * yw;
  if (pix == 0 || F == 0) return GH_OK;
  // one image per grid z where z can count them and an image's stored pixels fill most of their
  // workgroups' lanes; else the batch's stored pixels in one numbering
  const bool per_image = B <= 65535 && (int64_t)yh * yw < (1ll << 31) &&
                         cdiv((int64_t)yh * yw, 256) * 256 * 10 <= (int64_t)yh * yw * 14;
  const int64_t bx = per_image ? cdiv((int64_t)yh * yw, 256) : cdiv(pix, 256);
  const int64_t nblocks = per_image ? bx * B : bx;
  // enough filter groups to give every SIMD a few wavefronts, at least 4 filters each
  int64_t groups = cdiv((int64_t)ctx->cu_count * 16, nblocks * 4);
  if (groups > F / 4) groups = F / 4;
  if (groups < 1) groups = 1;
  const int fper = (int)cdiv(F, groups);
  const dim3 grid((unsigned)bx, (unsigned)cdiv(F, fper), per_image ? (unsigned)B : 1u);
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  const float* w = (const float*)(uintptr_t)c.ptr[1];
  float* y = (float*)(uintptr_t)c.ptr[2];
  const ConvTail tail = conv_tail(c);
#define GH_DIRECT(C_)                                                                                \
  do {                                                                                               \
    if (pool)                                                                                        \
      hipLaunchKernelGGL((k_conv3x3_direct<C_, 2>), grid, dim3(256), 0, ctx->stream, x, w, y, B, H, W, \
                         F, pad, yh, yw, fper, tail);                                                \
    else                                                                                             \
      hipLaunchKernelGGL((k_conv3x3_direct<C_, 1>), grid, dim3(256), 0, ctx->stream, x, w, y, B, H, W, \
                         F, pad, yh, yw, fper, tail);                                                \
  } while (0)
  switch (C) {
    case 1: GH_DIRECT(1); break;
    case 2: GH_DIRECT(2); break;
    case 3: GH_DIRECT(3); break;
    default: GH_DIRECT(4); break;
  }
#undef GH_DIRECT
  return gh_check_hip(ctx, hipGetLastError(), "direct conv launch");
}

int gh_launch_conv2d(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_conv2d_f64(ctx, c);
  if (c.flags & GH_FLAG_CONV_PRE) {
    const int rcp = gh_conv2d_can_pre(&c) ? gh_try_launch_conv_rows(ctx, c) : -1;
    if (rcp >= 0) return rcp;
    return gh_fail(ctx, GH_EINVAL, "conv2d: no folded first layer for this shape (see gh_conv2d_can_pre)");
  }
  if ((c.flags & GH_FLAG_CONV_KEEP) && !((c.flags & GH_FLAG_CONV_POOL2) && gh_conv2d_can_keep(&c)))
    return gh_fail(ctx, GH_EINVAL, "conv2d: the unpooled result cannot be kept for this command (see gh_conv2d_can_keep)");
  const int rc0 = gh_try_launch_conv_rows1(ctx, c);
  if (rc0 >= 0) return rc0;
  if (conv_direct_takes(c)) return launch_conv_direct(ctx, c);
  const int rcs = gh_try_launch_conv_small(ctx, c);
  if (rcs >= 0) return rcs;
  const int rcp = gh_try_launch_conv_patch(ctx, c);
  if (rcp >= 0) return rcp;
  const int rcw = gh_try_launch_conv_wide(ctx, c);
  if (rcw >= 0) return rcw;
  const int rc1 = gh_try_launch_conv_pointwise(ctx, c);
  if (rc1 >= 0) return rc1;
  const int rc3 = try_launch_conv3(ctx, c);
  if (rc3 >= 0) return rc3;
  if (c.flags & GH_FLAG_CONV_POOL2)
    return gh_fail(ctx, GH_EINVAL, "conv2d: no fused pooling for this shape (see gh_conv2d_can_pool)");
  ConvGeom g;
  g.C = (int)c.dim[1]; g.H = (int)c.dim[2]; g.W = (int)c.dim[3];
  g.kh = (int)c.dim[5]; g.kw = (int)c.dim[6];
  g.padH = (int)c.dim[7]; g.padW = (int)c.dim[8];
  g.strideH = (int)c.dim[9]; g.strideW = (int)c.dim[10];
  g.dilH = (int)c.dim[11]; g.dilW = (int)c.dim[12];
  g.oh = (int)gh_conv_out(g.H, g.kh, g.padH, g.strideH, g.dilH);
  g.ow = (int)gh_conv_out(g.W, g.kw, g.padW, g.strideW, g.dilW);
  g.P = (int)c.dim[0] * g.oh * g.ow;
  const int F = (int)c.dim[4], K = g.C * g.kh * g.kw;
  const TilePlan p = plan_tiles(ctx, F, g.P, K, 1, true);
  if (ctx->err) return ctx->err;
  if (p.tile == kTile128) return launch_conv_k<128, 128, 2>(ctx, c, g, F, K, p.splits);
  if (p.tile == kTile32x256) return launch_conv_k<32, 256, 1>(ctx, c, g, F, K, p.splits);
  return launch_conv_k<64, 64, 2>(ctx, c, g, F, K, p.splits);
}

static ConvGeom conv_geom(const gh_cmd& c) {
  ConvGeom g;
  g.C = (int)c.dim[1]; g.H = (int)c.dim[2]; g.W = (int)c.dim[3];
  g.kh = (int)c.dim[5]; g.kw = (int)c.dim[6];
  g.padH = (int)c.dim[7]; g.padW = (int)c.dim[8];
  g.strideH = (int)c.dim[9]; g.strideW = (int)c.dim[10];
  g.dilH = (int)c.dim[11]; g.dilW = (int)c.dim[12];
  g.oh = (int)gh_conv_out(g.H, g.kh, g.padH, g.strideH, g.dilH);
  g.ow = (int)gh_conv_out(g.W, g.kw, g.padW, g.strideW, g.dilW);
  g.P = (int)c.dim[0] * g.oh * g.ow;
  return g;
}

// Sum `splits` slabs of F x CKK partial filter gradients from the workspace into dw, in slab order.
static int launch_slab_reduce(gh_ctx* ctx, const float* ws, int splits, int F, int CKK, float* dw) {
  const int64_t total = (int64_t)F * CKK;
  if (splits >= 64) {
    hipLaunchKernelGGL((k_splitk_reduce_lanes<StoreRowMajor, 16>), dim3((int)cdiv(total * 16, 256)), dim3(256), 0,
                       ctx->stream, ws, splits, F, CKK, StoreRowMajor{dw, CKK}, 0, 0.f);
  } else if (splits >= 8) {
    hipLaunchKernelGGL((k_splitk_reduce_lanes<StoreRowMajor, 4>), dim3((int)cdiv(total * 4, 256)), dim3(256), 0,
                       ctx->stream, ws, splits, F, CKK, StoreRowMajor{dw, CKK}, 0, 0.f);
  } else {
    int64_t blocks = cdiv(total, 256);
    if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
    hipLaunchKernelGGL((k_splitk_reduce<StoreRowMajor>), dim3((int)blocks), dim3(256), 0, ctx->stream, ws, splits, F,
                       CKK, StoreRowMajor{dw, CKK}, 0, 0.f);
  }
  return gh_check_hip(ctx, hipGetLastError(), "split-K reduce launch");
}

// The direct kernel's shapes that k_conv3x3_wgrad_c1 takes: one channel, a padded image of at most 60 KB, at least
// a wavefront of output pixels.
static bool wgrad_c1_takes(const gh_cmd& c) {
  if (!conv_direct_shape(c) || c.dim[1] != 1 || c.dim[4] > 65535) return false;
  const ConvGeom g = conv_geom(c);
  const size_t img_bytes = (size_t)(g.H + 2 * g.padH) * (g.W + 2 * g.padH) * 4;
  return img_bytes <= 60 * 1024 && g.oh * g.ow >= 64 && g.ow >= 2 && !getenv("GORGONIA_HIP_WGRAD_NO_C1");   // (tuning switch)
}

// dW = dY2d^T . col  (ptr[0] = x, ptr[1] = dy, ptr[2] = dw)
int gh_launch_conv2d_bwd_filter(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_conv2d_bwd_filter_f64(ctx, c);
  const ConvGeom g = conv_geom(c);
  const int F = (int)c.dim[4], CKK = g.C * g.kh * g.kw;
  if (conv_direct_shape(c) && F <= 65535) {
    const int B = (int)c.dim[0];
    int G = B < 64 ? B : 64;
    if ((int64_t)G * F * CKK * 4 > ctx->workspace_bytes) {
      if (int rc = gh_ws_short(ctx, (int64_t)G * F * CKK * 4)) return rc;
      while (G > 1 && (int64_t)G * F * CKK * 4 > ctx->workspace_bytes) G--;
      if ((int64_t)G * F * CKK * 4 > ctx->workspace_bytes)
        return gh_fail(ctx, GH_ESTATE, "conv2d filter gradient: partial sums do not fit the workspace");
    }
    float* wsd = (float*)ctx->workspace;
    const float* xd = (const float*)(uintptr_t)c.ptr[0];
    const float* dyd = (const float*)(uintptr_t)c.ptr[1];
    const size_t img_bytes = (size_t)(g.H + 2 * g.padH) * (g.W + 2 * g.padH) * 4;
    if (wgrad_c1_takes(c)) {
      // as many slabs as give every compute unit a workgroup, within what the images and the workspace allow
      const int fby = (int)cdiv(F, 4);
      // a workgroup's images follow each other (stage, barrier, sum), so few per workgroup; 128 images of 28 x 28,
      // 32 filters: 25.8 us with 16 slabs, 16.0 with 32, 12.5 with 64, 13.0 with 128 (slab sum included; 15.8 on the
      // kernel below)
      int G1 = 64;
      if (const char* e = getenv("GORGONIA_HIP_WGRAD_C1_SLABS")) G1 = atoi(e);   // tuning override
      if (G1 > 256) G1 = 256;
      if (G1 > B) G1 = B;
      while (G1 > 1 && (int64_t)G1 * F * CKK * 4 > ctx->workspace_bytes) G1--;
      if (G1 < 1) G1 = 1;
      // exact while i * d < 2^32: ceil(2^32 / d)
      auto magic = [](int d) { return (unsigned)((0x100000000ull + (unsigned)d - 1) / (unsigned)d); };
      const int PW = g.W + 2 * g.padH;
      hipLaunchKernelGGL(k_conv3x3_wgrad_c1, dim3((unsigned)G1, (unsigned)fby), dim3(256), img_bytes, ctx->stream, xd, dyd,
                         wsd, B, g.H, g.W, F, g.padH, g.oh, g.ow, magic(g.ow), magic(PW));
      int rc1 = gh_check_hip(ctx, hipGetLastError(), "single-channel filter-gradient launch");
      if (rc1) return rc1;
      hipLaunchKernelGGL((k_splitk_reduce_lanes<StoreRowMajor, 4>), dim3((int)cdiv((int64_t)F * CKK * 4, 256)), dim3(256),
                         0, ctx->stream, wsd, G1, F, CKK, StoreRowMajor{(float*)(uintptr_t)c.ptr[2], CKK}, 0, 0.f);
      return gh_check_hip(ctx, hipGetLastError(), "split-K reduce launch");
    }
#define GH_WGRAD_DIRECT(C_, FB_)                                                                             \
  hipLaunchKernelGGL((k_conv3x3_wgrad_direct<C_, FB_>), dim3((unsigned)G, (unsigned)cdiv(F, FB_)), dim3(256), 0, \
                     ctx->stream, xd, dyd, wsd, B, g.H, g.W, F, g.padH, g.oh, g.ow)
    // two filters per workgroup pay for one channel (28x28, 32 filters, 128 images: 15.8 us
    // against 17.4); four filters, or more channels, spend the gain on the longer fold
    switch (g.C) {
      case 1: GH_WGRAD_DIRECT(1, 2); break;
      case 2: GH_WGRAD_DIRECT(2, 1); break;
      case 3: GH_WGRAD_DIRECT(3, 1); break;
      default: GH_WGRAD_DIRECT(4, 1); break;
    }
#undef GH_WGRAD_DIRECT
    int rc = gh_check_hip(ctx, hipGetLastError(), "direct filter-gradient launch");
    if (rc) return rc;
    hipLaunchKernelGGL((k_splitk_reduce_lanes<StoreRowMajor, 4>), dim3((int)cdiv((int64_t)F * CKK * 4, 256)), dim3(256),
                       0, ctx->stream, wsd, G, F, CKK, StoreRowMajor{(float*)(uintptr_t)c.ptr[2], CKK}, 0, 0.f);
    return gh_check_hip(ctx, hipGetLastError(), "split-K reduce launch");
  }
  {
    // small images: the kernel that keeps dy and x of a few images in LDS; slabs summed as below
    int sp = 0;
    const int rcs = gh_try_launch_conv_wgrad_small(ctx, c, &sp);
    if (rcs > 0 || (rcs == 0 && sp <= 1)) return rcs;
    if (rcs == 0) return launch_slab_reduce(ctx, (const float*)ctx->workspace, sp, F, CKK, (float*)(uintptr_t)c.ptr[2]);
  }
  constexpr int BM = 64, BN = 64, BK = 32;
  const int64_t tiles = cdiv(F, BM) * cdiv(CKK, BN);
  const int64_t nk = cdiv(g.P, BK);
  int64_t splits = cdiv(5 * (int64_t)ctx->cu_count / 2, tiles);   // ~2.5 workgroups per CU
  if (splits > nk / 4) splits = nk / 4;
  if (splits > 64) splits = 64;
  const int64_t slab = (int64_t)F * CKK * 4;
  if (splits > 1 && ctx->workspace_bytes / slab < splits) {
    if (int rc = gh_ws_short(ctx, splits * slab)) return rc;
    splits = ctx->workspace_bytes / slab;
  }
  if (splits < 1) splits = 1;
  const float* x = (const float*)(uintptr_t)c.ptr[0];
  const float* dy = (const float*)(uintptr_t)c.ptr[1];
  float* dw = (float*)(uintptr_t)c.ptr[2];
  float* ws = (float*)ctx->workspace;
  const dim3 grid((unsigned)cdiv(CKK, BN), (unsigned)cdiv(F, BM), (unsigned)splits);
  hipLaunchKernelGGL((k_conv2d_wgrad<BM, BN, BK, 2>), grid, dim3(kThreads), 0, ctx->stream, x, dy, dw, g, F,
                     CKK, (int)splits, ws);
  int rc = gh_check_hip(ctx, hipGetLastError(), "conv filter-gradient launch");
  if (rc || splits <= 1) return rc;
  return launch_slab_reduce(ctx, ws, (int)splits, F, CKK, dw);
}

// dX = col2im(dY2d . Wflat)  (ptr[0] = dy, ptr[1] = w, ptr[2] = dx)
int gh_launch_conv2d_bwd_data(gh_ctx* ctx, const gh_cmd& c) {
  if (gh_dtype_of(c.flags) == GH_F64) return gh_launch_conv2d_bwd_data_f64(ctx, c);
  const ConvGeom g = conv_geom(c);
  const int B = (int)c.dim[0], F = (int)c.dim[4];
  const float* dy = (const float*)(uintptr_t)c.ptr[0];
  const float* w = (const float*)(uintptr_t)c.ptr[1];
  float* dx = (float*)(uintptr_t)c.ptr[2];
  const int64_t wbytes = ((int64_t)F * g.C * g.kh * g.kw * 4 + 255) / 256 * 256;
  const int padH = g.dilH * (g.kh - 1) - g.padH, padW = g.dilW * (g.kw - 1) - g.padW;
  const bool mirror_shape = g.strideH == 1 && g.strideW == 1 && padH >= 0 && padW >= 0;
  if (mirror_shape && wbytes > ctx->workspace_bytes / 2)
    if (int rc = gh_ws_short(ctx, 2 * wbytes)) return rc;
  if (mirror_shape && wbytes <= ctx->workspace_bytes / 2) {
    // mirrored filters live at the top of the workspace; the forward launch
    // below may use what is left of it for its own split-K slabs
    float* wt = (float*)((char*)ctx->workspace + ctx->workspace_bytes - wbytes);
    int64_t blocks = cdiv((int64_t)F * g.C * g.kh * g.kw, 256);
    if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
    hipLaunchKernelGGL(k_flip_filters<float>, dim3((int)blocks), dim3(256), 0, ctx->stream, w, wt, F, g.C, g.kh, g.kw);
    int rc = gh_check_hip(ctx, hipGetLastError(), "filter mirror launch");
    if (rc) return rc;
    gh_cmd f{};
    f.opcode = GH_OP_CONV2D;
    f.ptr[0] = c.ptr[0]; f.ptr[1] = (uint64_t)(uintptr_t)wt; f.ptr[2] = c.ptr[2];
    f.dim[0] = B; f.dim[1] = F; f.dim[2] = g.oh; f.dim[3] = g.ow; f.dim[4] = g.C;
    f.dim[5] = g.kh; f.dim[6] = g.kw; f.dim[7] = padH; f.dim[8] = padW;
    f.dim[9] = 1; f.dim[10] = 1; f.dim[11] = g.dilH; f.dim[12] = g.dilW;
    const int64_t keep = ctx->workspace_bytes;
    ctx->workspace_bytes = keep - wbytes;
    rc = gh_launch_conv2d(ctx, f);
    ctx->workspace_bytes = keep;
    return rc;
  }
  const int64_t total = (int64_t)B * g.C * g.H * g.W;
  int64_t blocks = cdiv(total, 256);
  if (blocks > (int64_t)ctx->cu_count * 32) blocks = (int64_t)ctx->cu_count * 32;
  hipLaunchKernelGGL(k_conv2d_dgrad_gather, dim3((int)blocks), dim3(256), 0, ctx->stream, dy, w, dx, g, B, F);
  return gh_check_hip(ctx, hipGetLastError(), "conv input-gradient launch");
}

int gh_launch_gemv(gh_ctx* ctx, const gh_cmd& c) {
  const int m = (int)c.dim[0], n = (int)c.dim[1], lda = (int)c.dim[2];
  if (gh_dtype_of(c.flags) == GH_F64) {
    const double* A = (const double*)(uintptr_t)c.ptr[0];
    const double* x = (const double*)(uintptr_t)c.ptr[1];
    double* y = (double*)(uintptr_t)c.ptr[2];
    if (c.flags & GH_FLAG_TRANS_A)
      hipLaunchKernelGGL(k_dgemv_t, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, A, x, y, m, n, lda);
    else
      hipLaunchKernelGGL(k_dgemv_n, dim3((m + 3) / 4), dim3(256), 0, ctx->stream, A, x, y, m, n, lda);
    return gh_check_hip(ctx, hipGetLastError(), "dgemv launch");
  }
  const float* A = (const float*)(uintptr_t)c.ptr[0];
  const float* x = (const float*)(uintptr_t)c.ptr[1];
  float* y = (float*)(uintptr_t)c.ptr[2];
  if (c.flags & GH_FLAG_TRANS_A) {
    // (column block, row range) pairs: about half as many workgroups as compute
    // units, each with at least 64 rows to stream
    const bool vec = al16(c.ptr[0]) && al16(c.ptr[2]) && lda % 4 == 0 && n % 4 == 0 && n >= 4;
    const int cols = vec ? 2048 : 512;
    const int cblocks = (n + cols - 1) / cols;
    int chunks = (int)std::min<int64_t>(std::max<int64_t>(1, (int64_t)ctx->cu_count / 2 / cblocks), (m + 63) / 64);
    if (chunks > 1 && (int64_t)chunks * n * 4 > ctx->workspace_bytes) {
      if (gh_ws_short(ctx, (int64_t)chunks * n * 4)) return ctx->err;
      chunks = 1;
    }
    const int rows = ((m + chunks - 1) / chunks + 7) / 8 * 8;
    chunks = (m + rows - 1) / rows;
    float* out = chunks > 1 ? (float*)ctx->workspace : y;
    const dim3 grid(cblocks, chunks);
    if (vec) hipLaunchKernelGGL((k_gemv_t<4, 2, 8>), grid, dim3(256), 0, ctx->stream, A, x, out, m, n, lda, rows);
    else hipLaunchKernelGGL((k_gemv_t<1, 2, 8>), grid, dim3(256), 0, ctx->stream, A, x, out, m, n, lda, rows);
    if (chunks > 1)
      hipLaunchKernelGGL(k_gemv_t_sum, dim3((n + 63) / 64), dim3(256), 0, ctx->stream, out, y, chunks, n);
  } else {
    const int vec = al16(c.ptr[0]) && al16(c.ptr[1]) && lda % 4 == 0;
    hipLaunchKernelGGL(k_gemv_n, dim3((m + 3) / 4), dim3(256), 0, ctx->stream, A, x, y, m, n, lda, vec);
  }
  return gh_check_hip(ctx, hipGetLastError(), "gemv launch");
}

int gh_launch_outer(gh_ctx* ctx, const gh_cmd& c) {
  const int64_t m = c.dim[0], n = c.dim[1];
  int64_t blocks = (m * n + 1023) / 1024;
  if (blocks > (int64_t)ctx->cu_count * 8) blocks = (int64_t)ctx->cu_count * 8;
  if (gh_dtype_of(c.flags) == GH_F64) {
    hipLaunchKernelGGL(k_douter, dim3((int)blocks), dim3(256), 0, ctx->stream,
                       (const double*)(uintptr_t)c.ptr[0], (const double*)(uintptr_t)c.ptr[1],
                       (double*)(uintptr_t)c.ptr[2], m, n);
    return gh_check_hip(ctx, hipGetLastError(), "outer launch");
  }
  hipLaunchKernelGGL(k_outer, dim3((int)blocks), dim3(256), 0, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], m, n);
  return gh_check_hip(ctx, hipGetLastError(), "outer launch");
}

extern "C" int gh_gemm_can_softmax(const gh_cmd* c) {
  if (!c || c->opcode != GH_OP_GEMM || gh_dtype_of(c->flags) != GH_F32) return 0;
  if (c->flags & (GH_FLAG_TRANS_A | GH_FLAG_TRANS_B)) return 0;
  const int64_t batch = c->dim[6] <= 0 ? 1 : c->dim[6];
  if (batch != 1 || getenv("GORGONIA_HIP_GEMM_PLAN")) return 0;
  // the small-output kernel must take the product (one workgroup per 32 rows)
  return c->dim[1] >= 1 && c->dim[1] <= 32 && c->dim[0] >= 1 && c->dim[0] <= 2048 && c->dim[2] >= 32;
}

// The dispatch order of gh_launch_conv2d, asked without launching.  The plans are functions of the
// command; the one figure of the device they use, its compute units, is the MI355X's here.
extern "C" int gh_conv2d_route(const gh_cmd* c) {
  if (!c || c->opcode != GH_OP_CONV2D || gh_dtype_of(c->flags) != GH_F32) return -1;
  if (gh_conv_rows1_takes(*c)) return GH_CONV_ROUTE_ROWS1;
  if (conv_direct_takes(*c)) return GH_CONV_ROUTE_DIRECT;
  if (gh_conv_rows_takes(*c)) return GH_CONV_ROUTE_ROWS;
  if (gh_conv_small_takes(*c)) return GH_CONV_ROUTE_SMALL;
  if (gh_conv_patch_takes(*c)) return GH_CONV_ROUTE_PATCH;
  if (gh_conv_wide_takes(*c)) return GH_CONV_ROUTE_WIDE;
  if (gh_conv_pointwise_takes(*c, 256)) return GH_CONV_ROUTE_POINTWISE;
  Conv3Geom g;
  int BM, BN, per_thread;
  size_t lds;
  if (conv3_plan<8>(*c, false, &g, &BM, &BN, &lds, &per_thread)) return GH_CONV_ROUTE_TILED;
  return GH_CONV_ROUTE_GATHER;
}

// The dispatch order of gh_launch_conv2d_bwd_filter, asked without launching.
extern "C" int gh_conv2d_bwd_filter_route(const gh_cmd* c) {
  if (!c || c->opcode != GH_OP_CONV2D_BWD_FILTER) return -1;
  if (gh_dtype_of(c->flags) == GH_F64) return GH_WGRAD_ROUTE_F64;
  if (wgrad_c1_takes(*c)) return GH_WGRAD_ROUTE_SINGLE_CHANNEL;
  if (conv_direct_shape(*c) && c->dim[4] <= 65535) return GH_WGRAD_ROUTE_DIRECT;
  if (gh_conv_wgrad_small_takes(*c)) return GH_WGRAD_ROUTE_SMALL;
  return GH_WGRAD_ROUTE_GEMM;
}

extern "C" int gh_conv2d_can_keep(const gh_cmd* c) {
  if (!c || c->opcode != GH_OP_CONV2D || gh_dtype_of(c->flags) != GH_F32) return 0;
  if (getenv("GORGONIA_HIP_CONV_NO_KEEP")) return 0;   // tuning switch: the pool stays a kernel of its own
  if (gh_conv_rows1_takes(*c)) return 1;
  return gh_conv_rows_takes(*c) && gh_conv_rows_can_pool(*c) ? 1 : 0;
}

extern "C" int gh_conv2d_can_pre(const gh_cmd* c) {
  if (!c || c->opcode != GH_OP_CONV2D || gh_dtype_of(c->flags) != GH_F32) return 0;
  if (getenv("GORGONIA_HIP_CONV_NO_PRE")) return 0;   // tuning switch: the first layer stays a kernel of its own
  return gh_conv_rows_takes(*c) && gh_conv_rows_can_pre(*c) ? 1 : 0;
}

extern "C" int gh_conv2d_can_pool(const gh_cmd* c) {
  if (!c || c->opcode != GH_OP_CONV2D || gh_dtype_of(c->flags) != GH_F32) return 0;
  if (gh_conv_rows1_takes(*c)) return 1;   // even output extents are part of what it takes
  if (conv_direct_takes(*c)) {
    const int64_t oh = c->dim[2] + 2 * c->dim[7] - 2, ow = c->dim[3] + 2 * c->dim[7] - 2;
    return oh >= 2 && ow >= 2;
  }
  if (getenv("GORGONIA_HIP_CONV_NO_POOL")) return 0;  // tuning switch: keep MaxPool2D a kernel of its own
  // a shape the small-image, the patch or the wide-image kernel takes is pooled there or not at all (the plain and the
  // pooled command must sum in the same order)
  if (gh_conv_small_takes(*c)) return gh_conv_small_can_pool(*c) ? 1 : 0;
  if (gh_conv_patch_takes(*c)) return gh_conv_patch_can_pool(*c) ? 1 : 0;
  if (gh_conv_wide_takes(*c)) return gh_conv_wide_can_pool(*c) ? 1 : 0;
  Conv3Geom g;
  int BM, BN, per_thread;
  size_t lds;
  return conv3_plan<8>(*c, true, &g, &BM, &BN, &lds, &per_thread) ? 1 : 0;
}
