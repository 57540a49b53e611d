// Conv2d with a 1x1 filter, stride 1, no padding, float32, on the 16x16x4 MFMA, for results too
// small to fill the device with 64x64 tiles: y[b][f][p] = sum_c w[f][c] x[b][c][p].
//
// Replaces cuDNN ConvolutionForward (ops/nn/convolution_cuda.go:111-117) for these layers, where
// the tiled kernel has to cut K into slices over several workgroups and add the slabs in a second
// launch.  The GEMM view is that of the other convolution kernels (M = filters, N = output pixels
// of all images, K = C; op_nn.go:418-437 with kh = kw = 1), results go straight into NCHW.
//
//   * One workgroup of eight wavefronts owns a tile of 16 TM filters x 64 pixels and all of K.
//     K is split over the wavefronts in groups of 16 channels, group q to wavefront q mod 8, and
//     nothing is shared between them: a wavefront loads its operands from global memory straight
//     into the MFMA's register layout, every load 128 bits wide, and keeps one to three groups in
//     flight behind the one it multiplies.  No LDS, no barrier inside the K loop.  A lane's four k
//     values of a filter row are one load (step s of a group multiplies channel
//     16 q + 4 (lane / 16) + s, the same permutation on both operands).  On the pixel side column c
//     of the workgroup's four MFMA tiles is one quad of consecutive pixels of one image, so one
//     load of a channel row feeds all four tiles.  An image's last quad is moved back to end with
//     the image; the pixels it then shares with the quad before are computed twice and stored once.
//   * The eight partial tiles are then added through LDS in wavefront order, so a result does not
//     depend on the tile shape; the epilogue (BatchNorm, activation) runs on the sums, and a thread
//     stores a quad: 256 contiguous bytes per filter row and 16 lanes.
//   * What bounds it is the operand traffic out of L2, not the matrix cores: a 48 x 64 tile fetches
//     48 + 64 floats per k for 48 * 64 multiply-adds, and the 200-odd workgroups that a result of
//     this size gives the 256 compute units cannot have larger tiles.  With the loads of the K loop
//     taken out the same MFMAs run in 1.27 us per 128 channels, with them in 2.2 (8 x 1024 x 13 x 13
//     -> 425 filters: 23.3 us against 26.8 for 64x64 tiles over four K slices plus their sum).
//   * Workgroup ids are dealt round-robin over the 8 XCDs; the id is turned into a tile so that an
//     XCD owns a contiguous run of tiles, pixel-tile major: its L2 then holds a few pixel tiles
//     of x and the filters, each fetched from memory once per XCD.
#include <cstdlib>
#include <mutex>

#include "gh_conv_common.h"
#include "gh_internal.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

inline unsigned magic_of(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
__device__ __forceinline__ int mdiv(int n, unsigned magic) {
  const unsigned q = __umulhi((unsigned)n, magic);
  return (int)(q | ((unsigned)n & (0u - (unsigned)(magic == 0))));
}

struct PwGeom {
  int B, C, F, HW;
  int QI;           // quads per image: ceil(HW / 4)
  int NQ;           // B * QI
  int NG;           // groups of 16 channels per wavefront: C / 128
  int tilesM, ntiles, per_xcd;
  unsigned mQI;
};

constexpr int kWaves = 8;
constexpr int kTN = 4;   // pixel tiles per workgroup = floats per quad

// D operand sets per wavefront: one multiplied, the others in flight; NG is a multiple of D
template <int TM, int D>
__global__ __launch_bounds__(kWaves * 64) void k_conv1x1(const float* __restrict__ x, const float* __restrict__ w,
                                                         float* __restrict__ y, PwGeom g, ConvTail tail) {
  constexpr int TN = kTN, NT = TM * TN, BM = 16 * TM;
  extern __shared__ float lds[];
  f32x4* const part = reinterpret_cast<f32x4*>(lds);   // [wave][tile][lane]
  float* const ftab = lds + kWaves * NT * 256;          // [4][BM] BatchNorm constants
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lk = lane >> 4;
  const int lin = ((int)blockIdx.x & 7) * g.per_xcd + ((int)blockIdx.x >> 3);
  if (lin >= g.ntiles) return;
  const int nt = lin / g.tilesM, mt = lin - nt * g.tilesM;
  const int f0 = mt * BM, q0 = nt * 16;
  if (tid < BM) conv_tail_table(tail, ftab, BM, tid, min(f0 + tid, g.F - 1));

  // a lane's filter rows (at its four k of group 0) and its quad of pixels (at its first k)
  const float* wa[TM];
#pragma unroll
  for (int a = 0; a < TM; a++) wa[a] = w + (int64_t)min(f0 + 16 * a + li, g.F - 1) * g.C + 4 * lk;
  unsigned xo;   // byte offset from x
  {
    const int quad = min(q0 + li, g.NQ - 1);
    const int img = mdiv(quad, g.mQI);
    const int pb = min(4 * (quad - img * g.QI), g.HW - 4);
    xo = 4u * (unsigned)((img * g.C + 4 * lk) * g.HW + pb);
  }

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  f32x4 av[D][TM], bv[D][4];
  auto fetch = [&](int d, int i) {   // set d <- this wavefront's i-th group
    const int q = wave + kWaves * i;
#pragma unroll
    for (int a = 0; a < TM; a++) av[d][a] = *reinterpret_cast<const f32x4*>(wa[a] + 16 * q);
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const char* const xs = reinterpret_cast<const char*>(x + (int64_t)(16 * q + s) * g.HW);
      bv[d][s] = *reinterpret_cast<const f32x4_a4*>(xs + xo);
    }
  };
  auto multiply = [&](int d) {
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[d][a][s], bv[d][s][b], acc[a][b], 0, 0, 0);
  };
  // no branch between a set's loads and its MFMAs: the wait before a multiply then counts only
  // the loads issued after its own set's, and those stay in flight.  The scheduling barriers keep
  // the compiler from gathering a whole round's loads behind its last multiply.
#pragma unroll
  for (int d = 0; d < D; d++) {
    fetch(d, d);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int i = D; i < g.NG; i += D) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      multiply(d);
      __builtin_amdgcn_sched_barrier(0);
      fetch(d, i + d);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#pragma unroll
  for (int d = 0; d < D; d++) multiply(d);

  // the eight partial tiles, added in wavefront order by the thread that stores the quad
#pragma unroll
  for (int a = 0; a < TM; a++)
#pragma unroll
    for (int b = 0; b < TN; b++) part[(wave * NT + a * TN + b) * 64 + lane] = acc[a][b];
  __syncthreads();
  const float* const pf = lds;
  conv_tail_dispatch(tail, [&](auto bn_c, auto act_c) {
    constexpr bool BN = decltype(bn_c)::value;
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int j0 = 0; j0 < BM * 16; j0 += kWaves * 64) {
      const int j = j0 + tid;                 // (filter row fi, column ci): j = (fi / 4 * 16 + ci) * 4 + fi % 4
      if (BM * 16 % (kWaves * 64) != 0 && j >= BM * 16) break;
      const int r = j & 3, ci = (j >> 2) & 15, f4 = j >> 6;   // f4 = fi / 4: tile row a = f4 / 4, lane group f4 % 4
      const int fi = 4 * f4 + r;
      const int cell = ((f4 >> 2) * TN * 64 + (f4 & 3) * 16 + ci) * 4 + r;   // value r of lane (f4 % 4, ci) of tile (a, 0)
      float v[TN];
#pragma unroll
      for (int b = 0; b < TN; b++) {
        v[b] = pf[cell + b * 256];
#pragma unroll
        for (int wv = 1; wv < kWaves; wv++) v[b] = v[b] + pf[wv * NT * 256 + cell + b * 256];
        v[b] = tail_apply_fixed<BN, ACT>(ftab, BM, fi, v[b], tail.alpha);
      }
      const int quad = q0 + ci;
      if (f0 + fi < g.F && quad < g.NQ) {
        const int img = mdiv(quad, g.mQI);
        const int p4 = 4 * (quad - img * g.QI), pb = min(p4, g.HW - 4);
        float* const out = y + ((int64_t)img * g.F + f0 + fi) * g.HW + pb;
        if (p4 == pb) {
          *reinterpret_cast<f32x4_a4*>(out) = f32x4_a4{v[0], v[1], v[2], v[3]};
        } else {   // an image's last quad, moved back to end with the image: its first pixels are the quad before's
#pragma unroll
          for (int b = 0; b < TN; b++)
            if (pb + b >= p4) out[b] = v[b];
        }
      }
    }
  });
}

struct PwPlan { PwGeom g; int TM, D; size_t lds; };

// force_tm: 0, or the filter-tile height to use whatever the estimate says
bool pointwise_plan(const gh_cmd& c, int cus, PwPlan* out, int force_tm = 0) {
  if (gh_dtype_of(c.flags) != GH_F32 || (c.flags & GH_FLAG_CONV_POOL2)) return false;
  const int64_t B = c.dim[0], C = c.dim[1], H = c.dim[2], W = c.dim[3], F = c.dim[4];
  if (c.dim[5] != 1 || c.dim[6] != 1 || c.dim[7] != 0 || c.dim[8] != 0 || c.dim[9] != 1 || c.dim[10] != 1) return false;
  if (C % (16 * kWaves * 2) != 0) return false;                 // two or four groups of 16 channels per wavefront at a time
  if ((c.ptr[1] & 15) != 0) return false;                       // 128-bit loads of filter rows
  const int64_t HW = H * W, P = B * HW;
  if (HW < 4) return false;                                     // a quad of pixels per lane
  if (getenv("GORGONIA_HIP_CONV_NO_POINTWISE")) return false;   // tuning switch: the tiled kernel only
  if (B * C * HW * 4 >= (1ll << 32) || P * F >= (1ll << 31) || P >= (1 << 24)) return false;
  // only where 64x64 tiles would leave compute units idle, or nearly, without cutting K across workgroups
  // measured against the tiled kernel (batch 8): ahead up to about 2 cus of its tiles, by up to 2x below
  // one per compute unit; with 256 channels (few k-tiles for the tiled kernel to overlap its loads with)
  // up to about 8 cus (256 -> 256 at 52 x 52: 40.6 us against 52.8), level at 2700 tiles
  int64_t max_tiles = (C <= 256 ? 8 : 2) * (int64_t)cus;
  if (const char* e = getenv("GORGONIA_HIP_CONV_POINTWISE_TILES")) max_tiles = atoll(e);   // tuning override
  if (((F + 63) / 64) * ((P + 63) / 64) >= max_tiles) return false;
  PwGeom g{};
  g.B = (int)B; g.C = (int)C; g.F = (int)F; g.HW = (int)HW;
  g.QI = (int)((HW + 3) / 4); g.NQ = g.B * g.QI;
  g.NG = (int)(C / (16 * kWaves));
  g.mQI = magic_of((unsigned)g.QI);
  const int tilesN = (g.NQ + 15) / 16;
  // filter tile: the height whose rounds over the device, times its MFMAs per k step, are fewest
  int bestTM = 0; double best = 0;
  for (int TM : {3, 2, 1}) {
    const int64_t tiles = (int64_t)((F + 16 * TM - 1) / (16 * TM)) * tilesN;
    const double est = (double)((tiles + cus - 1) / cus) * (TM * kTN + 1.0);
    if (!bestTM || est < best) { best = est; bestTM = TM; }
  }
  if (force_tm) bestTM = force_tm;
  if (const char* e = getenv("GORGONIA_HIP_CONV_POINTWISE_TM")) { const int t = atoi(e); if (t >= 1 && t <= 3) bestTM = t; }   // tuning override
  g.tilesM = (int)((F + 16 * bestTM - 1) / (16 * bestTM));
  g.ntiles = g.tilesM * tilesN;
  g.per_xcd = (g.ntiles + 7) / 8;
  out->g = g; out->TM = bestTM; out->D = g.NG % 4 == 0 ? 4 : 2;
  out->lds = (size_t)(kWaves * bestTM * kTN * 256 + 4 * 16 * bestTM) * sizeof(float);
  return true;
}

template <int TM, int D>
int launch_pointwise(gh_ctx* ctx, const gh_cmd& c, const PwPlan& p) {
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [] {
    attr_rc = hipFuncSetAttribute((const void*)k_conv1x1<TM, D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024);
  });
  if (attr_rc != hipSuccess) return gh_check_hip(ctx, attr_rc, "hipFuncSetAttribute(conv1x1)");
  hipLaunchKernelGGL((k_conv1x1<TM, D>), dim3((unsigned)(8 * p.g.per_xcd)), dim3(kWaves * 64), p.lds, ctx->stream,
                     (const float*)(uintptr_t)c.ptr[0], (const float*)(uintptr_t)c.ptr[1],
                     (float*)(uintptr_t)c.ptr[2], p.g, conv_tail(c));
  return gh_check_hip(ctx, hipGetLastError(), "conv1x1 launch");
}

}  // namespace

bool gh_conv_pointwise_takes(const gh_cmd& c, int cus) {
  PwPlan p;
  return pointwise_plan(c, cus, &p);
}

// Returns -1 when the shape is not one this kernel takes.
int gh_try_launch_conv_pointwise(gh_ctx* ctx, const gh_cmd& c) {
  PwPlan p;
  if (!pointwise_plan(c, ctx->cu_count, &p)) return -1;
  // A result written straight into pinned host memory travels over the bus: the lowest tiles then, whose
  // workgroups store 4 KB each and finish at different moments, so that the bus is busy before the last
  // of them has multiplied (8 x 1024 x 13 x 13 -> 425 filters into host memory: 61.8 us against 68.9 with
  // 48-filter tiles, which are ahead by 1.6 us on device memory).  The sums are those of any tile shape.
  if (p.TM > 1)
    for (const auto& r : ctx->host_ranges)
      if (c.ptr[2] >= r.first && c.ptr[2] < r.second) { pointwise_plan(c, ctx->cu_count, &p, 1); break; }
#define GH_PW(TM_) return p.D == 4 ? launch_pointwise<TM_, 4>(ctx, c, p) : launch_pointwise<TM_, 2>(ctx, c, p)
  switch (p.TM) {
    case 3: GH_PW(3);
    case 2: GH_PW(2);
    default: GH_PW(1);
  }
#undef GH_PW
}
