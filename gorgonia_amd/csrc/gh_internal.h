// Internal declarations shared by the translation units of libgorgonia_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "gorgonia_hip.h"

struct gh_graph_slot {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  bool used = false;
};

// A model of what the 256 MB last-level cache still holds, for the streaming kernels'
// choice between plain and non-temporal accesses: the buffers commands touched lately and
// how many bytes of streaming traffic have gone by since.  Operands the cache still holds are
// quicker through plain accesses (non-temporal ones lose 5-10 % there), operands it has lost
// are quicker streamed (6-13 % on a binary kernel).  The model only steers that choice; both
// forms store the same bits.
struct gh_llc_model {
  struct Entry { uint64_t lo, hi, stamp; };
  static constexpr int kEntries = 48;
  Entry e[kEntries] = {};
  int next = 0;
  uint64_t clock = 0;   // bytes the streaming kernels have moved so far
  // a buffer starting at p was touched within the last `window` bytes of traffic
  bool warm(uint64_t p, uint64_t window) const {
    for (const Entry& x : e)
      if (x.hi > x.lo && p >= x.lo && p < x.hi && clock - x.stamp <= window) return true;
    return false;
  }
  void touch(uint64_t p, uint64_t bytes, bool counts) {
    if (!p) return;
    if (counts) clock += bytes;
    const uint64_t hi = p + (bytes ? bytes : 1);   // size unknown: the start address alone
    for (Entry& x : e)
      if (x.hi > x.lo && p < x.hi && x.lo < hi) { x = Entry{p, hi, clock}; return; }
    e[next] = Entry{p, hi, clock};
    next = (next + 1) % kEntries;
  }
};

struct gh_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  void* arena = nullptr;
  int64_t arena_bytes = 0;
  int err = GH_OK;          // sticky status
  std::string errmsg;
  bool capturing = false;
  std::vector<gh_graph_slot> graphs;
  hipEvent_t events[64] = {};
  int cu_count = 256;
  // scratch owned by the context (split-K partials, reduction flags)
  void* workspace = nullptr;
  int64_t workspace_bytes = 0;
  // set while gh_submit_noalloc runs: the scratch is the library's fixed array and a
  // plan may not shrink to fit it (results must not depend on the scratch size)
  bool ws_strict = false;
  bool sync_spin = false;  // gh_sync polls the stream instead of blocking in the runtime
  gh_llc_model llc;
  // pinned host buffers handed out by gh_host_alloc: [start, end)
  std::vector<std::pair<uint64_t, uint64_t>> host_ranges;
};

// A launcher calls this where `need` bytes of scratch do not fit the workspace,
// before it shrinks its plan (fewer split-K slices, a kernel without scratch).
// Returns GH_OK to go on shrinking; under gh_submit_noalloc it records the
// sticky error instead and returns its code, which the launcher passes on.
int gh_ws_short(gh_ctx* ctx, int64_t need);

// Record a sticky error on the context and return its code.
int gh_fail(gh_ctx* ctx, int code, const std::string& msg);
int gh_check_hip(gh_ctx* ctx, hipError_t e, const char* what);

// Per-family validators (host only) and launchers.  Launchers assume a
// validated command.  Each returns GH_OK or a code with `msg` filled in.
int gh_validate_cmd(const gh_cmd& c, std::string& msg);

int gh_launch_elem_bin(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_elem_unary(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bcast_bin(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_relu(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_relu_bwd(gh_ctx* ctx, const gh_cmd& c);
// float64 twins of the backward operators (k_bwd64.hip)
int gh_launch_relu_bwd_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_dropout_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_dropout_bwd_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_softmax_bwd_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_maxpool2d_bwd_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_solver_step_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bn_train_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bn_bwd_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_conv2d_bwd_data_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_conv2d_bwd_filter_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_leaky_relu(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_fill(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_has_nan_inf(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_gemm(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_gemv(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_outer(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_conv2d(gh_ctx* ctx, const gh_cmd& c);
// small-image 3x3 convolution (k_conv_small.hip): -1 when the shape is not one it takes
int gh_try_launch_conv_small(gh_ctx* ctx, const gh_cmd& c);
int gh_try_launch_conv_wgrad_small(gh_ctx* ctx, const gh_cmd& c, int* splits);
bool gh_conv_wgrad_small_takes(const gh_cmd& c);
bool gh_conv_small_takes(const gh_cmd& c);
bool gh_conv_small_can_pool(const gh_cmd& c);
// its 32- and 64-channel kernel (k_conv_rows.hip), same conventions
int gh_try_launch_conv_rows(gh_ctx* ctx, const gh_cmd& c);
bool gh_conv_rows_takes(const gh_cmd& c);
bool gh_conv_rows_can_pool(const gh_cmd& c);
bool gh_conv_rows_can_pre(const gh_cmd& c);
// single-channel 3x3 convolution on the matrix cores (k_conv_rows1.hip), same conventions
int gh_try_launch_conv_rows1(gh_ctx* ctx, const gh_cmd& c);
bool gh_conv_rows1_takes(const gh_cmd& c);
// 3x3 convolution over patches with K split across wavefronts (k_conv_patch.hip), same conventions
int gh_try_launch_conv_patch(gh_ctx* ctx, const gh_cmd& c);
bool gh_conv_patch_takes(const gh_cmd& c);
bool gh_conv_patch_can_pool(const gh_cmd& c);
// k_conv_wide.hip: 3x3 stride-1 convolution over large images with up to 64 channels
int gh_try_launch_conv_wide(gh_ctx* ctx, const gh_cmd& c);
bool gh_conv_wide_takes(const gh_cmd& c);
bool gh_conv_wide_can_pool(const gh_cmd& c);
// k_conv_pointwise.hip: 1x1 stride-1 convolution whose result is too small for K-wide 64x64 tiles to fill the device
int gh_try_launch_conv_pointwise(gh_ctx* ctx, const gh_cmd& c);
bool gh_conv_pointwise_takes(const gh_cmd& c, int cus);
int gh_launch_maxpool2d(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bn_infer(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_softmax(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_maxpool2d_bwd(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_conv2d_bwd_data(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_conv2d_bwd_filter(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bn_train(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bn_bwd(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_softmax_bwd(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_solver_step(gh_ctx* ctx, const gh_cmd& c);
int gh_solver_run_length(const gh_cmd* cmds, int n);
int gh_launch_solver_steps(gh_ctx* ctx, const gh_cmd* cmds, int count);
int gh_launch_rand_uniform(gh_ctx* ctx, const gh_cmd& c);
// float64 twins of the forward neural-network operators (k_nn64.hip)
int gh_launch_relu_f64(gh_ctx* ctx, const gh_cmd& c, bool leaky);
int gh_launch_maxpool2d_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_bn_infer_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_softmax_f64(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_conv2d_f64(gh_ctx* ctx, const gh_cmd& c);
bool gh_try_launch_conv2d_f64_mfma(gh_ctx* ctx, const gh_cmd& c);
bool gh_try_launch_conv2d_bwd_data_f64_mfma(gh_ctx* ctx, const gh_cmd& c);
bool gh_try_launch_conv2d_bwd_filter_f64_mfma(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_dropout(gh_ctx* ctx, const gh_cmd& c);
int gh_launch_dropout_bwd(gh_ctx* ctx, const gh_cmd& c);

// A convolution kernel's plan (geometry and workgroup shape) is a function of the command's shape,
// its dtype and of whether a pooling rides in the epilogue - and of tuning switches in the environment,
// which are read when a shape is first seen.  Finding one costs tens of microseconds on the host and a
// command asks several times (validation, the pooling query, the launcher), which an eager submit
// cannot hide behind kernels of a few microseconds: gh_plan_memo keeps the answers.  One table per call
// site (the lambda's type makes the instantiation unique); bounded, cleared when full.
template <class Plan, class Fn>
bool gh_plan_memo(const gh_cmd& c, bool pool, Plan* out, Fn&& compute) {
  struct Entry { int64_t dim[13]; uint32_t dtype; bool pool, ok; Plan plan; };
  static std::mutex mu;
  static std::vector<Entry> table;
  const uint32_t dtype = (c.flags >> 12) & 0xfu;
  {
    std::lock_guard<std::mutex> lock(mu);
    for (const Entry& e : table)
      if (e.pool == pool && e.dtype == dtype && memcmp(e.dim, c.dim, sizeof(e.dim)) == 0) {
        if (e.ok) *out = e.plan;
        return e.ok;
      }
  }
  Entry e;
  memcpy(e.dim, c.dim, sizeof(e.dim));
  e.dtype = dtype; e.pool = pool;
  e.ok = compute(&e.plan);
  std::lock_guard<std::mutex> lock(mu);
  if (table.size() >= 256) table.clear();
  table.push_back(e);
  if (e.ok) *out = e.plan;
  return e.ok;
}

static inline uint32_t gh_fn(uint32_t flags) { return flags & 0xffu; }
static inline uint32_t gh_mode(uint32_t flags) { return (flags >> 8) & 0xfu; }
static inline uint32_t gh_dtype_of(uint32_t flags) { return (flags >> 12) & 0xfu; }

// Output sizes shared by validators, launchers and the host mirror.
static inline int64_t gh_conv_out(int64_t in, int64_t k, int64_t pad, int64_t stride, int64_t dil) {
  return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;  // op_nn.go:311-315
}
static inline int64_t gh_pool_out(int64_t in, int64_t k, int64_t padA, int64_t padB, int64_t stride) {
  return (in + padA + padB - (k - 1) - 1) / stride + 1;      // op_nn.go:810-816
}
