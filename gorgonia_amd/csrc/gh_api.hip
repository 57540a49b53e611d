// Context, memory, submission and graph entry points of libgorgonia_hip.so.
// Replaces what Gorgonia's cuda.Engine gets from gorgonia.org/cu's
// BatchedContext: context creation (cuda/external.go:112-170), queued copies,
// kernel launch (cuda/arith.go:62) and DoWork/Signal (cuda/external.go:223).
#include <cstdio>
#include <cstring>

#include <mutex>

#include "gh_internal.h"

int gh_fail(gh_ctx* ctx, int code, const std::string& msg) {
  if (ctx && ctx->err == GH_OK) {
    ctx->err = code;
    ctx->errmsg = msg;
  }
  return code;
}

// Scratch of gh_submit_noalloc: part of the library's device image, so it exists
// on every GPU the library runs on from load time to process exit and no call
// has to allocate it.  In host code this name only stands for the symbol; the
// per-device address comes from hipGetSymbolAddress (static_scratch below) and
// is the only thing ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[GH_NOALLOC_SCRATCH_BYTES];

static constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices] = {};   // address of `scratch` on device i; filled by gh_init

// Address of the static scratch on `device`, which must be current.  Resolved
// once per device (every GPU holds its own copy at its own address).
static hipError_t static_scratch(int device, void** out) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  static std::mutex mu;   // contexts may be opened from several host threads at once
  std::lock_guard<std::mutex> lock(mu);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = p;
  }
  *out = g_scratch_ptr[device];
  return hipSuccess;
}

int gh_ws_short(gh_ctx* ctx, int64_t need) {
  if (!ctx->ws_strict) return GH_OK;
  return gh_fail(ctx, GH_EINVAL,
                 "gh_submit_noalloc: operator needs " + std::to_string(need) + " bytes of scratch, the fixed scratch holds " +
                     std::to_string((int64_t)GH_NOALLOC_SCRATCH_BYTES) + " (use gh_submit)");
}

int gh_check_hip(gh_ctx* ctx, hipError_t e, const char* what) {
  if (e == hipSuccess) return GH_OK;
  std::string m = std::string(what) + ": " + hipGetErrorString(e);
  return gh_fail(ctx, GH_EDEVICE, m);
}

extern "C" {

const char* gh_version(void) { return "gorgonia_hip 0.1 (gfx950)"; }

int gh_device_count(int* out) {
  if (!out) return GH_EINVAL;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) { *out = 0; return GH_EDEVICE; }
  *out = n;
  return GH_OK;
}

int gh_init(int device, int64_t arena_bytes, gh_ctx** out) {
  if (!out || arena_bytes < 0) return GH_EINVAL;
  *out = nullptr;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) return GH_EDEVICE;
  if (hipSetDevice(device) != hipSuccess) return GH_EDEVICE;
  gh_ctx* ctx = new gh_ctx();
  ctx->device = device;
  // Default priority only: mixed stream priorities are not used anywhere.
  if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
    delete ctx;
    return GH_EDEVICE;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->cu_count = prop.multiProcessorCount;
  if (const char* sm = getenv("GORGONIA_HIP_SYNC")) ctx->sync_spin = strcmp(sm, "spin") == 0;
  if (arena_bytes > 0) {
    size_t free_b = 0, total_b = 0;
    hipMemGetInfo(&free_b, &total_b);
    if ((size_t)arena_bytes >= free_b) {  // cuda/external.go:159-161
      hipStreamDestroy(ctx->stream);
      delete ctx;
      return GH_EOOM;
    }
    if (hipMalloc(&ctx->arena, (size_t)arena_bytes) != hipSuccess) {
      (void)hipGetLastError();
      hipStreamDestroy(ctx->stream);
      delete ctx;
      return GH_EOOM;
    }
    ctx->arena_bytes = arena_bytes;
  }
  // Context-owned scratch: split-K partial sums, reduction partials, mirrored
  // filters.  Mandatory: the launchers index it without asking again.
  ctx->workspace_bytes = 64ll << 20;
  void* fixed = nullptr;
  if (hipMalloc(&ctx->workspace, (size_t)ctx->workspace_bytes) != hipSuccess ||
      static_scratch(device, &fixed) != hipSuccess) {
    (void)hipGetLastError();
    if (ctx->workspace) hipFree(ctx->workspace);
    if (ctx->arena) hipFree(ctx->arena);
    hipStreamDestroy(ctx->stream);
    delete ctx;
    return GH_EOOM;
  }
  *out = ctx;
  return GH_OK;
}

int gh_close(gh_ctx* ctx) {
  if (!ctx) return GH_EINVAL;
  hipSetDevice(ctx->device);
  hipStreamSynchronize(ctx->stream);
  for (auto& g : ctx->graphs) {
    if (g.exec) hipGraphExecDestroy(g.exec);
    if (g.graph) hipGraphDestroy(g.graph);
  }
  for (auto& e : ctx->events)
    if (e) hipEventDestroy(e);
  if (ctx->workspace) hipFree(ctx->workspace);
  if (ctx->arena) hipFree(ctx->arena);
  hipStreamDestroy(ctx->stream);
  delete ctx;
  return GH_OK;
}

int gh_device_info(gh_ctx* ctx, gh_devinfo* out) {
  if (!ctx || !out) return GH_EINVAL;
  hipDeviceProp_t p;
  int rc = gh_check_hip(ctx, hipGetDeviceProperties(&p, ctx->device), "hipGetDeviceProperties");
  if (rc) return rc;
  memset(out, 0, sizeof(*out));
  out->wavefront_size = p.warpSize;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  out->max_grid_x = p.maxGridSize[0];
  out->max_grid_y = p.maxGridSize[1];
  out->max_grid_z = p.maxGridSize[2];
  out->max_block_x = p.maxThreadsDim[0];
  out->max_block_y = p.maxThreadsDim[1];
  out->max_block_z = p.maxThreadsDim[2];
  out->compute_units = p.multiProcessorCount;
  out->lds_bytes_per_block = (int32_t)p.sharedMemPerBlock;
  size_t f = 0, t = 0;
  hipMemGetInfo(&f, &t);
  out->free_mem = (int64_t)f;
  out->total_mem = (int64_t)t;
  snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
  return GH_OK;
}

gh_devptr gh_arena_base(gh_ctx* ctx) { return ctx ? (gh_devptr)(uintptr_t)ctx->arena : 0; }
int64_t gh_arena_size(gh_ctx* ctx) { return ctx ? ctx->arena_bytes : 0; }

int gh_malloc(gh_ctx* ctx, int64_t bytes, gh_devptr* out) {
  if (!ctx || !out || bytes <= 0) return GH_EINVAL;
  void* p = nullptr;
  if (hipMalloc(&p, (size_t)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return GH_EOOM;
  }
  *out = (gh_devptr)(uintptr_t)p;
  return GH_OK;
}

int gh_free(gh_ctx* ctx, gh_devptr p) {
  if (!ctx) return GH_EINVAL;
  if (!p) return GH_OK;
  return gh_check_hip(ctx, hipFree((void*)(uintptr_t)p), "hipFree");
}

int gh_host_alloc(gh_ctx* ctx, int64_t bytes, void** out) {
  if (!ctx || !out || bytes <= 0) return GH_EINVAL;
  if (hipHostMalloc(out, (size_t)bytes, hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return GH_EOOM;
  }
  ctx->host_ranges.emplace_back((uint64_t)(uintptr_t)*out, (uint64_t)(uintptr_t)*out + (uint64_t)bytes);
  return GH_OK;
}

int gh_host_free(gh_ctx* ctx, void* p) {
  if (!ctx) return GH_EINVAL;
  if (!p) return GH_OK;
  for (size_t i = 0; i < ctx->host_ranges.size(); i++)
    if (ctx->host_ranges[i].first == (uint64_t)(uintptr_t)p) {
      ctx->host_ranges.erase(ctx->host_ranges.begin() + (long)i);
      break;
    }
  return gh_check_hip(ctx, hipHostFree(p), "hipHostFree");
}

int gh_memcpy_h2d(gh_ctx* ctx, gh_devptr dst, const void* src, int64_t bytes) {
  if (!ctx || bytes < 0 || (bytes > 0 && (!dst || !src))) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  if (bytes == 0) return GH_OK;
  return gh_check_hip(ctx,
                      hipMemcpyAsync((void*)(uintptr_t)dst, src, (size_t)bytes,
                                     hipMemcpyHostToDevice, ctx->stream),
                      "hipMemcpyAsync(H2D)");
}

int gh_memcpy_d2h(gh_ctx* ctx, void* dst, gh_devptr src, int64_t bytes) {
  if (!ctx || bytes < 0 || (bytes > 0 && (!dst || !src))) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  if (bytes == 0) return GH_OK;
  return gh_check_hip(ctx,
                      hipMemcpyAsync(dst, (const void*)(uintptr_t)src, (size_t)bytes,
                                     hipMemcpyDeviceToHost, ctx->stream),
                      "hipMemcpyAsync(D2H)");
}

// Copies done by a kernel: a kernel node costs less inside a captured graph than
// a copy-engine node, and either side may be pinned host memory (results staged
// out to the host, inputs staged in from it over PCIe).
__global__ __launch_bounds__(256) void k_copy_words(uint32_t* __restrict__ dst,
                                                    const uint32_t* __restrict__ src, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}
// 16 bytes per lane, two in flight; the tail (< 16 bytes, a multiple of 4) goes word by word.
__global__ __launch_bounds__(256) void k_copy_vec(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                  int64_t n16, int64_t tail_words) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + stride < n16; i += 2 * stride) {
    const uint4 a = src[i], b = src[i + stride];
    dst[i] = a;
    dst[i + stride] = b;
  }
  if (i < n16) dst[i] = src[i];
  if (blockIdx.x == 0 && (int64_t)threadIdx.x < tail_words)
    ((uint32_t*)(dst + n16))[threadIdx.x] = ((const uint32_t*)(src + n16))[threadIdx.x];
}

static constexpr int64_t kKernelCopyLimit = 16 << 20;
// From pinned host memory the copy engine asks the bus for larger pieces than a kernel's 64-byte
// loads do: 16.6 MB in 299 us against 334 (55.6 / 49.8 GB/s); the kernel is ahead below about
// 2.5 MB (0.4 MB: 10.7 us against 16.6), where the engine's 9 us of start-up count.
static constexpr int64_t kHostDmaFrom = 4 << 20;

static bool in_pinned_host(const gh_ctx* ctx, uint64_t p) {
  for (const auto& r : ctx->host_ranges)
    if (p >= r.first && p < r.second) return true;
  return false;
}

int gh_memcpy_d2d(gh_ctx* ctx, gh_devptr dst, gh_devptr src, int64_t bytes) {
  if (!ctx || bytes < 0 || (bytes > 0 && (!dst || !src))) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  if (bytes == 0) return GH_OK;
  const bool dma_from_host = bytes >= kHostDmaFrom && in_pinned_host(ctx, src);
  if (!dma_from_host && bytes <= kKernelCopyLimit && ((dst | src | (uint64_t)bytes) & 3) == 0) {
    if (((dst | src) & 15) == 0 && bytes >= 4096) {
      const int64_t n16 = bytes / 16;
      int64_t blocks = (n16 + 511) / 512;
      if (blocks > 1024) blocks = 1024;
      hipLaunchKernelGGL(k_copy_vec, dim3((int)blocks), dim3(256), 0, ctx->stream, (uint4*)(uintptr_t)dst,
                         (const uint4*)(uintptr_t)src, n16, (bytes % 16) / 4);
    } else {
      const int64_t n = bytes / 4;
      int64_t blocks = (n + 255) / 256;
      if (blocks > 1024) blocks = 1024;
      hipLaunchKernelGGL(k_copy_words, dim3((int)blocks), dim3(256), 0, ctx->stream,
                         (uint32_t*)(uintptr_t)dst, (const uint32_t*)(uintptr_t)src, n);
    }
    return gh_check_hip(ctx, hipGetLastError(), "copy launch");
  }
  return gh_check_hip(ctx,
                      hipMemcpyAsync((void*)(uintptr_t)dst, (const void*)(uintptr_t)src,
                                     (size_t)bytes, hipMemcpyDefault, ctx->stream),
                      "hipMemcpyAsync(D2D)");
}

static int dispatch(gh_ctx* ctx, const gh_cmd& c) {
  // the streaming kernels keep their own account of what they touch; everything else marks its
  // operands as recently used (sizes unknown here: by start address), so that an elementwise
  // kernel behind a product or a convolution reads the result as the cache-resident data it is
  if (c.opcode != GH_OP_ELEM_BIN && c.opcode != GH_OP_ELEM_UNARY && c.opcode != GH_OP_BCAST_BIN && c.opcode != GH_OP_NOP)
    for (uint64_t p : c.ptr) ctx->llc.touch(p, 0, false);
  switch (c.opcode) {
    case GH_OP_NOP: return GH_OK;
    case GH_OP_ELEM_BIN: return gh_launch_elem_bin(ctx, c);
    case GH_OP_ELEM_UNARY: return gh_launch_elem_unary(ctx, c);
    case GH_OP_BCAST_BIN: return gh_launch_bcast_bin(ctx, c);
    case GH_OP_MEMCPY_D2D: return gh_memcpy_d2d(ctx, c.ptr[0], c.ptr[1], c.dim[0]);
    case GH_OP_GEMM: return gh_launch_gemm(ctx, c);
    case GH_OP_GEMV: return gh_launch_gemv(ctx, c);
    case GH_OP_OUTER: return gh_launch_outer(ctx, c);
    case GH_OP_CONV2D: return gh_launch_conv2d(ctx, c);
    case GH_OP_MAXPOOL2D: return gh_launch_maxpool2d(ctx, c);
    case GH_OP_BN_INFER: return gh_launch_bn_infer(ctx, c);
    case GH_OP_RELU: return gh_launch_relu(ctx, c);
    case GH_OP_LEAKY_RELU: return gh_launch_leaky_relu(ctx, c);
    case GH_OP_SOFTMAX: return gh_launch_softmax(ctx, c);
    case GH_OP_HAS_NAN:
    case GH_OP_HAS_INF: return gh_launch_has_nan_inf(ctx, c);
    case GH_OP_FILL: return gh_launch_fill(ctx, c);
    case GH_OP_MAXPOOL2D_BWD: return gh_launch_maxpool2d_bwd(ctx, c);
    case GH_OP_CONV2D_BWD_DATA: return gh_launch_conv2d_bwd_data(ctx, c);
    case GH_OP_CONV2D_BWD_FILTER: return gh_launch_conv2d_bwd_filter(ctx, c);
    case GH_OP_BN_TRAIN: return gh_launch_bn_train(ctx, c);
    case GH_OP_BN_BWD: return gh_launch_bn_bwd(ctx, c);
    case GH_OP_SOFTMAX_BWD: return gh_launch_softmax_bwd(ctx, c);
    case GH_OP_SOLVER_STEP: return gh_launch_solver_step(ctx, c);
    case GH_OP_RAND_UNIFORM: return gh_launch_rand_uniform(ctx, c);
    case GH_OP_DROPOUT: return gh_launch_dropout(ctx, c);
    case GH_OP_DROPOUT_BWD: return gh_launch_dropout_bwd(ctx, c);
    case GH_OP_RELU_BWD: return gh_launch_relu_bwd(ctx, c);
  }
  return GH_ENOFUNC;
}

int gh_validate(const gh_cmd* cmds, int n, char* msg, int msg_len) {
  if (n < 0 || (n > 0 && !cmds)) return GH_EINVAL;
  for (int i = 0; i < n; i++) {
    std::string m;
    int rc = gh_validate_cmd(cmds[i], m);
    if (rc) {
      if (msg && msg_len > 0) snprintf(msg, (size_t)msg_len, "cmd %d: %s", i, m.c_str());
      return rc;
    }
  }
  if (msg && msg_len > 0) msg[0] = 0;
  return GH_OK;
}

static int submit_cmds(gh_ctx* ctx, const gh_cmd* cmds, int n) {
  for (int i = 0; i < n; i++) {
    std::string m;
    int rc = gh_validate_cmd(cmds[i], m);
    if (rc) return gh_fail(ctx, rc, "cmd " + std::to_string(i) + ": " + m);
    // a run of solver steps with the same settings (a model's weight tensors) is one launch
    const int run = gh_solver_run_length(cmds + i, n - i);
    if (run > 1) {
      for (int j = 1; j < run; j++) {
        rc = gh_validate_cmd(cmds[i + j], m);
        if (rc) return gh_fail(ctx, rc, "cmd " + std::to_string(i + j) + ": " + m);
      }
      rc = gh_launch_solver_steps(ctx, cmds + i, run);
      if (rc) return rc;
      i += run - 1;
      continue;
    }
    rc = dispatch(ctx, cmds[i]);
    if (rc) return rc;
  }
  return GH_OK;
}

int gh_submit(gh_ctx* ctx, const gh_cmd* cmds, int n) {
  if (!ctx || n < 0 || (n > 0 && !cmds)) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  return submit_cmds(ctx, cmds, n);
}

int gh_submit_noalloc(gh_ctx* ctx, const gh_cmd* cmds, int n) {
  if (!ctx || n < 0 || (n > 0 && !cmds)) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  void* fixed = ctx->device >= 0 && ctx->device < kMaxDevices ? g_scratch_ptr[ctx->device] : nullptr;
  if (!fixed) return gh_fail(ctx, GH_ESTATE, "gh_submit_noalloc: the fixed scratch was not resolved on this device");
  // Same launchers, same plans: only the scratch they index changes, and a plan
  // that would not fit it is refused instead of shrunk (gh_ws_short).  Nothing
  // in the scratch has to start at zero: every slab and partial is written
  // before it is read.
  void* const keep = ctx->workspace;
  const int64_t keep_bytes = ctx->workspace_bytes;
  ctx->workspace = fixed;
  ctx->workspace_bytes = GH_NOALLOC_SCRATCH_BYTES;
  ctx->ws_strict = true;
  const int rc = submit_cmds(ctx, cmds, n);
  ctx->ws_strict = false;
  ctx->workspace = keep;
  ctx->workspace_bytes = keep_bytes;
  return rc;
}

int gh_sync(gh_ctx* ctx) {
  if (!ctx) return GH_EINVAL;
  if (ctx->capturing) return gh_fail(ctx, GH_ESTATE, "gh_sync during graph capture");
  hipError_t e;
  if (ctx->sync_spin) {
    // poll the stream from this thread instead of blocking in the runtime's wait
    while ((e = hipStreamQuery(ctx->stream)) == hipErrorNotReady) {
    }
  } else {
    e = hipStreamSynchronize(ctx->stream);
  }
  if (e != hipSuccess) gh_check_hip(ctx, e, "hipStreamSynchronize");
  return ctx->err;
}

int gh_graph_begin(gh_ctx* ctx) {
  if (!ctx) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  if (ctx->capturing) return gh_fail(ctx, GH_ESTATE, "graph capture already active");
  int rc = gh_check_hip(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal),
                        "hipStreamBeginCapture");
  if (rc) return rc;
  ctx->capturing = true;
  return GH_OK;
}

int gh_graph_end(gh_ctx* ctx, int* graph_id) {
  if (!ctx || !graph_id) return GH_EINVAL;
  if (!ctx->capturing) return gh_fail(ctx, GH_ESTATE, "no graph capture active");
  ctx->capturing = false;
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g);
  if (e != hipSuccess) return gh_check_hip(ctx, e, "hipStreamEndCapture");
  if (ctx->err) {  // a submit failed while capturing: drop the graph
    if (g) hipGraphDestroy(g);
    return ctx->err;
  }
  hipGraphExec_t ex = nullptr;
  e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    hipGraphDestroy(g);
    return gh_check_hip(ctx, e, "hipGraphInstantiate");
  }
  int id = -1;
  for (size_t i = 0; i < ctx->graphs.size(); i++)
    if (!ctx->graphs[i].used) { id = (int)i; break; }
  if (id < 0) {
    ctx->graphs.emplace_back();
    id = (int)ctx->graphs.size() - 1;
  }
  ctx->graphs[id].graph = g;
  ctx->graphs[id].exec = ex;
  ctx->graphs[id].used = true;
  *graph_id = id;
  return GH_OK;
}

int gh_graph_launch(gh_ctx* ctx, int id) {
  if (!ctx) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  if (id < 0 || id >= (int)ctx->graphs.size() || !ctx->graphs[id].used)
    return gh_fail(ctx, GH_EINVAL, "unknown graph id");
  return gh_check_hip(ctx, hipGraphLaunch(ctx->graphs[id].exec, ctx->stream), "hipGraphLaunch");
}

int gh_graph_destroy(gh_ctx* ctx, int id) {
  if (!ctx) return GH_EINVAL;
  if (id < 0 || id >= (int)ctx->graphs.size() || !ctx->graphs[id].used) return GH_EINVAL;
  hipStreamSynchronize(ctx->stream);
  hipGraphExecDestroy(ctx->graphs[id].exec);
  hipGraphDestroy(ctx->graphs[id].graph);
  ctx->graphs[id] = gh_graph_slot();
  return GH_OK;
}

int gh_last_error(gh_ctx* ctx, char* buf, int len) {
  if (!ctx) return GH_EINVAL;
  if (buf && len > 0) snprintf(buf, (size_t)len, "%s", ctx->errmsg.c_str());
  return ctx->err;
}

int gh_clear_error(gh_ctx* ctx) {
  if (!ctx) return GH_EINVAL;
  ctx->err = GH_OK;
  ctx->errmsg.clear();
  (void)hipGetLastError();
  return GH_OK;
}

int gh_event_record(gh_ctx* ctx, int slot) {
  if (!ctx || slot < 0 || slot >= 64) return GH_EINVAL;
  if (ctx->err) return ctx->err;
  if (!ctx->events[slot]) {
    int rc = gh_check_hip(ctx, hipEventCreate(&ctx->events[slot]), "hipEventCreate");
    if (rc) return rc;
  }
  return gh_check_hip(ctx, hipEventRecord(ctx->events[slot], ctx->stream), "hipEventRecord");
}

int gh_event_elapsed_ms(gh_ctx* ctx, int start, int stop, float* ms) {
  if (!ctx || !ms || start < 0 || start >= 64 || stop < 0 || stop >= 64) return GH_EINVAL;
  if (!ctx->events[start] || !ctx->events[stop]) return GH_ESTATE;
  int rc = gh_check_hip(ctx, hipEventSynchronize(ctx->events[stop]), "hipEventSynchronize");
  if (rc) return rc;
  return gh_check_hip(ctx, hipEventElapsedTime(ms, ctx->events[start], ctx->events[stop]),
                      "hipEventElapsedTime");
}

}  // extern "C"
