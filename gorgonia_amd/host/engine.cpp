#include "engine.hpp"

#include <cstdio>
#include <cstring>

namespace gorgonia {

static const char* kTypeMismatch = "TypeMismatch: a %s and b %s";              // cuda/errors.go:16
static const char* kShapeMismatch = "Shape mismatch. Expected %s. Got %s";    // cuda/errors.go:17

static std::string dtype_name(Dtype d) {
  return d == Dtype::Float32 ? "float32" : d == Dtype::Float64 ? "float64" : "other";
}

static std::string fmt2(const char* f, const std::string& a, const std::string& b) {
  char buf[512];
  snprintf(buf, sizeof(buf), f, a.c_str(), b.c_str());
  return buf;
}

std::string Shape::String() const {
  std::string s = "(";
  for (size_t i = 0; i < d.size(); i++) s += (i ? ", " : "") + std::to_string(d[i]);
  return s + ")";
}

Engine::~Engine() { Close(); }

Status Engine::fail(int rc, const std::string& what) {
  char buf[512] = {0};
  if (ctx_) gh_last_error(ctx_, buf, sizeof(buf));
  return Status::Err(rc, what + (buf[0] ? std::string(": ") + buf : std::string()));
}

Status Engine::Init(int device, int64_t size) {
  if (ctx_) return Status::OK();  // already initialised (cuda/external.go:93-95)
  if (size < 0) return Status::Err(GH_EINVAL, "negative arena size");
  // reserve 2*size + size/2 + minAllocSize (cuda/external.go:158)
  const int64_t allocsize = 2 * size + size / 2 + 256;
  int rc = gh_init(device, allocsize, &ctx_);
  if (rc != GH_OK) {
    ctx_ = nullptr;
    char buf[160];
    snprintf(buf, sizeof(buf), "Failed to initialize HIP Engine with size %lld for device %d",
             (long long)size, device);
    return Status::Err(rc, buf);
  }
  gh_device_info(ctx_, &info_);
  a_ = BFC(32);
  a_.reserve(gh_arena_base(ctx_), allocsize);
  uint64_t fm = 0;
  a_.alloc(4, &fm);
  flag_mem_ = fm;
  a_.reset_stats();
  return Status::OK();
}

Status Engine::Close() {
  if (!ctx_) return Status::OK();
  segment_.clear();
  a_.release();
  int rc = gh_close(ctx_);
  ctx_ = nullptr;
  return rc == GH_OK ? Status::OK() : Status::Err(rc, "Failed to close HIP context");
}

bool Engine::HasFunc(const std::string& name) const { return gh_has_func(name.c_str()) == 1; }

static int calc_blocks(int64_t n, int64_t max_threads) {  // cuda/utils.go calcBlocks
  return (int)((n + max_threads - 1) / max_threads);
}

// Kept for callers of the External interface; the HIP kernels size their own
// grids (grid-stride loops), so nothing on the launch path consumes this.
GridSize Engine::ElemGridSize(int n) const {
  const int64_t mt = info_.max_threads_per_block ? info_.max_threads_per_block : 1024;
  const int64_t mgx = info_.max_grid_x ? info_.max_grid_x : 2147483647;
  const int64_t mgy = info_.max_grid_y ? info_.max_grid_y : 65535;
  const int64_t mgz = info_.max_grid_z ? info_.max_grid_z : 65535;
  GridSize g{1, 1, 1, 1, 1, 1};
  const int64_t blocks = calc_blocks(n, mt);
  if (blocks == 1) g.bx = n;
  else if ((double)blocks >= (double)mgx * (double)mgy * (double)mgz) { /* unrepresentable */ }
  else if ((double)blocks >= (double)mgx * (double)mgy) {
    g.gx = (int)mgx; g.gy = (int)mgy; g.gz = calc_blocks(blocks % (mgx * mgy), mgz); g.bx = (int)mt;
  } else if (blocks >= mgx) {
    g.gx = (int)mgx; g.gy = calc_blocks(blocks % mgx, mgy); g.bx = (int)mt;
  } else { g.gx = (int)blocks; g.bx = (int)mt; }
  return g;
}

Status Engine::DoWork() {
  if (!ctx_) return Status::Err(GH_ESTATE, "engine not initialised");
  if (!segment_.empty()) {
    int rc = gh_submit(ctx_, segment_.data(), (int)segment_.size());
    submit_calls_++;
    segment_.clear();
    if (rc != GH_OK) return fail(rc, "gh_submit");
  }
  int rc = gh_sync(ctx_);
  if (rc != GH_OK) return fail(rc, "gh_sync");
  return Status::OK();
}

Status Engine::Errors() {
  if (!ctx_) return Status::OK();
  char buf[512] = {0};
  int rc = gh_last_error(ctx_, buf, sizeof(buf));
  return rc == GH_OK ? Status::OK() : Status::Err(rc, buf);
}

// ---- arena ---------------------------------------------------------------------
Status Engine::Get(int64_t size, uint64_t* mem) {
  OomError oom;
  int rc = a_.alloc(size, mem, &oom);
  if (rc == 1) return Status::Err(GH_EINVAL, "Cannot allocate memory with size 0 or less");
  if (rc == 2) {
    char buf[96];
    snprintf(buf, sizeof(buf), "allocated/reserved: %lld/%lld", (long long)oom.allocated,
             (long long)oom.reserved);  // cuda/errors.go:13
    return Status::Err(GH_EOOM, buf);
  }
  return Status::OK();
}

void Engine::Put(uint64_t mem, int64_t) { a_.free(mem); }

void Engine::ResetAllocator() {
  a_.reset_allocator();
  if (ctx_) {  // keep the NaN/Inf flag cell
    uint64_t fm = 0;
    a_.alloc(4, &fm);
    flag_mem_ = fm;
    a_.reset_stats();
  }
}

Status Engine::Memcpy(uint64_t dst, int64_t dsize, uint64_t src, int64_t ssize) {
  // copies min(dst, src) bytes and is eager (cuda/engine.go:103-127)
  const int64_t size = dsize < ssize ? dsize : ssize;
  gh_cmd c{};
  c.opcode = GH_OP_MEMCPY_D2D;
  c.ptr[0] = dst; c.ptr[1] = src; c.dim[0] = size;
  Enqueue(c);
  return DoWork();
}

Status Engine::MemcpyHtoD(uint64_t dst, const void* src, int64_t bytes) {
  if (!ctx_) return Status::Err(GH_ESTATE, "engine not initialised");
  // stream order: everything recorded so far runs before the copy
  if (!segment_.empty()) {
    int rc = gh_submit(ctx_, segment_.data(), (int)segment_.size());
    submit_calls_++;
    segment_.clear();
    if (rc != GH_OK) return fail(rc, "gh_submit");
  }
  int rc = gh_memcpy_h2d(ctx_, dst, src, bytes);
  return rc == GH_OK ? Status::OK() : fail(rc, "MemcpyHtoD");
}

Status Engine::MemcpyDtoH(void* dst, uint64_t src, int64_t bytes, bool synchronous) {
  if (!ctx_) return Status::Err(GH_ESTATE, "engine not initialised");
  if (!segment_.empty()) {
    int rc = gh_submit(ctx_, segment_.data(), (int)segment_.size());
    submit_calls_++;
    segment_.clear();
    if (rc != GH_OK) return fail(rc, "gh_submit");
  }
  int rc = gh_memcpy_d2h(ctx_, dst, src, bytes);
  if (rc != GH_OK) return fail(rc, "MemcpyDtoH");
  return synchronous ? DoWork() : Status::OK();
}

Status Engine::HostAlloc(int64_t bytes, void** out) {
  if (!ctx_) return Status::Err(GH_ESTATE, "engine not initialised");
  int rc = gh_host_alloc(ctx_, bytes, out);
  return rc == GH_OK ? Status::OK() : fail(rc, "HostAlloc");
}

void Engine::HostFree(void* p) {
  if (ctx_ && p) gh_host_free(ctx_, p);
}

void Engine::RecordCopy(uint64_t dst, uint64_t src, int64_t bytes) {
  gh_cmd c{};
  c.opcode = GH_OP_MEMCPY_D2D;
  c.ptr[0] = dst; c.ptr[1] = src; c.dim[0] = bytes;
  Enqueue(c);
}

// ---- checks (cuda/utils.go:22-112) ---------------------------------------------------
static Status binaryCheck(const Tensor& a, const Tensor& b) {
  if (a.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype for a: " + dtype_name(a.dt));
  if (b.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype for b: " + dtype_name(b.dt));
  if (a.dt != b.dt) return Status::Err(GH_EINVAL, fmt2(kTypeMismatch, dtype_name(a.dt), dtype_name(b.dt)));
  if (!a.shape.Eq(b.shape))
    return Status::Err(GH_EINVAL, fmt2(kShapeMismatch, b.shape.String(), a.shape.String()));
  if (a.requires_iterator) return Status::Err(GH_EINVAL, "unsupported operation: a requires an iterator");
  if (b.requires_iterator) return Status::Err(GH_EINVAL, "unsupported operation: b requires an iterator");
  return Status::OK();
}

static Status unaryCheck(const Tensor& a) {
  if (a.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype for a: " + dtype_name(a.dt));
  if (a.requires_iterator) return Status::Err(GH_EINVAL, "unsupported operation: a requires an iterator");
  return Status::OK();
}

static Status handleFuncOpts(const Shape& expShape, Dtype expType, const FuncOpts& o) {
  if (!o.reuse) return Status::OK();
  if (o.reuse->dt != expType)
    return Status::Err(GH_EINVAL, "Cannot use reuse: " +
                                      fmt2(kTypeMismatch, dtype_name(expType), dtype_name(o.reuse->dt)));
  if (o.reuse->DataSize() != expShape.TotalSize() && !expShape.IsScalar())
    return Status::Err(GH_EINVAL, "Cannot use reuse: shape mismatch - " +
                                      fmt2(kShapeMismatch, o.reuse->shape.String(), expShape.String()));
  return Status::OK();
}

static std::string binName(const char* fn, int mode, Dtype dt) {
  static const char* modes[4] = {"vv", "vs", "sv", "ss"};
  char buf[96];
  snprintf(buf, sizeof(buf), "elembinop.%s_%s_f%d", fn, modes[mode], (int)dtype_size(dt) * 8);
  return buf;
}

static const char* kFnNames[GH_BINFN__COUNT] = {"add", "sub", "mul", "div", "pow", "lt",
                                                "lte", "gt",  "gte", "eq",  "ne",  "mod"};

// Destination selection shared by all arithmetic methods (cuda/arith.go:34-49):
// with a reuse tensor the result lands there and a is left alone (the
// reference copies a into reuse and runs the in-place kernel on the copy; the
// three-address form of the command gives the same bytes in one pass);
// otherwise the op must be unsafe and works in place on a.
Status Engine::prepBinary(const char* go_name, Tensor& a, const FuncOpts& o, uint64_t* mem,
                          int64_t* size, Tensor** ret) {
  Status st = handleFuncOpts(a.shape, a.dt, o);
  if (!st.ok()) return st.Wrap("Unable to handle funcOpts");
  if (o.incr)
    return Status::Err(GH_EINVAL, std::string(go_name) + ": Incr operations are not supported");
  if (o.reuse) {
    *mem = o.reuse->mem;
    *size = o.reuse->DataSize();
    if (ret) *ret = o.reuse;
  } else if (!o.safe) {
    *mem = a.mem;
    *size = a.DataSize();
    if (ret) *ret = &a;
  } else {
    return Status::Err(GH_EINVAL,
                       "Impossible state: A reuse tensor must be passed in, or the operation must be "
                       "unsafe. Incr and safe operations are not supported");
  }
  return Status::OK();
}

Status Engine::BinOp(int fn, const char* go_name, Tensor& a, Tensor& b, const FuncOpts& o, Tensor** ret) {
  const int mode = a.shape.IsScalar() ? (b.shape.IsScalar() ? GH_SS : GH_SV)
                                      : (b.shape.IsScalar() ? GH_VS : GH_VV);  // constructName2
  const std::string name = binName(kFnNames[fn], mode, a.dt);
  if (!HasFunc(name))
    return Status::Err(GH_ENOFUNC, std::string("Unable to perform ") + go_name +
                                       "(). The tensor engine does not have the function \"" + name + "\"");
  Status st = binaryCheck(a, b);
  if (!st.ok()) return st.Wrap(std::string("Basic checks failed for ") + go_name);
  uint64_t mem; int64_t size;
  st = prepBinary(go_name, a, o, &mem, &size, ret);
  if (!st.ok()) return st;
  gh_cmd c{};
  c.opcode = GH_OP_ELEM_BIN;
  c.flags = GH_FLAG_FN(fn) | GH_FLAG_MODE(mode) | GH_FLAG_DTYPE((int)a.dt);
  c.ptr[0] = a.mem; c.ptr[1] = b.mem; c.ptr[2] = mem; c.dim[0] = size;
  Enqueue(c);
  return Status::OK();
}

Status Engine::BinOpScalar(int fn, const char* go_name, Tensor& a, uint64_t b_mem, bool left_tensor,
                           const FuncOpts& o, Tensor** ret) {
  const int mode = left_tensor ? GH_VS : GH_SV;  // constructName1
  const std::string name = binName(kFnNames[fn], mode, a.dt);
  if (!HasFunc(name))
    return Status::Err(GH_ENOFUNC, std::string("Unable to perform ") + go_name +
                                       "(). The tensor engine does not have the function \"" + name + "\"");
  if (!b_mem) return Status::Err(GH_EINVAL, "b has to be a tensor.Memory. Got <nil> instead");
  Status st = unaryCheck(a);
  if (!st.ok()) return st.Wrap(std::string("Basic checks failed for ") + go_name);
  uint64_t mem; int64_t size;
  st = prepBinary(go_name, a, o, &mem, &size, ret);
  if (!st.ok()) return st;
  gh_cmd c{};
  c.opcode = GH_OP_ELEM_BIN;
  c.flags = GH_FLAG_FN(fn) | GH_FLAG_MODE(mode) | GH_FLAG_DTYPE((int)a.dt);
  // vs: (tensor, scalar); sv: (scalar, tensor) - the reference swaps the two
  // pointers for sv because that kernel writes its second operand
  c.ptr[0] = left_tensor ? a.mem : b_mem;
  c.ptr[1] = left_tensor ? b_mem : a.mem;
  c.ptr[2] = mem;
  c.dim[0] = size;
  Enqueue(c);
  return Status::OK();
}

Status Engine::Mod(Tensor& a, Tensor& b, const FuncOpts& o, Tensor** ret) {
  return BinOp(GH_MOD, "Mod", a, b, o, ret);
}

Status Engine::UnaryTo(const std::string& op_name, Tensor& a, uint64_t dst_mem) {
  char nm[96];
  snprintf(nm, sizeof(nm), "elemunaryop.%s_f%d", op_name.c_str(), (int)dtype_size(a.dt) * 8);
  uint32_t opcode = 0, flags = 0;
  if (gh_lookup_func(nm, &opcode, &flags) != GH_OK)
    return Status::Err(GH_ENOFUNC, std::string("The tensor engine does not have the function \"") + nm + "\"");
  Status st = unaryCheck(a);
  if (!st.ok()) return st;
  gh_cmd c{};
  c.opcode = opcode; c.flags = flags;
  c.ptr[0] = a.mem; c.ptr[1] = dst_mem == a.mem ? 0 : dst_mem; c.dim[0] = a.DataSize();
  Enqueue(c);
  return Status::OK();
}

Status Engine::BroadcastBinOp(int fn, Tensor& big, Tensor& small, int64_t outer, int64_t mid,
                              int64_t inner, bool small_left, uint64_t dst_mem) {
  if (fn < 0 || fn >= GH_BINFN__COUNT) return Status::Err(GH_ENOFUNC, "unknown binary function");
  if (big.dt != small.dt) return Status::Err(GH_EINVAL, "broadcast: operands of different Dtypes");
  if (big.DataSize() != outer * mid * inner || small.DataSize() != mid)
    return Status::Err(GH_EINVAL, fmt2(kShapeMismatch, big.shape.String(), small.shape.String()));
  gh_cmd c{};
  c.opcode = GH_OP_BCAST_BIN;
  c.flags = GH_FLAG_FN(fn) | GH_FLAG_DTYPE(big.dt == Dtype::Float64 ? GH_F64 : GH_F32) | (small_left ? GH_FLAG_SMALL_LEFT : 0);
  c.ptr[0] = dst_mem; c.ptr[1] = big.mem; c.ptr[2] = small.mem;
  c.dim[0] = outer; c.dim[1] = mid; c.dim[2] = inner;
  Enqueue(c);
  return Status::OK();
}

Status Engine::SubmitPending() {
  if (!ctx_) return Status::Err(GH_ESTATE, "engine not initialised");
  if (segment_.empty()) return Status::OK();
  int rc = gh_submit(ctx_, segment_.data(), (int)segment_.size());
  submit_calls_++;
  segment_.clear();
  return rc == GH_OK ? Status::OK() : fail(rc, "gh_submit");
}

Status Engine::Sync() {
  if (!ctx_) return Status::Err(GH_ESTATE, "engine not initialised");
  int rc = gh_sync(ctx_);
  return rc == GH_OK ? Status::OK() : fail(rc, "gh_sync");
}

Status Engine::GraphBegin() {
  int rc = gh_graph_begin(ctx_);
  return rc == GH_OK ? Status::OK() : fail(rc, "gh_graph_begin");
}
Status Engine::GraphEnd(int* id) {
  int rc = gh_graph_end(ctx_, id);
  return rc == GH_OK ? Status::OK() : fail(rc, "gh_graph_end");
}
Status Engine::GraphLaunch(int id) {
  int rc = gh_graph_launch(ctx_, id);
  return rc == GH_OK ? Status::OK() : fail(rc, "gh_graph_launch");
}
Status Engine::GraphDestroy(int id) {
  if (!ctx_ || id < 0) return Status::OK();
  int rc = gh_graph_destroy(ctx_, id);
  return rc == GH_OK ? Status::OK() : fail(rc, "gh_graph_destroy");
}

// ---- linalg -------------------------------------------------------------------------
static Status checkThreeFloat(const Tensor& a, const Tensor& b, const Tensor& ret) {
  if (!a.manually_managed)
    return Status::Err(GH_EINVAL, "HIP Engine only takes non-natively accessible memory (memory on graphics cards). a isn't.");
  if (!b.manually_managed)
    return Status::Err(GH_EINVAL, "HIP Engine only takes non-natively accessible memory (memory on graphics cards). b isn't");
  if (!ret.manually_managed)
    return Status::Err(GH_EINVAL, "HIP Engine only takes non-natively accessible memory (memory on graphics cards). ret isn't");
  if (a.dt != b.dt || b.dt != ret.dt)
    return Status::Err(GH_EINVAL, "Expected a and b and retVal all to have the same Dtype");
  return Status::OK();
}

Status Engine::MatVecMul(Tensor& a, Tensor& b, Tensor& prealloc) {
  Status st = checkThreeFloat(a, b, prealloc);
  if (!st.ok()) return st.Wrap("MatVecMul failed pre check");
  if (a.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype");
  if (a.shape.Dims() != 2) return Status::Err(GH_EINVAL, "MatVecMul: a must be a matrix");
  const int64_t m = a.shape[0], n = a.shape[1];  // logical shape
  if (b.DataSize() != n || prealloc.DataSize() != m)
    return Status::Err(GH_EINVAL, fmt2(kShapeMismatch, Shape{n}.String(), b.shape.String()));
  gh_cmd c{};
  c.opcode = GH_OP_GEMV;
  c.ptr[0] = a.mem; c.ptr[1] = b.mem; c.ptr[2] = prealloc.mem;
  c.flags = GH_FLAG_DTYPE(a.dt == Dtype::Float64 ? GH_F64 : GH_F32);  // Dgemv / Sgemv, cuda/linalg.go:94-127
  // The four cases of cuda/linalg.go:57-75.  A column-major (m, n) matrix is the row-major matrix
  // (n, m) in memory, and so is a transposed view of a row-major one; column-major and transposed
  // together is plain row-major again.
  if (a.transposed != a.col_major) {  // stored (n x m) row-major: y = A_stored^T x
    c.flags |= GH_FLAG_TRANS_A;
    c.dim[0] = n; c.dim[1] = m; c.dim[2] = m;
  } else {
    c.dim[0] = m; c.dim[1] = n; c.dim[2] = n;
  }
  Enqueue(c);
  return Status::OK();
}

Status Engine::MatMul(Tensor& a, Tensor& b, Tensor& prealloc, int act, float alpha, bool softmax,
                      uint64_t bias) {
  Status st = checkThreeFloat(a, b, prealloc);
  if (!st.ok()) return st.Wrap("MatMul failed pre check");
  if (a.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype " + dtype_name(a.dt));
  if (a.dt == Dtype::Float64 && (act || bias))
    return Status::Err(GH_EINVAL, "MatMul: no fused activation or bias for float64");
  if (a.shape.Dims() != 2 || b.shape.Dims() != 2 || prealloc.shape.Dims() != 2)
    return Status::Err(GH_EINVAL, "MatMul: operands must be matrices");
  const int64_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
  if (b.shape[0] != k)
    return Status::Err(GH_EINVAL, fmt2(kShapeMismatch, Shape{k, n}.String(), b.shape.String()));
  if (prealloc.shape[0] != m || prealloc.shape[1] != n)
    return Status::Err(GH_EINVAL, fmt2(kShapeMismatch, Shape{m, n}.String(), prealloc.shape.String()));
  if (a.col_major != b.col_major)   // cuda/linalg.go:118-122
    return Status::Err(GH_EINVAL, std::string("a does not have the same data order as b. a is ") +
                                      (a.col_major ? "ColMajor" : "RowMajor") + ". b is " +
                                      (b.col_major ? "ColMajor" : "RowMajor"));
  gh_cmd c{};
  c.opcode = GH_OP_GEMM;
  c.flags = (act == 1 ? GH_FLAG_ACT_RELU : act == 2 ? GH_FLAG_ACT_LEAKY : 0) |
            (softmax ? GH_FLAG_GEMM_SOFTMAX : 0) | (bias ? GH_FLAG_GEMM_BIAS : 0) |
            GH_FLAG_DTYPE(a.dt == Dtype::Float64 ? GH_F64 : GH_F32);  // Dgemm / Sgemm, cuda/linalg.go:204-227
  c.f[0] = alpha;
  c.ptr[2] = prealloc.mem; c.ptr[3] = bias;
  c.dim[2] = k;
  c.dim[6] = 1;
  if (!a.col_major) {
    // Row-major case table of cuda/linalg.go:161-202 without the operand swap: the kernel is
    // row-major itself, so a transposed view just flips the flag and takes the stored width as
    // its leading dimension.
    c.flags |= (a.transposed ? GH_FLAG_TRANS_A : 0) | (b.transposed ? GH_FLAG_TRANS_B : 0);
    c.ptr[0] = a.mem; c.ptr[1] = b.mem;
    c.dim[0] = m; c.dim[1] = n;
    c.dim[3] = a.transposed ? m : k;
    c.dim[4] = b.transposed ? k : n;
    c.dim[5] = prealloc.shape[1];
  } else {
    // Column-major case table of cuda/linalg.go:142-160 (the result is column-major too, leading
    // dimension its row count): in row-major terms the memory holds C^T = B^T A^T, and a
    // column-major (r, c) operand is the row-major (c, r) matrix - the reference's operand swap the
    // other way round.  B^T (n x k) is the left operand, A^T (k x m) the right one; an operand whose
    // transposed flag is set is stored the other way and becomes a transposed view of that.
    if (act || bias || softmax)
      return Status::Err(GH_EINVAL, "MatMul: no fused bias, activation or softmax for column-major operands");
    c.flags |= (b.transposed ? GH_FLAG_TRANS_A : 0) | (a.transposed ? GH_FLAG_TRANS_B : 0);
    c.ptr[0] = b.mem; c.ptr[1] = a.mem;
    c.dim[0] = n; c.dim[1] = m;
    c.dim[3] = b.transposed ? n : k;   // ldb of the reference's table
    c.dim[4] = a.transposed ? k : m;   // lda
    c.dim[5] = prealloc.shape[0];      // ldc
  }
  c.dim[6] = 1;
  Enqueue(c);
  return Status::OK();
}

Status Engine::Outer(Tensor& a, Tensor& b, Tensor& prealloc) {
  Status st = checkThreeFloat(a, b, prealloc);
  if (!st.ok()) return st.Wrap("Outer failed pre check");
  if (a.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype");
  const int64_t m = a.DataSize(), n = b.DataSize();
  if (prealloc.DataSize() != m * n)
    return Status::Err(GH_EINVAL, fmt2(kShapeMismatch, Shape{m, n}.String(), prealloc.shape.String()));
  gh_cmd c{};
  c.opcode = GH_OP_OUTER;
  c.flags = GH_FLAG_DTYPE(a.dt == Dtype::Float64 ? GH_F64 : GH_F32);  // Dger / Sger, cuda/linalg.go:129-159
  c.ptr[0] = a.mem; c.ptr[1] = b.mem; c.ptr[2] = prealloc.mem;
  c.dim[0] = m; c.dim[1] = n;
  Enqueue(c);
  return Status::OK();
}

Status Engine::BatchedMatMul(Tensor& a, Tensor& b, Tensor& c, bool transA, bool transB) {
  Status st = checkThreeFloat(a, b, c);
  if (!st.ok()) return st.Wrap("BatchedMatMul failed pre check");
  if (a.dt == Dtype::Other) return Status::Err(GH_EINVAL, "Unsupported Dtype");
  const int da = a.shape.Dims(), db = b.shape.Dims();
  if (da < 3 || db != da) return Status::Err(GH_EINVAL, "BatchedMatMul: operands need equal rank >= 3");
  int64_t batch = 1;
  for (int i = 0; i < da - 2; i++) {
    if (a.shape[i] != b.shape[i]) return Status::Err(GH_EINVAL, "BatchedMatMul: batch dims differ");
    batch *= a.shape[i];
  }
  int64_t ar = a.shape[da - 2], ac = a.shape[da - 1], br = b.shape[da - 2], bc = b.shape[da - 1];
  const int64_t m = transA ? ac : ar, k = transA ? ar : ac;
  const int64_t kb = transB ? bc : br, n = transB ? br : bc;
  if (k != kb) return Status::Err(GH_EINVAL, "BatchedMatMul: inner dimensions differ");
  if (c.DataSize() != batch * m * n) return Status::Err(GH_EINVAL, "BatchedMatMul: bad result shape");
  gh_cmd cmd{};
  cmd.opcode = GH_OP_GEMM;
  cmd.flags = (transA ? GH_FLAG_TRANS_A : 0) | (transB ? GH_FLAG_TRANS_B : 0) |
              GH_FLAG_DTYPE(a.dt == Dtype::Float64 ? GH_F64 : GH_F32);
  cmd.ptr[0] = a.mem; cmd.ptr[1] = b.mem; cmd.ptr[2] = c.mem;
  cmd.dim[0] = m; cmd.dim[1] = n; cmd.dim[2] = k;
  cmd.dim[3] = ac; cmd.dim[4] = bc; cmd.dim[5] = n;
  cmd.dim[6] = batch; cmd.dim[7] = ar * ac; cmd.dim[8] = br * bc; cmd.dim[9] = m * n;
  Enqueue(cmd);
  return Status::OK();
}

// ---- NaN / Inf ------------------------------------------------------------------------
static Status has_check(Engine& e, gh_ctx* ctx, uint64_t flag_mem, int opcode, Tensor& a, bool* out) {
  if (a.dt == Dtype::Other) return Status::Err(GH_ENOFUNC, "Unable to perform HasNaN/HasInf(): unsupported dtype");
  gh_cmd c{};
  c.opcode = (uint32_t)opcode;
  c.flags = GH_FLAG_DTYPE((int)a.dt);
  c.ptr[0] = a.mem; c.ptr[1] = flag_mem; c.dim[0] = a.DataSize();
  e.Enqueue(c);
  Status st = e.DoWork();
  if (!st.ok()) return st;
  int32_t v = 0;
  int rc = gh_memcpy_d2h(ctx, &v, flag_mem, 4);
  if (rc == GH_OK) rc = gh_sync(ctx);
  if (rc != GH_OK) return Status::Err(rc, "reading NaN/Inf flag failed");
  *out = v > 0;
  return Status::OK();
}

Status Engine::HasNaN(Tensor& a, bool* out) { return has_check(*this, ctx_, flag_mem_, GH_OP_HAS_NAN, a, out); }
Status Engine::HasInf(Tensor& a, bool* out) { return has_check(*this, ctx_, flag_mem_, GH_OP_HAS_INF, a, out); }

}  // namespace gorgonia
