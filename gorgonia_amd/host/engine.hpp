// C++ mirror of Gorgonia's device engine (package cuda: Engine, External,
// Arena) written against the C ABI of include/gorgonia_hip.h only - the same
// calls a Go/cgo shim would make.  Method names, argument meaning and error
// behaviour follow the Go methods they stand in for; each one cites its
// counterpart.
//
// The engine never launches anything itself.  Every operator appends one
// gh_cmd to the current tape segment; DoWork()/Signal() hand the whole segment
// to gh_submit() in one call and wait (the reference's BatchedContext queues
// driver calls the same way and drains them in DoWork, cuda/external.go:223).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "bfc.hpp"
#include "gorgonia_hip.h"

namespace gorgonia {

enum class Dtype : int32_t { Float32 = 0, Float64 = 1, Other = 2 };
inline int64_t dtype_size(Dtype d) { return d == Dtype::Float64 ? 8 : 4; }

// tensor.Shape: empty = scalar.
struct Shape {
  std::vector<int64_t> d;
  Shape() {}
  Shape(std::initializer_list<int64_t> l) : d(l) {}
  explicit Shape(std::vector<int64_t> v) : d(std::move(v)) {}
  bool IsScalar() const { return d.empty(); }
  int Dims() const { return (int)d.size(); }
  int64_t TotalSize() const { int64_t n = 1; for (auto v : d) n *= v; return n; }
  bool Eq(const Shape& o) const { return d == o.d; }
  int64_t operator[](int i) const { return d[(size_t)i]; }
  std::string String() const;
};

// A dense tensor whose memory lives in the engine's arena ("manually managed",
// cuda/engine.go:81-83).  `transposed` is the DataOrder flag the linalg methods
// look at (cuda/linalg.go:57,135).
struct Tensor {
  uint64_t mem = 0;
  Dtype dt = Dtype::Float32;
  Shape shape;
  bool manually_managed = true;
  bool transposed = false;
  bool col_major = false;          // DataOrder.IsColMajor: element (i, j) of an untransposed (r, c) matrix at j * r + i
  bool requires_iterator = false;  // views the engine cannot walk (cuda/utils.go:83-89)
  int64_t DataSize() const { return shape.IsScalar() ? 1 : shape.TotalSize(); }
  int64_t MemSize() const { return DataSize() * dtype_size(dt); }
};

struct Status {
  int code = 0;  // 0 ok, otherwise a GH_E* code
  std::string msg;
  bool ok() const { return code == 0; }
  static Status OK() { return Status(); }
  static Status Err(int c, std::string m) { Status s; s.code = c; s.msg = std::move(m); return s; }
  Status Wrap(const std::string& ctx) const { return ok() ? *this : Err(code, ctx + ": " + msg); }
};

// tensor.FuncOpt subset the engine understands (cuda/utils.go:22-56):
// WithReuse(t), UseUnsafe(), WithIncr (rejected).
struct FuncOpts {
  Tensor* reuse = nullptr;
  bool safe = true;
  bool incr = false;
  static FuncOpts WithReuse(Tensor* t) { FuncOpts o; o.reuse = t; return o; }
  static FuncOpts UseUnsafe() { FuncOpts o; o.safe = false; return o; }
};

struct GridSize { int gx, gy, gz, bx, by, bz; };

class Engine {
 public:
  Engine() {}
  ~Engine();
  Engine(const Engine&) = delete;
  Engine& operator=(const Engine&) = delete;

  // ---- External (cuda/interfaces.go:23-65, cuda/external.go) ----------------
  Status Init(int device, int64_t size);           // cuda/external.go:88-170
  Status Close();                                  // cuda/external.go:173-220
  bool Initialized() const { return ctx_ != nullptr; }
  bool HasFunc(const std::string& name) const;     // cuda/external.go:26
  GridSize ElemGridSize(int n) const;              // cuda/external.go:52-85
  Status DoWork();                                 // cuda/external.go:223-226
  Status Signal() { return DoWork(); }             // cuda/external.go:32-34 (+ Sync)
  Status Errors();                                 // cuda/engine.go:141
  gh_ctx* Context() const { return ctx_; }         // stands in for *cu.BatchedContext
  const gh_devinfo& DeviceInfo() const { return info_; }

  // ---- Arena (cuda/arena.go:13-36) -----------------------------------------------
  Status Get(int64_t size, uint64_t* mem);
  void Put(uint64_t mem, int64_t size);
  void ResetAllocator();
  BFC& Allocator() { return a_; }

  // ---- tensor.Engine (cuda/engine.go:72-141) ---------------------------------------
  // Device memory is not host-dereferenceable (hipMalloc, not managed memory):
  bool AllocAccessible() const { return false; }
  Status Alloc(int64_t size, uint64_t* mem) { return Get(size, mem); }
  Status Free(uint64_t mem, int64_t size) { Put(mem, size); return Status::OK(); }
  Status Memcpy(uint64_t dst, int64_t dsize, uint64_t src, int64_t ssize);  // eager, min size
  bool WorksWith() const { return true; }
  // The reference leaves these three unimplemented and panics (cuda/engine.go:93-99,
  // 130-132); here they report the same words as an error instead of aborting.
  Status Memset(uint64_t, const void*) { return Status::Err(GH_ENOFUNC, "not implemented"); }
  Status Memclr(uint64_t) { return Status::Err(GH_ENOFUNC, "not implemented"); }
  Status Accessible(uint64_t, uint64_t*) { return Status::Err(GH_ENOFUNC, "not implemented"); }
  // AllocFlags (cuda/engine.go:81-83): manually managed memory, column-major tag.
  void AllocFlags(bool* manually_managed, bool* col_major) const { *manually_managed = true; *col_major = true; }
  void NonStdAlloc() {}                            // cuda/engine.go:138

  // Host <-> device transfers (ExternMetadata.Transfer, cuda.go:179-215); queued
  // behind the segment recorded so far.  `synchronous` flushes like Signal().
  Status MemcpyHtoD(uint64_t dst, const void* src, int64_t bytes);
  Status MemcpyDtoH(void* dst, uint64_t src, int64_t bytes, bool synchronous = true);
  // Pinned host memory the device can write; a copy into it can be recorded in
  // the segment like any operator (and so be captured and replayed with it).
  Status HostAlloc(int64_t bytes, void** out);
  void HostFree(void* p);
  void RecordCopy(uint64_t dst, uint64_t src, int64_t bytes);

  // ---- arithmetic and comparison (cuda/arith.go, cuda/cmp.go) -----------------------
  // fn is a gh_binfn.  Tensor-tensor form: Add/Sub/Mul/Div/Pow/Lt/Lte/Gt/Gte/ElEq/ElNe.
  Status BinOp(int fn, const char* go_name, Tensor& a, Tensor& b, const FuncOpts& o, Tensor** ret);
  // Tensor-scalar form (AddScalar ...): b is device memory holding one element.
  Status BinOpScalar(int fn, const char* go_name, Tensor& a, uint64_t b_mem, bool left_tensor,
                     const FuncOpts& o, Tensor** ret);
#define GORGONIA_BINOP(NAME, FN)                                                         \
  Status NAME(Tensor& a, Tensor& b, const FuncOpts& o, Tensor** ret = nullptr) {         \
    return BinOp(FN, #NAME, a, b, o, ret);                                               \
  }                                                                                      \
  Status NAME##Scalar(Tensor& a, uint64_t b, bool leftTensor, const FuncOpts& o,         \
                      Tensor** ret = nullptr) {                                          \
    return BinOpScalar(FN, #NAME "Scalar", a, b, leftTensor, o, ret);                    \
  }
  GORGONIA_BINOP(Add, GH_ADD) GORGONIA_BINOP(Sub, GH_SUB) GORGONIA_BINOP(Mul, GH_MUL)
  GORGONIA_BINOP(Div, GH_DIV) GORGONIA_BINOP(Pow, GH_POW) GORGONIA_BINOP(Lt, GH_LT)
  GORGONIA_BINOP(Lte, GH_LTE) GORGONIA_BINOP(Gt, GH_GT) GORGONIA_BINOP(Gte, GH_GTE)
  GORGONIA_BINOP(ElEq, GH_EQ) GORGONIA_BINOP(ElNe, GH_NE)
#undef GORGONIA_BINOP
  // Mod: the reference engine declares the methods but ships no kernel, so its calls stop at
  // "does not have the function" (cuda/arith.go:589-701, elembinop.cu:201-210); here the
  // kernel exists and the call runs, with math.Mod's semantics.
  Status Mod(Tensor& a, Tensor& b, const FuncOpts& o, Tensor** ret = nullptr);

  // Unary kernels by the reference's op name ("tanh", "sigmoid", "inv" ...):
  // elemUnaryOp.CUDADo (op_math_cuda.go:23-85), in place on a.
  Status Unary(const std::string& op_name, Tensor& a) { return UnaryTo(op_name, a, 0); }
  // Same with a separate destination (prealloc != input: the reference copies
  // the input into prealloc first, op_math_cuda.go:62-70; one pass here).
  Status UnaryTo(const std::string& op_name, Tensor& a, uint64_t dst_mem);
  // Fused broadcast: dst = big op small (or small op big), `small` repeated
  // over (outer, inner).  Engine-level stand-in for Broadcast + repeatOp + the
  // plain op (broadcast.go:69-129, op_tensor.go:354-394, api_gen.go:129-135).
  Status BroadcastBinOp(int fn, Tensor& big, Tensor& small, int64_t outer, int64_t mid, int64_t inner,
                        bool small_left, uint64_t dst_mem);

  // ---- linalg (cuda/linalg.go:47-285) -----------------------------------------------------
  Status MatVecMul(Tensor& a, Tensor& b, Tensor& prealloc);
  // act: 0 none, 1 Rectify, 2 LeakyRelu(alpha) applied to the product (fused epilogue).
  // bias (device address of n floats, 0 = none) is added to every row before the activation
  Status MatMul(Tensor& a, Tensor& b, Tensor& prealloc, int act = 0, float alpha = 0.f, bool softmax = false,
                uint64_t bias = 0);
  Status Outer(Tensor& a, Tensor& b, Tensor& prealloc);
  // batchedMatMul (operatorLinAlg.go:435-502): one strided-batched launch.
  Status BatchedMatMul(Tensor& a, Tensor& b, Tensor& c, bool transA, bool transB);

  // ---- NaN / Inf watch (cuda/engine.go:144-191) ---------------------------------------------
  Status HasNaN(Tensor& a, bool* out);
  Status HasInf(Tensor& a, bool* out);

  // ---- segment recording ----------------------------------------------------------------------
  void Enqueue(const gh_cmd& c) { segment_.push_back(c); }
  size_t PendingCommands() const { return segment_.size(); }
  const std::vector<gh_cmd>& Segment() const { return segment_; }
  void DropSegment() { segment_.clear(); }
  int64_t SubmitCalls() const { return submit_calls_; }  // C-ABI crossings made by DoWork
  Status SubmitPending();                 // gh_submit of the segment, no wait
  Status Sync();                          // wait only
  // hipGraph replay of a segment (gh_graph_* pass-throughs)
  Status GraphBegin();
  Status GraphEnd(int* id);
  Status GraphLaunch(int id);
  Status GraphDestroy(int id);

 private:
  Status fail(int rc, const std::string& what);
  Status prepBinary(const char* go_name, Tensor& a, const FuncOpts& o, uint64_t* mem, int64_t* size,
                    Tensor** ret);
  gh_ctx* ctx_ = nullptr;
  gh_devinfo info_{};
  BFC a_{32};  // memalign = 32 (cuda/external.go:21)
  std::vector<gh_cmd> segment_;
  int64_t submit_calls_ = 0;
  uint64_t flag_mem_ = 0;  // 4-byte device flag for HasNaN/HasInf
};

}  // namespace gorgonia
