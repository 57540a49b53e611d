#include "tape.hpp"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <sstream>

namespace gorgonia {

// Outputs up to this size leave through pinned host memory, written by their own
// kernel where nothing else on the device reads them.  (The 2.3 MB result of the
// yolo-shaped stack written by its last kernel costs ~57 us of PCIe time; the
// explicit copy behind the segment it replaces cost ~85 us.)
static constexpr int64_t kStageLimit = 8 << 20;
// inputs re-uploaded on every run are staged through pinned memory up to these sizes
static constexpr int64_t kStageInLimit = 16 << 20;    // per input (what one copy kernel moves)
static constexpr int64_t kStageInTotal = 512ll << 20; // per machine
// inputs from this size on are uploaded in pieces, the host copy into pinned memory overlapping the bus
static constexpr int64_t kPipelinedUpload = 4 << 20;
static constexpr int64_t kUploadPiece = 2 << 20;

static Status bad(const std::string& m) { return Status::Err(GH_EINVAL, m); }

static int64_t conv_out(int64_t in, int64_t k, int64_t pad, int64_t stride, int64_t dil) {
  return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;  // op_nn.go:311-315
}
static int64_t pool_out(int64_t in, int64_t k, int64_t pa, int64_t pb, int64_t stride) {
  return (in + pa + pb - (k - 1) - 1) / stride + 1;  // op_nn.go:810-816
}

// Broadcast decomposition: the small operand has size-1 dims everywhere except
// one contiguous run of axes, which must match the big operand.
static bool bcast_decompose(const Shape& big, const Shape& small, int64_t* outer, int64_t* mid,
                            int64_t* inner) {
  if (big.Dims() != small.Dims()) return false;
  int first = -1, last = -1;
  for (int i = 0; i < big.Dims(); i++) {
    if (small[i] == big[i] && big[i] != 1) { if (first < 0) first = i; last = i; }
    else if (small[i] != 1) return false;
  }
  if (first < 0) { *outer = big.TotalSize(); *mid = 1; *inner = 1; return true; }
  for (int i = first; i <= last; i++) if (small[i] != big[i]) return false;
  *outer = *mid = *inner = 1;
  for (int i = 0; i < first; i++) *outer *= big[i];
  for (int i = first; i <= last; i++) *mid *= big[i];
  for (int i = last + 1; i < big.Dims(); i++) *inner *= big[i];
  return true;
}

Status InferShape(const OpSpec& op, const std::vector<const Shape*>& in, Shape* out) {
  auto need = [&](size_t n) { return in.size() == n; };
  switch (op.kind) {
    case OpKind::ElemBin:
      if (!need(2)) return bad("binary op needs 2 inputs");
      if (in[0]->IsScalar()) { *out = *in[1]; return Status::OK(); }
      if (in[1]->IsScalar()) { *out = *in[0]; return Status::OK(); }
      if (!in[0]->Eq(*in[1]))
        return bad("Shape mismatch. Expected " + in[0]->String() + ". Got " + in[1]->String());
      *out = *in[0];
      return Status::OK();
    case OpKind::ElemUnary:
    case OpKind::Rectify:
    case OpKind::LeakyRelu:
      if (!need(1)) return bad("unary op needs 1 input");
      *out = *in[0];
      return Status::OK();
    case OpKind::BroadcastBin: {
      if (!need(2)) return bad("broadcast op needs 2 inputs");
      int64_t o, m, i;
      const bool left_small = in[0]->TotalSize() < in[1]->TotalSize();
      const Shape& big = left_small ? *in[1] : *in[0];
      const Shape& small = left_small ? *in[0] : *in[1];
      if (!bcast_decompose(big, small, &o, &m, &i))
        return bad("cannot broadcast " + small.String() + " to " + big.String());
      *out = big;
      return Status::OK();
    }
    case OpKind::MatMul: {
      if (!need(2) || in[0]->Dims() != 2 || in[1]->Dims() != 2) return bad("MatMul needs two matrices");
      const int64_t m = op.transA ? (*in[0])[1] : (*in[0])[0], k = op.transA ? (*in[0])[0] : (*in[0])[1];
      const int64_t kb = op.transB ? (*in[1])[1] : (*in[1])[0], n = op.transB ? (*in[1])[0] : (*in[1])[1];
      if (k != kb) return bad("MatMul: inner dimensions differ");
      *out = Shape{m, n};
      return Status::OK();
    }
    case OpKind::MatVecMul: {
      if (!need(2) || in[0]->Dims() != 2 || in[1]->Dims() != 1) return bad("MatVecMul needs a matrix and a vector");
      const int64_t m = op.transA ? (*in[0])[1] : (*in[0])[0], n = op.transA ? (*in[0])[0] : (*in[0])[1];
      if ((*in[1])[0] != n) return bad("MatVecMul: dimension mismatch");
      *out = Shape{m};
      return Status::OK();
    }
    case OpKind::Outer:
      if (!need(2) || in[0]->Dims() != 1 || in[1]->Dims() != 1) return bad("Outer needs two vectors");
      *out = Shape{(*in[0])[0], (*in[1])[0]};
      return Status::OK();
    case OpKind::BatchedMatMul: {
      if (!need(2) || in[0]->Dims() < 3 || in[0]->Dims() != in[1]->Dims()) return bad("BatchedMatMul needs equal rank >= 3");
      const int d = in[0]->Dims();
      std::vector<int64_t> o(in[0]->d.begin(), in[0]->d.end() - 2);
      const int64_t ar = (*in[0])[d - 2], ac = (*in[0])[d - 1], br = (*in[1])[d - 2], bc = (*in[1])[d - 1];
      const int64_t m = op.transA ? ac : ar, k = op.transA ? ar : ac, kb = op.transB ? bc : br,
                    n = op.transB ? br : bc;
      if (k != kb) return bad("BatchedMatMul: inner dimensions differ");
      o.push_back(m); o.push_back(n);
      *out = Shape(o);
      return Status::OK();
    }
    case OpKind::Conv2d: {
      if (!need(2)) return bad("Conv2d needs image and filter");
      if (in[0]->Dims() != 4) return bad("im should have 4 dims, got " + std::to_string(in[0]->Dims()) + " dims");
      if (in[1]->Dims() != 4) return bad("filter should have 4 dims, got " + std::to_string(in[1]->Dims()) + " dims");
      if (op.ints.size() != 8) return bad("Conv2d needs kernel, pad, stride, dilation");
      const auto& p = op.ints;
      if (p[4] <= 0 || p[5] <= 0) return bad("Cannot use strides of less than or equal 0");
      if (p[2] < 0 || p[3] < 0) return bad("Cannot use padding of less than 0");
      if (p[6] <= 0 || p[7] <= 0) return bad("Cannot use dilation less than or eq 0");
      if ((*in[1])[1] != (*in[0])[1] || (*in[1])[2] != p[0] || (*in[1])[3] != p[1])
        return bad("filter shape " + in[1]->String() + " does not fit image " + in[0]->String());
      const int64_t oh = conv_out((*in[0])[2], p[0], p[2], p[4], p[6]);
      const int64_t ow = conv_out((*in[0])[3], p[1], p[3], p[5], p[7]);
      if (oh <= 0 || ow <= 0) return bad("Conv2d: empty output");
      *out = Shape{(*in[0])[0], (*in[1])[0], oh, ow};
      return Status::OK();
    }
    case OpKind::MaxPool2D: {
      if (!need(1)) return bad("MaxPool2D needs 1 input");
      if (in[0]->Dims() != 4) return bad("Expected input to have a shape with dimension 4");
      const auto& p = op.ints;  // kh kw npad pads... sh sw
      if (p.size() < 3 || (p[2] != 2 && p[2] != 4) || (int64_t)p.size() != 3 + p[2] + 2)
        return bad("MaxPool2D needs kernel, 2 or 4 pads, stride");
      const int64_t np = p[2];
      const int64_t pn = p[3], ps = np == 4 ? p[4] : p[3], pw = np == 4 ? p[5] : p[4], pe = np == 4 ? p[6] : p[4];
      const int64_t sh = p[3 + np], sw = p[4 + np];
      if (sh <= 0 || sw <= 0) return bad("Cannot use strides of less than or equal 0");
      for (int64_t i = 0; i < np; i++) if (p[3 + i] < 0) return bad("Cannot use padding of less than 0");
      if ((*in[0])[2] - p[0] + pn + ps < 0) return bad("Impossible height/kernel/pad combination");
      if ((*in[0])[3] - p[1] + pw + pe < 0) return bad("Impossible width/kernel/pad combination");
      *out = Shape{(*in[0])[0], (*in[0])[1], pool_out((*in[0])[2], p[0], pn, ps, sh),
                   pool_out((*in[0])[3], p[1], pw, pe, sw)};
      return Status::OK();
    }
    case OpKind::BatchNorm: {
      if (in.size() != 3 && in.size() != 5) return bad("BatchNorm needs x, mean, var[, scale, bias]");
      if (in[0]->Dims() != 2 && in[0]->Dims() != 4) return bad("BatchNorm input must be (B, N) or (B, C, H, W)");
      const int64_t C = (*in[0])[1];
      for (size_t i = 1; i < in.size(); i++)
        if (in[i]->TotalSize() != C)
          return bad("invalid runningMean shape " + in[i]->String() + ". Expected: (" + std::to_string(C) + ")");
      *out = *in[0];
      return Status::OK();
    }
    case OpKind::SoftMax:
      if (!need(1) || in[0]->IsScalar()) return bad("SoftMax needs a tensor");
      *out = *in[0];
      return Status::OK();
    case OpKind::MaxPool2DDiff: {
      if (!need(2)) return bad("MaxPool2DDiff needs input and gradient");
      OpSpec fwd = op;
      fwd.kind = OpKind::MaxPool2D;
      Shape pooled;
      std::vector<const Shape*> one{in[0]};
      Status st = InferShape(fwd, one, &pooled);
      if (!st.ok()) return st;
      if (!pooled.Eq(*in[1])) return bad("MaxPool2DDiff: gradient shape " + in[1]->String() + ", expected " + pooled.String());
      *out = *in[0];
      return Status::OK();
    }
    case OpKind::Conv2dDiffData: {
      if (!need(2) || op.ints.size() != 12) return bad("Conv2dDiffData needs gradient, filter and the image shape");
      Shape xs{op.ints[8], op.ints[9], op.ints[10], op.ints[11]};
      OpSpec fwd = op;
      fwd.kind = OpKind::Conv2d;
      fwd.ints.resize(8);
      Shape ys;
      std::vector<const Shape*> two{&xs, in[1]};
      Status st = InferShape(fwd, two, &ys);
      if (!st.ok()) return st;
      if (!ys.Eq(*in[0])) return bad("Conv2dDiffData: gradient shape " + in[0]->String() + ", expected " + ys.String());
      *out = xs;
      return Status::OK();
    }
    case OpKind::Conv2dDiffFilter: {
      if (!need(2) || op.ints.size() != 8) return bad("Conv2dDiffFilter needs image, gradient and the conv parameters");
      if (in[0]->Dims() != 4 || in[1]->Dims() != 4) return bad("Conv2dDiffFilter: 4-D operands expected");
      Shape ws{(*in[1])[1], (*in[0])[1], op.ints[0], op.ints[1]};
      OpSpec fwd = op;
      fwd.kind = OpKind::Conv2d;
      Shape ys;
      std::vector<const Shape*> two{in[0], &ws};
      Status st = InferShape(fwd, two, &ys);
      if (!st.ok()) return st;
      if (!ys.Eq(*in[1])) return bad("Conv2dDiffFilter: gradient shape " + in[1]->String() + ", expected " + ys.String());
      *out = ws;
      return Status::OK();
    }
    case OpKind::BatchNormTrain:
    case OpKind::BatchNormDiff: {
      const size_t want = op.kind == OpKind::BatchNormTrain ? 5 : 4;
      if (in.size() != want) return bad("BatchNorm training ops need x[, grad] and the statistics tensors");
      if (in[0]->Dims() != 2 && in[0]->Dims() != 4) return bad("BatchNorm input must be (B, N) or (B, C, H, W)");
      const int64_t C = (*in[0])[1];
      const size_t first = op.kind == OpKind::BatchNormTrain ? 1 : 2;
      if (op.kind == OpKind::BatchNormDiff && !in[1]->Eq(*in[0])) return bad("BatchNormDiff: gradient shape mismatch");
      for (size_t i = first; i < in.size(); i++)
        if (in[i]->TotalSize() != C)
          return bad("invalid runningMean shape " + in[i]->String() + ". Expected: (" + std::to_string(C) + ")");
      *out = *in[0];
      return Status::OK();
    }
    case OpKind::SoftMaxDiff:
      if (!need(2) || !in[0]->Eq(*in[1])) return bad("SoftMaxDiff needs output and gradient of one shape");
      *out = *in[0];
      return Status::OK();
    case OpKind::Set:
      if (!need(2) || in[0]->TotalSize() != in[1]->TotalSize()) return bad("Set: sizes differ");
      *out = *in[0];
      return Status::OK();
    case OpKind::SolverStep: {
      if (op.fn < 0 || op.fn >= GH_SOLVER__COUNT) return bad("SolverStep: unknown solver");
      // Adam may take one more input: its two bias corrections as a tensor (a new value every step)
      const bool corr = op.fn == GH_SOLVER_ADAM && in.size() == 5;
      if (in.size() != (size_t)(2 + op.fn) && !corr) return bad("SolverStep: weights, grad and the solver's caches expected");
      for (size_t i = 1; i < (size_t)(2 + op.fn); i++)
        if (in[i]->TotalSize() != in[0]->TotalSize()) return bad("SolverStep: sizes differ");
      if (corr && in[4]->TotalSize() != 2) return bad("SolverStep: the bias corrections are two values");
      if (op.fs.size() < 10 || op.ints.empty()) return bad("SolverStep: constants missing");
      *out = *in[0];
      return Status::OK();
    }
    case OpKind::RandUniform: {
      if (in.size() > 1 || (in.size() == 1 && in[0]->TotalSize() != 1)) return bad("RandUniform: at most one counter input");
      if (op.ints.size() < 2) return bad("RandUniform: seed and offset missing");
      Shape s(std::vector<int64_t>(op.ints.begin() + 2, op.ints.end()));
      for (int64_t d : s.d) if (d < 0) return bad("RandUniform: negative dimension");
      *out = s;
      return Status::OK();
    }
    case OpKind::RectifyDiff:
      if (!need(2) || !in[0]->Eq(*in[1]))
        return bad("RectifyDiff: Shape mismatch. Expected " + in[0]->String() + ". Got " + (need(2) ? in[1]->String() : "nothing"));
      *out = *in[0];
      return Status::OK();
    case OpKind::Dropout:
    case OpKind::DropoutDiff:
      if (!need(2) || in[0]->TotalSize() != in[1]->TotalSize()) return bad("Dropout: operand sizes differ");
      if (!(op.f0 >= 0.0 && op.f0 < 1.0)) return bad("Dropout: probability must be in [0, 1)");
      *out = *in[0];
      return Status::OK();
    case OpKind::Reshape: {
      if (!need(1)) return bad("Reshape needs 1 input");
      Shape s(op.ints);
      if (s.TotalSize() != in[0]->TotalSize()) return bad("Reshape: size mismatch " + in[0]->String() + " -> " + s.String());
      *out = s;
      return Status::OK();
    }
  }
  return bad("unknown op");
}

int OverwritesInput(const OpSpec& op) {
  // elementwise ops may overwrite their tensor argument (op_math.go:285-294,
  // 476-481); everything else writes a fresh value
  if (op.kind == OpKind::ElemUnary) return 0;
  if (op.kind == OpKind::ElemBin) return 0;
  if (op.kind == OpKind::RectifyDiff) return 1;   // the gradient is masked in place
  return -1;
}

static uint32_t dtype_flag(Dtype dt) { return GH_FLAG_DTYPE(dt == Dtype::Float64 ? GH_F64 : GH_F32); }

// float64 scalars ride in a dim slot as their bit pattern (gh_cmd.f is float32)
static int64_t double_bits(double v) {
  int64_t b;
  std::memcpy(&b, &v, sizeof(b));
  return b;
}

static std::string op_name(const OpSpec& op) {
  static const char* bins[] = {"add", "sub", "mul", "div", "pow", "lt", "lte", "gt", "gte", "eq", "ne", "mod"};
  switch (op.kind) {
    case OpKind::ElemBin: return std::string("elembin.") + bins[op.fn];
    case OpKind::ElemUnary: return "elemunary." + op.name;
    case OpKind::BroadcastBin: return std::string("broadcast.") + bins[op.fn];
    case OpKind::MatMul:
      return std::string("matmul") + (op.fuse_bias ? "+bias" : "") + (op.fuse_act_relu ? "+rectify" : op.fuse_act_leaky ? "+leakyrelu" : "") +
             (op.fuse_softmax ? "+softmax" : "");
    case OpKind::MatVecMul: return "matvecmul";
    case OpKind::Outer: return "outer";
    case OpKind::BatchedMatMul: return "batchedmatmul";
    case OpKind::Conv2d:
      return std::string(op.fuse_pre ? "conv2d+rectify+maxpool2d+conv2d" : op.fuse_keep ? "conv2d(kept)" : "conv2d") + (op.fuse_bn ? "+batchnorm(eval)" : "") +
             (op.fuse_act_relu ? "+rectify" : op.fuse_act_leaky ? "+leakyrelu" : "") +
             (op.fuse_pool2 ? "+maxpool2d" : "");
    case OpKind::MaxPool2D: return op.relu_input ? "rectify+maxpool2d" : "maxpool2d";
    case OpKind::BatchNorm: return "batchnorm(eval)";
    case OpKind::Rectify: return "rectify";
    case OpKind::LeakyRelu: return "leakyrelu";
    case OpKind::SoftMax: return "softmax";
    case OpKind::Reshape: return "reshape";
    case OpKind::MaxPool2DDiff: return op.relu_input ? "rectify+maxpool2d.diff" : "maxpool2d.diff";
    case OpKind::Conv2dDiffData: return "conv2d.diff.image";
    case OpKind::Conv2dDiffFilter: return "conv2d.diff.filter";
    case OpKind::BatchNormTrain: return "batchnorm(train)";
    case OpKind::BatchNormDiff: return "batchnorm.diff";
    case OpKind::SoftMaxDiff: return "softmax.diff";
    case OpKind::Set: return "set";
    case OpKind::RandUniform: return "rand.uniform";
    case OpKind::Dropout: return "dropout";
    case OpKind::DropoutDiff: return "dropoutDiff";
    case OpKind::RectifyDiff: return "rectifyDiff";
    case OpKind::SolverStep: return op.fn == GH_SOLVER_ADAM ? "solver.adam" : op.fn == GH_SOLVER_RMSPROP ? "solver.rmsprop" : "solver.vanilla";
  }
  return "?";
}

Status CUDADo(Engine& e, const OpSpec& op, Tensor& prealloc, const std::vector<Tensor*>& in) {
  switch (op.kind) {
    case OpKind::ElemBin: {
      Tensor& a = *in[0];
      Tensor& b = *in[1];
      static const char* names[GH_BINFN__COUNT] = {"Add", "Sub", "Mul", "Div", "Pow", "Lt",
                                                   "Lte", "Gt",  "Gte", "ElEq", "ElNe", "Mod"};
      if (op.fn < 0 || op.fn >= GH_BINFN__COUNT) return Status::Err(GH_ENOFUNC, "no binary function " + std::to_string(op.fn));
      const bool as = a.shape.IsScalar(), bs = b.shape.IsScalar();
      if (as != bs) {  // tensor-scalar: the *Scalar methods (operatorPointwise_binary.go:359-426)
        Tensor& t = as ? b : a;
        Tensor& s = as ? a : b;
        FuncOpts o = prealloc.mem == t.mem ? FuncOpts::UseUnsafe() : FuncOpts::WithReuse(&prealloc);
        return e.BinOpScalar(op.fn, names[op.fn], t, s.mem, /*leftTensor=*/!as, o, nullptr);
      }
      FuncOpts o = prealloc.mem == a.mem ? FuncOpts::UseUnsafe() : FuncOpts::WithReuse(&prealloc);
      return e.BinOp(op.fn, names[op.fn], a, b, o, nullptr);
    }
    case OpKind::ElemUnary:
      return e.UnaryTo(op.name, *in[0], prealloc.mem);
    case OpKind::BroadcastBin: {
      const bool left_small = in[0]->shape.TotalSize() < in[1]->shape.TotalSize();
      Tensor& big = left_small ? *in[1] : *in[0];
      Tensor& small = left_small ? *in[0] : *in[1];
      int64_t o, m, i;
      if (!bcast_decompose(big.shape, small.shape, &o, &m, &i)) return bad("cannot broadcast");
      return e.BroadcastBinOp(op.fn, big, small, o, m, i, left_small, prealloc.mem);
    }
    case OpKind::MatMul: {
      // op.transA/transB are applied as transposed views (op_math_cuda.go:210-224)
      Tensor a = *in[0], b = *in[1];
      if (op.transA) { std::swap(a.shape.d[0], a.shape.d[1]); a.transposed = !a.transposed; }
      if (op.transB) { std::swap(b.shape.d[0], b.shape.d[1]); b.transposed = !b.transposed; }
      const int act = op.fuse_act_relu ? 1 : op.fuse_act_leaky ? 2 : 0;
      if (op.fuse_bias && in.size() != 3) return bad("MatMul: fused bias needs a third input");
      return e.MatMul(a, b, prealloc, act, (float)op.f0, op.fuse_softmax, op.fuse_bias ? in[2]->mem : 0);
    }
    case OpKind::MatVecMul: {
      Tensor a = *in[0];
      if (op.transA) { std::swap(a.shape.d[0], a.shape.d[1]); a.transposed = !a.transposed; }
      return e.MatVecMul(a, *in[1], prealloc);
    }
    case OpKind::Outer:
      return e.Outer(*in[0], *in[1], prealloc);
    case OpKind::BatchedMatMul:
      return e.BatchedMatMul(*in[0], *in[1], prealloc, op.transA, op.transB);
    case OpKind::Conv2d: {
      const Tensor& x = *in[0];
      const Tensor& w = *in[1];
      if (x.dt == Dtype::Other || w.dt != x.dt) return bad("Conv2d: Unsupported Dtype");
      if (x.dt == Dtype::Float64 && (op.fuse_bn || op.fuse_act_relu || op.fuse_act_leaky || op.fuse_pool2 || op.fuse_pre))
        return bad("Conv2d: no epilogue operators for float64");
      if (op.fuse_pre && op.fuse_keep) return bad("Conv2d: a folded first layer and a kept result exclude each other");
      const size_t nin = in.size() - (op.fuse_pre || op.fuse_keep ? 1 : 0);   // a folded first layer's filters, or the tensor for the kept result, come last
      gh_cmd c{};
      c.opcode = GH_OP_CONV2D;
      c.flags = (op.fuse_act_relu ? GH_FLAG_ACT_RELU : op.fuse_act_leaky ? GH_FLAG_ACT_LEAKY : 0) | dtype_flag(x.dt);
      c.f[0] = (float)op.f0;
      c.ptr[0] = x.mem; c.ptr[1] = w.mem; c.ptr[2] = prealloc.mem;
      if (op.fuse_bn) {
        if (nin != 4 && nin != 6) return bad("Conv2d: fused BatchNorm needs mean, var[, scale, bias]");
        c.flags |= GH_FLAG_CONV_BN;
        c.ptr[3] = in[2]->mem; c.ptr[4] = in[3]->mem;
        if (nin == 6) {
          c.flags |= GH_FLAG_HAS_GAMMA | GH_FLAG_HAS_BETA;
          c.ptr[5] = in[4]->mem; c.ptr[6] = in[5]->mem;
        }
        c.f[1] = (float)op.f1;
      }
      if (op.fuse_pool2) c.flags |= GH_FLAG_CONV_POOL2;
      for (int i = 0; i < 4; i++) c.dim[i] = x.shape[i];
      if (op.fuse_pre) {
        // x holds the single-channel images; the command's B,C,H,W describe the input that is never stored
        if (nin < 2 || x.shape[1] != 1 || (x.shape[2] & 1) || (x.shape[3] & 1)) return bad("Conv2d: folded first layer needs B x 1 x 2H x 2W images");
        c.flags |= GH_FLAG_CONV_PRE;
        c.ptr[7] = in.back()->mem;
        c.dim[1] = w.shape[1]; c.dim[2] = x.shape[2] / 2; c.dim[3] = x.shape[3] / 2;
      }
      if (op.fuse_keep) {
        if (!op.fuse_pool2 || nin < 2) return bad("Conv2d: a kept result goes with fused pooling");
        c.flags |= GH_FLAG_CONV_KEEP;
        c.ptr[7] = in.back()->mem;
      }
      c.dim[4] = w.shape[0];
      for (int i = 0; i < 8; i++) c.dim[5 + i] = op.ints[(size_t)i];
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::MaxPool2D: {
      const Tensor& x = *in[0];
      if (x.dt == Dtype::Other) return bad("MaxPool2D: Unsupported Dtype");
      const auto& p = op.ints;
      const int64_t np = p[2];
      gh_cmd c{};
      c.opcode = GH_OP_MAXPOOL2D;
      c.flags = (np == 4 ? GH_FLAG_EXPLICIT_PAD : 0) | (op.relu_input ? GH_FLAG_ACT_RELU : 0) | dtype_flag(x.dt);
      c.ptr[0] = x.mem; c.ptr[1] = prealloc.mem;
      for (int i = 0; i < 4; i++) c.dim[i] = x.shape[i];
      c.dim[4] = p[0]; c.dim[5] = p[1];
      if (np == 4) { c.dim[6] = p[3]; c.dim[7] = p[4]; c.dim[8] = p[5]; c.dim[9] = p[6]; }
      else { c.dim[6] = c.dim[7] = p[3]; c.dim[8] = c.dim[9] = p[4]; }
      c.dim[10] = p[3 + np]; c.dim[11] = p[4 + np];
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::BatchNorm: {
      const Tensor& x = *in[0];
      if (x.dt == Dtype::Other) return bad("BatchNorm: Unsupported Dtype");
      for (size_t i = 1; i < in.size(); i++)
        if (in[i]->dt != x.dt) return bad("BatchNorm: statistics and input differ in dtype");
      gh_cmd c{};
      c.opcode = GH_OP_BN_INFER;
      c.flags = dtype_flag(x.dt);
      c.ptr[0] = x.mem; c.ptr[1] = prealloc.mem; c.ptr[2] = in[1]->mem; c.ptr[3] = in[2]->mem;
      if (in.size() == 5) {
        c.flags |= GH_FLAG_HAS_GAMMA | GH_FLAG_HAS_BETA;
        c.ptr[4] = in[3]->mem; c.ptr[5] = in[4]->mem;
      }
      c.dim[3] = double_bits(op.f0);   // epsilon for the float64 kernel
      const int64_t B = x.shape[0], C = x.shape[1];
      c.dim[0] = B; c.dim[1] = C; c.dim[2] = x.shape.TotalSize() / (B * C);
      c.f[0] = (float)op.f0;
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::Rectify:
    case OpKind::LeakyRelu: {
      gh_cmd c{};
      if (in[0]->dt == Dtype::Other) return bad("Unsupported Dtype");
      c.opcode = op.kind == OpKind::Rectify ? GH_OP_RELU : GH_OP_LEAKY_RELU;
      c.flags = dtype_flag(in[0]->dt);
      c.ptr[0] = in[0]->mem; c.ptr[1] = prealloc.mem;
      c.dim[0] = in[0]->DataSize();
      c.dim[1] = double_bits(op.f0);   // alpha for the float64 kernel
      c.f[0] = (float)op.f0;
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::SoftMax: {
      const Tensor& x = *in[0];
      gh_cmd c{};
      if (x.dt == Dtype::Other) return bad("SoftMax: Unsupported Dtype");
      c.opcode = GH_OP_SOFTMAX;
      c.flags = dtype_flag(x.dt);
      c.ptr[0] = x.mem; c.ptr[1] = prealloc.mem;
      const int64_t cols = x.shape[x.shape.Dims() - 1];
      c.dim[0] = x.shape.TotalSize() / cols; c.dim[1] = cols;
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::Reshape:
      return Status::OK();  // metadata only (op_tensor.go:1226-1246)
    case OpKind::MaxPool2DDiff: {
      const Tensor& x = *in[0];
      const auto& p = op.ints;
      const int64_t np = p[2];
      if (x.dt == Dtype::Other || in[1]->dt != x.dt) return bad("MaxPool2DDiff: Unsupported Dtype");
      gh_cmd c{};
      c.opcode = GH_OP_MAXPOOL2D_BWD;
      c.flags = (np == 4 ? GH_FLAG_EXPLICIT_PAD : 0) | (op.relu_input ? GH_FLAG_ACT_RELU : 0) | dtype_flag(x.dt);
      c.ptr[0] = x.mem; c.ptr[1] = in[1]->mem; c.ptr[2] = prealloc.mem;
      for (int i = 0; i < 4; i++) c.dim[i] = x.shape[i];
      c.dim[4] = p[0]; c.dim[5] = p[1];
      if (np == 4) { c.dim[6] = p[3]; c.dim[7] = p[4]; c.dim[8] = p[5]; c.dim[9] = p[6]; }
      else { c.dim[6] = c.dim[7] = p[3]; c.dim[8] = c.dim[9] = p[4]; }
      c.dim[10] = p[3 + np]; c.dim[11] = p[4 + np];
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::Conv2dDiffData:
    case OpKind::Conv2dDiffFilter: {
      const bool data = op.kind == OpKind::Conv2dDiffData;
      if (in[0]->dt == Dtype::Other || in[1]->dt != in[0]->dt) return bad("Conv2d gradients: Unsupported Dtype");
      gh_cmd c{};
      c.opcode = data ? GH_OP_CONV2D_BWD_DATA : GH_OP_CONV2D_BWD_FILTER;
      c.flags = dtype_flag(in[0]->dt);
      c.ptr[0] = in[0]->mem; c.ptr[1] = in[1]->mem; c.ptr[2] = prealloc.mem;
      const Shape& xs = data ? prealloc.shape : in[0]->shape;
      for (int i = 0; i < 4; i++) c.dim[i] = xs[i];
      c.dim[4] = data ? in[1]->shape[0] : prealloc.shape[0];
      for (int i = 0; i < 8; i++) c.dim[5 + i] = op.ints[(size_t)i];
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::BatchNormTrain:
    case OpKind::BatchNormDiff: {
      const Tensor& x = *in[0];
      if (x.dt == Dtype::Other) return bad("BatchNorm: Unsupported Dtype");
      for (size_t i = 1; i < in.size(); i++)
        if (in[i]->dt != x.dt) return bad("BatchNorm: Unsupported Dtype");
      gh_cmd c{};
      const int64_t B = x.shape[0], C = x.shape[1];
      c.flags = dtype_flag(x.dt);
      c.dim[0] = B; c.dim[1] = C; c.dim[2] = x.shape.TotalSize() / (B * C);
      c.f[0] = (float)op.f0;
      c.dim[3] = double_bits(op.f0);   // float64: epsilon (and momentum below) as doubles
      if (op.kind == OpKind::BatchNormTrain) {
        c.opcode = GH_OP_BN_TRAIN;
        c.ptr[0] = x.mem; c.ptr[1] = prealloc.mem;
        for (int i = 0; i < 4; i++) c.ptr[2 + i] = in[(size_t)(1 + i)]->mem;
        c.f[1] = (float)op.f1;
        c.dim[4] = double_bits(op.f1);
      } else {
        c.opcode = GH_OP_BN_BWD;
        c.ptr[0] = x.mem; c.ptr[1] = in[1]->mem; c.ptr[2] = prealloc.mem;
        c.ptr[3] = in[2]->mem; c.ptr[4] = in[3]->mem;
      }
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::SoftMaxDiff: {
      const Tensor& y = *in[0];
      if (y.dt == Dtype::Other || in[1]->dt != y.dt) return bad("SoftMaxDiff: Unsupported Dtype");
      gh_cmd c{};
      c.opcode = GH_OP_SOFTMAX_BWD;
      c.flags = dtype_flag(y.dt);
      c.ptr[0] = y.mem; c.ptr[1] = in[1]->mem; c.ptr[2] = prealloc.mem;
      const int64_t cols = y.shape[y.shape.Dims() - 1];
      c.dim[0] = y.shape.TotalSize() / cols; c.dim[1] = cols;
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::SolverStep: {
      gh_cmd c{};
      c.opcode = GH_OP_SOLVER_STEP;
      for (size_t i = 0; i < in.size(); i++)
        if (in[i]->dt == Dtype::Other || in[i]->dt != in[0]->dt) return bad("SolverStep: Unsupported Dtype");
      c.flags = GH_FLAG_FN(op.fn) | GH_FLAG_MODE(op.ints[0]) | dtype_flag(in[0]->dt);
      for (size_t i = 0; i < in.size(); i++) c.ptr[i] = in[i]->mem;   // Adam: in[4] = bias corrections in memory
      c.dim[0] = in[0]->DataSize();
      for (int i = 0; i < 10; i++) c.f[i] = (float)op.fs[(size_t)i];
      if (in[0]->dt == Dtype::Float64)   // float64 tensors take the constants as doubles
        for (int i = 0; i < 10; i++) c.dim[1 + i] = double_bits(op.fs[(size_t)i]);
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::RandUniform: {
      if (!in.empty() && in[0]->dt != Dtype::Float64) return bad("RandUniform: the counter must be an 8-byte scalar");
      gh_cmd c{};
      c.opcode = GH_OP_RAND_UNIFORM;
      c.ptr[0] = prealloc.mem;
      c.ptr[1] = in.empty() ? 0 : in[0]->mem;
      c.dim[0] = prealloc.shape.TotalSize(); c.dim[1] = op.ints[0]; c.dim[2] = op.ints[1];
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::RectifyDiff: {
      if (in[0]->dt == Dtype::Other || in[1]->dt != in[0]->dt) return bad("RectifyDiff: Unsupported Dtype");
      gh_cmd c{};
      c.opcode = GH_OP_RELU_BWD;
      c.flags = dtype_flag(in[0]->dt);
      c.ptr[0] = in[0]->mem; c.ptr[1] = in[1]->mem; c.ptr[2] = prealloc.mem;
      c.dim[0] = in[0]->shape.TotalSize();
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::Dropout:
    case OpKind::DropoutDiff: {
      if (in[0]->dt == Dtype::Other || in[1]->dt != in[0]->dt) return bad("Dropout: Unsupported Dtype");
      gh_cmd c{};
      c.opcode = op.kind == OpKind::Dropout ? GH_OP_DROPOUT : GH_OP_DROPOUT_BWD;
      c.flags = dtype_flag(in[0]->dt);
      c.dim[1] = double_bits(op.f0);
      if (op.kind == OpKind::Dropout) {
        if (!op.fn) c.flags |= GH_FLAG_BN_EVAL;
        c.ptr[0] = in[0]->mem; c.ptr[1] = prealloc.mem; c.ptr[2] = in[1]->mem;
      } else {
        c.ptr[0] = in[0]->mem; c.ptr[1] = in[1]->mem; c.ptr[2] = prealloc.mem;
      }
      c.dim[0] = in[0]->shape.TotalSize();
      c.f[0] = (float)op.f0;
      e.Enqueue(c);
      return Status::OK();
    }
    case OpKind::Set: {
      // prealloc is a's register (the node aliases a); copy b's bytes into it
      const int64_t bytes = in[1]->DataSize() * dtype_size(in[1]->dt);
      e.RecordCopy(prealloc.mem, in[1]->mem, bytes);
      return Status::OK();
    }
  }
  return bad("unknown op");
}

// ---- Graph ------------------------------------------------------------------------

int Graph::NewTensor(const Shape& s, Dtype dt, const void* host, bool resident) {
  Node n;
  n.id = (int)nodes_.size();
  n.shape = s; n.dt = dt; n.is_input = true; n.host = host; n.resident = resident;
  nodes_.push_back(n);
  return n.id;
}

Status Graph::Apply(const OpSpec& op, const std::vector<int>& inputs, int* out) {
  // an operator the engine has no function for is refused here, before any
  // table is indexed with it (the reference's HasFunc check, op_math_cuda.go:34-36)
  if ((int)op.kind < 0 || (int)op.kind > (int)OpKind::RectifyDiff)
    return Status::Err(GH_ENOFUNC, "Apply: no operator of kind " + std::to_string((int)op.kind));
  if ((op.kind == OpKind::ElemBin || op.kind == OpKind::BroadcastBin) && (op.fn < 0 || op.fn >= GH_BINFN__COUNT))
    return Status::Err(GH_ENOFUNC, "Apply: no binary function " + std::to_string(op.fn));
  if (op.kind == OpKind::SolverStep && (op.fn < 0 || op.fn >= GH_SOLVER__COUNT))
    return Status::Err(GH_ENOFUNC, "Apply: no solver " + std::to_string(op.fn));
  std::vector<const Shape*> shapes;
  for (int i : inputs) {
    if (i < 0 || i >= (int)nodes_.size()) return bad("Apply: unknown input node");
    shapes.push_back(&nodes_[(size_t)i].shape);
  }
  // the reference's type inference refuses operands of different Dtypes when the graph is built
  // ("Unification Fail: Float64 ~ Float32 cannot be unified"); so does this
  switch (op.kind) {
    case OpKind::ElemBin: case OpKind::BroadcastBin: case OpKind::MatMul: case OpKind::MatVecMul: case OpKind::Outer:
    case OpKind::BatchedMatMul: case OpKind::Conv2d: case OpKind::BatchNorm:
      for (size_t i = 1; i < inputs.size(); i++)
        if (nodes_[(size_t)inputs[i]].dt != nodes_[(size_t)inputs[0]].dt)
          return bad("Apply: operands of different Dtypes cannot be unified (input 0 and input " + std::to_string(i) + ")");
      break;
    default: break;
  }
  Node n;
  Status st = InferShape(op, shapes, &n.shape);
  if (!st.ok()) return st;
  n.id = (int)nodes_.size();
  n.dt = inputs.empty() || op.kind == OpKind::RandUniform ? Dtype::Float32 : nodes_[(size_t)inputs[0]].dt;
  n.op = op;
  n.inputs = inputs;
  if (op.kind == OpKind::Reshape || op.kind == OpKind::Set || op.kind == OpKind::SolverStep) n.alias_of = inputs[0];
  nodes_.push_back(n);
  if (out) *out = n.id;
  return Status::OK();
}

Status Graph::Let(int node, const void* host) {
  if (node < 0 || node >= (int)nodes_.size() || !nodes_[(size_t)node].is_input) return bad("Let: not an input node");
  nodes_[(size_t)node].host = host;
  nodes_[(size_t)node].host_borrowed = false;
  return Status::OK();
}

Status Graph::LetBorrowed(int node) {
  static const char marker = 0;   // host only has to be non-null: nothing is ever read through it
  if (node < 0 || node >= (int)nodes_.size() || !nodes_[(size_t)node].is_input) return bad("LetBorrowed: not an input node");
  nodes_[(size_t)node].host = &marker;
  nodes_[(size_t)node].host_borrowed = true;
  return Status::OK();
}

Status Graph::Read(int node, void* host_out) {
  if (node < 0 || node >= (int)nodes_.size()) return bad("Read: unknown node");
  Node& n = nodes_[(size_t)node];
  if (n.read_into && host_out != n.read_into) {   // a node may be read more than once (gorgonia.Read makes a readOp node per call, gorgonia.go:311-318)
    if (n.read_borrowed) return bad("Read: the node's value is lent out (ReadBorrowed)");
    n.read_also.push_back(host_out);
    return Status::OK();
  }
  n.read_into = host_out;
  n.read_borrowed = false;
  return Status::OK();
}

Status Graph::ReadBorrowed(int node) {
  static char marker;   // read_into only has to be non-null: nothing is ever copied there
  if (node < 0 || node >= (int)nodes_.size()) return bad("ReadBorrowed: unknown node");
  Node& n = nodes_[(size_t)node];
  if (n.read_into && !n.read_borrowed) return bad("ReadBorrowed: the node already has a Read");
  n.read_into = &marker;
  n.read_borrowed = true;
  return Status::OK();
}

int Graph::FuseActivations() {
  int fused = 0;
  std::vector<int> uses(nodes_.size(), 0);
  for (auto& n : nodes_) for (int i : n.inputs) uses[(size_t)i]++;
  for (auto& n : nodes_) {
    if (n.is_input || n.fused_away || n.inputs.empty()) continue;
    const OpKind k = n.op.kind;
    if (k != OpKind::Rectify && k != OpKind::LeakyRelu && k != OpKind::BatchNorm && k != OpKind::MaxPool2D &&
        k != OpKind::SoftMax && !(k == OpKind::BroadcastBin && n.op.fn == GH_ADD))
      continue;
    // the producer: the first input, or for a broadcast add whichever input is the product
    int pi = n.inputs[0];
    if (k == OpKind::BroadcastBin && n.inputs.size() == 2 && nodes_[(size_t)n.inputs[1]].op.kind == OpKind::MatMul &&
        !nodes_[(size_t)n.inputs[1]].is_input)
      pi = n.inputs[1];
    Node& p = nodes_[(size_t)pi];
    if (p.is_input || p.fused_away || p.read_into || uses[(size_t)p.id] != 1) continue;
    if (p.op.kind != OpKind::Conv2d && p.op.kind != OpKind::MatMul) continue;
    if (p.dt != Dtype::Float32) continue;   // the epilogues exist for float32 only
    OpSpec op = p.op;
    std::vector<int> inputs = p.inputs;
    const bool has_act = op.fuse_act_relu || op.fuse_act_leaky;
    if (op.fuse_softmax) continue;   // nothing rides behind a softmax
    if (k == OpKind::BroadcastBin) {
      // Add(Mul(x, w), b) with b one value per column: a + b and b + a are the same bits
      if (op.kind != OpKind::MatMul || has_act || op.fuse_bias || n.inputs.size() != 2 || n.shape.Dims() != 2) continue;
      if (op.transA || op.transB) continue;   // the bias epilogue exists for untransposed products
      const Node& small = nodes_[(size_t)(pi == n.inputs[0] ? n.inputs[1] : n.inputs[0])];
      if (small.dt != Dtype::Float32 || small.shape.Dims() != 2 || small.shape[0] != 1 || small.shape[1] != n.shape[1] ||
          n.shape[0] == 1)
        continue;
      op.fuse_bias = true;
      inputs.push_back(small.id);
    } else if (k == OpKind::SoftMax) {
      if (op.kind != OpKind::MatMul || op.transA || op.transB || n.shape.Dims() != 2) continue;
      gh_cmd c{};
      c.opcode = GH_OP_GEMM;
      c.flags = GH_FLAG_DTYPE(p.dt == Dtype::Float64 ? GH_F64 : GH_F32);
      c.dim[0] = n.shape[0]; c.dim[1] = n.shape[1]; c.dim[2] = nodes_[(size_t)inputs[0]].shape[1];
      c.dim[6] = 1;
      if (!gh_gemm_can_softmax(&c)) continue;
      op.fuse_softmax = true;
    } else if (k == OpKind::BatchNorm) {
      if (op.kind != OpKind::Conv2d || op.fuse_bn || has_act || op.fuse_pool2) continue;
      if (n.shape.Dims() != 4) continue;
      op.fuse_bn = true;
      op.f1 = n.op.f0;
      for (size_t i = 1; i < n.inputs.size(); i++) inputs.push_back(n.inputs[i]);
    } else if (k == OpKind::Rectify || k == OpKind::LeakyRelu) {
      if (has_act || op.fuse_pool2) continue;
      if (k == OpKind::Rectify) op.fuse_act_relu = true;
      else { op.fuse_act_leaky = true; op.f0 = n.op.f0; }
    } else {  // MaxPool2D: 2x2 window, stride 2, no padding, and a kernel that can take it
      if (op.kind != OpKind::Conv2d || op.fuse_pool2) continue;
      const auto& q = n.op.ints;  // kh kw npad pads... sh sw
      bool plain = q.size() >= 5 && q[0] == 2 && q[1] == 2;
      for (size_t i = 3; plain && i < q.size(); i++) plain = q[i] == (i >= 3 + (size_t)q[2] ? 2 : 0);
      if (!plain) continue;
      const Shape& xs = nodes_[(size_t)inputs[0]].shape;
      const Shape& ws = nodes_[(size_t)inputs[1]].shape;
      gh_cmd c{};
      c.opcode = GH_OP_CONV2D;
      for (int i = 0; i < 4; i++) c.dim[i] = xs[i];
      c.dim[4] = ws[0];
      for (int i = 0; i < 8; i++) c.dim[5 + i] = op.ints[(size_t)i];
      if (!gh_conv2d_can_pool(&c)) continue;
      op.fuse_pool2 = true;
    }
    n.op = op;
    n.inputs = inputs;
    p.fused_away = true;
    fused++;
  }
  fused += fuse_rectify_into_pool();
  fused += fuse_pooled_rectify();
  fused += fuse_first_layer();
  fused += fuse_kept_conv();
  return fused;
}

// z = Conv2d(x, w); p = MaxPool2D(z) 2x2/2 (read through a Rectify or not) where other nodes read z as well -
// a training graph, whose backward pass needs the unpooled values - and the library's kernel for the shape
// can store both (gh_conv2d_can_keep): p takes over the convolution, with z as its last input, the tensor the
// unpooled values go to; z keeps its register and loses its instruction.  Nothing may read z between the two.
int Graph::fuse_kept_conv() {
  int fused = 0;
  for (auto& pn : nodes_) {
    if (pn.is_input || pn.fused_away || pn.deferred || pn.op.kind != OpKind::MaxPool2D || pn.inputs.size() != 1) continue;
    if (pn.dt != Dtype::Float32 || pn.shape.Dims() != 4) continue;
    const auto& q = pn.op.ints;  // kh kw npad pads... sh sw
    bool plain = q.size() >= 5 && q[0] == 2 && q[1] == 2;
    for (size_t i = 3; plain && i < q.size(); i++) plain = q[i] == (i >= 3 + (size_t)q[2] ? 2 : 0);
    if (!plain) continue;
    Node& z = nodes_[(size_t)pn.inputs[0]];
    if (z.is_input || z.fused_away || z.deferred || z.alias_of >= 0 || z.op.kind != OpKind::Conv2d || z.inputs.size() != 2) continue;
    const OpSpec& zo = z.op;
    if (zo.fuse_bn || zo.fuse_act_relu || zo.fuse_act_leaky || zo.fuse_pool2 || zo.fuse_pre || zo.fuse_keep) continue;
    if (z.dt != Dtype::Float32 || z.id >= pn.id) continue;
    bool read_between = false;
    for (int j = z.id + 1; j < pn.id && !read_between; j++) {
      const Node& o = nodes_[(size_t)j];
      if (o.fused_away) continue;
      for (int in : o.inputs) if (in == z.id || nodes_[(size_t)in].alias_of == z.id) read_between = true;
    }
    if (read_between) continue;
    const Shape& xs = nodes_[(size_t)z.inputs[0]].shape;
    const Shape& ws = nodes_[(size_t)z.inputs[1]].shape;
    gh_cmd c{};
    c.opcode = GH_OP_CONV2D;
    for (int i = 0; i < 4; i++) c.dim[i] = xs[i];
    c.dim[4] = ws[0];
    for (int i = 0; i < 8; i++) c.dim[5 + i] = zo.ints[(size_t)i];
    if (!gh_conv2d_can_pool(&c) || !gh_conv2d_can_keep(&c)) continue;
    OpSpec op = zo;
    op.fuse_pool2 = true;
    op.fuse_keep = true;
    op.fuse_act_relu = pn.op.relu_input;
    pn.op = op;
    pn.inputs = {z.inputs[0], z.inputs[1], z.id};
    z.deferred = true;
    fused++;
  }
  return fused;
}

// p = MaxPool2D(Rectify(z)) where nothing else reads the activation and no producer took it into an epilogue
// (a float64 convolution has none): the pool reads z through the activation, whose result is never stored.
// The pooled values are those of the two operators: the same scan over the same x * (x >= 0).
int Graph::fuse_rectify_into_pool() {
  int fused = 0;
  std::vector<int> uses(nodes_.size(), 0);
  for (auto& n : nodes_)
    if (!n.fused_away) for (int i : n.inputs) uses[(size_t)i]++;
  for (auto& pn : nodes_) {
    if (pn.is_input || pn.fused_away || pn.op.kind != OpKind::MaxPool2D || pn.inputs.size() != 1 || pn.op.relu_input) continue;
    Node& a = nodes_[(size_t)pn.inputs[0]];
    if (a.is_input || a.fused_away || a.deferred || a.read_into || a.alias_of >= 0 || uses[(size_t)a.id] != 1) continue;
    if (a.op.kind != OpKind::Rectify || a.inputs.size() != 1) continue;
    if (a.dt != Dtype::Float32 && a.dt != Dtype::Float64) continue;
    pn.inputs[0] = a.inputs[0];
    pn.op.relu_input = true;
    a.fused_away = true;
    fused++;
  }
  return fused;
}

// conv(conv+rectify+pool(x0, w0), w1, ...) where the inner node is a single-channel 3x3 / pad 1 / stride 1
// convolution with Rectify and the 2x2 pool already in its epilogue, read by nothing but the outer convolution,
// and the library folds the pair (gh_conv2d_can_pre): the outer node takes x0 as input 0 and w0 as its last
// input; the tensor between the two layers is never stored.
int Graph::fuse_first_layer() {
  int fused = 0;
  std::vector<int> uses(nodes_.size(), 0);
  for (auto& n : nodes_)
    if (!n.fused_away) for (int i : n.inputs) uses[(size_t)i]++;
  for (auto& n : nodes_) {
    if (n.is_input || n.fused_away || n.op.kind != OpKind::Conv2d || n.op.fuse_pre || n.inputs.size() < 2) continue;
    if (n.dt != Dtype::Float32) continue;
    Node& p = nodes_[(size_t)n.inputs[0]];
    if (p.is_input || p.fused_away || p.read_into || uses[(size_t)p.id] != 1 || p.op.kind != OpKind::Conv2d) continue;
    const OpSpec& q = p.op;
    if (!q.fuse_act_relu || !q.fuse_pool2 || q.fuse_bn || q.fuse_act_leaky || q.fuse_pre || p.inputs.size() != 2) continue;
    static const int64_t first[8] = {3, 3, 1, 1, 1, 1, 1, 1};   // kernel, pad, stride, dilation
    bool plain = q.ints.size() >= 8;
    for (size_t i = 0; plain && i < 8; i++) plain = q.ints[i] == first[i];
    if (!plain) continue;
    const Shape& x0 = nodes_[(size_t)p.inputs[0]].shape;
    const Shape& ws = nodes_[(size_t)n.inputs[1]].shape;
    if (x0.Dims() != 4 || x0[1] != 1 || (x0[2] & 1) || (x0[3] & 1) || p.shape.Dims() != 4 || ws.Dims() != 4) continue;
    if (p.shape[2] != x0[2] / 2 || p.shape[3] != x0[3] / 2 || ws[1] != p.shape[1]) continue;
    gh_cmd c{};
    c.opcode = GH_OP_CONV2D;
    for (int i = 0; i < 4; i++) c.dim[i] = p.shape[i];
    c.dim[4] = ws[0];
    for (int i = 0; i < 8; i++) c.dim[5 + i] = n.op.ints[(size_t)i];
    if (!gh_conv2d_can_pre(&c)) continue;
    n.op.fuse_pre = true;
    n.inputs[0] = p.inputs[0];
    n.inputs.push_back(p.inputs[1]);
    p.fused_away = true;
    fused++;
  }
  return fused;
}

// The training pattern around a pooled activation:
//   a = Rectify(z); p = MaxPool2D(a); ...; da = MaxPool2DDiff(a, g); dz = RectifyDiff(z, da)
// with a read by nothing but the pool and its gradient, and da by nothing but dz.  The pool then
// reads z through the activation, and dz becomes one operator that scans the windows over
// z * (z >= 0) and masks the result with (z >= 0): a and da are never stored, and every value
// that is stored has the bits the four operators would have given it.
int Graph::fuse_pooled_rectify() {
  int fused = 0;
  const size_t N = nodes_.size();
  std::vector<std::vector<int>> users(N);
  for (auto& n : nodes_)
    if (!n.fused_away)
      for (int i : n.inputs) users[(size_t)i].push_back(n.id);
  for (auto& a : nodes_) {
    if (a.fused_away || a.is_input || a.read_into || a.op.kind != OpKind::Rectify || a.dt != Dtype::Float32) continue;
    if (a.inputs.size() != 1 || users[(size_t)a.id].size() != 2) continue;
    const int z = a.inputs[0];
    Node* pool = nullptr;
    Node* diff = nullptr;
    for (int u : users[(size_t)a.id]) {
      Node& n = nodes_[(size_t)u];
      if (n.op.kind == OpKind::MaxPool2D && n.inputs.size() == 1 && !n.op.relu_input) pool = &n;
      if (n.op.kind == OpKind::MaxPool2DDiff && n.inputs.size() == 2 && n.inputs[0] == a.id && n.inputs[1] != a.id &&
          !n.op.relu_input)
        diff = &n;
    }
    if (!pool || !diff || diff->read_into || diff->op.ints != pool->op.ints) continue;
    if (users[(size_t)diff->id].size() != 1) continue;
    Node& dz = nodes_[(size_t)users[(size_t)diff->id][0]];
    if (dz.op.kind != OpKind::RectifyDiff || dz.inputs.size() != 2 || dz.inputs[0] != z || dz.inputs[1] != diff->id) continue;
    if (nodes_[(size_t)z].dt != Dtype::Float32 || nodes_[(size_t)z].fused_away) continue;
    pool->op.relu_input = true;
    pool->inputs[0] = z;
    dz.op = diff->op;
    dz.op.relu_input = true;
    dz.inputs = {z, diff->inputs[1]};
    a.fused_away = true;
    diff->fused_away = true;
    fused += 2;
  }
  return fused;
}

// ---- TapeMachine --------------------------------------------------------------------

TapeMachine::~TapeMachine() { Close(); }

Status TapeMachine::Compile() {
  auto& nodes = g_->Nodes();
  const int N = (int)nodes.size();
  prog_.clear();
  auto bytes_of = [&](const Node& n) {
    return (n.shape.IsScalar() ? 1 : n.shape.TotalSize()) * dtype_size(n.dt);
  };
  // root value of a node: aliases (Reshape, fused activations) are views of it
  std::vector<int> root((size_t)N);
  for (int i = 0; i < N; i++) root[(size_t)i] = nodes[(size_t)i].alias_of >= 0 ? root[(size_t)nodes[(size_t)i].alias_of] : i;
  // last instruction that reads each root value
  std::vector<int> last_reader((size_t)N, -1);
  for (int i = 0; i < N; i++) {
    if (nodes[(size_t)i].fused_away) continue;  // its inputs are read by the node that absorbed it
    for (int in : nodes[(size_t)i].inputs) last_reader[(size_t)root[(size_t)in]] = i;
  }
  std::vector<char> value_kept((size_t)N, 0);  // read by the host, or a resident input
  for (int i = 0; i < N; i++)
    if (nodes[(size_t)i].read_into || (nodes[(size_t)i].is_input && nodes[(size_t)i].resident))
      value_kept[(size_t)root[(size_t)i]] = 1;

  // registers: a node that overwrites a dead input takes over that input's
  // register (regalloc.go:211-243); every other node gets a fresh one
  node_reg_.assign((size_t)N, -1);
  std::vector<char> inplace((size_t)N, 0);
  int nreg = 0;
  for (int i = 0; i < N; i++) {
    Node& n = nodes[(size_t)i];
    if (n.fused_away) continue;
    if (n.alias_of >= 0) { node_reg_[(size_t)i] = node_reg_[(size_t)root[(size_t)i]]; continue; }
    const int ow = n.is_input || opt_.node_at_a_time ? -1 : OverwritesInput(n.op);
    if (ow >= 0 && ow < (int)n.inputs.size()) {
      int src = n.inputs[(size_t)ow];
      if (n.op.kind == OpKind::ElemBin && n.inputs.size() == 2 && nodes[(size_t)src].shape.IsScalar())
        src = n.inputs[1];  // scalar (op) tensor: the tensor operand is the one overwritten
      const int rs = root[(size_t)src];
      if (last_reader[(size_t)rs] == i && !value_kept[(size_t)rs] && bytes_of(nodes[(size_t)src]) == bytes_of(n)) {
        node_reg_[(size_t)i] = node_reg_[(size_t)rs];
        inplace[(size_t)i] = 1;
        continue;
      }
    }
    node_reg_[(size_t)i] = nreg++;
  }
  // register liveness: last instruction touching any value held in it
  std::vector<int> reg_last((size_t)nreg, -1);
  std::vector<char> reg_kept((size_t)nreg, 0);
  for (int i = 0; i < N; i++) {
    const int r = node_reg_[(size_t)i];
    if (r < 0) continue;
    reg_last[(size_t)r] = std::max(reg_last[(size_t)r], std::max(i, last_reader[(size_t)root[(size_t)i]]));
    if (value_kept[(size_t)root[(size_t)i]]) reg_kept[(size_t)r] = 1;
  }
  // A small result that only the host reads is written by its kernel straight
  // into pinned host memory: no arena register, no staging copy at the end of
  // the segment.
  std::vector<char> host_out((size_t)N, 0);
  for (int i = 0; i < N; i++) {
    const Node& n = nodes[(size_t)i];
    if (!n.read_into || n.is_input || n.fused_away || n.alias_of >= 0 || inplace[(size_t)i]) continue;
    if ((bytes_of(n) > kStageLimit && !n.read_borrowed) || bytes_of(n) % 4 != 0 || last_reader[(size_t)i] >= 0) continue;
    bool shared = false;
    for (int j = 0; j < N; j++)
      if (j != i && (root[(size_t)j] == i || node_reg_[(size_t)j] == node_reg_[(size_t)i])) shared = true;
    if (!shared) host_out[(size_t)i] = 1;
  }
  regs_.assign((size_t)nreg, Tensor());
  reg_live_.assign((size_t)nreg, 0);
  resident_done_.assign((size_t)N, 0);
  reg_bytes_.assign((size_t)nreg, 0);
  std::vector<int64_t>& reg_bytes = reg_bytes_;
  gpumem_ = 0;

  // Inputs first, operators after: every upload sits at the head of the program
  // (the reference interleaves them, compile.go:16-60; the values an operator
  // sees are the same), so the operators of a run form one uninterrupted segment.
  for (int pass = 0; pass < 2; pass++)
  for (int i = 0; i < N; i++) {
    Node& n = nodes[(size_t)i];
    if (n.fused_away) continue;
    if ((pass == 0) != (n.is_input && n.alias_of < 0)) continue;
    if (n.alias_of >= 0 && n.op.kind != OpKind::Set && n.op.kind != OpKind::SolverStep) continue;  // a view: nothing to run
    const int r = node_reg_[(size_t)i];
    const int64_t bytes = bytes_of(n);
    if (n.alias_of >= 0) {
      // Set and SolverStep write into the register they alias
      prog_.push_back({InstrKind::ExecOp, i, r, bytes, true});
    } else if (n.is_input) {
      prog_.push_back({InstrKind::LoadArg, i, r, bytes, false});
      prog_.push_back({InstrKind::Alloc, i, r, bytes, false});
      prog_.push_back({InstrKind::Transport, i, r, bytes, false});
      reg_bytes[(size_t)r] = bytes;
      gpumem_ += bytes;
    } else {
      if (host_out[(size_t)i]) {
        prog_.push_back({InstrKind::AllocHost, i, r, bytes, false});
      } else if (!inplace[(size_t)i]) {
        prog_.push_back({InstrKind::Alloc, i, r, bytes, false});
        reg_bytes[(size_t)r] = bytes;
        gpumem_ += bytes;
      }
      if (!n.deferred) prog_.push_back({InstrKind::ExecOp, i, r, bytes, inplace[(size_t)i] != 0});
    }
    // registers whose last use is this instruction die here
    for (int q = 0; q < nreg; q++)
      if (reg_last[(size_t)q] == i && !reg_kept[(size_t)q] && reg_bytes[(size_t)q] > 0)
        prog_.push_back({InstrKind::Free, i, q, reg_bytes[(size_t)q], false});
  }
  // host reads: one flush, then the copies (compile.go:437-462 puts a flush in
  // front of every consumer that needs a finished value)
  for (int i = 0; i < N; i++)
    if (nodes[(size_t)i].read_into && !host_out[(size_t)i] &&
        (bytes_of(nodes[(size_t)i]) <= kStageLimit || nodes[(size_t)i].read_borrowed) && bytes_of(nodes[(size_t)i]) % 4 == 0)
      prog_.push_back({InstrKind::StageOut, i, node_reg_[(size_t)i], bytes_of(nodes[(size_t)i]), false});
  prog_.push_back({InstrKind::Flush, -1, -1, 0, false});
  std::vector<int> freed;
  for (int i = 0; i < N; i++)
    if (nodes[(size_t)i].read_into)
      prog_.push_back({InstrKind::Read, i, node_reg_[(size_t)i], bytes_of(nodes[(size_t)i]), false});
  for (int i = 0; i < N; i++) {
    Node& n = nodes[(size_t)i];
    const int r = node_reg_[(size_t)i];
    if (!n.read_into || host_out[(size_t)i]) continue;
    bool resident_reg = false;
    for (int j = 0; j < N; j++)
      if (node_reg_[(size_t)j] == r && nodes[(size_t)j].is_input && nodes[(size_t)j].resident) resident_reg = true;
    if (resident_reg || std::find(freed.begin(), freed.end(), r) != freed.end()) continue;
    prog_.push_back({InstrKind::Free, i, r, reg_bytes[(size_t)r], false});
    freed.push_back(r);
  }
  return Status::OK();
}

Status TapeMachine::Init(int device) {
  Status st = Compile();
  if (!st.ok()) return st;
  // every register is 32-byte aligned in the arena: size the reservation on
  // aligned sizes so that "2.5x the program's need" still holds for many small
  // tensors (the reference sums raw sizes, compile.go:148-216)
  int64_t need = 0;
  for (auto& in : prog_)
    if (in.kind == InstrKind::Alloc) need += (in.size + 31) / 32 * 32;
  if (borrowed_) {
    if (!eng_.Initialized()) return Status::Err(GH_ESTATE, "WithEngine: the engine is not initialised");
    int64_t room = 0;
    for (auto& hole : eng_.Allocator().freelist()) room += hole.second;
    if (need > room)
      return Status::Err(GH_EOOM, "WithEngine: the program needs " + std::to_string(need) +
                                      " bytes of registers, the engine's arena has " + std::to_string(room) + " free");
  } else {
    st = eng_.Init(device, need > gpumem_ ? need : gpumem_);
    if (!st.ok()) return st;
  }
  open_ = true;
  stage_.assign(g_->Nodes().size(), nullptr);
  stage_in_.assign(g_->Nodes().size(), nullptr);
  int64_t staged_in = 0;
  for (auto& in : prog_) {
    if (in.kind == InstrKind::StageOut || in.kind == InstrKind::AllocHost) {
      st = eng_.HostAlloc(in.size, &stage_[(size_t)in.node]);
      if (!st.ok()) return st;
    }
    // an input uploaded on every run goes through a pinned buffer of its own
    // (RunAll waits for the device before it returns, so one buffer per input
    // is the whole ring); inputs past the cap fall back to a direct copy
    if (in.kind == InstrKind::Transport) {
      const Node& n = g_->Nodes()[(size_t)in.node];
      if (n.host_borrowed) {   // the caller fills this buffer itself: it exists whatever the size
        if (in.size % 4 != 0)
          return Status::Err(GH_EINVAL, "LetBorrowed: input node " + std::to_string(in.node) + " is not a multiple of 4 bytes");
        st = eng_.HostAlloc(in.size, &stage_in_[(size_t)in.node]);
        if (!st.ok()) return st;
        continue;
      }
      if ((n.resident && !opt_.reupload_resident) || in.size % 4 != 0 || in.size > kStageInLimit ||
          staged_in + in.size > kStageInTotal)
        continue;
      st = eng_.HostAlloc(in.size, &stage_in_[(size_t)in.node]);
      if (!st.ok()) return st;
      staged_in += in.size;
    }
  }
  return Status::OK();
}

void* TapeMachine::InputBuffer(int node) const {
  if (node < 0 || node >= (int)stage_in_.size() || !g_->Nodes()[(size_t)node].host_borrowed) return nullptr;
  return stage_in_[(size_t)node];
}

const void* TapeMachine::ReadBuffer(int node) const {
  if (node < 0 || node >= (int)stage_.size() || !g_->Nodes()[(size_t)node].read_borrowed) return nullptr;
  return stage_[(size_t)node];
}

uint64_t TapeMachine::RegisterAddress(int node) const {
  if (node < 0 || node >= (int)node_reg_.size() || node_reg_[(size_t)node] < 0) return 0;
  return regs_[(size_t)node_reg_[(size_t)node]].mem;
}

static inline int64_t now_ns() {
  return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

Status TapeMachine::flush() {
  segments_++;
  // launch, then wait, with the host time of each kept for PhaseNs()
  auto launch_and_wait = [&](auto&& launch) -> Status {
    const int64_t t0 = now_ns();
    Status st = launch();
    const int64_t t1 = now_ns();
    ns_launch_ += t1 - t0;
    if (!st.ok()) return st;
    st = eng_.Sync();
    ns_wait_ += now_ns() - t1;
    return st;
  };
  auto eager = [&]() { return launch_and_wait([&]() { return eng_.SubmitPending(); }); };
  if (!opt_.graph_replay || opt_.watch_nan || opt_.watch_inf) return eager();
  const size_t idx = (size_t)seg_index_++;
  if (seg_cache_.size() <= idx) seg_cache_.resize(idx + 1);
  SegCache& sc = seg_cache_[idx];
  const std::vector<gh_cmd>& cur = eng_.Segment();
  const bool same = sc.cmds.size() == cur.size() &&
                    (cur.empty() || std::memcmp(sc.cmds.data(), cur.data(), cur.size() * sizeof(gh_cmd)) == 0);
  if (cur.empty()) return eng_.Sync();
  // A graph launch has a higher fixed cost than a handful of plain launches
  // (measured on MI355X: one small kernel per run 29 us replayed against 13 us
  // eager, break-even at about five kernels), so short segments stay eager.
  constexpr size_t kMinGraphCmds = 5;
  if (cur.size() < kMinGraphCmds) {
    sc.verdict = SegCache::Plain;
    return eager();
  }
  if (opt_.replay_measured && same && sc.verdict != SegCache::Replay) {
    // two timed plain runs, a capture, two timed replays, then the verdict
    constexpr int kTimed = 2;
    if (sc.verdict == SegCache::Plain) return eager();
    if (sc.plain_timed < kTimed) {
      const int64_t l0 = ns_launch_, w0 = ns_wait_;
      Status st = eager();
      sc.plain_ns = std::min(sc.plain_ns, (ns_launch_ - l0) + (ns_wait_ - w0));
      sc.plain_timed++;
      return st;
    }
    if (sc.graph_id >= 0 && sc.replay_timed < kTimed) {
      eng_.DropSegment();
      graph_launches_++;
      const int64_t l0 = ns_launch_, w0 = ns_wait_;
      Status st = launch_and_wait([&]() { return eng_.GraphLaunch(sc.graph_id); });
      sc.replay_ns = std::min(sc.replay_ns, (ns_launch_ - l0) + (ns_wait_ - w0));
      if (++sc.replay_timed == kTimed) {
        if (sc.replay_ns < sc.plain_ns) {
          sc.verdict = SegCache::Replay;
        } else {
          sc.verdict = SegCache::Plain;
          eng_.GraphDestroy(sc.graph_id);
          sc.graph_id = -1;
        }
      }
      return st;
    }
    // falls through to the capture below
  }
  if (sc.graph_id >= 0 && same) {
    eng_.DropSegment();
    graph_launches_++;
    return launch_and_wait([&]() { return eng_.GraphLaunch(sc.graph_id); });
  }
  if (same && runs_ >= 1) {
    // an identical run of this segment: capture it, then launch the capture
    Status st = eng_.GraphBegin();
    if (!st.ok()) return st;
    st = eng_.SubmitPending();
    int id = -1;
    Status st2 = eng_.GraphEnd(&id);
    if (!st.ok()) return st;
    if (!st2.ok()) return st2;
    sc.graph_id = id;
    graph_launches_++;
    return launch_and_wait([&]() { return eng_.GraphLaunch(id); });
  }
  sc.cmds = cur;  // first sight (or the pointer set changed): run eagerly, remember
  if (sc.graph_id >= 0) eng_.GraphDestroy(sc.graph_id);  // the capture of the old pointer set is dead
  sc.graph_id = -1;
  sc.plain_timed = sc.replay_timed = 0;
  sc.plain_ns = sc.replay_ns = INT64_MAX;
  sc.verdict = SegCache::Measuring;
  return eager();
}

Status TapeMachine::RunAll() {
  if (!eng_.Initialized()) return Status::Err(GH_ESTATE, "tape machine not initialised");
  auto& nodes = g_->Nodes();
  segments_ = 0;
  seg_index_ = 0;
  const int64_t t_run = now_ns();
  ns_launch_ = ns_wait_ = 0;
  for (size_t pc = 0; pc < prog_.size(); pc++) {
    const Instr& in = prog_[pc];
    Status st;
    switch (in.kind) {
      case InstrKind::LoadArg:
        if (!nodes[(size_t)in.node].host)
          return Status::Err(GH_EINVAL, "PC " + std::to_string(pc) + ": input node " +
                                            std::to_string(in.node) + " has no value bound");
        break;
      case InstrKind::Alloc:
        if (!reg_live_[(size_t)in.reg]) {  // skipped when the register still holds a value (vm_tape.go:594-597)
          uint64_t mem = 0;
          st = eng_.Get(in.size, &mem);
          if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": alloc");
          regs_[(size_t)in.reg].mem = mem;
          reg_live_[(size_t)in.reg] = 1;
        }
        break;
      case InstrKind::Transport: {
        Node& n = nodes[(size_t)in.node];
        if (n.resident && resident_done_[(size_t)in.node] && !opt_.reupload_resident) break;
        if (void* pinned = stage_in_[(size_t)in.node]) {
          // host value -> pinned buffer now, pinned buffer -> register as a command of
          // the segment: the upload is captured and replayed with the operators
          if (!n.host_borrowed && in.size >= kPipelinedUpload && eng_.Segment().empty()) {
            // a large value at the front of its segment: piece by piece, the host copy of one
            // piece runs while the copy engine moves the piece before it (stream order puts the
            // segment's operators behind the last piece)
            const char* src = static_cast<const char*>(n.host);
            char* stg = static_cast<char*>(pinned);
            for (int64_t off = 0; off < in.size; off += kUploadPiece) {
              const int64_t len = std::min(kUploadPiece, in.size - off);
              std::memcpy(stg + off, src + off, (size_t)len);
              st = eng_.MemcpyHtoD(regs_[(size_t)in.reg].mem + (uint64_t)off, stg + off, len);
              if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": devTrans");
            }
            resident_done_[(size_t)in.node] = 1;
            break;
          }
          if (!n.host_borrowed) std::memcpy(pinned, n.host, (size_t)in.size);
          eng_.RecordCopy(regs_[(size_t)in.reg].mem, (uint64_t)(uintptr_t)pinned, in.size);
          resident_done_[(size_t)in.node] = 1;
          break;
        }
        // a borrowed input has no host value of its own (Node::host is a marker): without the machine's
        // pinned buffer - LetBorrowed after Init, on an input this machine does not stage - there is
        // nothing to upload
        if (n.host_borrowed)
          return Status::Err(GH_ESTATE, "PC " + std::to_string(pc) + ": devTrans: input " + std::to_string(in.node) +
                                            " was lent (LetBorrowed) but this machine holds no pinned buffer for it; "
                                            "lend inputs before the machine is created");
        st = eng_.MemcpyHtoD(regs_[(size_t)in.reg].mem, n.host, in.size);
        if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": devTrans");
        resident_done_[(size_t)in.node] = 1;
        break;
      }
      case InstrKind::ExecOp: {
        Node& n = nodes[(size_t)in.node];
        Tensor out;
        out.mem = regs_[(size_t)in.reg].mem;
        out.dt = n.dt;
        out.shape = n.shape;
        std::vector<Tensor> ins(n.inputs.size());
        std::vector<Tensor*> inp(n.inputs.size());
        for (size_t k = 0; k < n.inputs.size(); k++) {
          const Node& s = nodes[(size_t)n.inputs[k]];
          ins[k].mem = regs_[(size_t)node_reg_[(size_t)s.id]].mem;
          ins[k].dt = s.dt;
          ins[k].shape = s.shape;
          inp[k] = &ins[k];
        }
        st = CUDADo(eng_, n.op, out, inp);
        if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": " + op_name(n.op));
        if (opt_.node_at_a_time) {
          st = flush();  // DoWork after every node (vm_genera.go:144)
          if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": " + op_name(n.op) + ": DoWork failed");
        }
        if (opt_.watch_nan || opt_.watch_inf) {
          // the value just written, checked before anything else runs (vm_tape.go:271-315)
          if (!opt_.node_at_a_time) {
            st = flush();
            if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": " + op_name(n.op) + ": DoWork failed");
          }
          char idhex[24];
          std::snprintf(idhex, sizeof idhex, "%x", (unsigned)n.id);
          bool hit = false;
          if (opt_.watch_nan && n.dt != Dtype::Other) {
            st = eng_.HasNaN(out, &hit);
            if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": watchNaN");
            if (hit) return Status::Err(GH_ESTATE, "NaN found in value. Node: " + op_name(n.op) + "(" + idhex + ")");
          }
          if (opt_.watch_inf && n.dt != Dtype::Other) {
            st = eng_.HasInf(out, &hit);
            if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": watchInf");
            if (hit) return Status::Err(GH_ESTATE, "Inf found in value. Node: " + op_name(n.op) + "(" + idhex + ")");
          }
        }
        break;
      }
      case InstrKind::Free:
        if (reg_live_[(size_t)in.reg]) {
          eng_.Put(regs_[(size_t)in.reg].mem, in.size);
          reg_live_[(size_t)in.reg] = 0;
        }
        break;
      case InstrKind::Flush:
        st = flush();
        if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": flush");
        break;
      case InstrKind::AllocHost:
        regs_[(size_t)in.reg].mem = (uint64_t)(uintptr_t)stage_[(size_t)in.node];
        break;
      case InstrKind::StageOut:
        eng_.RecordCopy((uint64_t)(uintptr_t)stage_[(size_t)in.node], regs_[(size_t)in.reg].mem, in.size);
        break;
      case InstrKind::Read: {
        Node& n = nodes[(size_t)in.node];
        if (in.node < (int)stage_.size() && stage_[(size_t)in.node]) {
          // the flush in front of the reads has waited for the staging copy; a borrowed
          // read is finished with that
          if (!n.read_borrowed) std::memcpy(n.read_into, stage_[(size_t)in.node], (size_t)in.size);
          for (void* more : n.read_also) std::memcpy(more, stage_[(size_t)in.node], (size_t)in.size);
          break;
        }
        st = eng_.MemcpyDtoH(n.read_into, regs_[(size_t)in.reg].mem, in.size, false);
        for (void* more : n.read_also)
          if (st.ok()) st = eng_.MemcpyDtoH(more, regs_[(size_t)in.reg].mem, in.size, false);
        if (!st.ok()) return st.Wrap("PC " + std::to_string(pc) + ": read");
        bool last = pc + 1 >= prog_.size() || prog_[pc + 1].kind != InstrKind::Read;
        if (last) {
          st = eng_.Sync();
          if (!st.ok()) return st;
        }
        break;
      }
    }
  }
  Status st = eng_.DoWork();  // final DoWork (vm_tape.go:236)
  runs_++;
  // Leave the arena in a state that depends only on what is still held
  // (resident inputs): merge the holes and zero the free/alloc counters, so the
  // next run's first-fit walk hands out the same addresses again and a captured
  // segment stays replayable.
  eng_.Allocator().coalesce();
  eng_.Allocator().reset_stats();
  ns_total_ = now_ns() - t_run;
  return st;
}

void TapeMachine::drop_graphs() {
  for (SegCache& sc : seg_cache_) {
    if (sc.graph_id >= 0) eng_.GraphDestroy(sc.graph_id);
    sc.graph_id = -1;
    sc.cmds.clear();
  }
}

// Give back what this machine holds in the arena (a shared engine's other
// users keep theirs).
void TapeMachine::release_registers() {
  for (size_t r = 0; r < reg_live_.size(); r++)
    if (reg_live_[r]) {
      eng_.Put(regs_[r].mem, reg_bytes_[r]);
      reg_live_[r] = 0;
    }
}

Status TapeMachine::Reset() {
  if (!open_ || !eng_.Initialized()) return Status::OK();
  eng_.DropSegment();
  if (borrowed_) release_registers();
  else eng_.ResetAllocator();
  std::fill(reg_live_.begin(), reg_live_.end(), 0);
  std::fill(resident_done_.begin(), resident_done_.end(), 0);
  return Status::OK();
}

Status TapeMachine::Close() {
  if (!open_) return Status::OK();
  open_ = false;
  if (eng_.Initialized()) {
    drop_graphs();
    for (auto* v : {&stage_, &stage_in_})
      for (void*& p : *v) {
        eng_.HostFree(p);
        p = nullptr;
      }
  }
  if (!borrowed_) return eng_.Close();
  if (eng_.Initialized()) {
    eng_.DropSegment();
    release_registers();
    eng_.Allocator().coalesce();
  }
  return Status::OK();
}

std::string TapeMachine::ProgramString() const {
  static const char* names[] = {"loadArg", "alloc", "devTrans", "execOp", "free", "flush", "read", "stageOut", "allocHost"};
  std::ostringstream os;
  os << "Instructions:\n";
  const auto& nodes = g_->Nodes();
  for (size_t pc = 0; pc < prog_.size(); pc++) {
    const Instr& in = prog_[pc];
    os << pc << "\t" << names[(int)in.kind];
    if (in.node >= 0) os << " node " << in.node;
    if (in.reg >= 0) os << " GPU" << in.reg;
    if (in.kind == InstrKind::ExecOp)
      os << " " << op_name(nodes[(size_t)in.node].op) << (in.use_unsafe ? " [unsafe]" : " [reuse]");
    if (in.size) os << " " << in.size << "B";
    os << "\n";
  }
  os << "GPU Memories: " << gpumem_ << "\n";
  return os.str();
}

}  // namespace gorgonia
