// Host-only command validation and the kernel-name registry.
// The checks mirror what cuda.Engine verifies before a launch
// (cuda/utils.go:58-112: float32/float64 only, sizes agree) plus the operand
// shape checks a hand-written kernel needs before it may be launched.
#include <cstdio>
#include <cstring>
#include <string>

#include "gh_internal.h"

static bool pos(int64_t v) { return v > 0; }
static double dim_double(int64_t bits) {   // a float64 scalar carried in a dim slot
  double v;
  memcpy(&v, &bits, sizeof(v));
  return v;
}

int gh_validate_cmd(const gh_cmd& c, std::string& msg) {
  auto bad = [&](const char* m) { msg = m; return (int)GH_EINVAL; };
  const uint32_t fn = gh_fn(c.flags), mode = gh_mode(c.flags), dt = gh_dtype_of(c.flags);
  switch (c.opcode) {
    case GH_OP_NOP: return GH_OK;
    case GH_OP_ELEM_BIN:
      if (fn >= GH_BINFN__COUNT) { msg = "unknown binary function"; return GH_ENOFUNC; }
      if (mode > GH_SS) return bad("unknown operand mode");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (!c.ptr[0] || !c.ptr[1]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      if (mode == GH_SS && c.dim[0] != 1) return bad("scalar-scalar op needs size 1");
      return GH_OK;
    case GH_OP_ELEM_UNARY:
      if (fn >= GH_UNARYFN__COUNT) { msg = "unknown unary function"; return GH_ENOFUNC; }
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (!c.ptr[0]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      return GH_OK;
    case GH_OP_BCAST_BIN:
      if (fn >= GH_BINFN__COUNT) { msg = "unknown binary function"; return GH_ENOFUNC; }
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (c.dim[0] < 0 || c.dim[1] <= 0 || c.dim[2] <= 0) return bad("bad broadcast shape");
      return GH_OK;
    case GH_OP_MEMCPY_D2D:
      if (c.dim[0] < 0) return bad("negative size");
      if (c.dim[0] > 0 && (!c.ptr[0] || !c.ptr[1])) return bad("null operand");
      return GH_OK;
    case GH_OP_GEMM: {
      const int64_t m = c.dim[0], n = c.dim[1], k = c.dim[2];
      const int64_t lda = c.dim[3], ldb = c.dim[4], ldc = c.dim[5];
      const int64_t batch = c.dim[6] <= 0 ? 1 : c.dim[6];
      const bool ta = c.flags & GH_FLAG_TRANS_A, tb = c.flags & GH_FLAG_TRANS_B;
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (!pos(m) || !pos(n) || !pos(k)) return bad("gemm: m, n, k must be positive");
      if (lda < (ta ? m : k)) return bad("gemm: lda too small");
      if (ldb < (tb ? k : n)) return bad("gemm: ldb too small");
      if (ldc < n) return bad("gemm: ldc too small");
      if (m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return bad("gemm: dimension too large");
      if (batch > 1 && (c.dim[7] < 0 || c.dim[8] < 0 || c.dim[9] < m * n))
        return bad("gemm: bad batch strides");
      if (batch > 65535 * 16) return bad("gemm: batch too large");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (dt == GH_F64 && (c.flags & (GH_FLAG_ACT_RELU | GH_FLAG_ACT_LEAKY)))
        return bad("gemm: no fused activation for float64");
      if (dt == GH_F64 && batch > 65535) return bad("gemm: batch too large");
      if ((c.flags & GH_FLAG_GEMM_BIAS) && (dt != GH_F32 || !c.ptr[3] || ta || tb))
        return bad("gemm: the fused row bias is float32 only, takes untransposed operands and needs ptr[3]");
      if ((c.flags & GH_FLAG_GEMM_SOFTMAX) && !gh_gemm_can_softmax(&c))
        return bad("gemm: no fused softmax for this shape (see gh_gemm_can_softmax)");
      return GH_OK;
    }
    case GH_OP_GEMV:
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (!pos(c.dim[0]) || !pos(c.dim[1])) return bad("gemv: m, n must be positive");
      if (c.dim[2] < c.dim[1]) return bad("gemv: lda too small");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_OUTER:
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (!pos(c.dim[0]) || !pos(c.dim[1])) return bad("outer: m, n must be positive");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_CONV2D_BWD_DATA:
    case GH_OP_CONV2D_BWD_FILTER:
      if (c.flags & (GH_FLAG_CONV_BN | GH_FLAG_CONV_POOL2 | GH_FLAG_ACT_RELU | GH_FLAG_ACT_LEAKY | GH_FLAG_CONV_PRE | GH_FLAG_CONV_KEEP))
        return bad("conv2d backward takes no epilogue flags");
      [[fallthrough]];
    case GH_OP_CONV2D: {
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      for (int i = 0; i <= 6; i++)
        if (!pos(c.dim[i])) return bad("conv2d: B,C,H,W,F,kh,kw must be positive");
      if (c.dim[7] < 0 || c.dim[8] < 0) return bad("Cannot use padding of less than 0");
      if (!pos(c.dim[9]) || !pos(c.dim[10])) return bad("Cannot use strides of less than or equal 0");
      if (!pos(c.dim[11]) || !pos(c.dim[12])) return bad("Cannot use dilation less than or eq 0");
      const int64_t oh = gh_conv_out(c.dim[2], c.dim[5], c.dim[7], c.dim[9], c.dim[11]);
      const int64_t ow = gh_conv_out(c.dim[3], c.dim[6], c.dim[8], c.dim[10], c.dim[12]);
      if (oh <= 0 || ow <= 0) return bad("conv2d: empty output");
      if (c.dim[0] * oh * ow > INT32_MAX || c.dim[1] * c.dim[5] * c.dim[6] > INT32_MAX ||
          c.dim[0] * c.dim[1] * c.dim[2] * c.dim[3] > INT32_MAX ||
          c.dim[0] * c.dim[4] * oh * ow > INT32_MAX)
        return bad("conv2d: tensor too large for 32-bit indexing");
      if ((c.flags & GH_FLAG_ACT_RELU) && (c.flags & GH_FLAG_ACT_LEAKY))
        return bad("conv2d: two activations requested");
      if (c.flags & GH_FLAG_CONV_BN) {
        if (!c.ptr[3] || !c.ptr[4]) return bad("conv2d: fused BatchNorm needs mean and variance");
        if ((c.flags & GH_FLAG_HAS_GAMMA) && !c.ptr[5]) return bad("conv2d: fused BatchNorm gamma is null");
        if ((c.flags & GH_FLAG_HAS_BETA) && !c.ptr[6]) return bad("conv2d: fused BatchNorm beta is null");
      }
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (dt == GH_F64 && (c.flags & (GH_FLAG_CONV_BN | GH_FLAG_CONV_POOL2 | GH_FLAG_ACT_RELU | GH_FLAG_ACT_LEAKY)))
        return bad("conv2d: no epilogue operators for float64");
      if ((c.flags & GH_FLAG_CONV_POOL2) && !gh_conv2d_can_pool(&c))
        return bad("conv2d: no fused pooling for this shape");
      if (c.flags & GH_FLAG_CONV_KEEP) {
        if (c.opcode != GH_OP_CONV2D || dt != GH_F32 || !(c.flags & GH_FLAG_CONV_POOL2) || (c.flags & GH_FLAG_CONV_PRE))
          return bad("conv2d: keeping the unpooled result is for the float32 forward command with fused pooling, without a folded first layer");
        if (!c.ptr[7]) return bad("conv2d: the tensor for the unpooled result (ptr[7]) is null");
        if (!gh_conv2d_can_keep(&c)) return bad("conv2d: the unpooled result cannot be kept for this shape");
      }
      if (c.flags & GH_FLAG_CONV_PRE) {
        if (c.opcode != GH_OP_CONV2D || dt != GH_F32) return bad("conv2d: a folded first layer is for the float32 forward command");
        if (!c.ptr[7]) return bad("conv2d: the folded first layer's filters (ptr[7]) are null");
        if (!gh_conv2d_can_pre(&c)) return bad("conv2d: no folded first layer for this shape");
      }
      return GH_OK;
    }
    case GH_OP_MAXPOOL2D_BWD:
      if (!c.ptr[2]) return bad("null operand");
      [[fallthrough]];
    case GH_OP_MAXPOOL2D: {
      if (!c.ptr[0] || !c.ptr[1]) return bad("null operand");
      for (int i = 0; i <= 5; i++)
        if (!pos(c.dim[i])) return bad("maxpool2d: B,C,H,W,kh,kw must be positive");
      for (int i = 6; i <= 9; i++)
        if (c.dim[i] < 0) return bad("Cannot use padding of less than 0");
      if (!pos(c.dim[10]) || !pos(c.dim[11])) return bad("Cannot use strides of less than or equal 0");
      if (c.dim[2] - c.dim[4] + c.dim[6] + c.dim[7] < 0)
        return bad("Impossible height/kernel/pad combination");
      if (c.dim[3] - c.dim[5] + c.dim[8] + c.dim[9] < 0)
        return bad("Impossible width/kernel/pad combination");
      if (c.dim[0] * c.dim[1] * c.dim[2] * c.dim[3] > INT32_MAX)
        return bad("maxpool2d: tensor too large for 32-bit indexing");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (dt == GH_F64 && (c.flags & GH_FLAG_ACT_RELU) && c.opcode == GH_OP_MAXPOOL2D_BWD)
        return bad("maxpool2d gradient: no Rectify on the input for float64");
      return GH_OK;
    }
    case GH_OP_BN_INFER:
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2] || !c.ptr[3]) return bad("null operand");
      if ((c.flags & GH_FLAG_HAS_GAMMA) && !c.ptr[4]) return bad("null gamma");
      if ((c.flags & GH_FLAG_HAS_BETA) && !c.ptr[5]) return bad("null beta");
      if (!pos(c.dim[0]) || !pos(c.dim[1]) || !pos(c.dim[2])) return bad("bn: B,C,S must be positive");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_BN_TRAIN:
      for (int i = 0; i < 6; i++)
        if (!c.ptr[i]) return bad("null operand");
      if (!pos(c.dim[0]) || !pos(c.dim[1]) || !pos(c.dim[2])) return bad("bn: B,C,S must be positive");
      if (c.dim[1] > 65535) return bad("bn: more than 65535 channels");
      if (c.dim[0] * c.dim[2] < 2) return bad("bn: training statistics need at least two values per channel");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_BN_BWD:
      for (int i = 0; i < 5; i++)
        if (!c.ptr[i]) return bad("null operand");
      if (!pos(c.dim[0]) || !pos(c.dim[1]) || !pos(c.dim[2])) return bad("bn: B,C,S must be positive");
      if (c.dim[1] > 65535) return bad("bn: more than 65535 channels");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_SOFTMAX_BWD:
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (c.dim[0] < 0 || !pos(c.dim[1])) return bad("softmax: bad shape");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_SOLVER_STEP:
      if (fn >= GH_SOLVER__COUNT) { msg = "unknown solver"; return GH_ENOFUNC; }
      if (!c.ptr[0] || !c.ptr[1]) return bad("null operand");
      if (fn >= GH_SOLVER_RMSPROP && !c.ptr[2]) return bad("solver cache is null");
      if (fn == GH_SOLVER_ADAM && !c.ptr[3]) return bad("Adam second-moment cache is null");
      if (c.ptr[4] && fn != GH_SOLVER_ADAM) return bad("only Adam takes bias corrections");
      if (c.ptr[4] & (dt == GH_F64 ? 7 : 3)) return bad("Adam bias corrections must be aligned to their type");
      if (c.dim[0] < 0) return bad("negative size");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_RAND_UNIFORM:
      if (!c.ptr[0]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      if (c.ptr[1] & 7) return bad("rand: state must be 8-byte aligned");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_RELU_BWD:
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_DROPOUT:
    case GH_OP_DROPOUT_BWD:
      if (!c.ptr[0] || !c.ptr[1] || !c.ptr[2]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (dt == GH_F64 ? !(dim_double(c.dim[1]) >= 0.0 && dim_double(c.dim[1]) < 1.0) : !(c.f[0] >= 0.0f && c.f[0] < 1.0f))
        return bad("dropout: probability must be in [0, 1)");
      return GH_OK;
    case GH_OP_RELU:
    case GH_OP_LEAKY_RELU:
      if (!c.ptr[0] || !c.ptr[1]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_SOFTMAX:
      if (!c.ptr[0] || !c.ptr[1]) return bad("null operand");
      if (c.dim[0] < 0 || !pos(c.dim[1])) return bad("softmax: bad shape");
      if (dt > GH_F64) return bad("Unsupported Dtype");
      return GH_OK;
    case GH_OP_HAS_NAN:
    case GH_OP_HAS_INF:
      if (dt > GH_F64) return bad("Unsupported Dtype");
      if (!c.ptr[0] || !c.ptr[1]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      return GH_OK;
    case GH_OP_FILL:
      if (!c.ptr[0]) return bad("null operand");
      if (c.dim[0] < 0) return bad("negative size");
      return GH_OK;
  }
  msg = "unknown opcode";
  return GH_ENOFUNC;
}

// ---- kernel names --------------------------------------------------------
// The reference names kernels "<module>.<fn>_<mode>_f<bits>" for binary ops
// (cuda/utils.go:114-139) and "<module>.<fn>_f<bits>" for unary ops
// (op_math_cuda.go:38).  "mod" is declared by the engine
// (cuda/arith.go:589-701) but its kernel is absent from elembinop.cu:201-210,
// so HasFunc is false for it there; here the kernel exists.

static const char* kBinNames[GH_BINFN__COUNT] = {"add", "sub", "mul", "div", "pow", "lt",
                                                 "lte", "gt",  "gte", "eq",  "ne",  "mod"};
static const char* kModeNames[4] = {"vv", "vs", "sv", "ss"};
// Kernel-file names (elemunaryop.cu:109-193) ...
static const char* kUnaryNames[GH_UNARYFN__COUNT] = {
    "abs",  "sign",   "ceil", "floor",   "sin",     "cos",  "exp",  "ln",      "log2",  "neg",
    "square", "sqrt", "inverse", "invsqrt", "cube", "tanh", "sigmoid", "log1p", "expm1", "softplus"};
// ... and the op String() forms the Go side actually asks for
// (operatorPointwise_unary_const.go:117-125): "inv" and "invSqrt" never
// matched a CUDA kernel and fell back to the CPU; both spellings resolve here.
static const struct { const char* alias; int fn; } kUnaryAlias[] = {{"inv", GH_INVERSE},
                                                                    {"invSqrt", GH_INVSQRT}};

extern "C" int gh_lookup_func(const char* name, uint32_t* opcode, uint32_t* flags) {
  if (!name) return GH_EINVAL;
  const char* dot = strchr(name, '.');
  if (!dot) return GH_ENOFUNC;
  std::string mod(name, dot - name), rest(dot + 1);
  // dtype suffix
  uint32_t dt;
  if (rest.size() > 4 && rest.compare(rest.size() - 4, 4, "_f32") == 0) dt = GH_F32;
  else if (rest.size() > 4 && rest.compare(rest.size() - 4, 4, "_f64") == 0) dt = GH_F64;
  else return GH_ENOFUNC;
  rest.resize(rest.size() - 4);
  uint32_t op = 0, fl = 0;
  if (mod == "elembinop") {
    size_t us = rest.rfind('_');
    if (us == std::string::npos) return GH_ENOFUNC;
    std::string fn = rest.substr(0, us), md = rest.substr(us + 1);
    int fi = -1, mi = -1;
    for (int i = 0; i < GH_BINFN__COUNT; i++) if (fn == kBinNames[i]) fi = i;
    for (int i = 0; i < 4; i++) if (md == kModeNames[i]) mi = i;
    if (fi < 0 || mi < 0) return GH_ENOFUNC;
    op = GH_OP_ELEM_BIN;
    fl = GH_FLAG_FN(fi) | GH_FLAG_MODE(mi) | GH_FLAG_DTYPE(dt);
  } else if (mod == "elemunaryop") {
    int fi = -1;
    for (int i = 0; i < GH_UNARYFN__COUNT; i++) if (rest == kUnaryNames[i]) fi = i;
    for (auto& a : kUnaryAlias) if (rest == a.alias) fi = a.fn;
    if (fi < 0) return GH_ENOFUNC;
    op = GH_OP_ELEM_UNARY;
    fl = GH_FLAG_FN(fi) | GH_FLAG_DTYPE(dt);
  } else if (mod == "misc") {
    if (rest == "hasNaN") op = GH_OP_HAS_NAN;
    else if (rest == "hasInf") op = GH_OP_HAS_INF;
    else return GH_ENOFUNC;
    fl = GH_FLAG_DTYPE(dt);
  } else {
    return GH_ENOFUNC;
  }
  if (opcode) *opcode = op;
  if (flags) *flags = fl;
  return GH_OK;
}

extern "C" int gh_has_func(const char* name) {
  return gh_lookup_func(name, nullptr, nullptr) == GH_OK ? 1 : 0;
}
