// Operators with a device path (the reference's CUDADoer implementers) and a
// tape machine that runs them in segments.
//
// What this mirrors:
//   - Op::CUDADo(extern, dev, prealloc, inputs...)            op.go:153-155
//       elemBinOp / elemUnaryOp / linAlgBinOp                 op_math_cuda.go:23-240
//       reshapeOp (metadata only)                             op_tensor.go:1226-1246
//       ops/nn convolution, maxpool, BatchNormOp, activation  ops/nn/*_cuda.go
//   - the tape program: loadArg / alloc / deviceTransport / execOp / free /
//     flushInstr / readInstr                                  vm_tape.go:584-793
//   - register reuse only when the overwritten input is dead  regalloc.go:211-243
//   - flushInstr only where a host read needs a finished value compile.go:437-462
//   - RunAll / Reset                                          vm_tape.go:123-134,213-249
//
// The expression-graph front end (type system, differentiation, CSE) is out of
// scope; Graph below is the minimum needed to produce the same instruction
// stream for forward graphs: nodes are appended in topological order, each
// with an Op and its input nodes.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "engine.hpp"

namespace gorgonia {

enum class OpKind : int32_t {
  ElemBin = 0,      // Add, Sub, HadamardProd, HadamardDiv, Pow, Lt, Lte, Gt, Gte, Eq, Ne
  ElemUnary = 1,    // Sigmoid, Tanh, Exp, ... (by the op's String() name)
  BroadcastBin = 2, // BroadcastAdd / BroadcastHadamardProd ... (broadcast.go:69-129)
  MatMul = 3,       // linAlgBinOp matMulOperator (+transA/transB)
  MatVecMul = 4,
  Outer = 5,
  BatchedMatMul = 6,
  Conv2d = 7,       // nnops.Conv2d
  MaxPool2D = 8,    // nnops.MaxPool2D
  BatchNorm = 9,    // nnops.BatchNorm in eval mode (+ the gamma/beta wrap of nn.go:429-440)
  Rectify = 10,     // nnops.Rectify
  LeakyRelu = 11,   // gorgonia.LeakyRelu
  SoftMax = 12,     // gorgonia.SoftMax (last axis)
  Reshape = 13,     // gorgonia.Reshape
  // the diff ops the reference's symbolic differentiation inserts, and Set
  MaxPool2DDiff = 14,    // maxPoolDiffOp (op_nn.go:962-1093): inputs x, grad
  Conv2dDiffData = 15,   // gradient of Conv2d wrt the image: inputs grad, filter; ints = conv params + image shape
  Conv2dDiffFilter = 16, // gradient wrt the filter: inputs image, grad; ints = conv params
  BatchNormTrain = 17,   // BatchNormOp in training mode (op_nn.go:1489-1635): inputs x, runningMean,
                         // runningVar, saveMean, saveVar; the four statistics tensors are updated in place
  BatchNormDiff = 18,    // batchnormDiffOp (op_nn.go:1834-1943): inputs x, grad, saveMean, saveVar
  SoftMaxDiff = 19,      // softmaxDiffOp (op_softmax.go:184-279): inputs y, grad
  Set = 20,              // gorgonia.Set(a, b): a's value becomes b's (operations.go); inputs a, b
  SolverStep = 21,       // one Step of VanillaSolver / RMSPropSolver / AdamSolver on one weight tensor
                         // (solvers.go:273-870): inputs weights, grad[, cache[, cache2]]; fn = gh_solver,
                         // ints[0] = use mask, fs = the ten constants; the weights are updated in place
  RandUniform = 22,      // the uniform [0,1) source gorgonia.Dropout draws from (nn.go:71-77), generated on
                         // the device: ints = seed, offset, shape...; optional input = one 8-byte counter
                         // (a Float64 scalar used as raw bits) read as the offset and advanced by the size
  Dropout = 23,          // dropoutOp (op_dropout.go:107-132): inputs x, uniform numbers; f0 = probability,
                         // fn = 1 while training, 0 for the identity of evaluation
  DropoutDiff = 24,      // dropoutDiffOp (op_dropout.go:205-238): inputs y, grad; f0 = probability
  RectifyDiff = 25       // activation backward (ops/nn/activation_cuda.go:130-153): inputs x, grad; grad * (x >= 0)
};

struct OpSpec {
  OpKind kind = OpKind::ElemBin;
  int32_t fn = 0;             // gh_binfn for ElemBin / BroadcastBin
  std::string name;           // unary op name ("sigmoid", "tanh", ...)
  bool transA = false, transB = false;
  std::vector<int64_t> ints;  // kernel/pad/stride/dilation, new shape, broadcast axes ...
  double f0 = 0.0;            // epsilon / alpha
  std::vector<double> fs;     // SolverStep constants
  // Followers folded into a Conv2d/MatMul epilogue by Graph::FuseActivations,
  // applied in this order: BatchNorm (Conv2d only; inputs 2.. = mean, var[,
  // scale, bias], f1 = epsilon), activation (f0 = alpha), 2x2/2 MaxPool2D.
  bool fuse_bn = false;
  double f1 = 0.0;
  bool fuse_act_relu = false;
  bool fuse_act_leaky = false;
  bool fuse_pool2 = false;
  bool fuse_bias = false;     // MatMul only: the BroadcastAdd of a row vector that follows (last input)
  bool fuse_softmax = false;  // MatMul only: the SoftMax that follows, where gh_gemm_can_softmax allows
  // Conv2d only: the operators in FRONT of it ride along (GH_FLAG_CONV_PRE).  Input 0 is then a batch of
  // single-channel images and the last input the filters of Conv2d 3x3 pad 1 -> Rectify -> MaxPool2D 2x2/2
  // whose result this convolution reads without it ever being stored.
  bool fuse_pre = false;
  // Conv2d only, with fuse_pool2: the convolution's own result is stored as well (GH_FLAG_CONV_KEEP), into the
  // register of the node given as the last input - a Conv2d node whose work this node has taken over
  // (Node::deferred) because other nodes, a backward pass, read the unpooled values too.
  bool fuse_keep = false;
  // MaxPool2D / MaxPool2DDiff: input 0 is the value before a Rectify and is read through it; the
  // diff also applies the Rectify's own gradient (it stands for RectifyDiff(z, MaxPool2DDiff(Rectify(z), g)))
  bool relu_input = false;
};

// Output shape of an op (InferShape of each reference op); error if the inputs
// do not fit.
Status InferShape(const OpSpec& op, const std::vector<const Shape*>& in, Shape* out);
// Which input the op may overwrite, -1 for none (OverwritesInput,
// op_math.go:285-294,476-481; the nn ops return -1).
int OverwritesInput(const OpSpec& op);
// Record the op's device work on the engine (one or more gh_cmd).
Status CUDADo(Engine& e, const OpSpec& op, Tensor& prealloc, const std::vector<Tensor*>& inputs);

struct Node {
  int id = -1;
  Shape shape;
  Dtype dt = Dtype::Float32;
  bool is_input = false;
  bool resident = false;          // uploaded once and kept (weights); else re-uploaded per run
  const void* host = nullptr;     // bound host value (Let / WithValue)
  bool host_borrowed = false;     // LetBorrowed: the caller writes the value into the machine's pinned buffer
  OpSpec op;
  std::vector<int> inputs;
  void* read_into = nullptr;      // Read(node, &host) target
  std::vector<void*> read_also;   // further Reads of the same node: each gets the value too
  bool read_borrowed = false;     // ReadBorrowed: the value stays in the machine's own pinned buffer
  bool fused_away = false;        // absorbed into the follower that now computes both: no register, no instruction
  bool deferred = false;          // keeps its register, but a later node (which lists it as its last input) writes it: no instruction
  int alias_of = -1;              // Reshape shares its input's register
};

class Graph {
 public:
  int NewTensor(const Shape& s, Dtype dt, const void* host, bool resident);
  Status Apply(const OpSpec& op, const std::vector<int>& inputs, int* out);
  Status Let(int node, const void* host);              // rebind an input value
  // The input's value is whatever the caller has written into the machine's pinned buffer for
  // it (TapeMachine::InputBuffer) when a run uploads it: Let without the host-to-host copy.
  Status LetBorrowed(int node);
  Status Read(int node, void* host_out);               // gorgonia.Read
  // Read without the last host copy: the machine keeps the value in pinned host memory of its
  // own (TapeMachine::ReadBuffer) and overwrites it on every run, as the reference rebinds
  // the Value a Read points at (op.go readOp.Do).
  Status ReadBorrowed(int node);
  // Fold BatchNorm (eval), Rectify/LeakyRelu and a 2x2/2 MaxPool2D into the
  // Conv2d that feeds them (activations into MatMul too) when nothing else reads
  // the intermediate value.  The follower takes over the producer's operator
  // and inputs; the values it stores are bit-identical to the unfused chain's.
  // Returns the number of operators folded away.
  int FuseActivations();
  int fuse_pooled_rectify();   // part of FuseActivations: the Rectify between a pool and both gradients
  int fuse_first_layer();      // part of FuseActivations: a single-channel first layer folded into the next convolution
  int fuse_rectify_into_pool();   // part of FuseActivations: a Rectify read by nothing but a pool (float64 convolutions have no epilogue)
  int fuse_kept_conv();        // part of FuseActivations: a pool into the convolution whose result other nodes read too
  const std::vector<Node>& Nodes() const { return nodes_; }
  std::vector<Node>& Nodes() { return nodes_; }

 private:
  std::vector<Node> nodes_;
};

enum class InstrKind : int32_t { LoadArg, Alloc, Transport, ExecOp, Free, Flush, Read, StageOut, AllocHost };

struct Instr {
  InstrKind kind;
  int node = -1;    // node the instruction is about
  int reg = -1;     // register written / freed
  int64_t size = 0; // bytes for Alloc/Free/Transport/Read
  bool use_unsafe = false;  // ExecOp reuses input 0's register
};

struct TapeOptions {
  bool graph_replay = false;      // capture each segment into a hipGraph and replay it
  // With graph_replay: time a segment's plain submits and its replays over its
  // first runs and keep whichever finishes sooner.  A replayed graph saves the
  // per-kernel launch calls but starts later than the first plain launch does,
  // so it only pays for segments of many short kernels.
  bool replay_measured = false;
  bool reupload_resident = false; // treat resident inputs like the reference does (H2D every run)
  // The lispMachine's way of running a graph (vm_genera.go:121-200,296-430): every
  // node is executed and waited for when it is reached - one submit and one wait
  // per operator, no segment batching, no replay - and no operator writes over
  // an input's register.  Same operators, same kernels: the values are those of
  // the batched machine, which is what running one graph on both machines checks.
  bool node_at_a_time = false;
  // WithNaNWatch() / WithInfWatch() (vm.go:138-166; the checks of vm_tape.go:271-315): after every operator
  // its value is searched for NaN / +-Inf on the device (the engine's HasNaN / HasInf) and the run stops
  // at the first hit with "NaN found in value. Node: ..." - later operators, weight updates included,
  // do not run.  Every operator is then submitted and waited for on its own, which "slows the execution
  // down" here as it does there; segments are neither batched across operators nor replayed.
  bool watch_nan = false;
  bool watch_inf = false;
};

class TapeMachine {
 public:
  TapeMachine(Graph* g, const TapeOptions& o) : g_(g), opt_(o), eng_(own_) {}
  // WithEngine(e) (vm.go:318-329): the machine computes on an engine its caller
  // created and initialised, takes its registers from that engine's arena and
  // leaves the engine open when it closes.  Machines that share an engine run
  // one after the other, never at the same time.
  TapeMachine(Graph* g, const TapeOptions& o, Engine* shared)
      : g_(g), opt_(o), eng_(shared ? *shared : own_), borrowed_(shared != nullptr) {}
  ~TapeMachine();
  // Compile (compile.go:16-60 for forward graphs), size the arena from the
  // program (compile.go:148-216) and create the engine (vm_tape_cuda.go:17-41).
  // With a shared engine nothing is created: the engine must be initialised
  // already and its arena must still have room for the program's registers.
  Status Init(int device);
  Status Compile();  // program only, no device
  Status RunAll();
  void SetWatch(bool nan, bool inf) { opt_.watch_nan = nan; opt_.watch_inf = inf; }
  Status Reset();   // vm_tape.go:123-134: pc = 0, arena reset
  Status Close();
  Engine& Eng() { return eng_; }
  const std::vector<Instr>& Program() const { return prog_; }
  int64_t GpuMem() const { return gpumem_; }
  int Segments() const { return segments_; }      // flush points in the last run
  // How segment `i` of the last run is executed: 0 still measuring, 1 plain submits, 2 graph replay.
  int SegmentVerdict(int i) const { return i >= 0 && i < (int)seg_cache_.size() ? (int)seg_cache_[(size_t)i].verdict : 0; }
  int GraphLaunches() const { return graph_launches_; }
  // Host time of the last RunAll in nanoseconds: [0] the whole call, [1] inside
  // graph launches and submits, [2] waiting for the device.
  void PhaseNs(int64_t out[3]) const { out[0] = ns_total_; out[1] = ns_launch_; out[2] = ns_wait_; }
  uint64_t RegisterAddress(int node) const;
  void* InputBuffer(int node) const;        // where a LetBorrowed input's next value goes (null: not such a node)
  const void* ReadBuffer(int node) const;   // where a ReadBorrowed node's value is after RunAll (null: not such a node)
  std::string ProgramString() const;              // program.String() (vm_tape.go:493-522)

 private:
  Status flush();
  void drop_graphs();   // destroy every captured segment graph
  void release_registers();
  Graph* g_;
  TapeOptions opt_;
  Engine own_;
  Engine& eng_;          // own_, or the caller's engine
  bool borrowed_ = false;
  bool open_ = false;    // Init done, Close not yet
  std::vector<Instr> prog_;
  std::vector<Tensor> regs_;       // one per register
  std::vector<int> node_reg_;      // node -> register
  std::vector<char> reg_live_;     // register currently holds arena memory
  std::vector<int64_t> reg_bytes_; // register -> bytes it was allocated with
  std::vector<char> resident_done_;
  // Small outputs leave through pinned host buffers written by a copy at the
  // end of the segment, so a replayed run is one graph launch and one wait;
  // node -> buffer (null: the output is read with a D2H copy after the flush).
  std::vector<void*> stage_;
  // Inputs uploaded on every run enter through pinned host buffers read by a
  // copy at the head of the segment; node -> buffer (null: direct H2D copy).
  std::vector<void*> stage_in_;
  int64_t gpumem_ = 0;
  int runs_ = 0, segments_ = 0, graph_launches_ = 0;
  int64_t ns_total_ = 0, ns_launch_ = 0, ns_wait_ = 0;
  // per-segment replay cache
  struct SegCache {
    std::vector<gh_cmd> cmds;
    int graph_id = -1;
    // replay_measured bookkeeping: host nanoseconds (launch + wait) of the best
    // plain and the best replayed run so far, and the verdict
    int plain_timed = 0, replay_timed = 0;
    int64_t plain_ns = INT64_MAX, replay_ns = INT64_MAX;
    enum { Measuring, Plain, Replay } verdict = Measuring;
  };
  std::vector<SegCache> seg_cache_;
  int seg_index_ = 0;
};

}  // namespace gorgonia
