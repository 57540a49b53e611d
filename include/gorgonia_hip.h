/*
 * gorgonia_hip.h - C ABI of libgorgonia_hip.so, the gfx950 device engine that
 * sits where Gorgonia's cuda/ package calls into gorgonia.org/cu, cuBLAS and
 * cuDNN.
 *
 * The calling model follows Gorgonia's own "fill a command array in Go, drain
 * it in one cgo call" precedent (blase/work.h:144-168): the host records one
 * gh_cmd per operator while the tape machine walks a segment, and hands the
 * whole array to gh_submit() when it reaches a flush point.  One cgo crossing
 * per tape segment instead of one per operator.
 *
 * Conventions
 *   - every entry point returns 0 on success, a GH_E* code otherwise;
 *   - device errors are sticky per context (cuda/external.go:223-226,251-257):
 *     once a call fails, later gh_submit()/gh_sync() calls return the same
 *     code until gh_clear_error(); gh_last_error() returns the message;
 *   - a context is used from one thread at a time (cuda/external.go:237);
 *   - all work is stream-ordered on the context's single stream; results are
 *     only guaranteed after gh_sync() (enqueue-then-flush, vm_tape.go:735-745);
 *   - device addresses are plain uint64_t (tensor.Memory.Uintptr()).
 */
#ifndef GORGONIA_HIP_H
#define GORGONIA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported from the shared library (everything else is built hidden). */
#if defined(__GNUC__)
#define GH_API __attribute__((visibility("default")))
#else
#define GH_API
#endif

typedef struct gh_ctx gh_ctx;
typedef uint64_t gh_devptr;

enum {
  GH_OK = 0,
  GH_EINVAL = 1,     /* bad argument / shape / opcode (cuda/utils.go:58-112) */
  GH_EDEVICE = 2,    /* HIP runtime error (sticky) */
  GH_EOOM = 3,       /* arena reservation failed (cuda/external.go:158-166) */
  GH_ENOFUNC = 4,    /* no such kernel (cuda/arith.go:17-19) */
  GH_ESTATE = 5      /* call not valid in the current state */
};

/* Device limits; replaces the attribute query at cuda/external.go:135-146. */
typedef struct gh_devinfo {
  int32_t wavefront_size;
  int32_t max_threads_per_block;
  int32_t max_grid_x, max_grid_y, max_grid_z;
  int32_t max_block_x, max_block_y, max_block_z;
  int32_t compute_units;
  int32_t lds_bytes_per_block;
  int64_t free_mem, total_mem;
  char    arch[32];
} gh_devinfo;

/* ---- operator command -------------------------------------------------- */

enum gh_opcode {
  GH_OP_NOP = 0,
  GH_OP_ELEM_BIN = 1,   /* elembinop.<fn>_{vv,vs,sv,ss}_f{32,64}              */
  GH_OP_ELEM_UNARY = 2, /* elemunaryop.<fn>_f{32,64}                          */
  GH_OP_BCAST_BIN = 3,  /* Broadcast{Add,Sub,HadamardProd,...}: fused repeat  */
  GH_OP_MEMCPY_D2D = 4, /* Engine.memcpy (cuda/engine.go:129-131)             */
  GH_OP_GEMM = 5,       /* Engine.MatMul / BatchedMatMul (cuda/linalg.go:110) */
  GH_OP_GEMV = 6,       /* Engine.MatVecMul (cuda/linalg.go:47)               */
  GH_OP_OUTER = 7,      /* Engine.Outer (cuda/linalg.go:232)                  */
  GH_OP_CONV2D = 8,     /* ops/nn/convolution_cuda.go:95-121                  */
  GH_OP_MAXPOOL2D = 9,  /* ops/nn/maxpool_cuda.go:94-111                      */
  GH_OP_BN_INFER = 10,  /* ops/nn/batchnorm_cuda.go:101-111 (CPU semantics)   */
  GH_OP_RELU = 11,      /* ops/nn/activation_cuda.go:72-94; nn.go:136-163     */
  GH_OP_LEAKY_RELU = 12,/* nn.go:83-131                                       */
  GH_OP_SOFTMAX = 13,   /* op_softmax.go:99-128                               */
  GH_OP_HAS_NAN = 14,   /* misc.hasNaN (cuda/engine.go:144-166)               */
  GH_OP_HAS_INF = 15,   /* misc.hasInf (cuda/engine.go:169-191)               */
  GH_OP_FILL = 16,      /* Memset of a float value                            */
  /* backward passes and the training-mode BatchNorm forward */
  GH_OP_MAXPOOL2D_BWD = 17,     /* ops/nn/maxpool_cuda.go:177-188; CPU op_nn.go:1042-1093      */
  GH_OP_CONV2D_BWD_DATA = 18,   /* ops/nn/convolution_cuda.go:192-229; CPU col2im op_nn.go:605 */
  GH_OP_CONV2D_BWD_FILTER = 19, /* ops/nn/convolution_cuda.go:230-267                          */
  GH_OP_BN_TRAIN = 20,          /* ops/nn/batchnorm_cuda.go:87-100; CPU op_nn.go:1489-1635     */
  GH_OP_BN_BWD = 21,            /* ops/nn/batchnorm_cuda.go:192-219; CPU op_nn.go:1834-1943    */
  GH_OP_SOFTMAX_BWD = 22,       /* softmaxDiffOp, op_softmax.go:266-279                        */
  GH_OP_SOLVER_STEP = 23,       /* Vanilla/RMSProp/Adam Step on a float32 tensor, solvers.go:273-870 */
  GH_OP_RAND_UNIFORM = 24,      /* the random source of Dropout (nn.go:71-77), generated on the device */
  GH_OP_DROPOUT = 25,           /* dropoutOp.do, op_dropout.go:107-132; ops/nn/dropout_cuda.go    */
  GH_OP_DROPOUT_BWD = 26,       /* dropoutDiffOp, op_dropout.go:205-238                            */
  GH_OP_RELU_BWD = 27,          /* activation backward, ops/nn/activation_cuda.go:130-153; CPU: dy * (x >= 0) */
  GH_OP__COUNT
};

/* GH_OP_SOLVER_STEP: which solver (flags FN field) */
enum gh_solver { GH_SOLVER_VANILLA = 0, GH_SOLVER_RMSPROP = 1, GH_SOLVER_ADAM = 2, GH_SOLVER__COUNT };

/* flags for GH_OP_ELEM_BIN / GH_OP_BCAST_BIN: fn | mode<<8 | dtype<<12 | ... */
enum gh_binfn {
  GH_ADD = 0, GH_SUB = 1, GH_MUL = 2, GH_DIV = 3, GH_POW = 4,
  GH_LT = 5, GH_LTE = 6, GH_GT = 7, GH_GTE = 8, GH_EQ = 9, GH_NE = 10,
  GH_MOD = 11, /* Engine.Mod / ModScalar (cuda/arith.go:589-701): the reference declares the
                  methods but ships no "mod" kernel, so they fail there; math.Mod semantics */
  GH_BINFN__COUNT
};
enum gh_binmode { GH_VV = 0, GH_VS = 1, GH_SV = 2, GH_SS = 3 };
enum gh_dtype { GH_F32 = 0, GH_F64 = 1 };

/* flags for GH_OP_ELEM_UNARY: fn | dtype<<12 */
enum gh_unaryfn {
  GH_ABS = 0, GH_SIGN = 1, GH_CEIL = 2, GH_FLOOR = 3, GH_SIN = 4, GH_COS = 5,
  GH_EXP = 6, GH_LN = 7, GH_LOG2 = 8, GH_NEG = 9, GH_SQUARE = 10, GH_SQRT = 11,
  GH_INVERSE = 12, GH_INVSQRT = 13, GH_CUBE = 14, GH_TANH = 15, GH_SIGMOID = 16,
  GH_LOG1P = 17, GH_EXPM1 = 18, GH_SOFTPLUS = 19,
  GH_UNARYFN__COUNT
};

#define GH_FLAG_FN(f)        ((uint32_t)(f) & 0xffu)
#define GH_FLAG_MODE(m)      (((uint32_t)(m) & 0xfu) << 8)
#define GH_FLAG_DTYPE(d)     (((uint32_t)(d) & 0xfu) << 12)
#define GH_FLAG_TRANS_A      (1u << 16)   /* GEMM/GEMV: logical transpose of A */
#define GH_FLAG_TRANS_B      (1u << 17)   /* GEMM: logical transpose of B      */
#define GH_FLAG_SMALL_LEFT   (1u << 18)   /* BCAST_BIN: small operand on left  */
#define GH_FLAG_EXPLICIT_PAD (1u << 19)   /* MAXPOOL2D: 4-value padding given  */
#define GH_FLAG_HAS_GAMMA    (1u << 20)   /* BN_INFER: ptr[4] = gamma          */
#define GH_FLAG_HAS_BETA     (1u << 21)   /* BN_INFER: ptr[5] = beta           */
#define GH_FLAG_ACT_RELU     (1u << 22)   /* CONV2D/GEMM epilogue: x*(x>=0)    */
#define GH_FLAG_ACT_LEAKY    (1u << 23)   /* epilogue: leaky relu, alpha=f[0]  */
#define GH_FLAG_CONV_BN      (1u << 24)   /* CONV2D: BatchNorm (eval) on the result, ptr[3..6] */
#define GH_FLAG_BN_EVAL      (1u << 26)   /* BN_BWD: eval-mode gradient dy/sqrt(var+eps)       */
#define GH_FLAG_CONV_POOL2   (1u << 25)   /* CONV2D: 2x2 stride-2 unpadded MaxPool2D on the result */
#define GH_FLAG_GEMM_SOFTMAX (1u << 27)   /* GEMM: row SoftMax on the result (after the activation) */
#define GH_FLAG_CONV_PRE     (1u << 29)   /* CONV2D: the input is made on the fly from single-channel images, see below */
#define GH_FLAG_CONV_KEEP    (1u << 30)   /* CONV2D with CONV_POOL2: ptr[7] also receives the unpooled result, see below */
#define GH_FLAG_GEMM_BIAS    (1u << 28)   /* GEMM (untransposed): ptr[3] = N floats added to every row of the product (before the activation) */

/*
 * One operator.  Field use per opcode:
 *
 * ELEM_BIN    ptr[0]=A ptr[1]=B [ptr[2]=dst]  dim[0]=n
 *             without dst: vv/vs/ss write A, sv writes B (elembinop.cu:13-35);
 *             with dst the operands are left alone (the reference reaches the
 *             same state by memcpy(reuse <- a) + in-place op, cuda/arith.go:36-44)
 * ELEM_UNARY  ptr[0]=A [ptr[1]=dst]        dim[0]=n ; in place without dst
 * BCAST_BIN   ptr[0]=dst ptr[1]=big ptr[2]=small
 *             dim[0]=outer dim[1]=mid dim[2]=inner; small has `mid` elements,
 *             element (o,m,i) pairs big[o,m,i] with small[m]; float32 or
 *             float64 by the dtype field, both operands alike
 * MEMCPY_D2D  ptr[0]=dst ptr[1]=src        dim[0]=bytes
 *             either side may be pinned host memory from gh_host_alloc (the
 *             device reads or writes it over the bus): this is how a segment
 *             carries its own input uploads and result downloads
 * GEMM        ptr[0]=A ptr[1]=B ptr[2]=C   dim[0..2]=m,n,k  dim[3..5]=lda,ldb,ldc
 *             dim[6]=batch (0/1 = single)  dim[7..9]=strideA,strideB,strideC
 *             row-major; C(m x n) = op(A)(m x k) * op(B)(k x n)
 *             float64 with GH_FLAG_DTYPE(GH_F64) (no fused activation)
 *             float32 epilogue, stored bits those of the separate commands, in
 *             this order: GEMM_BIAS (ptr[3] = n floats, added to every row - the
 *             BroadcastAdd of a dense layer's bias), ACT_RELU / ACT_LEAKY,
 *             GEMM_SOFTMAX (see gh_gemm_can_softmax)
 * GEMV        ptr[0]=A ptr[1]=x ptr[2]=y   dim[0..2]=m,n,lda ; A is (m x n) row-major,
 *             y(m)=A x, or with TRANS_A y(n)=A^T x
 * OUTER       ptr[0]=x ptr[1]=y ptr[2]=A   dim[0..1]=m,n ; A(m x n) = x y^T
 * CONV2D      ptr[0]=x ptr[1]=w ptr[2]=y   dim[0..3]=B,C,H,W dim[4]=F dim[5..6]=kh,kw
 *             dim[7..8]=padH,padW dim[9..10]=strideH,strideW dim[11..12]=dilH,dilW
 *             Operators that follow the convolution can ride in its epilogue; the
 *             stored values are bit for bit those of the separate commands, in
 *             this order: CONV_BN (ptr[3]=mean ptr[4]=var, with HAS_GAMMA ptr[5]=gamma,
 *             with HAS_BETA ptr[6]=beta, f[1]=eps; BN_INFER's arithmetic per filter),
 *             then ACT_RELU / ACT_LEAKY, then CONV_POOL2 (y then has the pooled
 *             shape B,F,oh/2,ow/2; only where gh_conv2d_can_pool says so)
 *             CONV_KEEP (float32, with CONV_POOL2, only where gh_conv2d_can_keep says so): ptr[7] =
 *             a (B,F,oh,ow) tensor that also receives the convolution's result as the activation
 *             and the pool read it (after a fused BatchNorm, before the activation) - what a
 *             training step keeps for the backward pass; both tensors hold the bits of the
 *             separate commands.  Not together with CONV_PRE.
 *             CONV_PRE (float32, only where gh_conv2d_can_pre says so): the operators in front
 *             of the convolution ride along too.  ptr[0] then holds single-channel images
 *             (B,1,2H,2W) and ptr[7] C filters (C,1,3,3); the convolution's input (B,C,H,W) is
 *             MaxPool2D 2x2/2 (Rectify (Conv2d 3x3 pad 1 (ptr[0], ptr[7]))), computed where it is
 *             needed and never stored; y holds the bits the three commands would give
 * MAXPOOL2D   ptr[0]=x ptr[1]=y            dim[0..3]=B,C,H,W dim[4..5]=kh,kw
 *             dim[6..9]=padN,padS,padW,padE dim[10..11]=strideH,strideW
 *             GH_FLAG_ACT_RELU: x is read through Rectify, y = pool(x*(x>=0));
 *             the activation's result is never stored
 * BN_INFER    ptr[0]=x ptr[1]=y ptr[2]=mean ptr[3]=var [ptr[4]=gamma ptr[5]=beta]
 *             dim[0..2]=B,C,S  f[0]=eps
 * RELU        ptr[0]=x ptr[1]=y            dim[0]=n
 * LEAKY_RELU  ptr[0]=x ptr[1]=y            dim[0]=n f[0]=alpha
 * SOFTMAX     ptr[0]=x ptr[1]=y            dim[0]=rows dim[1]=cols
 * HAS_NAN/INF ptr[0]=A ptr[1]=int32 flag (device)  dim[0]=n ; flag is set to 1
 *             if any element matches, else 0
 * FILL        ptr[0]=A                     dim[0]=n f[0]=value
 * MAXPOOL2D_BWD     ptr[0]=x ptr[1]=dy ptr[2]=dx ; dims as MAXPOOL2D.  dx gets, per element,
 *             the dy of every window whose argmax it is (first maximum in scan order)
 *             GH_FLAG_ACT_RELU (float32): x is the value before a Rectify whose result was
 *             pooled; dx = (x>=0) * that gradient taken over x*(x>=0) - MaxPool2DDiff then the
 *             activation's gradient, with their bits, in one pass
 * CONV2D_BWD_DATA   ptr[0]=dy ptr[1]=w ptr[2]=dx ; dims as CONV2D (B,C,H,W describe x / dx)
 * CONV2D_BWD_FILTER ptr[0]=x ptr[1]=dy ptr[2]=dw ; dims as CONV2D
 * BN_TRAIN    ptr[0]=x ptr[1]=y ptr[2]=running_mean ptr[3]=running_var (both updated)
 *             ptr[4]=save_mean ptr[5]=save_var (outputs; save_var is the SUM of squared
 *             deviations, op_nn.go:1536-1541)  dim[0..2]=B,C,S  f[0]=eps f[1]=momentum
 * BN_BWD      ptr[0]=x ptr[1]=dy ptr[2]=dx ptr[3]=save_mean ptr[4]=save_var
 *             dim[0..2]=B,C,S  f[0]=eps ; BN_EVAL selects dx = dy/sqrt(save_var/n + eps)
 * SOFTMAX_BWD ptr[0]=y ptr[1]=dy ptr[2]=dx        dim[0]=rows dim[1]=cols
 * float64: CONV2D (no epilogue flags), MAXPOOL2D, BN_INFER, RELU, LEAKY_RELU, SOFTMAX,
 *             CONV2D_BWD_DATA, CONV2D_BWD_FILTER, MAXPOOL2D_BWD, SOFTMAX_BWD, RELU_BWD, DROPOUT,
 *             DROPOUT_BWD and SOLVER_STEP take
 *             GH_FLAG_DTYPE(GH_F64); their scalars then travel as the bit pattern of a double
 *             in a dim slot (LEAKY_RELU alpha: dim[1]; BN_INFER epsilon: dim[3]; DROPOUT and
 *             DROPOUT_BWD probability: dim[1]; SOLVER_STEP's ten constants: dim[1..10]).
 *             BN_TRAIN (epsilon dim[3], momentum dim[4]), BN_BWD (epsilon dim[3]) and
 *             RAND_UNIFORM (53 random bits: the top 53 of the same 64-bit value) likewise
 * RAND_UNIFORM ptr[0]=out [ptr[1]=state]          dim[0]=n dim[1]=seed dim[2]=offset
 *             float32 in [0,1) with 24 random bits, element i = SplitMix64 output function
 *             of seed*0xD1342543DE82EF95 + (offset + i + 1)*0x9E3779B97F4A7C15.  With a
 *             state pointer (one uint64 on the device) the offset is read from it and n
 *             is added to it afterwards, so a replayed segment draws fresh numbers
 * DROPOUT     ptr[0]=x ptr[1]=y ptr[2]=r (uniform numbers, one per element)  dim[0]=n
 *             f[0]=drop probability ; y = r < 1-p ? x/(1-p) : 0 ; BN_EVAL or p == 0: y = x
 * DROPOUT_BWD ptr[0]=y ptr[1]=dy ptr[2]=dx         dim[0]=n f[0]=drop probability
 *             dx = (p != 0 && y != 0) ? dy/p : 0   (the reference divides by p)
 * RELU_BWD    ptr[0]=x ptr[1]=dy ptr[2]=dx         dim[0]=n ; dx = dy * (x >= 0 ? 1 : 0), the bits of
 *             Gte(x, 0) followed by HadamardProd; dx may be dy (in place)
 * SOLVER_STEP ptr[0]=weights ptr[1]=grad [ptr[2]=cache (RMSProp cache / Adam m) ptr[3]=Adam v]
 *             dim[0]=n ; flags: FN = gh_solver, MODE = use mask (1 l1reg, 2 l2reg, 4 clip,
 *             8 batch) ; f[0]=eta f[1]=eps f[2]=l1reg f[3]=l2reg f[4]=clip f[5]=1/batch
 *             f[6]=decay|beta1 f[7]=(1-decay)|beta2 f[8]=1/(1-beta1^t) f[9]=1/(1-beta2^t).
 *             Adam only: [ptr[4]=two values of the weights' type in device memory (or pinned
 *             host memory) that replace f[8], f[9] when the step runs] - the bias corrections
 *             change every iteration, and read from memory they leave the command, and with
 *             it a captured segment, unchanged from step to step.
 *             Weights and caches are updated in place with the reference's sequence of
 *             tensor ops, one rounding each; grad is left untouched (the reference zeroes it)
 */
typedef struct gh_cmd {
  uint32_t opcode;
  uint32_t flags;
  uint64_t ptr[8];
  int64_t  dim[16];
  float    f[12];
} gh_cmd;

/* ---- context / device -------------------------------------------------- */

/* Engine.Init/doInit (cuda/external.go:88-170): make the device current,
 * create the stream, reserve `arena_bytes` of device memory in one hipMalloc
 * (arena_bytes may be 0: no reservation). */
GH_API int gh_init(int device, int64_t arena_bytes, gh_ctx** out);
/* Engine.Close (cuda/external.go:173-220). */
GH_API int gh_close(gh_ctx* ctx);
/* Device attribute query (cuda/external.go:135-146, cu.MemInfo :153). */
GH_API int gh_device_info(gh_ctx* ctx, gh_devinfo* out);
/* Number of visible devices; does not create a context. */
GH_API int gh_device_count(int* out);

/* Base and size of the reservation handed to the host-side BFC arena
 * (bfc.reserve, cuda/external.go:166). */
GH_API gh_devptr gh_arena_base(gh_ctx* ctx);
GH_API int64_t gh_arena_size(gh_ctx* ctx);

/* Stand-alone device allocations outside the arena (cu.MemAlloc). */
GH_API int gh_malloc(gh_ctx* ctx, int64_t bytes, gh_devptr* out);
GH_API int gh_free(gh_ctx* ctx, gh_devptr p);

/* Pinned host staging memory for H2D/D2H (the reference relies on managed
 * memory, cuda/external.go:162; explicit copies need a pinned source to be
 * asynchronous). */
GH_API int gh_host_alloc(gh_ctx* ctx, int64_t bytes, void** out);
GH_API int gh_host_free(gh_ctx* ctx, void* p);

/* Queued copies: cuda.go:141,186,199 and vm_tape_cuda.go:220-243
 * (MemcpyHtoD / MemcpyDtoH), cuda/engine.go:103-127 (Memcpy D2D).  Stream
 * ordered; the host buffer must stay valid until the next gh_sync(). */
GH_API int gh_memcpy_h2d(gh_ctx* ctx, gh_devptr dst, const void* src, int64_t bytes);
GH_API int gh_memcpy_d2h(gh_ctx* ctx, void* dst, gh_devptr src, int64_t bytes);
GH_API int gh_memcpy_d2d(gh_ctx* ctx, gh_devptr dst, gh_devptr src, int64_t bytes);

/* ---- work submission --------------------------------------------------- */

/* Validate and enqueue n operators in order (replaces the per-operator
 * BatchedContext.LaunchAndSync of cuda/arith.go:62, the cuBLAS calls at
 * cuda/linalg.go:102,223,282 and the cuDNN calls in ops/nn/ *_cuda.go files).
 * A command that fails validation enqueues nothing from that command on and
 * returns GH_EINVAL/GH_ENOFUNC with the index in gh_last_error(). */
GH_API int gh_submit(gh_ctx* ctx, const gh_cmd* cmds, int n);
/* No counterpart in the reference.  For callers that cannot allocate device
 * memory around a submit - code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc: gh_submit with the same commands, kernels and
 * results, except that the operators' scratch (split-K partial sums, reduction
 * partials, mirrored filters for the image gradient) is a fixed array of
 * GH_NOALLOC_SCRATCH_BYTES inside the library's device image instead of the
 * context's workspace, and the call itself allocates and frees nothing.  An
 * operator whose plan needs more scratch than that is refused with GH_EINVAL
 * (message names the need) and nothing from it on is enqueued; plans never
 * shrink to fit, so accepted commands store the bits gh_submit stores.  All
 * contexts on one GPU share the array: calls whose work overlaps in time on one
 * GPU (two contexts, two threads) race on it. */
#define GH_NOALLOC_SCRATCH_BYTES (16 << 20)
GH_API int gh_submit_noalloc(gh_ctx* ctx, const gh_cmd* cmds, int n);
/* Validate only: same checks as gh_submit, touches no device. */
GH_API int gh_validate(const gh_cmd* cmds, int n, char* msg, int msg_len);
/* 1 when this CONV2D command may carry GH_FLAG_CONV_POOL2 (a convolution whose
 * kernel keeps a whole pooling window in one thread), else 0.  Host only.  The
 * reference has no fused form: this folds maxpool.CUDADo
 * (ops/nn/maxpool_cuda.go:94-111) into convolution.CUDADo (convolution_cuda.go:95-121). */
GH_API int gh_conv2d_can_pool(const gh_cmd* conv);
/* 1 when gh_submit accepts GH_FLAG_CONV_PRE on this float32 CONV2D command (dims as for the
 * unfolded command: B,C,H,W describe the input that is never stored).  Host only.  The reference
 * runs the first layer of its convolutional example as three operators with two stored tensors
 * between them (examples/convnet/main.go:86-112); folded, a step has one kernel and one tensor less. */
GH_API int gh_conv2d_can_pre(const gh_cmd* conv);
/* 1 when gh_submit accepts GH_FLAG_CONV_KEEP on this float32 CONV2D command with CONV_POOL2.  Host only.
 * The reference's training graph stores the convolution's result and runs the activation and the pool
 * as operators of their own (examples/convnet/main.go:86-112); here the convolution stores both. */
GH_API int gh_conv2d_can_keep(const gh_cmd* conv);
/* Which of the library's convolution kernels gh_submit runs this float32 CONV2D command on, a
 * function of its shape, its flags and (for the filter operand's alignment) its pointers: one of
 * GH_CONV_ROUTE_*, or -1 for a command that is no float32 CONV2D.  Host only.  The reference
 * leaves this choice to cuDNN (algorithm ImplicitGemm, ops/nn/convolution_cuda.go:111-117); here
 * the summing order, and with it the bits, belong to the kernel, so tests and callers can ask.
 * The three route queries take no context: where a launcher's choice depends on the number of
 * compute units (the 1x1 kernel, the small-output product, the K slices of a product) they
 * answer for 256 of them, the MI355X's count; on a device with another count gh_submit may
 * choose differently there. */
enum gh_conv_route {
  GH_CONV_ROUTE_DIRECT = 0,     /* 3x3, at most four channels: vector ALUs               */
  GH_CONV_ROUTE_SMALL = 1,      /* 3x3 over images up to 16 x 16, K split over wavefronts */
  GH_CONV_ROUTE_PATCH = 2,      /* 3x3, 64 channels or more, patch per workgroup          */
  GH_CONV_ROUTE_WIDE = 3,       /* 3x3 over large images, persistent workgroups           */
  GH_CONV_ROUTE_POINTWISE = 4,  /* 1x1 with a small result                                */
  GH_CONV_ROUTE_TILED = 5,      /* 3x3 staged through LDS tiles (+ K slices)              */
  GH_CONV_ROUTE_GATHER = 6,     /* every other geometry                                   */
  GH_CONV_ROUTE_ROWS = 7,       /* 3x3, 32 or 64 channels, images up to 16 x 16: pixels on
                                   the MFMA rows, the 2x2 pool inside a lane's registers  */
  GH_CONV_ROUTE_ROWS1 = 8       /* 3x3, one channel, images up to 64 x 64 with even output
                                   extents: the same layout, K = 9 taps                   */
};
GH_API int gh_conv2d_route(const gh_cmd* conv);
/* The same for a CONV2D_BWD_FILTER command (ConvolutionBackwardFilter,
 * ops/nn/convolution_cuda.go:230-267): GH_WGRAD_ROUTE_*, or -1. */
enum gh_wgrad_route {
  GH_WGRAD_ROUTE_DIRECT = 0,  /* 3x3, at most four channels: reduction on the vector ALUs     */
  GH_WGRAD_ROUTE_SMALL = 1,   /* 3x3 over images up to 16 x 16: dy and x in LDS, MFMA          */
  GH_WGRAD_ROUTE_GEMM = 2,    /* every other geometry: implicit GEMM over the output pixels    */
  GH_WGRAD_ROUTE_F64 = 3,     /* float64 (its own kernels)                                     */
  GH_WGRAD_ROUTE_SINGLE_CHANNEL = 4   /* 3x3 over one channel: the image in LDS, a wavefront per filter */
};
GH_API int gh_conv2d_bwd_filter_route(const gh_cmd* conv_bwd_filter);
/* The same for a GEMM command (Engine.MatMul, cuda/linalg.go:110-229, where cuBLAS chooses):
 * GH_GEMM_ROUTE_*, or -1; *splits (may be null) receives the number of K slices whose slabs a
 * second launch adds, 1 for a single launch. */
enum gh_gemm_route {
  GH_GEMM_ROUTE_SMALL_OUTPUT = 0, /* few output tiles: K split over the wavefronts of a workgroup */
  GH_GEMM_ROUTE_TILE128 = 1,      /* 128 x 128 tiles through LDS                                 */
  GH_GEMM_ROUTE_TILE64 = 2,       /* 64 x 64 tiles (+ K slices)                                  */
  GH_GEMM_ROUTE_TILE128X64 = 3,
  GH_GEMM_ROUTE_F64 = 4           /* float64 (its own kernels)                                   */
};
GH_API int gh_gemm_route(const gh_cmd* gemm, int* splits);

/* 1 when this GEMM command may carry GH_FLAG_GEMM_SOFTMAX: a float32 product of
 * untransposed operands with at most 32 columns and at most 2048 rows, whose
 * rows are whole inside one workgroup.  The stored values are those of the
 * SOFTMAX command applied to the plain product. */
GH_API int gh_gemm_can_softmax(const gh_cmd* gemm);
/* Engine.DoWork / Signal+Sync (cuda/external.go:223-226): block until the
 * stream drains, return the sticky error. */
GH_API int gh_sync(gh_ctx* ctx);

/* Optional replay of a whole tape segment: record the submits between begin
 * and end into a hipGraph, launch it again while the segment's pointer set is
 * unchanged (arena offsets are deterministic, cuda/bfc.go:351-382). */
GH_API int gh_graph_begin(gh_ctx* ctx);
GH_API int gh_graph_end(gh_ctx* ctx, int* graph_id);
GH_API int gh_graph_launch(gh_ctx* ctx, int graph_id);
GH_API int gh_graph_destroy(gh_ctx* ctx, int graph_id);

/* ---- kernel registry ---------------------------------------------------- */

/* Engine.HasFunc (cuda/external.go:26) over the reference's kernel names,
 * e.g. "elembinop.add_vv_f32", "elemunaryop.tanh_f32", "misc.hasNaN_f32"
 * (cuda/utils.go:114-139, op_math_cuda.go:38).  Returns 1/0. */
GH_API int gh_has_func(const char* name);
/* Resolve such a name into opcode+flags for a gh_cmd. 0 on success. */
GH_API int gh_lookup_func(const char* name, uint32_t* opcode, uint32_t* flags);

/* ---- errors -------------------------------------------------------------- */

/* Engine.Errors (cuda/engine.go:141): sticky status; copies the message. */
GH_API int gh_last_error(gh_ctx* ctx, char* buf, int len);
GH_API int gh_clear_error(gh_ctx* ctx);

/* ---- timing (benchmark support; no reference counterpart) ---------------- */

/* Record a HIP event on the context's stream into slot [0,64). */
GH_API int gh_event_record(gh_ctx* ctx, int slot);
/* Milliseconds between two recorded slots (synchronises on `stop`). */
GH_API int gh_event_elapsed_ms(gh_ctx* ctx, int start, int stop, float* ms);

/* Library version string. */
GH_API const char* gh_version(void);

#ifdef __cplusplus
}
#endif
#endif /* GORGONIA_HIP_H */
