/*
 * gorgonia_host.h - C view of libgorgonia_host.so, the C++ host mirror of
 * Gorgonia's device engine (package cuda: Engine/External/Arena/bfc), of the
 * operators with a device path (CUDADoer) and of the tape machine's segment
 * runner.  The Go toolchain is not available in this build's environment, so
 * the logic a Go shim would hold lives here in C++; it reaches the GPU only
 * through the C ABI of gorgonia_hip.h.  These wrappers exist so that tests and
 * the benchmark can drive that logic from Python via ctypes.
 *
 * Status convention: 0 = ok, otherwise a GH_E* code; the message of the last
 * failure on a handle is returned by the *_last_error call of its family.
 */
#ifndef GORGONIA_HOST_H
#define GORGONIA_HOST_H

#include <stdint.h>

#include "gorgonia_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Dense device tensor descriptor (tensor.Dense with engine-owned memory). */
typedef struct ghh_tensor {
  uint64_t mem;
  int32_t  dtype;        /* 0 float32, 1 float64, 2 other (rejected, cuda/utils.go:62-72) */
  int32_t  ndim;         /* 0 = scalar */
  int64_t  shape[8];
  uint32_t flags;        /* GHH_T_* */
} ghh_tensor;

#define GHH_T_NOT_MANAGED  1u  /* host memory: !IsManuallyManaged (cuda/linalg.go:19-29) */
#define GHH_T_TRANSPOSED   2u  /* DataOrder.IsTransposed (cuda/linalg.go:57,135) */
#define GHH_T_NEEDS_ITER   4u  /* RequiresIterator (cuda/utils.go:83-89) */
#define GHH_T_COL_MAJOR    8u  /* DataOrder.IsColMajor (cuda/linalg.go:57-75,118-160) */

/* ---- bfc: cuda/bfc.go, cuda/bfc_test.go (no GPU needed) ------------------- */
typedef struct ghh_bfc ghh_bfc;
GH_API ghh_bfc* ghh_bfc_new(int64_t alignment);                       /* newBFC */
GH_API void ghh_bfc_destroy(ghh_bfc* b);
GH_API void ghh_bfc_reserve(ghh_bfc* b, uint64_t start, int64_t size); /* reserve */
GH_API uint64_t ghh_bfc_release(ghh_bfc* b);                          /* release */
/* alloc: 0 ok, 1 size <= 0, 2 out of memory (oom[0]=reserved, oom[1]=allocated) */
GH_API int ghh_bfc_alloc(ghh_bfc* b, int64_t size, uint64_t* addr, int64_t* oom);
GH_API void ghh_bfc_free(ghh_bfc* b, uint64_t addr);
GH_API void ghh_bfc_coalesce(ghh_bfc* b);
GH_API void ghh_bfc_reset_allocator(ghh_bfc* b);                      /* Engine.ResetAllocator */
GH_API int ghh_bfc_freelist_len(ghh_bfc* b);
/* copies up to cap (offset, size) pairs in address order; returns the count */
GH_API int ghh_bfc_freelist(ghh_bfc* b, uint64_t* offsets, int64_t* sizes, int cap);
GH_API int64_t ghh_bfc_align(ghh_bfc* b, int64_t size);
GH_API int64_t ghh_bfc_allocated(ghh_bfc* b);
GH_API int ghh_bfc_used_count(ghh_bfc* b);

/* ---- engine: cuda.Engine ----------------------------------------------------- */
typedef struct ghh_engine ghh_engine;
GH_API ghh_engine* ghh_engine_new(void);
GH_API void ghh_engine_destroy(ghh_engine* e);
GH_API int ghh_engine_init(ghh_engine* e, int device, int64_t size);     /* Engine.Init */
GH_API int ghh_engine_close(ghh_engine* e);                              /* Engine.Close */
GH_API const char* ghh_engine_last_error(ghh_engine* e);
GH_API int ghh_engine_get(ghh_engine* e, int64_t size, uint64_t* mem);   /* Arena.Get */
GH_API int ghh_engine_put(ghh_engine* e, uint64_t mem, int64_t size);    /* Arena.Put */
GH_API int ghh_engine_reset_allocator(ghh_engine* e);
GH_API int ghh_engine_alloc_accessible(ghh_engine* e);                   /* AllocAccessible */
/* Memset, Memclr, Accessible: "not implemented" in the reference (cuda/engine.go:93-99,
 * 130-132, a panic there); GH_ENOFUNC with that message here. */
GH_API int ghh_engine_memset(ghh_engine* e, uint64_t mem, const void* val);
GH_API int ghh_engine_memclr(ghh_engine* e, uint64_t mem);
GH_API int ghh_engine_accessible(ghh_engine* e, uint64_t mem, uint64_t* out);
/* AllocFlags (cuda/engine.go:81-83): out[0] = manually managed, out[1] = column-major tag */
GH_API int ghh_engine_alloc_flags(ghh_engine* e, int32_t out[2]);
GH_API int ghh_engine_memcpy(ghh_engine* e, uint64_t dst, int64_t dsize, uint64_t src, int64_t ssize);
GH_API int ghh_engine_h2d(ghh_engine* e, uint64_t dst, const void* src, int64_t bytes);
GH_API int ghh_engine_d2h(ghh_engine* e, void* dst, uint64_t src, int64_t bytes);
GH_API int ghh_engine_has_func(ghh_engine* e, const char* name);         /* HasFunc */
GH_API int ghh_engine_elem_grid_size(ghh_engine* e, int n, int32_t out[6]);
/* arithmetic / comparison: fn is a gh_binfn (11 = Mod, which has no kernel).
 * reuse may be NULL; safe != 0 without reuse is the reference's error. */
GH_API int ghh_engine_binop(ghh_engine* e, int fn, const ghh_tensor* a, const ghh_tensor* b,
                            const ghh_tensor* reuse, int safe, int incr, uint64_t* ret_mem);
GH_API int ghh_engine_binop_scalar(ghh_engine* e, int fn, const ghh_tensor* a, uint64_t b_mem,
                                   int left_tensor, const ghh_tensor* reuse, int safe,
                                   uint64_t* ret_mem);
GH_API int ghh_engine_unary(ghh_engine* e, const char* op_name, const ghh_tensor* a, uint64_t dst_mem);
GH_API int ghh_engine_matmul(ghh_engine* e, const ghh_tensor* a, const ghh_tensor* b, const ghh_tensor* c);
GH_API int ghh_engine_matvecmul(ghh_engine* e, const ghh_tensor* a, const ghh_tensor* b, const ghh_tensor* c);
GH_API int ghh_engine_outer(ghh_engine* e, const ghh_tensor* a, const ghh_tensor* b, const ghh_tensor* c);
GH_API int ghh_engine_has_nan(ghh_engine* e, const ghh_tensor* a, int* out);
GH_API int ghh_engine_has_inf(ghh_engine* e, const ghh_tensor* a, int* out);
GH_API int ghh_engine_do_work(ghh_engine* e);                            /* DoWork / Signal */
GH_API int ghh_engine_pending(ghh_engine* e);        /* commands recorded, not yet submitted */
GH_API int64_t ghh_engine_submit_calls(ghh_engine* e);

/* ---- graph + tape machine ------------------------------------------------------ */
typedef struct ghh_graph ghh_graph;
typedef struct ghh_tape ghh_tape;

/* op kinds follow gorgonia::OpKind (host/tape.hpp) */
typedef struct ghh_op {
  int32_t kind;
  int32_t fn;
  char    name[24];
  int32_t trans_a, trans_b;
  int32_t n_ints;
  int64_t ints[16];
  double  f0;
  double  f1;      /* second scalar parameter (BatchNorm momentum) */
  double  fs[10];  /* SolverStep: the constants of GH_OP_SOLVER_STEP's f[0..9] */
} ghh_op;

GH_API ghh_graph* ghh_graph_new(void);
GH_API void ghh_graph_destroy(ghh_graph* g);
GH_API const char* ghh_graph_last_error(ghh_graph* g);
/* NewTensor + WithValue: an input bound to host memory.  Returns the node, or -1 (message in
 * ghh_graph_last_error) for more than 8 dimensions or an extent that is not positive. */
GH_API int ghh_graph_new_tensor(ghh_graph* g, const int64_t* shape, int ndim, int dtype,
                                const void* host, int resident);
GH_API int ghh_graph_apply(ghh_graph* g, const ghh_op* op, const int* inputs, int n_inputs, int* out);
GH_API int ghh_graph_let(ghh_graph* g, int node, const void* host);
GH_API int ghh_graph_read(ghh_graph* g, int node, void* host_out);
/* Read without the last host copy (op.go:readOp rebinds the Value a Read points at; here the
 * caller borrows the machine's buffer instead): after every RunAll the node's value is in
 * pinned host memory the machine owns, at ghh_tape_read_buffer(t, node) - the same address for
 * the machine's lifetime, overwritten by the next run, freed by ghh_tape_close.  The producing
 * kernel or a staging copy inside the segment writes it there; nothing is copied afterwards. */
GH_API int ghh_graph_read_borrowed(ghh_graph* g, int node);
/* Let without the host-to-host copy (the counterpart of ghh_graph_read_borrowed for inputs): the
 * input's value is what the caller has written to ghh_tape_input_buffer(t, node) - pinned host
 * memory the machine owns, one address for its life - when a run uploads it.  A data loader
 * that decodes a batch straight into that buffer saves the copy ghh_graph_let's value takes. */
GH_API int ghh_graph_let_borrowed(ghh_graph* g, int node);
GH_API int ghh_graph_node_shape(ghh_graph* g, int node, int64_t* shape, int cap);
/* Node.Dtype(): 0 float32, 1 float64, 2 other; -1 for a bad node id */
GH_API int ghh_graph_node_dtype(ghh_graph* g, int node);
GH_API int ghh_graph_fuse_activations(ghh_graph* g);

/* graph_replay: 0 every segment is submitted command by command on every run;
 * 1 a segment whose commands repeat is captured into a hipGraph on its second
 * run and replayed from then on; 2 as 1, but the machine first times two plain
 * runs and two replays of the segment and keeps the quicker way
 * (ghh_tape_segment_verdict tells which).  reupload_resident: resident inputs
 * are uploaded on every run like all others (vm_tape_cuda.go:220-243). */
GH_API ghh_tape* ghh_tape_new(ghh_graph* g, int graph_replay, int reupload_resident);
/* NewLispMachine(g) (vm_genera.go:43-120), forward execution only: the same handle type and calls
 * as a tape machine, but every node is submitted and waited for on its own when it is reached
 * (vm_genera.go:144) and no operator overwrites an input.  It exists for what the reference uses
 * its second machine for in tests: run one graph on both, require equal values. */
GH_API ghh_tape* ghh_lisp_new(ghh_graph* g, int reupload_resident);
/* NewTapeMachine(g, WithEngine(e)) (vm.go:318-329): the machine runs on the
 * caller's engine, which must be initialised (ghh_engine_init) before
 * ghh_tape_init and must outlive the machine.  Registers come out of that
 * engine's arena and go back to it on ghh_tape_reset / ghh_tape_close; the
 * engine itself stays open.  ghh_tape_init's device argument is ignored, and
 * it returns GH_ESTATE for an engine that is not initialised, GH_EOOM when the
 * arena has less free space than the program's registers need.  Machines on
 * one engine run one after the other. */
GH_API ghh_tape* ghh_tape_new_with_engine(ghh_graph* g, ghh_engine* e, int graph_replay, int reupload_resident);
GH_API void ghh_tape_destroy(ghh_tape* t);
GH_API const char* ghh_tape_last_error(ghh_tape* t);
GH_API int ghh_tape_init(ghh_tape* t, int device);   /* compile + engine init */
GH_API int ghh_tape_run_all(ghh_tape* t);            /* RunAll */
/* WithNaNWatch() / WithInfWatch() (vm.go:138-166; vm_tape.go:271-315): from the next RunAll on, every
 * operator is submitted and waited for on its own and its value searched for NaN / +-Inf on the device;
 * the run stops at the first hit with GH_ESTATE and "NaN found in value. Node: <operator>(<id>)" (or
 * "Inf found ..."), the operators behind it - weight updates included - not run.  nan = inf = 0 turns
 * the watch off again.  The values checked are those of the graph's commands: after
 * ghh_graph_fuse_activations a folded command is checked as one (a max-pool folded behind a convolution
 * drops a NaN the convolution produced), so watch graphs that were not folded. */
GH_API int ghh_tape_watch(ghh_tape* t, int nan, int inf);
/* n RunAll calls one after the other, stopping at the first error: the loop of a compiled caller
 * (`for i := 0; i < n; i++ { vm.RunAll(); vm.Reset() }`, cuda_test.go:125-141) without an
 * interpreter's call overhead between the steps; every step still ends with its results on the host. */
GH_API int ghh_tape_run_all_n(ghh_tape* t, int n);
GH_API int ghh_tape_reset(ghh_tape* t);              /* Reset */
GH_API int ghh_tape_close(ghh_tape* t);
GH_API int64_t ghh_tape_gpumem(ghh_tape* t);
GH_API int ghh_tape_segments(ghh_tape* t);
GH_API int ghh_tape_graph_launches(ghh_tape* t);
GH_API int64_t ghh_tape_submit_calls(ghh_tape* t);
GH_API uint64_t ghh_tape_register_address(ghh_tape* t, int node);
/* Where a ghh_graph_read_borrowed node's value lies after RunAll; NULL for any other node. */
GH_API const void* ghh_tape_read_buffer(ghh_tape* t, int node);
/* Where a ghh_graph_let_borrowed input's next value is to be written; NULL for any other node. */
GH_API void* ghh_tape_input_buffer(ghh_tape* t, int node);
GH_API int ghh_tape_program_string(ghh_tape* t, char* buf, int cap);
GH_API ghh_engine* ghh_tape_engine(ghh_tape* t);     /* borrowed: do not destroy */
/* How segment `segment` of the last run executes: 0 undecided (still being timed, or graph_replay
 * is not 2), 1 plain submits, 2 graph replay. */
GH_API int ghh_tape_segment_verdict(ghh_tape* t, int segment);
/* Host time of the last RunAll in nanoseconds: out3[0] the whole call, out3[1]
 * inside gh_submit / gh_graph_launch, out3[2] waiting for the device. */
GH_API void ghh_tape_phase_ns(ghh_tape* t, int64_t* out3);
/* compile only (no device): lets CPU tests inspect the instruction stream */
GH_API int ghh_tape_compile_only(ghh_tape* t);

#ifdef __cplusplus
}
#endif
#endif /* GORGONIA_HOST_H */
