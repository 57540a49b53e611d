// extern "C" wrappers of the host mirror (include/gorgonia_host.h).
#include <cstdio>
#include <cstring>
#include <string>

#include "gorgonia_host.h"
#include "tape.hpp"

using namespace gorgonia;

struct ghh_bfc { BFC b; explicit ghh_bfc(int64_t a) : b(a) {} };
struct ghh_engine { Engine* e; bool owned; std::string err; };
struct ghh_graph { Graph g; std::string err; };
struct ghh_tape { TapeMachine* t; std::string err; ghh_engine eng; };

static Tensor to_tensor(const ghh_tensor* t) {
  Tensor r;
  r.mem = t->mem;
  r.dt = t->dtype == 0 ? Dtype::Float32 : t->dtype == 1 ? Dtype::Float64 : Dtype::Other;
  for (int i = 0; i < t->ndim && i < 8; i++) r.shape.d.push_back(t->shape[i]);
  r.manually_managed = !(t->flags & GHH_T_NOT_MANAGED);
  r.transposed = t->flags & GHH_T_TRANSPOSED;
  r.col_major = t->flags & GHH_T_COL_MAJOR;
  r.requires_iterator = t->flags & GHH_T_NEEDS_ITER;
  return r;
}

template <class H>
static int ret(H* h, const Status& s) {
  if (!s.ok()) h->err = s.msg;
  return s.code;
}

extern "C" {

// ---- bfc ---------------------------------------------------------------------
ghh_bfc* ghh_bfc_new(int64_t alignment) { return new ghh_bfc(alignment); }
void ghh_bfc_destroy(ghh_bfc* b) { delete b; }
void ghh_bfc_reserve(ghh_bfc* b, uint64_t start, int64_t size) { b->b.reserve(start, size); }
uint64_t ghh_bfc_release(ghh_bfc* b) { return b->b.release(); }
int ghh_bfc_alloc(ghh_bfc* b, int64_t size, uint64_t* addr, int64_t* oom) {
  OomError o;
  int rc = b->b.alloc(size, addr, &o);
  if (rc == 2 && oom) { oom[0] = o.reserved; oom[1] = o.allocated; }
  return rc;
}
void ghh_bfc_free(ghh_bfc* b, uint64_t addr) { b->b.free(addr); }
void ghh_bfc_coalesce(ghh_bfc* b) { b->b.coalesce(); }
void ghh_bfc_reset_allocator(ghh_bfc* b) { b->b.reset_allocator(); }
int ghh_bfc_freelist_len(ghh_bfc* b) { return b->b.freelist_len(); }
int ghh_bfc_freelist(ghh_bfc* b, uint64_t* offsets, int64_t* sizes, int cap) {
  auto fl = b->b.freelist();
  int n = 0;
  for (auto& kv : fl) {
    if (n >= cap) break;
    offsets[n] = kv.first;
    sizes[n] = kv.second;
    n++;
  }
  return (int)fl.size();
}
int64_t ghh_bfc_align(ghh_bfc* b, int64_t size) { return b->b.align(size); }
int64_t ghh_bfc_allocated(ghh_bfc* b) { return b->b.allocated(); }
int ghh_bfc_used_count(ghh_bfc* b) { return b->b.used_count(); }

// ---- engine --------------------------------------------------------------------
ghh_engine* ghh_engine_new(void) { return new ghh_engine{new Engine(), true, ""}; }
void ghh_engine_destroy(ghh_engine* e) {
  if (!e) return;
  if (e->owned) delete e->e;
  delete e;
}
int ghh_engine_init(ghh_engine* e, int device, int64_t size) { return ret(e, e->e->Init(device, size)); }
int ghh_engine_close(ghh_engine* e) { return ret(e, e->e->Close()); }
const char* ghh_engine_last_error(ghh_engine* e) { return e->err.c_str(); }
int ghh_engine_get(ghh_engine* e, int64_t size, uint64_t* mem) { return ret(e, e->e->Get(size, mem)); }
int ghh_engine_put(ghh_engine* e, uint64_t mem, int64_t size) { e->e->Put(mem, size); return 0; }
int ghh_engine_reset_allocator(ghh_engine* e) { e->e->ResetAllocator(); return 0; }
int ghh_engine_alloc_accessible(ghh_engine* e) { return e->e->AllocAccessible() ? 1 : 0; }
int ghh_engine_memset(ghh_engine* e, uint64_t mem, const void* val) { return ret(e, e->e->Memset(mem, val)); }
int ghh_engine_memclr(ghh_engine* e, uint64_t mem) { return ret(e, e->e->Memclr(mem)); }
int ghh_engine_accessible(ghh_engine* e, uint64_t mem, uint64_t* out) { return ret(e, e->e->Accessible(mem, out)); }
int ghh_engine_alloc_flags(ghh_engine* e, int32_t out[2]) {
  bool mm, cm;
  e->e->AllocFlags(&mm, &cm);
  out[0] = mm; out[1] = cm;
  return 0;
}
int ghh_engine_memcpy(ghh_engine* e, uint64_t dst, int64_t dsize, uint64_t src, int64_t ssize) {
  return ret(e, e->e->Memcpy(dst, dsize, src, ssize));
}
int ghh_engine_h2d(ghh_engine* e, uint64_t dst, const void* src, int64_t bytes) {
  Status s = e->e->MemcpyHtoD(dst, src, bytes);
  if (s.ok()) s = e->e->DoWork();  // the host buffer may be pageable: finish before returning
  return ret(e, s);
}
int ghh_engine_d2h(ghh_engine* e, void* dst, uint64_t src, int64_t bytes) {
  return ret(e, e->e->MemcpyDtoH(dst, src, bytes, true));
}
int ghh_engine_has_func(ghh_engine* e, const char* name) { return e->e->HasFunc(name) ? 1 : 0; }
int ghh_engine_elem_grid_size(ghh_engine* e, int n, int32_t out[6]) {
  GridSize g = e->e->ElemGridSize(n);
  out[0] = g.gx; out[1] = g.gy; out[2] = g.gz; out[3] = g.bx; out[4] = g.by; out[5] = g.bz;
  return 0;
}

static FuncOpts make_opts(Tensor* reuse, int safe, int incr) {
  FuncOpts o;
  o.reuse = reuse;
  o.safe = safe != 0;
  o.incr = incr != 0;
  return o;
}

int ghh_engine_binop(ghh_engine* e, int fn, const ghh_tensor* a, const ghh_tensor* b,
                     const ghh_tensor* reuse, int safe, int incr, uint64_t* ret_mem) {
  static const char* names[] = {"Add", "Sub", "Mul", "Div", "Pow", "Lt", "Lte", "Gt", "Gte", "ElEq", "ElNe"};
  Tensor ta = to_tensor(a), tb = to_tensor(b), tr;
  if (reuse) tr = to_tensor(reuse);
  FuncOpts o = make_opts(reuse ? &tr : nullptr, safe, incr);
  Tensor* r = nullptr;
  Status s = fn == 11 ? e->e->Mod(ta, tb, o, &r)
             : (fn < 0 || fn > 11) ? Status::Err(GH_ENOFUNC, "unknown function")
                                   : e->e->BinOp(fn, names[fn], ta, tb, o, &r);
  if (s.ok() && ret_mem && r) *ret_mem = r->mem;
  return ret(e, s);
}

int ghh_engine_binop_scalar(ghh_engine* e, int fn, const ghh_tensor* a, uint64_t b_mem, int left_tensor,
                            const ghh_tensor* reuse, int safe, uint64_t* ret_mem) {
  static const char* names[] = {"AddScalar", "SubScalar", "MulScalar", "DivScalar", "PowScalar", "LtScalar",
                                "LteScalar", "GtScalar", "GteScalar", "ElEqScalar", "ElNeScalar", "ModScalar"};
  if (fn < 0 || fn > 11) { e->err = "unknown function"; return GH_ENOFUNC; }
  Tensor ta = to_tensor(a), tr;
  if (reuse) tr = to_tensor(reuse);
  FuncOpts o = make_opts(reuse ? &tr : nullptr, safe, 0);
  Tensor* r = nullptr;
  Status s = e->e->BinOpScalar(fn, names[fn], ta, b_mem, left_tensor != 0, o, &r);
  if (s.ok() && ret_mem && r) *ret_mem = r->mem;
  return ret(e, s);
}

int ghh_engine_unary(ghh_engine* e, const char* op_name, const ghh_tensor* a, uint64_t dst_mem) {
  Tensor ta = to_tensor(a);
  return ret(e, e->e->UnaryTo(op_name, ta, dst_mem));
}
int ghh_engine_matmul(ghh_engine* e, const ghh_tensor* a, const ghh_tensor* b, const ghh_tensor* c) {
  Tensor ta = to_tensor(a), tb = to_tensor(b), tc = to_tensor(c);
  return ret(e, e->e->MatMul(ta, tb, tc));
}
int ghh_engine_matvecmul(ghh_engine* e, const ghh_tensor* a, const ghh_tensor* b, const ghh_tensor* c) {
  Tensor ta = to_tensor(a), tb = to_tensor(b), tc = to_tensor(c);
  return ret(e, e->e->MatVecMul(ta, tb, tc));
}
int ghh_engine_outer(ghh_engine* e, const ghh_tensor* a, const ghh_tensor* b, const ghh_tensor* c) {
  Tensor ta = to_tensor(a), tb = to_tensor(b), tc = to_tensor(c);
  return ret(e, e->e->Outer(ta, tb, tc));
}
int ghh_engine_has_nan(ghh_engine* e, const ghh_tensor* a, int* out) {
  Tensor ta = to_tensor(a);
  bool v = false;
  Status s = e->e->HasNaN(ta, &v);
  *out = v;
  return ret(e, s);
}
int ghh_engine_has_inf(ghh_engine* e, const ghh_tensor* a, int* out) {
  Tensor ta = to_tensor(a);
  bool v = false;
  Status s = e->e->HasInf(ta, &v);
  *out = v;
  return ret(e, s);
}
int ghh_engine_do_work(ghh_engine* e) { return ret(e, e->e->DoWork()); }
int ghh_engine_pending(ghh_engine* e) { return (int)e->e->PendingCommands(); }
int64_t ghh_engine_submit_calls(ghh_engine* e) { return e->e->SubmitCalls(); }

// ---- graph / tape ------------------------------------------------------------------
ghh_graph* ghh_graph_new(void) { return new ghh_graph(); }
void ghh_graph_destroy(ghh_graph* g) { delete g; }
const char* ghh_graph_last_error(ghh_graph* g) { return g->err.c_str(); }
int ghh_graph_new_tensor(ghh_graph* g, const int64_t* shape, int ndim, int dtype, const void* host,
                         int resident) {
  if (!g) return -1;
  if (ndim < 0 || ndim > 8 || (ndim > 0 && !shape)) { g->err = "NewTensor: between 0 and 8 dimensions"; return -1; }
  for (int i = 0; i < ndim; i++)
    if (shape[i] <= 0) { g->err = "NewTensor: every extent of a shape must be positive"; return -1; }
  Shape s;
  for (int i = 0; i < ndim; i++) s.d.push_back(shape[i]);
  return g->g.NewTensor(s, dtype == 1 ? Dtype::Float64 : dtype == 0 ? Dtype::Float32 : Dtype::Other, host,
                        resident != 0);
}
int ghh_graph_apply(ghh_graph* g, const ghh_op* op, const int* inputs, int n_inputs, int* out) {
  OpSpec s;
  s.kind = (OpKind)op->kind;
  s.fn = op->fn;
  s.name = std::string(op->name, strnlen(op->name, sizeof(op->name)));
  s.transA = op->trans_a != 0;
  s.transB = op->trans_b != 0;
  for (int i = 0; i < op->n_ints && i < 16; i++) s.ints.push_back(op->ints[i]);
  s.f0 = op->f0;
  s.f1 = op->f1;
  s.fs.assign(op->fs, op->fs + 10);
  std::vector<int> in(inputs, inputs + n_inputs);
  return ret(g, g->g.Apply(s, in, out));
}
int ghh_graph_let(ghh_graph* g, int node, const void* host) { return ret(g, g->g.Let(node, host)); }
int ghh_graph_read(ghh_graph* g, int node, void* host_out) { return ret(g, g->g.Read(node, host_out)); }
int ghh_graph_read_borrowed(ghh_graph* g, int node) { return ret(g, g->g.ReadBorrowed(node)); }
int ghh_graph_let_borrowed(ghh_graph* g, int node) { return ret(g, g->g.LetBorrowed(node)); }
int ghh_graph_node_shape(ghh_graph* g, int node, int64_t* shape, int cap) {
  if (node < 0 || node >= (int)g->g.Nodes().size()) return -1;
  const Shape& s = g->g.Nodes()[(size_t)node].shape;
  for (int i = 0; i < s.Dims() && i < cap; i++) shape[i] = s[i];
  return s.Dims();
}
int ghh_graph_node_dtype(ghh_graph* g, int node) {
  if (node < 0 || node >= (int)g->g.Nodes().size()) return -1;
  return (int)g->g.Nodes()[(size_t)node].dt;
}
int ghh_graph_fuse_activations(ghh_graph* g) { return g->g.FuseActivations(); }

ghh_tape* ghh_tape_new(ghh_graph* g, int graph_replay, int reupload_resident) {
  TapeOptions o;
  o.graph_replay = graph_replay != 0;
  o.replay_measured = graph_replay == 2;
  o.reupload_resident = reupload_resident != 0;
  ghh_tape* t = new ghh_tape();
  t->t = new TapeMachine(&g->g, o);
  t->eng.e = &t->t->Eng();
  t->eng.owned = false;
  return t;
}
ghh_tape* ghh_lisp_new(ghh_graph* g, int reupload_resident) {
  if (!g) return nullptr;
  TapeOptions o;
  o.node_at_a_time = true;
  o.reupload_resident = reupload_resident != 0;
  ghh_tape* t = new ghh_tape();
  t->t = new TapeMachine(&g->g, o);
  t->eng.e = &t->t->Eng();
  t->eng.owned = false;
  return t;
}
ghh_tape* ghh_tape_new_with_engine(ghh_graph* g, ghh_engine* e, int graph_replay, int reupload_resident) {
  if (!g || !e || !e->e) return nullptr;
  TapeOptions o;
  o.graph_replay = graph_replay != 0;
  o.replay_measured = graph_replay == 2;
  o.reupload_resident = reupload_resident != 0;
  ghh_tape* t = new ghh_tape();
  t->t = new TapeMachine(&g->g, o, e->e);
  t->eng.e = e->e;
  t->eng.owned = false;
  return t;
}
void ghh_tape_destroy(ghh_tape* t) {
  if (!t) return;
  delete t->t;
  delete t;
}
const char* ghh_tape_last_error(ghh_tape* t) { return t ? t->err.c_str() : "null machine handle"; }
// (a null handle - a machine that was never made, or one already destroyed by the caller - is an argument error)
int ghh_tape_init(ghh_tape* t, int device) { return t ? ret(t, t->t->Init(device)) : GH_EINVAL; }
int ghh_tape_compile_only(ghh_tape* t) { return t ? ret(t, t->t->Compile()) : GH_EINVAL; }
int ghh_tape_run_all(ghh_tape* t) { return t ? ret(t, t->t->RunAll()) : GH_EINVAL; }
int ghh_tape_run_all_n(ghh_tape* t, int n) {
  if (!t) return GH_EINVAL;
  for (int i = 0; i < n; i++) {
    const int rc = ret(t, t->t->RunAll());
    if (rc) return rc;
  }
  return 0;
}
int ghh_tape_watch(ghh_tape* t, int nan, int inf) {
  if (!t) return GH_EINVAL;
  t->t->SetWatch(nan != 0, inf != 0);
  return 0;
}
int ghh_tape_reset(ghh_tape* t) { return t ? ret(t, t->t->Reset()) : GH_EINVAL; }
int ghh_tape_close(ghh_tape* t) { return t ? ret(t, t->t->Close()) : GH_EINVAL; }
int64_t ghh_tape_gpumem(ghh_tape* t) { return t ? t->t->GpuMem() : 0; }
int ghh_tape_segments(ghh_tape* t) { return t ? t->t->Segments() : 0; }
int ghh_tape_graph_launches(ghh_tape* t) { return t ? t->t->GraphLaunches() : 0; }
int64_t ghh_tape_submit_calls(ghh_tape* t) { return t ? t->t->Eng().SubmitCalls() : 0; }
uint64_t ghh_tape_register_address(ghh_tape* t, int node) { return t ? t->t->RegisterAddress(node) : 0; }
const void* ghh_tape_read_buffer(ghh_tape* t, int node) { return t ? t->t->ReadBuffer(node) : nullptr; }
void* ghh_tape_input_buffer(ghh_tape* t, int node) { return t ? t->t->InputBuffer(node) : nullptr; }
int ghh_tape_program_string(ghh_tape* t, char* buf, int cap) {
  if (!t) return 0;
  std::string s = t->t->ProgramString();
  if (buf && cap > 0) snprintf(buf, (size_t)cap, "%s", s.c_str());
  return (int)s.size();
}
ghh_engine* ghh_tape_engine(ghh_tape* t) { return t ? &t->eng : nullptr; }
int ghh_tape_segment_verdict(ghh_tape* t, int segment) { return t ? t->t->SegmentVerdict(segment) : 0; }
void ghh_tape_phase_ns(ghh_tape* t, int64_t* out3) { if (t) t->t->PhaseNs(out3); }

}  // extern "C"
