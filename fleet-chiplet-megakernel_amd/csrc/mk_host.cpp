// Host side of the persistent decode megakernel: records the PersistentKernel task
// list, lowers it to the stage program the kernel walks, owns intermediate tensors
// and runtime state, and launches the kernel cooperatively.
//
// Replaces, for the decode path: src/kernel/graph.cc (register_task, attach_*,
// shuffle_tensors), src/kernel/task_register.cc (per-task validation),
// src/kernel/runtime.cc (register_mugraph / print_task_graph) and the host half of
// include/mirage/persistent_kernel/persistent_kernel.cuh:1960-2429.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <array>
#include <map>
#include <numeric>
#include <string>
#include <vector>

#include "../../include/fleet_mk.h"
#include "mk_types.h"


namespace {

thread_local std::string g_err;

int fail(int code, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

#define HIP_TRY(expr)                                                                         \
  do {                                                                                        \
    hipError_t e_ = (expr);                                                                   \
    if (e_ != hipSuccess) return fail(MK_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

enum TensorKind { T_ATTACHED, T_OWNED, T_SHUFFLED };

struct Tensor {
  std::string name;
  int ndims = 0;
  int64_t dims[4] = {1, 1, 1, 1};
  int64_t strides[4] = {1, 1, 1, 1};
  int dtype = MK_DT_BF16;
  TensorKind kind = T_ATTACHED;
  void *ptr = nullptr;
  std::vector<int> sources;  // T_SHUFFLED
  int num_groups = 1;
  bool interleave = true;
  int io_category = 0;
  size_t elems() const {
    size_t n = 1;
    for (int i = 0; i < ndims; i++) n *= (size_t)dims[i];
    return n;
  }
};

struct Task {
  std::string name;
  int grid[3], block[3];
  std::vector<int> ops;
  std::vector<std::array<int, 3>> maps;
  std::vector<int> forloop;
  std::vector<int> params;
};

size_t dtype_size(int dt) {
  switch (dt) {
    case MK_DT_BF16:
    case MK_DT_F16: return 2;
    case MK_DT_F32:
    case MK_DT_I32: return 4;
    case MK_DT_I64:
    case MK_DT_U64: return 8;
    default: return 0;
  }
}

}  // namespace

struct mk_graph {
  mk_config cfg;
  int num_cus = 0;
  int G = 0;
  std::vector<Tensor> tensors;
  std::vector<Task> tasks;
  std::vector<Task> ltasks;  // what lower() walks: `tasks` with composite tasks expanded
  bool compiled = false;
  bool host_only = false;  // created with device < 0: records, validates, lowers and emits the task graph, never launches
  std::vector<void *> allocs;
  std::vector<void *> host_allocs;
  std::vector<MkStage> stages;
  std::vector<std::string> stage_desc;
  MkRuntime h_rt;
  MkRuntime *d_rt = nullptr;
  MkStage *d_stages = nullptr;
  MkSync *d_sync = nullptr;
  MkSched *d_sched = nullptr;
  long long *d_timing = nullptr;
  int timing_cap = 0;
  std::string json, program_text;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  bool launch_pending = false;
  MkSync *pending_sync = nullptr;  // barrier state of the pending / last launch (the graph's own or the static scratch)
  int max_kv_heads = 1, max_qpk = 1;  // over the attention stages
  double last_ms = 0.0;
  int last_nxcd = 0, last_aborted = 0;
  int64_t weight_bytes = 0;
  int64_t packed_bytes = 0;  // matrix-core copies of the weights held by the handle
  size_t attn_cnt_n = 0;
  int num_ref_tasks = 0, num_ref_events = 0;
  int last_linear_task = -1, last_linear_stage = -1;  // lowering: the most recent linear task and the stage it became
  std::vector<int> stage_weight;      // per stage: tensor id of a LINEAR stage's weight operand (-1: none)
  std::vector<char> releasable;       // per tensor (single-weight-copy graphs, after mk_compile): the handle never reads it again
  bool single_copy = false;
  int spec_len = 0;  // guesses per decoding request (set by a find_ngram_global task)
  void *profiler_ptr = nullptr;  // the caller's profiler tensor (mk_set_profiler)
  long long profiler_cap = 0;
  int64_t row_major_bytes = 0;
};

namespace {

int dev_alloc(mk_graph *g, void **out, size_t bytes, bool zero = true) {
  if (bytes == 0) bytes = 16;
  if (g->host_only) {  // stand-in address: only its identity matters to the lowering
    *out = malloc(16);
    if (!*out) return fail(MK_EINVAL, "out of host memory");
    g->host_allocs.push_back(*out);
    return MK_OK;
  }
  HIP_TRY(hipMalloc(out, bytes));
  g->allocs.push_back(*out);
  if (zero) HIP_TRY(hipMemset(*out, 0, bytes));
  return MK_OK;
}

bool is_norm(const std::string &n) { return n == "rmsnorm" || n == "gang_rmsnorm_mi300"; }

// Classify linear-type task names: returns false if `n` is not a linear.
bool linear_kind(const std::string &n, bool *res, bool *silu, int *n_extra_inputs) {
  *res = false;
  *silu = false;
  *n_extra_inputs = 0;
  static const char *plain[] = {"linear", "gang_linear_mi300", "gang_linear_n_tiling_mi300", "gang_linear_msplit_mi300",
                                "splitk_linear_mi300"};
  static const char *with_res[] = {"linear_with_residual", "gang_linear_res_mi300", "gang_linear_res_n_tiling_mi300",
                                   "gang_linear_res_msplit_mi300"};
  static const char *fused_silu[] = {"linear_silu_mi300", "gang_linear_silu_mi300"};
  for (auto p : plain)
    if (n == p) return true;
  for (auto p : with_res)
    if (n == p) {
      *res = true;
      return true;
    }
  for (auto p : fused_silu)
    if (n == p) {
      *silu = true;
      return true;
    }
  if (n == "splitk_linear_res_atomic_mi300") {  // [input, weight, residual, workspace, done_counter, output]
    *res = true;
    *n_extra_inputs = 2;
    return true;
  }
  if (n == "gang_splitk_linear_res_mi300") {  // [input, weight, residual, workspace, output]
    *res = true;
    *n_extra_inputs = 1;
    return true;
  }
  return false;
}

int resolve_weight(mk_graph *g, int id, int64_t k, MkWeight *w, int64_t *rows_out, int *group_half) {
  const Tensor &t = g->tensors[id];
  memset(w, 0, sizeof(*w));
  if (t.ndims != 2) return fail(MK_EINVAL, "weight '%s' must be 2-D", t.name.c_str());
  if (t.dtype != MK_DT_BF16) return fail(MK_EINVAL, "weight '%s' must be bf16", t.name.c_str());
  if (t.dims[1] != k) return fail(MK_EINVAL, "weight '%s' has k=%lld, expected %lld", t.name.c_str(), (long long)t.dims[1], (long long)k);
  *rows_out = t.dims[0];
  *group_half = 0;
  if (t.kind != T_SHUFFLED) {
    if (!t.ptr) return fail(MK_EINVAL, "weight '%s' has no storage", t.name.c_str());
    w->nseg = 1;
    w->seg[0] = t.ptr;
    w->seg_rows[0] = (int)t.dims[0];
    w->group_rows = (int)t.dims[0];
    return MK_OK;
  }
  const int n = (int)t.sources.size();
  if (n > MK_MAX_SEGS) return fail(MK_EUNSUPPORTED, "shuffled weight '%s' has %d sources (max %d)", t.name.c_str(), n, MK_MAX_SEGS);
  int groups = t.interleave ? t.num_groups : 1;
  int total = 0;
  for (int i = 0; i < n; i++) {
    const Tensor &s = g->tensors[t.sources[i]];
    if (s.kind == T_SHUFFLED || !s.ptr) return fail(MK_EINVAL, "source '%s' of '%s' has no storage", s.name.c_str(), t.name.c_str());
    if (s.dims[0] % groups) return fail(MK_EINVAL, "source '%s' rows %lld not divisible by %d groups", s.name.c_str(), (long long)s.dims[0], groups);
    w->seg[i] = s.ptr;
    w->seg_rows[i] = (int)(s.dims[0] / groups);
    total += w->seg_rows[i];
  }
  w->nseg = n;
  w->group_rows = total;
  if (n == 2 && w->seg_rows[0] == w->seg_rows[1]) *group_half = w->seg_rows[0];
  return MK_OK;
}

std::string fmt(const char *f, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, f);
  vsnprintf(buf, sizeof(buf), f, ap);
  va_end(ap);
  return buf;
}

// operands are listed inputs first, outputs last: how many of a task's operands are outputs
int num_outputs(const Task &t) {
  if (t.name == "argmax_partial") return 2;
  if (t.name == "gang_attn_split_kv_mi300") return 3;
  if (t.name == "paged_attention_ck_fmha_split_kv_mi300" || t.name == "paged_attention_split_kv_mi300") return 2;
  if (t.name == "moe_topk_softmax_mi300") return 3;
  return 1;
}

// Lower one linear-type task (optionally preceded by a norm task whose output it consumes, optionally
// followed by a silu_mul consuming its output) into stages.
int lower_linear(mk_graph *g, size_t &i) {
  const Task *norm = nullptr;
  if (is_norm(g->ltasks[i].name)) {
    norm = &g->ltasks[i];
    i++;
  }
  const Task &lt = g->ltasks[i];
  bool res, silu;
  int extra;
  if (!linear_kind(lt.name, &res, &silu, &extra)) return fail(MK_EINVAL, "internal: '%s' is not a linear", lt.name.c_str());
  const size_t need_ops = 3 + (res ? 1 : 0) + extra;
  if (lt.ops.size() != need_ops) return fail(MK_EINVAL, "task '%s' expects %zu operands, got %zu", lt.name.c_str(), need_ops, lt.ops.size());
  const int in_id = lt.ops[0], w_id = lt.ops[1];
  int res_id = res ? lt.ops[2] : -1, out_id = lt.ops.back();
  size_t consumed_linear = 1;
  if (lt.name == "splitk_linear_mi300" && g->tensors[out_id].dtype == MK_DT_F32) {
    // the reference's two-task split-K: partial products into an fp32 workspace, then splitk_reduce [workspace, residual,
    // output] sums the slices and adds the residual.  The pair is one stage here; the workspace is never written.
    const Task *rd = i + 1 < g->ltasks.size() ? &g->ltasks[i + 1] : nullptr;
    if (!rd || rd->name != "splitk_reduce_mi300" || rd->ops.size() != 3 || rd->ops[0] != out_id)
      return fail(MK_EUNSUPPORTED, "splitk_linear_mi300 into an fp32 workspace must be followed by splitk_reduce_mi300 over that workspace");
    res = true;
    res_id = rd->ops[1];
    out_id = rd->ops[2];
    consumed_linear = 2;
  }
  const Tensor &tin = g->tensors[in_id];
  Tensor &tout = g->tensors[out_id];
  if (tin.ndims != 2 || tout.ndims != 2) return fail(MK_EINVAL, "task '%s': input/output must be 2-D", lt.name.c_str());
  if (tin.dtype != MK_DT_BF16 || tout.dtype != MK_DT_BF16) return fail(MK_EINVAL, "task '%s': activations must be bf16", lt.name.c_str());
  MkStage st;
  memset(&st, 0, sizeof(st));
  st.op = MK_OP_LINEAR;
  st.k = (int)tin.dims[1];
  if (st.k % 8) return fail(MK_EINVAL, "task '%s': reduction length %d must be a multiple of 8", lt.name.c_str(), st.k);
  if (g->cfg.max_num_batched_tokens > 1 && st.k % 32) return fail(MK_EINVAL, "task '%s': reduction length %d must be a multiple of 32 when more than one token is batched", lt.name.c_str(), st.k);
  int64_t rows;
  int half;
  int rc = resolve_weight(g, w_id, st.k, &st.w, &rows, &half);
  if (rc) return rc;
  st.n = (int)rows;
  st.eps = g->cfg.rms_eps;
  // a following silu_mul over this linear's (library-owned) output is folded into the epilogue
  const Task *act = nullptr;
  if (!silu && !res && i + 1 < g->ltasks.size() && g->ltasks[i + 1].name == "silu_mul" && g->ltasks[i + 1].ops.size() == 2 &&
      g->ltasks[i + 1].ops[0] == out_id && tout.kind == T_OWNED) {
    act = &g->ltasks[i + 1];
  }
  int final_out = out_id;
  if (silu || act) {
    st.flags |= MK_F_SILU;
    if (act) {
      final_out = act->ops[1];
      const int groups = act->grid[0] * act->grid[1] * act->grid[2];
      if (groups <= 0 || (rows / 2) % groups) return fail(MK_EINVAL, "silu_mul grid %d does not divide %lld outputs", groups, (long long)(rows / 2));
      st.silu_half = (int)(rows / 2 / groups);
    } else {
      st.silu_half = half ? half : 128;  // physically interleaved weight: reference layout [gate128 ; up128]
    }
    if (half && half != st.silu_half) return fail(MK_EINVAL, "task '%s': shuffled group half %d != activation half %d", lt.name.c_str(), half, st.silu_half);
    if (rows % (2 * st.silu_half)) return fail(MK_EINVAL, "task '%s': %lld rows not a multiple of %d", lt.name.c_str(), (long long)rows, 2 * st.silu_half);
  }
  const Tensor &tfo = g->tensors[final_out];
  const int n_out = (st.flags & MK_F_SILU) ? st.n / 2 : st.n;
  if (tfo.ndims != 2 || tfo.dims[1] < n_out) return fail(MK_EINVAL, "task '%s': output '%s' has %lld columns, need %d", lt.name.c_str(), tfo.name.c_str(), (long long)tfo.dims[1], n_out);
  if (tin.dims[0] < g->cfg.max_num_batched_tokens || tfo.dims[0] < g->cfg.max_num_batched_tokens)
    return fail(MK_EINVAL, "task '%s': activations need at least max_num_batched_tokens=%d rows", lt.name.c_str(), g->cfg.max_num_batched_tokens);
  st.in = tin.ptr;
  st.ld_in = (int)tin.strides[0];
  st.out = tfo.ptr;
  st.ld_out = (int)tfo.strides[0];
  if (res) {
    const Tensor &tr = g->tensors[res_id];
    if (tr.ndims != 2 || tr.dims[1] < n_out || tr.dtype != MK_DT_BF16) return fail(MK_EINVAL, "task '%s': bad residual '%s'", lt.name.c_str(), tr.name.c_str());
    st.flags |= MK_F_RES;
    st.res = tr.ptr;
    st.ld_res = (int)tr.strides[0];
  }
  if (norm) {
    const Tensor &nx = g->tensors[norm->ops[0]];
    const Tensor &nw = g->tensors[norm->ops[1]];
    const Tensor &no = g->tensors[norm->ops[2]];
    if (nx.ndims != 2 || nx.dims[1] != st.k || nw.elems() != (size_t)st.k || nw.dtype != MK_DT_BF16)
      return fail(MK_EINVAL, "task '%s': norm shapes do not match k=%d", norm->name.c_str(), st.k);
    MkStage ns;
    memset(&ns, 0, sizeof(ns));
    ns.op = MK_OP_NORM;
    ns.flags = MK_F_ONLY_MULTI;
    ns.k = st.k;
    ns.eps = g->cfg.rms_eps;
    ns.in = nx.ptr;
    ns.ld_in = (int)nx.strides[0];
    ns.norm_w = nw.ptr;
    ns.out = no.ptr;
    ns.ld_out = (int)no.strides[0];
    if (!g->stages.empty()) {
      // a plain or residual linear whose whole output this norm reads may leave its split-K sum to the norm stage
      MkStage &pl = g->stages.back();
      const bool rows_ok = (ns.k & 15) == 0 && ns.k / 8 <= 6 * MK_THREADS && (ns.ld_in & 7) == 0 && (ns.ld_out & 7) == 0 && ((uintptr_t)ns.in & 15) == 0;
      const bool res_ok = !(pl.flags & MK_F_RES) || ((pl.ld_res & 7) == 0 && ((uintptr_t)pl.res & 15) == 0);
      if (pl.op == MK_OP_LINEAR && !(pl.flags & MK_F_SILU) && pl.out == ns.in && pl.ld_out == ns.ld_in && pl.n == ns.k && rows_ok && res_ok)
        pl.flags |= MK_F_DEFER_SUM;
    }
    g->stages.push_back(ns);
    g->stage_desc.push_back(fmt("NORM[multi-token only] %s -> %s k=%d", nx.name.c_str(), no.name.c_str(), st.k));
    st.flags |= MK_F_NORM;
    st.in = nx.ptr;
    st.ld_in = (int)nx.strides[0];
    st.norm_w = nw.ptr;
    st.norm_out = no.ptr;
    st.ld_norm = (int)no.strides[0];
  }
  g->stages.push_back(st);
  g->stage_desc.push_back(fmt("LINEAR%s%s%s %s x %s -> %s n=%d k=%d segs=%d", (st.flags & MK_F_NORM) ? "+norm" : "", (st.flags & MK_F_RES) ? "+res" : "",
                              (st.flags & MK_F_SILU) ? "+silu" : "", tin.name.c_str(), g->tensors[w_id].name.c_str(), tfo.name.c_str(), st.n, st.k,
                              st.w.nseg));
  g->weight_bytes += (int64_t)st.n * st.k * 2;
  g->stage_weight.resize(g->stages.size(), -1);
  g->stage_weight.back() = w_id;
  g->last_linear_task = (int)i;
  g->last_linear_stage = (int)g->stages.size() - 1;
  i += act ? 2 : consumed_linear;
  return MK_OK;
}

// silu_mul_linear_with_residual [input [tokens, 2I], weight [H, I], residual, output]: out = silu_mul(input) W^T + residual.
// Which columns of `input` are gate and which are up:
//   * `input` was produced by the linear stage right before it through a shuffled [gate ; up] weight view: the view says so;
//   * params[0] > 0 (the builder that interleaved a physical weight passes its group size): groups of
//     [gate x params[0] ; up x params[0]];
//   * otherwise [gate | up] halves, the layout the reference task kernel reads (tasks/mi300/silu_mul_linear_mi300.cuh:40-42,
//     tasks/ampere/silu_mul_linear.cuh:78-80).
// When the producer is that linear stage and no later task reads `input`, the activation moves into the producer's
// epilogue (single rounding, like the fused gate/up task) writing a library-owned [tokens, I] tensor and the gate/up tensor
// itself is no longer written.  Otherwise a standalone activation stage reads `input`.
int lower_silu_mul_linear(mk_graph *g, size_t &i) {
  const Task &t = g->ltasks[i];
  if (t.ops.size() != 4) return fail(MK_EINVAL, "silu_mul_linear_with_residual expects 4 operands");
  const Tensor &x = g->tensors[t.ops[0]], &w = g->tensors[t.ops[1]], &r = g->tensors[t.ops[2]], &o = g->tensors[t.ops[3]];
  const int B = g->cfg.max_num_batched_tokens;
  if (x.ndims != 2 || w.ndims != 2 || r.ndims != 2 || o.ndims != 2 || x.dtype != MK_DT_BF16 || o.dtype != MK_DT_BF16 || r.dtype != MK_DT_BF16)
    return fail(MK_EINVAL, "silu_mul_linear_with_residual: operands must be 2-D bf16");
  const int I = (int)w.dims[1], H = (int)w.dims[0];
  if (x.dims[1] != 2 * (int64_t)I || o.dims[1] < H || r.dims[1] < H || x.dims[0] < B || o.dims[0] < B || r.dims[0] < B)
    return fail(MK_EINVAL, "silu_mul_linear_with_residual: input must be [tokens, 2*%d], residual/output [tokens, >=%d]", I, H);
  if (I % 8 || (B > 1 && I % 32)) return fail(MK_EINVAL, "silu_mul_linear_with_residual: intermediate size %d must be a multiple of 8 (32 when batching)", I);
  void *mid = nullptr;
  int rc = dev_alloc(g, &mid, (size_t)B * I * 2);
  if (rc) return rc;
  const bool have_producer = g->last_linear_stage >= 0 && g->last_linear_stage == (int)g->stages.size() - 1;
  MkStage *prev = have_producer ? &g->stages.back() : nullptr;
  if (prev && !(prev->op == MK_OP_LINEAR && prev->out == x.ptr && !(prev->flags & (MK_F_SILU | MK_F_RES)) && prev->n == 2 * I)) prev = nullptr;
  int half = I;
  const char *how = "[gate | up] halves";
  if (prev && prev->w.nseg == 2 && prev->w.seg_rows[0] == prev->w.seg_rows[1]) {
    half = prev->w.seg_rows[0];
    how = "groups of the producer's shuffled weight view";
  } else if (!t.params.empty() && t.params[0] > 0) {
    half = t.params[0];
    how = "groups given by the caller";
  }
  if (half <= 0 || I % half) return fail(MK_EINVAL, "silu_mul_linear_with_residual: gate/up groups of %d rows do not divide the intermediate size %d", half, I);
  // folding stops the gate/up tensor from being written: no later task may read it before some task writes it again
  // (drivers reuse one gate/up buffer for every layer)
  bool read_later = false;
  for (size_t j = i + 1; j < g->ltasks.size() && !read_later; j++) {
    const Task &lt = g->ltasks[j];
    const size_t n_in = lt.ops.size() - (size_t)num_outputs(lt);
    bool rewritten = false;
    for (size_t a = 0; a < lt.ops.size(); a++) {
      if (lt.ops[a] != t.ops[0]) continue;
      if (a < n_in) read_later = true;
      else rewritten = true;
    }
    if (rewritten) break;
  }
  if (prev && !read_later) {
    prev->flags |= MK_F_SILU;
    prev->silu_half = half;
    prev->out = mid;
    prev->ld_out = I;
    g->stage_desc.back() += fmt(" [+silu half=%d (%s) folded in from silu_mul_linear_with_residual; output is library-owned]", half, how);
  } else {
    MkStage a;
    memset(&a, 0, sizeof(a));
    a.op = MK_OP_SILU_MUL;
    a.n = I;
    a.silu_half = half;
    a.groups = I / half;
    a.in = x.ptr;
    a.ld_in = (int)x.strides[0];
    a.out = mid;
    a.ld_out = I;
    g->stages.push_back(a);
    g->stage_desc.push_back(fmt("SILU_MUL %s -> (library) n=%d half=%d (%s)", x.name.c_str(), I, half, how));
  }
  MkStage st;
  memset(&st, 0, sizeof(st));
  st.op = MK_OP_LINEAR;
  st.flags = MK_F_RES;
  st.k = I;
  int64_t rows;
  int halfw;
  rc = resolve_weight(g, t.ops[1], I, &st.w, &rows, &halfw);
  if (rc) return rc;
  st.n = (int)rows;
  st.eps = g->cfg.rms_eps;
  st.in = mid;
  st.ld_in = I;
  st.out = o.ptr;
  st.ld_out = (int)o.strides[0];
  st.res = r.ptr;
  st.ld_res = (int)r.strides[0];
  g->stages.push_back(st);
  g->stage_desc.push_back(fmt("LINEAR+res silu_mul(%s) x %s -> %s n=%d k=%d", x.name.c_str(), w.name.c_str(), o.name.c_str(), st.n, st.k));
  g->weight_bytes += (int64_t)st.n * st.k * 2;
  g->stage_weight.resize(g->stages.size(), -1);
  g->stage_weight.back() = t.ops[1];
  i++;
  return MK_OK;
}

// A merge task that closes a split-KV attention task: [lse, chunked output, final output].  Returns the final
// output's tensor id when task `j` is such a merge over the attention's chunked output, -1 otherwise.
int merge_output_of(mk_graph *g, size_t j, const char *merge_name, int chunked_out_id) {
  if (j >= g->ltasks.size()) return -1;
  const Task &m = g->ltasks[j];
  if (m.name != merge_name || m.ops.size() != 3 || m.ops[1] != chunked_out_id) return -1;
  return m.ops[2];
}

// Every attention flavour of the API becomes ONE stage (q/k-norm, RoPE, KV append, attention over a KV split the stage
// chooses itself, merge): the fused tasks directly, kv_cache_update + attention as a pair, and any of them built with
// num_kv_chunks > 1 together with the merge task that must follow (the stage writes the merge's output; the chunked
// accumulator and the log-sum-exp tensor of the reference's two-task form are never touched).
int lower_attention(mk_graph *g, size_t &i) {
  const Task &t0 = g->ltasks[i];
  int in_id, kc_id, vc_id, qn_id, kn_id, cos_id, sin_id, out_id, qws_id = -1, nq = 0, chunks = 1;
  size_t consumed = 1;
  const char *merge = nullptr;
  if (t0.name == "gang_attn_split_kv_mi300") {
    if (t0.ops.size() != 10 || t0.params.size() < 10) return fail(MK_EINVAL, "gang_attn_split_kv_mi300 expects 10 operands / 10 params");
    in_id = t0.ops[0]; kc_id = t0.ops[1]; vc_id = t0.ops[2]; qn_id = t0.ops[3]; kn_id = t0.ops[4]; cos_id = t0.ops[5]; sin_id = t0.ops[6];
    out_id = t0.ops[8]; qws_id = t0.ops[9];
    nq = t0.params[0];
    chunks = t0.params[6];
    merge = "gang_attn_merge_mi300";
  } else if (t0.name == "paged_attention" || t0.name == "paged_attention_split_kv_mi300" || t0.name == "attention" || t0.name == "single_batch_extend_attention") {
    // "attention" (python/mirage/mpk/persistent_kernel.py:587-650) is the form with one contiguous cache row range per
    // request, [requests, seq_len, kv heads, head_dim]: a paged cache whose pages are max_seq_length long
    const bool split = t0.name == "paged_attention_split_kv_mi300";
    // ("single_batch_extend_attention", persistent_kernel.py:653-730: the same cache form for the rows of a speculating
    // request -- its newest token and the guesses behind it; params 4, 5 = number of guesses, output stride)
    const size_t need_params = t0.name == "attention" ? 4u : (split ? 7u : 6u);
    if (t0.ops.size() != (split ? 9u : 8u) || t0.params.size() < need_params) return fail(MK_EINVAL, "%s: wrong number of operands / params", t0.name.c_str());
    in_id = t0.ops[0]; kc_id = t0.ops[1]; vc_id = t0.ops[2]; qn_id = t0.ops[3]; kn_id = t0.ops[4]; cos_id = t0.ops[5]; sin_id = t0.ops[6];
    out_id = t0.ops.back();
    nq = t0.params[0];
    if (split) {
      chunks = 2;  // the chunked [tokens, chunks * heads * head_dim, kv heads] output always needs the merge task
      merge = "paged_attention_split_kv_merge_mi300";
    }
  } else if (t0.name == "kv_cache_update_mi300") {
    if (t0.ops.size() != 8 || t0.params.size() < 7) return fail(MK_EINVAL, "kv_cache_update_mi300 expects 8 operands / 7 params");
    if (i + 1 >= g->ltasks.size() || g->ltasks[i + 1].name != "paged_attention_ck_fmha_split_kv_mi300")
      return fail(MK_EUNSUPPORTED, "kv_cache_update_mi300 must be followed by paged_attention_ck_fmha_split_kv_mi300");
    const Task &t1 = g->ltasks[i + 1];
    if (t1.ops.size() != 5 || t1.params.size() < 9) return fail(MK_EINVAL, "paged_attention_ck_fmha_split_kv_mi300 expects 5 operands / 9 params");
    in_id = t0.ops[0]; kc_id = t0.ops[1]; vc_id = t0.ops[2]; qn_id = t0.ops[3]; kn_id = t0.ops[4]; cos_id = t0.ops[5]; sin_id = t0.ops[6];
    qws_id = t0.ops[7];
    if (t1.ops[0] != qws_id || t1.ops[1] != kc_id || t1.ops[2] != vc_id) return fail(MK_EINVAL, "attention does not consume the q workspace / caches of the preceding kv_cache_update");
    out_id = t1.ops[3];
    nq = t0.params[0];
    chunks = t1.params[5];
    merge = "paged_attention_ck_fmha_merge_mi300";
    consumed = 2;
  } else {
    return fail(MK_EUNSUPPORTED, "attention task '%s' is not supported", t0.name.c_str());
  }
  if (chunks < 1) return fail(MK_EINVAL, "%s: num_kv_chunks=%d", t0.name.c_str(), chunks);
  if (chunks > 1) {
    const int fin = merge_output_of(g, i + consumed, merge, out_id);
    if (fin < 0) return fail(MK_EUNSUPPORTED, "%s with num_kv_chunks=%d must be followed by %s over its chunked output", t0.name.c_str(), chunks, merge);
    out_id = fin;
    consumed++;
  }
  const Tensor &tin = g->tensors[in_id], &kc = g->tensors[kc_id], &vc = g->tensors[vc_id], &to = g->tensors[out_id];
  if (kc.ndims != 4 || vc.ndims != 4) return fail(MK_EINVAL, "k/v cache must be 4-D [pages, page_size, kv_heads, head_dim]");
  const int nkv = (int)kc.dims[2], D = (int)kc.dims[3];
  if (D != 128) return fail(MK_EUNSUPPORTED, "head_dim %d: only 128 is supported", D);
  if (kc.dims[0] < g->cfg.max_num_pages || vc.dims[0] < g->cfg.max_num_pages)
    return fail(MK_EINVAL, "k/v cache holds %lld / %lld pages, fewer than max_num_pages=%d", (long long)kc.dims[0], (long long)vc.dims[0], g->cfg.max_num_pages);
  for (int d = 1; d < 4; d++)
    if (kc.dims[d] != vc.dims[d]) return fail(MK_EINVAL, "k and v cache shapes differ");
  if (kc.dtype != MK_DT_BF16 || vc.dtype != MK_DT_BF16) return fail(MK_EINVAL, "k/v cache must be bf16");
  if (kc.dims[1] != g->cfg.page_size) return fail(MK_EINVAL, "k cache page size %lld != configured %d", (long long)kc.dims[1], g->cfg.page_size);
  if (nkv <= 0 || nq % nkv) return fail(MK_EINVAL, "q heads %d not a multiple of kv heads %d", nq, nkv);
  const int qpk = nq / nkv;
  if (qpk != 4 && qpk != 8) return fail(MK_EUNSUPPORTED, "q heads per kv head = %d: supported 4 and 8", qpk);
  if (tin.ndims != 2 || tin.dims[1] != (int64_t)(nq + 2 * nkv) * D) return fail(MK_EINVAL, "attention input must be [tokens, (q+2kv)*head_dim]");
  if (to.ndims != 2 || to.dims[1] < (int64_t)nq * D) return fail(MK_EINVAL, "attention output must be [tokens, q_heads*head_dim]");
  MkStage st;
  memset(&st, 0, sizeof(st));
  st.op = MK_OP_ATTN;
  st.eps = g->cfg.rms_eps;
  st.in = tin.ptr;
  st.ld_in = (int)tin.strides[0];
  st.out = to.ptr;
  st.ld_out = (int)to.strides[0];
  st.k_cache = kc.ptr;
  st.v_cache = vc.ptr;
  st.num_q_heads = nq;
  st.num_kv_heads = nkv;
  st.head_dim = D;
  st.sm_scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
  if (qn_id >= 0 && kn_id >= 0) {
    st.flags |= MK_F_QK_NORM;
    st.q_norm_w = g->tensors[qn_id].ptr;
    st.k_norm_w = g->tensors[kn_id].ptr;
    if (g->tensors[qn_id].elems() != (size_t)D || g->tensors[kn_id].elems() != (size_t)D) return fail(MK_EINVAL, "q/k norm weights must have head_dim elements");
  }
  if (cos_id >= 0 && sin_id >= 0) {
    const Tensor &c = g->tensors[cos_id];
    if (c.ndims != 2 || c.dims[1] < D / 2 || c.dims[0] < g->cfg.max_seq_length) return fail(MK_EINVAL, "cos/sin tables must be [>=max_seq_length, >=head_dim/2]");
    st.flags |= MK_F_ROPE;
    st.cos_tab = c.ptr;
    st.sin_tab = g->tensors[sin_id].ptr;
    st.ld_cos = (int)c.strides[0];
  }
  if (qws_id >= 0) {
    st.q_ws = g->tensors[qws_id].ptr;
    st.ld_qws = (int)g->tensors[qws_id].strides[0];
  }
  if (!g->stages.empty()) {
    // a plain linear whose whole output is this stage's q/k/v rows may leave its split-K sum to this stage's row fetch
    MkStage &pl = g->stages.back();
    if (pl.op == MK_OP_LINEAR && !(pl.flags & (MK_F_SILU | MK_F_RES)) && pl.out == st.in && pl.ld_out == st.ld_in && pl.n == (nq + 2 * nkv) * D)
      pl.flags |= MK_F_DEFER_SUM;
  }
  g->stages.push_back(st);
  g->stage_desc.push_back(fmt("ATTN %s -> %s q=%d kv=%d d=%d norm=%d rope=%d", tin.name.c_str(), to.name.c_str(), nq, nkv, D, !!(st.flags & MK_F_QK_NORM),
                              !!(st.flags & MK_F_ROPE)));
  i += consumed;
  return MK_OK;
}


bool is_moe_linear(const std::string &n) {
  return n == "moe_w13_linear_mi300" || n == "moe_w2_linear_mi300" || n == "gang_moe_w13_linear_mi300" || n == "gang_moe_w2_linear_mi300";
}

// dims 0 and 1 of a [tokens, topk, width] tensor must form one contiguous run of rows
bool rows_contiguous_3d(const Tensor &t) { return t.ndims == 3 && t.strides[2] == 1 && t.strides[0] == t.dims[1] * t.strides[1]; }

// Router: moe_topk_softmax_mi300 [logits, topk_weight, routing_indices, mask].  When the per-expert linear that consumes
// the routing follows directly, single-token iterations route inside that linear and this stage runs for multi-token
// iterations only.
int lower_moe_topk(mk_graph *g, size_t &i, bool *inline_next) {
  const Task &t = g->ltasks[i];
  if (t.ops.size() != 4) return fail(MK_EINVAL, "%s expects 4 operands", t.name.c_str());
  const Tensor &lg = g->tensors[t.ops[0]], &tw = g->tensors[t.ops[1]], &ri = g->tensors[t.ops[2]], &mk = g->tensors[t.ops[3]];
  const int B = g->cfg.max_num_batched_tokens;
  if (lg.ndims != 2 || lg.dtype != MK_DT_BF16 || lg.dims[0] < B) return fail(MK_EINVAL, "%s: logits must be [tokens, experts] bf16", t.name.c_str());
  const int E = (int)lg.dims[1];
  if (E < 1 || E > MK_MOE_MAX_EXPERTS) return fail(MK_EUNSUPPORTED, "%s: %d experts (max %d)", t.name.c_str(), E, MK_MOE_MAX_EXPERTS);
  if (tw.ndims != 2 || tw.dtype != MK_DT_F32 || tw.dims[0] < B || tw.strides[1] != 1) return fail(MK_EINVAL, "%s: routing weights must be [tokens, topk] fp32", t.name.c_str());
  const int topk = (int)tw.dims[1];
  if (topk < 1 || topk > MK_MOE_MAX_TOPK || topk > E) return fail(MK_EUNSUPPORTED, "%s: top-%d of %d experts (max %d)", t.name.c_str(), topk, E, MK_MOE_MAX_TOPK);
  if (ri.ndims != 2 || ri.dtype != MK_DT_I32 || ri.dims[0] != E || ri.dims[1] < B || ri.strides[1] != 1)
    return fail(MK_EINVAL, "%s: routing indices must be [experts, tokens] int32", t.name.c_str());
  if (mk.dtype != MK_DT_I32 || mk.elems() < (size_t)E + 1) return fail(MK_EINVAL, "%s: mask must hold experts+1 int32", t.name.c_str());
  if (i + 1 >= g->ltasks.size() || !is_moe_linear(g->ltasks[i + 1].name) || g->ltasks[i + 1].ops.size() != 5 || g->ltasks[i + 1].ops[2] != t.ops[2] ||
      g->ltasks[i + 1].ops[3] != t.ops[3])
    return fail(MK_EUNSUPPORTED, "%s must be followed by the per-expert linear that consumes its routing table (it publishes the active-expert mask)", t.name.c_str());
  *inline_next = g->tensors[g->ltasks[i + 1].ops[0]].ndims == 2;
  MkStage st;
  memset(&st, 0, sizeof(st));
  st.op = MK_OP_MOE_TOPK;
  if (*inline_next) st.flags |= MK_F_ONLY_MULTI;
  st.moe_logits = lg.ptr;
  st.ld_logits = (int)lg.strides[0];
  st.moe_topk_w = (float *)tw.ptr;
  st.ld_topk_w = (int)tw.strides[0];
  st.moe_routing = (int *)ri.ptr;
  st.ld_routing = (int)ri.strides[0];
  st.moe_mask = (int *)mk.ptr;
  st.num_experts = E;
  st.topk = topk;
  g->stages.push_back(st);
  g->stage_desc.push_back(fmt("MOE_TOPK%s %s -> %s,%s experts=%d topk=%d", *inline_next ? "[multi-token only]" : "", lg.name.c_str(), tw.name.c_str(), ri.name.c_str(), E, topk));
  i++;
  return MK_OK;
}

// Per-expert linear [input, weight[E,N,K], routing_indices, mask, output[tokens,topk,N]]; input is [tokens, K] (every
// slot of a token sees the same row: W13) or [tokens, topk, K] (W2).  A directly following moe_silu_mul / moe_mul_sum_add
// over its output becomes the epilogue.
int lower_moe_linear(mk_graph *g, size_t &i, const MkStage *router) {
  const Task &t = g->ltasks[i];
  if (t.ops.size() != 5) return fail(MK_EINVAL, "%s expects 5 operands", t.name.c_str());
  const Tensor &x = g->tensors[t.ops[0]], &w = g->tensors[t.ops[1]], &ri = g->tensors[t.ops[2]], &mk = g->tensors[t.ops[3]], &y = g->tensors[t.ops[4]];
  const int B = g->cfg.max_num_batched_tokens;
  if (w.ndims != 3 || w.dtype != MK_DT_BF16 || !w.ptr || w.strides[2] != 1 || w.strides[1] != w.dims[2] || w.strides[0] != w.dims[1] * w.dims[2])
    return fail(MK_EINVAL, "%s: weight '%s' must be a contiguous [experts, rows, k] bf16 tensor", t.name.c_str(), w.name.c_str());
  const int E = (int)w.dims[0], N = (int)w.dims[1], K = (int)w.dims[2];
  if (E > MK_MOE_MAX_EXPERTS) return fail(MK_EUNSUPPORTED, "%s: %d experts (max %d)", t.name.c_str(), E, MK_MOE_MAX_EXPERTS);
  if (K % 8 || K > 4096) return fail(MK_EUNSUPPORTED, "%s: k=%d must be a multiple of 8 and at most 4096", t.name.c_str(), K);
  if (ri.ndims != 2 || ri.dtype != MK_DT_I32 || ri.dims[0] != E || ri.dims[1] < B || ri.strides[1] != 1)
    return fail(MK_EINVAL, "%s: routing indices must be [experts, tokens] int32", t.name.c_str());
  if (mk.dtype != MK_DT_I32 || mk.elems() < (size_t)E + 1) return fail(MK_EINVAL, "%s: mask must hold experts+1 int32", t.name.c_str());
  if (!rows_contiguous_3d(y) || y.dtype != MK_DT_BF16 || y.dims[0] < B || y.dims[2] < N) return fail(MK_EINVAL, "%s: output must be [tokens, topk, %d] bf16", t.name.c_str(), N);
  const int topk = (int)y.dims[1];
  if (topk < 1 || topk > MK_MOE_MAX_TOPK) return fail(MK_EUNSUPPORTED, "%s: topk=%d (max %d)", t.name.c_str(), topk, MK_MOE_MAX_TOPK);
  MkStage st;
  memset(&st, 0, sizeof(st));
  st.op = MK_OP_MOE_LINEAR;
  st.n = N;
  st.k = K;
  st.num_experts = E;
  st.topk = topk;
  st.w.nseg = 1;
  st.w.seg[0] = w.ptr;
  st.w.seg_rows[0] = st.w.group_rows = E * N;
  st.moe_routing = (int *)ri.ptr;
  st.ld_routing = (int)ri.strides[0];
  st.moe_mask = (int *)mk.ptr;
  st.in = x.ptr;
  if (x.dtype != MK_DT_BF16 || x.dims[0] < B) return fail(MK_EINVAL, "%s: input must be bf16 with at least %d token rows", t.name.c_str(), B);
  if (x.ndims == 2) {
    if (x.dims[1] != K || x.strides[1] != 1) return fail(MK_EINVAL, "%s: input must be [tokens, %d]", t.name.c_str(), K);
    st.ld_in = (int)x.strides[0];
  } else if (x.ndims == 3) {
    if (x.dims[1] != topk || x.dims[2] != K || x.strides[2] != 1) return fail(MK_EINVAL, "%s: input must be [tokens, %d, %d]", t.name.c_str(), topk, K);
    st.ld_in = (int)x.strides[0];
    st.ld_in_slot = (int)x.strides[1];
  } else {
    return fail(MK_EINVAL, "%s: input must be 2-D or 3-D", t.name.c_str());
  }
  if ((st.ld_in % 8) || (st.ld_in_slot % 8)) return fail(MK_EINVAL, "%s: input rows must be 16-byte aligned", t.name.c_str());
  st.out = y.ptr;
  st.ld_out = (int)y.strides[0];
  st.ld_out_slot = (int)y.strides[1];
  if (router) {
    st.flags |= MK_F_MOE_INLINE_TOPK;
    st.moe_logits = router->moe_logits;
    st.ld_logits = router->ld_logits;
    st.moe_topk_w = router->moe_topk_w;
    st.ld_topk_w = router->ld_topk_w;
    if (router->topk != topk || router->num_experts != E) return fail(MK_EINVAL, "%s: router has %d experts / top-%d, linear has %d / %d", t.name.c_str(), router->num_experts, router->topk, E, topk);
  }
  size_t consumed = 1;
  std::string extra;
  const Task *nx = i + 1 < g->ltasks.size() ? &g->ltasks[i + 1] : nullptr;
  if (nx && nx->name == "moe_silu_mul" && nx->ops.size() == 2 && nx->ops[0] == t.ops[4] && N % 2 == 0) {
    const Tensor &o = g->tensors[nx->ops[1]];
    if (!rows_contiguous_3d(o) || o.dtype != MK_DT_BF16 || o.dims[0] < B || o.dims[1] != topk || o.dims[2] != N / 2)
      return fail(MK_EINVAL, "moe_silu_mul: output must be [tokens, %d, %d] bf16", topk, N / 2);
    st.flags |= MK_F_SILU;
    st.out2 = o.ptr;
    st.ld_out2 = (int)o.strides[0];
    st.ld_out2_slot = (int)o.strides[1];
    consumed = 2;
    extra = "+silu -> " + o.name;
  } else if (nx && nx->name == "moe_mul_sum_add_mi300" && nx->ops.size() == 4 && nx->ops[0] == t.ops[4] && x.ndims == 3) {
    // fused for single-token iterations; the combine stage emitted by lower_moe_combine covers the others
    const Tensor &tw = g->tensors[nx->ops[1]], &r = g->tensors[nx->ops[2]], &o = g->tensors[nx->ops[3]];
    if (tw.ndims != 2 || tw.dtype != MK_DT_F32 || tw.dims[1] != topk || tw.strides[1] != 1 || r.ndims != 2 || o.ndims != 2 || r.dims[1] < N || o.dims[1] < N ||
        r.dtype != MK_DT_BF16 || o.dtype != MK_DT_BF16)
      return fail(MK_EINVAL, "moe_mul_sum_add_mi300: shapes do not match the expert outputs");
    st.flags |= MK_F_MOE_COMBINE;
    st.moe_topk_w = (float *)tw.ptr;
    st.ld_topk_w = (int)tw.strides[0];
    st.res = r.ptr;
    st.ld_res = (int)r.strides[0];
    st.out2 = o.ptr;
    st.ld_out2 = (int)o.strides[0];
    extra = "+combine(single token) -> " + o.name;
  }
  g->stages.push_back(st);
  g->stage_desc.push_back(fmt("MOE_LINEAR%s %s x %s -> %s experts=%d topk=%d n=%d k=%d%s", router ? "+route(single token)" : "", x.name.c_str(), w.name.c_str(), y.name.c_str(), E,
                              topk, N, K, extra.c_str()));
  g->weight_bytes += (int64_t)topk * N * K * 2;  // bytes a single-token iteration streams
  i += consumed;
  return MK_OK;
}

// moe_mul_sum_add_mi300 [expert outputs [tokens,topk,n], routing weights [tokens,topk], residual, output]
int lower_moe_combine(mk_graph *g, size_t &i, bool fused_single) {
  const Task &t = g->ltasks[i];
  if (t.ops.size() != 4) return fail(MK_EINVAL, "%s expects 4 operands", t.name.c_str());
  const Tensor &x = g->tensors[t.ops[0]], &tw = g->tensors[t.ops[1]], &r = g->tensors[t.ops[2]], &o = g->tensors[t.ops[3]];
  const int B = g->cfg.max_num_batched_tokens;
  if (x.ndims != 3 || x.dtype != MK_DT_BF16 || x.strides[2] != 1 || x.dims[0] < B) return fail(MK_EINVAL, "%s: input must be [tokens, topk, n] bf16", t.name.c_str());
  const int topk = (int)x.dims[1], N = (int)x.dims[2];
  if (tw.ndims != 2 || tw.dtype != MK_DT_F32 || tw.dims[1] != topk || tw.strides[1] != 1 || tw.dims[0] < B) return fail(MK_EINVAL, "%s: weights must be [tokens, %d] fp32", t.name.c_str(), topk);
  if (r.ndims != 2 || o.ndims != 2 || r.dims[1] < N || o.dims[1] < N || r.dtype != MK_DT_BF16 || o.dtype != MK_DT_BF16 || r.dims[0] < B || o.dims[0] < B)
    return fail(MK_EINVAL, "%s: residual/output must be [tokens, >=%d] bf16", t.name.c_str(), N);
  MkStage st;
  memset(&st, 0, sizeof(st));
  st.op = MK_OP_MOE_COMBINE;
  if (fused_single) st.flags |= MK_F_ONLY_MULTI;
  st.n = N;
  st.topk = topk;
  st.in = x.ptr;
  st.ld_in = (int)x.strides[0];
  st.ld_in_slot = (int)x.strides[1];
  st.moe_topk_w = (float *)tw.ptr;
  st.ld_topk_w = (int)tw.strides[0];
  st.res = r.ptr;
  st.ld_res = (int)r.strides[0];
  st.out = o.ptr;
  st.ld_out = (int)o.strides[0];
  g->stages.push_back(st);
  g->stage_desc.push_back(fmt("MOE_COMBINE%s %s * %s + %s -> %s n=%d topk=%d", fused_single ? "[multi-token only]" : "", x.name.c_str(), tw.name.c_str(), r.name.c_str(), o.name.c_str(), N, topk));
  i++;
  return MK_OK;
}

int lower(mk_graph *g) {
  g->stages.clear();
  g->stage_desc.clear();
  g->stage_weight.clear();
  g->weight_bytes = 0;
  g->last_linear_task = g->last_linear_stage = -1;
  const int B = g->cfg.max_num_batched_tokens;
  // The list that is lowered: the recorded tasks, with the composite ones spelt out as the tasks they stand for (the
  // task graph handed back to the caller keeps them as recorded).
  g->ltasks.clear();
  for (const Task &t : g->tasks) {
    if (t.name == "rmsnorm_linear") {
      // [input, norm weight, linear weight, output] (python/mirage/mpk/persistent_kernel.py:566-585): RMSNorm into a
      // library-owned row buffer, then a plain linear over it
      if (t.ops.size() != 4) return fail(MK_EINVAL, "rmsnorm_linear expects 4 operands");
      const Tensor &x = g->tensors[t.ops[0]];
      if (x.ndims != 2) return fail(MK_EINVAL, "rmsnorm_linear: input must be 2-D");
      const std::string nm = "rmsnorm_linear_norm_out_" + std::to_string(g->ltasks.size());
      int nid = -1;
      for (size_t k = 0; k < g->tensors.size(); k++)
        if (g->tensors[k].name == nm) nid = (int)k;
      if (nid < 0) {
        Tensor nt;
        nt.name = nm;
        nt.ndims = 2;
        nt.dtype = x.dtype;
        nt.kind = T_OWNED;
        nt.dims[0] = x.dims[0];
        nt.dims[1] = x.dims[1];
        nt.strides[0] = x.dims[1];
        nt.strides[1] = 1;
        void *p = nullptr;
        int rc = dev_alloc(g, &p, (size_t)x.dims[0] * x.dims[1] * dtype_size(x.dtype));
        if (rc) return rc;
        nt.ptr = p;
        g->tensors.push_back(nt);
        nid = (int)g->tensors.size() - 1;
      }
      Task n = t, l = t;
      n.name = "rmsnorm";
      n.ops = {t.ops[0], t.ops[1], nid};
      n.maps = {t.maps[0], t.maps[1], t.maps[0]};
      n.forloop = {t.forloop[0], t.forloop[1], t.forloop[0]};
      n.params.clear();
      l.name = "linear";
      l.ops = {nid, t.ops[2], t.ops[3]};
      l.maps = {t.maps[0], t.maps[2], t.maps[3]};
      l.forloop = {t.forloop[0], t.forloop[2], t.forloop[3]};
      l.params.clear();
      g->ltasks.push_back(n);
      g->ltasks.push_back(l);
    } else {
      g->ltasks.push_back(t);
    }
  }
  size_t i = 0;
  while (i < g->ltasks.size()) {
    const Task &t = g->ltasks[i];
    bool res, silu;
    int extra;
    if (t.name == "embedding") {
      if (t.ops.size() != 3) return fail(MK_EINVAL, "embedding expects 3 operands");
      const Tensor &ids = g->tensors[t.ops[0]], &w = g->tensors[t.ops[1]], &o = g->tensors[t.ops[2]];
      if (ids.dtype != MK_DT_I64) return fail(MK_EINVAL, "embedding ids must be int64");
      if (w.ndims != 2 || o.ndims != 2 || w.dims[1] != o.dims[1] || w.dims[1] % 8 || w.dtype != MK_DT_BF16) return fail(MK_EINVAL, "embedding shapes mismatch");
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_EMBED;
      st.k = (int)w.dims[1];
      st.in = ids.ptr;
      st.out = o.ptr;
      st.ld_out = (int)o.strides[0];
      st.w.nseg = 1;
      st.w.seg[0] = w.ptr;
      if (!t.params.empty() && t.params[0] == 0) st.flags |= MK_F_EMBED_FROM_TOKENS;
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("EMBED %s[%s] -> %s k=%d", w.name.c_str(), ids.name.c_str(), o.name.c_str(), st.k));
      i++;
    } else if (is_norm(t.name)) {
      if (t.ops.size() != 3) return fail(MK_EINVAL, "%s expects 3 operands", t.name.c_str());
      if (i + 1 < g->ltasks.size() && linear_kind(g->ltasks[i + 1].name, &res, &silu, &extra) && g->ltasks[i + 1].ops[0] == t.ops[2]) {
        int rc = lower_linear(g, i);
        if (rc) return rc;
      } else {
        const Tensor &x = g->tensors[t.ops[0]], &w = g->tensors[t.ops[1]], &o = g->tensors[t.ops[2]];
        if (x.ndims != 2 || o.ndims != 2 || x.dims[1] != o.dims[1] || w.elems() != (size_t)x.dims[1] || x.dims[1] % 8)
          return fail(MK_EINVAL, "%s shapes mismatch", t.name.c_str());
        MkStage st;
        memset(&st, 0, sizeof(st));
        st.op = MK_OP_NORM;
        st.k = (int)x.dims[1];
        st.eps = g->cfg.rms_eps;
        st.in = x.ptr;
        st.ld_in = (int)x.strides[0];
        st.norm_w = w.ptr;
        st.out = o.ptr;
        st.ld_out = (int)o.strides[0];
        g->stages.push_back(st);
        g->stage_desc.push_back(fmt("NORM %s -> %s k=%d", x.name.c_str(), o.name.c_str(), st.k));
        i++;
      }
    } else if (linear_kind(t.name, &res, &silu, &extra)) {
      int rc = lower_linear(g, i);
      if (rc) return rc;
    } else if (t.name == "silu_mul_linear_with_residual") {
      int rc = lower_silu_mul_linear(g, i);
      if (rc) return rc;
    } else if (t.name == "silu_mul") {
      if (t.ops.size() != 2) return fail(MK_EINVAL, "silu_mul expects 2 operands");
      const Tensor &x = g->tensors[t.ops[0]], &o = g->tensors[t.ops[1]];
      const int groups = t.grid[0] * t.grid[1] * t.grid[2];
      if (x.ndims != 2 || o.ndims != 2 || x.dims[1] != 2 * o.dims[1] || groups <= 0 || o.dims[1] % groups) return fail(MK_EINVAL, "silu_mul shapes mismatch");
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_SILU_MUL;
      st.n = (int)o.dims[1];
      st.silu_half = (int)(o.dims[1] / groups);
      st.groups = groups;
      st.in = x.ptr;
      st.ld_in = (int)x.strides[0];
      st.out = o.ptr;
      st.ld_out = (int)o.strides[0];
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("SILU_MUL %s -> %s n=%d half=%d", x.name.c_str(), o.name.c_str(), st.n, st.silu_half));
      i++;
    } else if (t.name == "gang_attn_split_kv_mi300" || t.name == "kv_cache_update_mi300" || t.name == "paged_attention" ||
               t.name == "paged_attention_split_kv_mi300" || t.name == "attention" || t.name == "single_batch_extend_attention") {
      int rc = lower_attention(g, i);
      if (rc) return rc;
    } else if (t.name == "moe_topk_softmax_mi300") {
      bool inline_next = false;
      int rc = lower_moe_topk(g, i, &inline_next);
      if (rc) return rc;
      const MkStage router = g->stages.back();
      rc = lower_moe_linear(g, i, inline_next ? &router : nullptr);
      if (rc) return rc;
    } else if (is_moe_linear(t.name)) {
      int rc = lower_moe_linear(g, i, nullptr);
      if (rc) return rc;
    } else if (t.name == "moe_mul_sum_add_mi300") {
      const bool fused = !g->stages.empty() && g->stages.back().op == MK_OP_MOE_LINEAR && (g->stages.back().flags & MK_F_MOE_COMBINE) &&
                         g->stages.back().out == g->tensors[t.ops.empty() ? 0 : t.ops[0]].ptr;
      int rc = lower_moe_combine(g, i, fused);
      if (rc) return rc;
    } else if (t.name == "moe_silu_mul") {
      if (t.ops.size() != 2) return fail(MK_EINVAL, "moe_silu_mul expects 2 operands");
      const Tensor &x = g->tensors[t.ops[0]], &o = g->tensors[t.ops[1]];
      if (!rows_contiguous_3d(x) || !rows_contiguous_3d(o) || x.dims[2] != 2 * o.dims[2] || x.dims[1] != o.dims[1] || x.dtype != MK_DT_BF16 || o.dtype != MK_DT_BF16)
        return fail(MK_EINVAL, "moe_silu_mul shapes mismatch");
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_SILU_MUL;
      st.n = (int)o.dims[2];
      st.silu_half = st.n;  // [gate ; up] halves of every (token, slot) row
      st.groups = 1;
      st.topk = (int)x.dims[1];
      st.in = x.ptr;
      st.ld_in = (int)x.strides[1];
      st.out = o.ptr;
      st.ld_out = (int)o.strides[1];
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("SILU_MUL(moe) %s -> %s n=%d rows/token=%d", x.name.c_str(), o.name.c_str(), st.n, st.topk));
      i++;
    } else if (t.name == "identity") {
      // [input, output], same shape (python/mirage/mpk/persistent_kernel.py:2153-2172; tasks/ampere/identity.cuh:24-37)
      if (t.ops.size() != 2) return fail(MK_EINVAL, "identity expects 2 operands");
      const Tensor &x = g->tensors[t.ops[0]], &o = g->tensors[t.ops[1]];
      if (x.ndims != o.ndims || x.ndims < 2 || x.dtype != o.dtype || x.kind == T_SHUFFLED || o.kind == T_SHUFFLED) return fail(MK_EINVAL, "identity: input and output must be stored tensors of one shape and dtype");
      int64_t inner = 1;
      for (int d = 0; d < x.ndims; d++) {
        if (x.dims[d] != o.dims[d] || x.strides[d] != o.strides[d]) return fail(MK_EINVAL, "identity: input and output shapes differ");
        if (d) inner *= x.dims[d];
      }
      if (x.strides[0] != inner) return fail(MK_EINVAL, "identity: rows must be contiguous");
      if (x.dims[0] < B) return fail(MK_EINVAL, "identity: tensors need at least max_num_batched_tokens=%d rows", B);
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_COPY;
      st.n = (int)(inner * (int64_t)dtype_size(x.dtype) / 2);  // 16-bit units per token row
      st.in = x.ptr;
      st.out = o.ptr;
      st.ld_in = st.ld_out = st.n;
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("COPY %s -> %s units=%d", x.name.c_str(), o.name.c_str(), st.n));
      i++;
    } else if (t.name == "argmax") {
      // [logits, output] in one task (python/mirage/mpk/persistent_kernel.py:2195-2205): the same two stages as the
      // partial + reduce pair, over library-owned partials
      if (t.ops.size() != 2) return fail(MK_EINVAL, "argmax expects 2 operands");
      const Tensor &x = g->tensors[t.ops[0]], &o = g->tensors[t.ops[1]];
      if (x.ndims != 2 || x.dtype != MK_DT_BF16 || o.dtype != MK_DT_I64) return fail(MK_EINVAL, "argmax: logits must be 2-D bf16 and the output int64");
      void *pv = nullptr, *pi = nullptr;
      int rc = dev_alloc(g, &pv, sizeof(float) * (size_t)B * g->G);
      if (rc) return rc;
      rc = dev_alloc(g, &pi, sizeof(int) * (size_t)B * g->G);
      if (rc) return rc;
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_ARGMAX_PARTIAL;
      st.n = (int)x.dims[1];
      st.in = x.ptr;
      st.ld_in = (int)x.strides[0];
      st.aux0 = pv;
      st.aux1 = pi;
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("ARGMAX_PARTIAL %s n=%d", x.name.c_str(), st.n));
      MkStage sr;
      memset(&sr, 0, sizeof(sr));
      sr.op = MK_OP_ARGMAX_REDUCE;
      sr.aux0 = pv;
      sr.aux1 = pi;
      sr.out = o.ptr;
      g->stages.push_back(sr);
      g->stage_desc.push_back(fmt("ARGMAX_REDUCE -> %s", o.name.c_str()));
      i++;
    } else if (t.name == "argmax_partial") {
      if (t.ops.size() != 3) return fail(MK_EINVAL, "argmax_partial expects 3 operands");
      if (i + 1 >= g->ltasks.size() || g->ltasks[i + 1].name != "argmax_reduce" || g->ltasks[i + 1].ops.size() != 3)
        return fail(MK_EUNSUPPORTED, "argmax_partial must be followed by argmax_reduce");
      const Tensor &x = g->tensors[t.ops[0]], &o = g->tensors[g->ltasks[i + 1].ops[2]];
      if (x.ndims != 2 || x.dtype != MK_DT_BF16 || o.dtype != MK_DT_I64) return fail(MK_EINVAL, "argmax: logits must be 2-D bf16 and the output int64");
      void *pv = nullptr, *pi = nullptr;
      int rc = dev_alloc(g, &pv, sizeof(float) * (size_t)B * g->G);
      if (rc) return rc;
      rc = dev_alloc(g, &pi, sizeof(int) * (size_t)B * g->G);
      if (rc) return rc;
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_ARGMAX_PARTIAL;
      st.n = (int)x.dims[1];
      st.in = x.ptr;
      st.ld_in = (int)x.strides[0];
      st.aux0 = pv;
      st.aux1 = pi;
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("ARGMAX_PARTIAL %s n=%d", x.name.c_str(), st.n));
      MkStage sr;
      memset(&sr, 0, sizeof(sr));
      sr.op = MK_OP_ARGMAX_REDUCE;
      sr.aux0 = pv;
      sr.aux1 = pi;
      sr.out = o.ptr;
      g->stages.push_back(sr);
      g->stage_desc.push_back(fmt("ARGMAX_REDUCE -> %s", o.name.c_str()));
      i += 2;
    } else if (t.name == "find_ngram_partial") {
      // (tokens, partial) + [ngram size]; src/kernel/task_register.cc:1689-1719
      if (t.ops.size() != 2 || t.params.size() != 1) return fail(MK_EINVAL, "find_ngram_partial expects (tokens, partial results) and the n-gram size");
      const Tensor &tk = g->tensors[t.ops[0]], &po = g->tensors[t.ops[1]];
      if (tk.ptr != (void *)g->cfg.tokens) return fail(MK_EINVAL, "find_ngram_partial searches the `tokens` meta tensor: attach that tensor as its input");
      if (po.ndims != 2 || po.dtype != MK_DT_I64 || po.dims[0] < g->cfg.max_num_batched_requests || po.dims[1] < 1)
        return fail(MK_EINVAL, "find_ngram_partial: the partial results are an int64 [batch slots >= %d, tasks] tensor", g->cfg.max_num_batched_requests);
      if (t.params[0] < 1 || t.params[0] > 16) return fail(MK_EINVAL, "find_ngram_partial: n-gram size %d outside [1, 16]", t.params[0]);
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_NGRAM_PARTIAL;
      st.n = (int)po.dims[1];
      st.k = t.params[0];
      st.out = po.ptr;
      st.ld_out = (int)po.strides[0];
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("NGRAM_PARTIAL %s -> %s ngram=%d tasks=%d", tk.name.c_str(), po.name.c_str(), st.k, st.n));
      i++;
    } else if (t.name == "find_ngram_global") {
      // (partial, tokens, spec tokens) + [ngram size, spec length]; task_register.cc:1721-1754
      if (t.ops.size() != 3 || t.params.size() != 2) return fail(MK_EINVAL, "find_ngram_global expects (partial results, tokens, spec tokens) and (n-gram size, spec length)");
      const Tensor &pi = g->tensors[t.ops[0]], &tk = g->tensors[t.ops[1]], &so = g->tensors[t.ops[2]];
      if (tk.ptr != (void *)g->cfg.tokens) return fail(MK_EINVAL, "find_ngram_global reads the `tokens` meta tensor: attach that tensor as its input");
      if (pi.ndims != 2 || pi.dtype != MK_DT_I64 || pi.dims[0] < g->cfg.max_num_batched_requests) return fail(MK_EINVAL, "find_ngram_global: bad partial-result tensor");
      if (so.dtype != MK_DT_I64 || (long long)so.elems() < B) return fail(MK_EINVAL, "find_ngram_global: the spec-token tensor holds one int64 id per token row of an iteration (>= %d)", B);
      const int spec_len = t.params[1];
      if (spec_len < 1) return fail(MK_EINVAL, "find_ngram_global: spec length %d < 1", spec_len);
      if (g->cfg.mode != MK_MODE_OFFLINE) return fail(MK_EUNSUPPORTED, "speculative decoding needs the offline scheduler (mode offline): it sizes the token groups of decoding requests");
      if (B < spec_len + 1) return fail(MK_EINVAL, "speculative decoding with %d guesses needs max_num_batched_tokens >= %d", spec_len, spec_len + 1);
      if ((g->cfg.max_tokens_per_request > 0 ? g->cfg.max_tokens_per_request : 8) < spec_len + 1)
        return fail(MK_EINVAL, "speculative decoding with %d guesses needs max_tokens_per_request >= %d (a decoding request brings that many rows)", spec_len, spec_len + 1);
      if (g->spec_len && g->spec_len != spec_len) return fail(MK_EINVAL, "two find_ngram_global tasks with different spec lengths");
      g->spec_len = spec_len;
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_NGRAM_GLOBAL;
      st.n = (int)pi.dims[1];
      st.k = t.params[0];
      st.topk = spec_len;
      st.in = pi.ptr;
      st.ld_in = (int)pi.strides[0];
      st.out = so.ptr;
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("NGRAM_GLOBAL %s, %s -> %s ngram=%d spec=%d", pi.name.c_str(), tk.name.c_str(), so.name.c_str(), st.k, spec_len));
      i++;
    } else if (t.name == "target_verify_greedy") {
      // (spec tokens, target tokens, accepted length); task_register.cc:1756-1784
      if (t.ops.size() != 3) return fail(MK_EINVAL, "target_verify_greedy expects (spec tokens, target tokens, output)");
      const Tensor &sp = g->tensors[t.ops[0]], &tg = g->tensors[t.ops[1]], &vo = g->tensors[t.ops[2]];
      if (sp.dtype != MK_DT_I64 || tg.dtype != MK_DT_I64 || vo.dtype != MK_DT_I64 || (long long)sp.elems() < B || (long long)tg.elems() < B || vo.elems() < 1)
        return fail(MK_EINVAL, "target_verify_greedy: spec and target tokens hold one int64 id per token row (>= %d), the output one int64", B);
      if (!g->cfg.num_new_tokens) return fail(MK_EINVAL, "target_verify_greedy writes the num_new_tokens meta tensor: it must be given");
      if (!g->spec_len) return fail(MK_EINVAL, "target_verify_greedy without a find_ngram_global task before it");
      MkStage st;
      memset(&st, 0, sizeof(st));
      st.op = MK_OP_VERIFY;
      st.in = sp.ptr;
      st.aux0 = tg.ptr;
      st.out = vo.ptr;
      g->stages.push_back(st);
      g->stage_desc.push_back(fmt("VERIFY %s vs %s -> num_new_tokens, %s", sp.name.c_str(), tg.name.c_str(), vo.name.c_str()));
      i++;
    } else if (t.name == "paged_attention_split_kv_merge_mi300" || t.name == "paged_attention_ck_fmha_merge_mi300" || t.name == "gang_attn_merge_mi300" ||
               t.name == "splitk_reduce_mi300") {
      return fail(MK_EUNSUPPORTED, "task '%s' must directly follow the split task whose partial results it combines", t.name.c_str());
    } else {
      return fail(MK_EUNSUPPORTED, "task '%s' has no MI355X lowering", t.name.c_str());
    }
  }
  g->stage_weight.resize(g->stages.size(), -1);
  for (auto &st : g->stages) {  // the task type a stage is shown as in a profiler trace (runtime_header.h:91-188)
    switch (st.op) {
      case MK_OP_EMBED: st.prof_event = 101; break;
      case MK_OP_NORM: st.prof_event = 119; break;
      case MK_OP_LINEAR: st.prof_event = (st.flags & MK_F_NORM) ? 102 : ((st.flags & MK_F_RES) ? 108 : 120); break;
      case MK_OP_SILU_MUL: st.prof_event = 118; break;
      case MK_OP_ATTN: st.prof_event = 116; break;
      case MK_OP_ARGMAX_PARTIAL: st.prof_event = 110; break;
      case MK_OP_ARGMAX_REDUCE: st.prof_event = 111; break;
      case MK_OP_MOE_TOPK: st.prof_event = 172; break;
      case MK_OP_MOE_LINEAR: st.prof_event = (st.flags & MK_F_MOE_COMBINE) || st.ld_in_slot ? 171 : 170; break;
      case MK_OP_MOE_COMBINE: st.prof_event = 173; break;
      case MK_OP_NGRAM_PARTIAL: st.prof_event = 112; break;
      case MK_OP_NGRAM_GLOBAL: st.prof_event = 113; break;
      case MK_OP_VERIFY: st.prof_event = 114; break;
      default: st.prof_event = 121; break;
    }
  }
  g->program_text.clear();
  for (size_t s = 0; s < g->stage_desc.size(); s++) g->program_text += fmt("%3zu ", s) + g->stage_desc[s] + "\n";
  return MK_OK;
}

// ---- reference-shaped task graph (JSON) ------------------------------------------------------
// The task / event graph the reference's Graph::generate_task_graph builds for the recorded operators
// (src/kernel/runtime.cc:164-612, printed by print_task_graph :948-1437), re-derived:
//   * task 0 = TERMINATE, task 1 = BEGIN_TASK_GRAPH; event 0 = TERMINATION, event 1 = LAUNCH_DEPENDENT_TASKS over
//     [2, #tasks); the last event = END_OF_TASK_GRAPH, triggered by every task of the last operator (:176-182,580-595);
//   * the first operator's tasks follow in (bid.x, bid.y, bid.z) order and are the "first_tasks" (:499-513);
//   * between operators i and i+1 the dependency is carried by ONE tensor -- the last (consumer input, producer output)
//     pair naming the same tensor (:519-531); along each of its dims the number of events is gcd(producer partition,
//     consumer partition) (:533-557); an event holds the consumer blocks whose index along the mapped grid axis falls
//     into its slice, in bid order, and is triggered by the producer blocks of the matching slice (:53-140).  Consumer
//     tasks are therefore stored event by event, not in plain bid order;
//   * every launch event ends as EVENT_EMPTY, its tasks carrying `dependent_event` (:593-611; the LAUNCH_TASKS /
//     LAUNCH_MASSIVE_TASKS distinction of :102-105 does not survive that rewrite); tasks without a dependency and the
//     two bookkeeping tasks carry EVENT_INVALID_ID.
// The six metadata keys are views of one 8-byte union that starts as all ones (runtime_header.h:223-256) and receives
// the writes of runtime.cc:365-452 in that order -- including the request_id = bid.x every task gets through the
// always-true term at :380.  Two operators that share no tensor (the reference asserts) get one event from all
// producer blocks to all consumer blocks.
struct RefTask {
  int op_index;
  int bid[3];
  unsigned long long trigger_event, dependent_event;
};
struct RefEvent {
  int type, num_triggers, first_task, last_task;
};
static const unsigned long long REF_EVENT_INVALID = 0x7ffffffffffffffeull;

int task_type_id(const std::string &n) {
  // runtime_header.h:91-188 task ids for the tasks this library lowers
  static const std::map<std::string, int> ids = {
      {"embedding", 101},       {"rmsnorm", 119},          {"gang_rmsnorm_mi300", 143}, {"linear", 120},
      {"linear_with_residual", 108}, {"silu_mul", 118},    {"argmax_partial", 110},     {"argmax_reduce", 111},
      {"splitk_linear_res_atomic_mi300", 133}, {"gang_linear_mi300", 136}, {"gang_linear_res_mi300", 137},
      {"gang_attn_split_kv_mi300", 138}, {"kv_cache_update_mi300", 140}, {"paged_attention_ck_fmha_split_kv_mi300", 141},
      {"gang_linear_silu_mi300", 142}, {"linear_silu_mi300", 182}, {"splitk_linear_mi300", 129}, {"gang_splitk_linear_res_mi300", 144},
      {"gang_linear_n_tiling_mi300", 147}, {"gang_linear_res_n_tiling_mi300", 148}, {"gang_linear_msplit_mi300", 183},
      {"gang_linear_res_msplit_mi300", 184}, {"moe_w13_linear_mi300", 170}, {"moe_w2_linear_mi300", 171}, {"moe_topk_softmax_mi300", 172},
      {"moe_mul_sum_add_mi300", 173}, {"gang_moe_w13_linear_mi300", 174}, {"gang_moe_w2_linear_mi300", 175}, {"moe_silu_mul", 118},
      {"paged_attention", 116}, {"paged_attention_split_kv_mi300", 130}, {"paged_attention_split_kv_merge_mi300", 131},
      {"paged_attention_ck_fmha_merge_mi300", 131}, {"gang_attn_merge_mi300", 139}, {"splitk_reduce_mi300", 132},
      {"silu_mul_linear_with_residual", 105}, {"rmsnorm_linear", 102}, {"identity", 121}, {"argmax", 109}, {"attention", 103},
      {"find_ngram_partial", 112}, {"find_ngram_global", 113}, {"target_verify_greedy", 114}, {"single_batch_extend_attention", 115}};
  auto it = ids.find(n);
  return it == ids.end() ? 0 : it->second;
}

// which param of a gang task is its tiles-per-XCD count (src/kernel/graph.cc:584-675,825-838); -1: not a gang task
int gang_tiles_param(const std::string &n) {
  if (n == "gang_linear_mi300" || n == "gang_linear_n_tiling_mi300" || n == "gang_linear_res_mi300" || n == "gang_linear_res_n_tiling_mi300" ||
      n == "gang_linear_silu_mi300")
    return 4;
  if (n == "gang_linear_msplit_mi300" || n == "gang_linear_res_msplit_mi300") return 3;
  if (n == "gang_rmsnorm_mi300") return 0;
  if (n == "gang_attn_split_kv_mi300") return 7;
  if (n == "gang_attn_merge_mi300") return 5;
  if (n == "gang_moe_w13_linear_mi300" || n == "gang_moe_w2_linear_mi300") return 2;
  if (n == "gang_splitk_linear_res_mi300") return -2;  // params[2] * params[3]
  return -1;
}

// The 8-byte metadata union of a task (runtime_header.h:238-256), little endian: bytes 0-1 request_id / n_tile_start,
// bytes 2-3 kv_idx / n_tile_count, bytes 0-3 expert_offset, bytes 4-7 merge_task_offset / _linear_reserved.
unsigned long long ref_task_metadata(const Task &t, const int bid[3]) {
  unsigned long long m = ~0ull;
  auto set16 = [&](int at, unsigned v) { m = (m & ~(0xffffull << (8 * at))) | ((unsigned long long)(v & 0xffffu) << (8 * at)); };
  auto set32 = [&](int at, unsigned v) { m = (m & ~(0xffffffffull << (8 * at))) | ((unsigned long long)v << (8 * at)); };
  const int type = task_type_id(t.name);
  set16(0, (unsigned)bid[0]);  // request_id: written for every task (runtime.cc:380 is a bare enumerator in an || chain)
  if (type == 170 || type == 171 || type == 182) set32(0, (unsigned)((bid[1] << 16) | (bid[0] & 0xFFFF)));
  const int gp = gang_tiles_param(t.name);
  if (gp != -1) {
    int tiles = 0;
    if (gp == -2) tiles = t.params.size() > 3 ? t.params[2] * t.params[3] : 0;
    else tiles = (int)t.params.size() > gp ? t.params[gp] : 0;
    set16(2, (unsigned)tiles);
    if (type == 183 || type == 184) {
      set16(0, 0);
      set32(4, (unsigned)bid[0]);
    } else if (type == 138 || type == 139) {
      set16(0, (unsigned)(bid[0] * tiles));
    } else {
      set16(0, 0);
    }
  }
  if (type == 130 || type == 131 || type == 141) {
    set16(2, (unsigned)bid[2]);
    set32(4, (unsigned)bid[1]);
  }
  return m;
}

// partition of a tensor along each of its dims by one operand's grid mapping (later axes override earlier ones)
void partition_of(const Task &t, int operand, int part[4]) {
  for (int d = 0; d < 4; d++) part[d] = 1;
  for (int a = 0; a < 3; a++) {
    const int d = t.maps[operand][a];
    if (d >= 0 && d < 4) part[d] = t.grid[a];
  }
}

int build_task_graph_json(mk_graph *g) {
  std::vector<RefTask> tasks;
  std::vector<RefEvent> events;
  tasks.push_back({-1, {0, 0, 0}, REF_EVENT_INVALID, REF_EVENT_INVALID});  // TERMINATE
  tasks.push_back({-1, {0, 0, 0}, 1, REF_EVENT_INVALID});                  // BEGIN_TASK_GRAPH triggers event 1
  events.push_back({911 /*EVENT_TERMINATION*/, 1, 0, 0});
  events.push_back({903 /*EVENT_LAUNCH_DEPENDENT_TASKS*/, 1, 2, 0});
  std::vector<int> first_tasks;
  std::map<std::array<int, 3>, int> pre_map, cur_map;  // bid -> task index, of the previous / current operator
  for (size_t oi = 0; oi < g->tasks.size(); oi++) {
    const Task &c = g->tasks[oi];
    cur_map.clear();
    if (oi == 0) {
      for (int x = 0; x < c.grid[0]; x++)
        for (int y = 0; y < c.grid[1]; y++)
          for (int z = 0; z < c.grid[2]; z++) {
            cur_map[{x, y, z}] = (int)tasks.size();
            first_tasks.push_back((int)tasks.size());
            tasks.push_back({(int)oi, {x, y, z}, REF_EVENT_INVALID, REF_EVENT_INVALID});
          }
      pre_map = cur_map;
      continue;
    }
    const Task &p = g->tasks[oi - 1];
    // the tensor that carries the dependency: the last (consumer input, producer output) pair naming the same tensor
    const int c_in = (int)c.ops.size() - num_outputs(c), p_in = (int)p.ops.size() - num_outputs(p);
    int co = -1, po = -1;
    for (int a = 0; a < c_in; a++)
      for (int b = p_in; b < (int)p.ops.size(); b++)
        if (c.ops[a] >= 0 && c.ops[a] == p.ops[b]) {
          co = a;
          po = b;
        }
    int ev_dims[4] = {1, 1, 1, 1};
    std::array<int, 3> in_map = {-1, -1, -1}, out_map = {-1, -1, -1};
    if (co >= 0) {
      int pp[4], cp[4];
      in_map = c.maps[co];
      out_map = p.maps[po];
      partition_of(c, co, cp);
      partition_of(p, po, pp);
      for (int d = 0; d < 4; d++) ev_dims[d] = std::gcd(pp[d], cp[d]);
    }
    // depth-first over the tensor's dims: each combination of slices is one event
    int idx[4];
    for (idx[0] = 0; idx[0] < ev_dims[0]; idx[0]++)
      for (idx[1] = 0; idx[1] < ev_dims[1]; idx[1]++)
        for (idx[2] = 0; idx[2] < ev_dims[2]; idx[2]++)
          for (idx[3] = 0; idx[3] < ev_dims[3]; idx[3]++) {
            int clo[3] = {0, 0, 0}, chi[3] = {c.grid[0], c.grid[1], c.grid[2]}, plo[3] = {0, 0, 0}, phi[3] = {p.grid[0], p.grid[1], p.grid[2]};
            for (int d = 0; d < 4; d++)
              for (int a = 0; a < 3; a++) {
                if (in_map[a] == d) {
                  const int f = c.grid[a] / ev_dims[d];
                  clo[a] = idx[d] * f;
                  chi[a] = (idx[d] + 1) * f;
                }
                if (out_map[a] == d) {
                  const int f = p.grid[a] / ev_dims[d];
                  plo[a] = idx[d] * f;
                  phi[a] = (idx[d] + 1) * f;
                }
              }
            const int ev = (int)events.size();
            RefEvent e = {900 /*EVENT_EMPTY: its tasks carry dependent_event*/, 0, (int)tasks.size(), 0};
            for (int x = clo[0]; x < chi[0]; x++)
              for (int y = clo[1]; y < chi[1]; y++)
                for (int z = clo[2]; z < chi[2]; z++) {
                  cur_map[{x, y, z}] = (int)tasks.size();
                  tasks.push_back({(int)oi, {x, y, z}, REF_EVENT_INVALID, (unsigned long long)ev});
                }
            e.last_task = (int)tasks.size();
            for (int x = plo[0]; x < phi[0]; x++)
              for (int y = plo[1]; y < phi[1]; y++)
                for (int z = plo[2]; z < phi[2]; z++) {
                  auto it = pre_map.find({x, y, z});
                  if (it == pre_map.end()) return fail(MK_EINVAL, "task graph: producer block (%d,%d,%d) of '%s' has no task", x, y, z, p.name.c_str());
                  tasks[it->second].trigger_event = (unsigned long long)ev;
                  e.num_triggers++;
                }
            events.push_back(e);
          }
    if ((int)cur_map.size() != c.grid[0] * c.grid[1] * c.grid[2])
      return fail(MK_EINVAL, "task graph: the partitions of '%s' and '%s' over their shared tensor leave blocks of '%s' without an event", p.name.c_str(),
                  c.name.c_str(), c.name.c_str());
    pre_map = cur_map;
  }
  // the last operator's tasks trigger END_OF_TASK_GRAPH
  const int end_ev = (int)events.size();
  for (auto &kv : pre_map)
    if (tasks[kv.second].trigger_event == REF_EVENT_INVALID) tasks[kv.second].trigger_event = (unsigned long long)end_ev;
  events.push_back({910 /*EVENT_END_OF_TASK_GRAPH*/, (int)pre_map.size(), 0, 0});
  events[1].last_task = (int)tasks.size();
  g->num_ref_tasks = (int)tasks.size();
  g->num_ref_events = (int)events.size();
  // sanity check (reference: runtime.cc:614-674): run the graph once from the first tasks; every task must run exactly
  // once, every event between operators fire exactly once, and END_OF_TASK_GRAPH be reached
  {
    std::vector<int> left(events.size()), fired(events.size(), 0), ran(tasks.size(), 0);
    for (size_t e = 0; e < events.size(); e++) left[e] = events[e].num_triggers;
    std::vector<int> queue(first_tasks.begin(), first_tasks.end());
    size_t head = 0;
    while (head < queue.size()) {
      const int k = queue[head++];
      if (ran[k]++) return fail(MK_EINVAL, "task graph sanity check: task %d scheduled twice", k);
      const unsigned long long ev = tasks[k].trigger_event;
      if (ev == REF_EVENT_INVALID) continue;
      if (left[ev] <= 0) return fail(MK_EINVAL, "task graph sanity check: event %llu triggered more often than it counts", ev);
      if (--left[ev] == 0) {
        if (fired[ev]++) return fail(MK_EINVAL, "task graph sanity check: event %llu fired twice", ev);
        if (events[ev].type == 900)
          for (int c2 = events[ev].first_task; c2 < events[ev].last_task; c2++) queue.push_back(c2);
      }
    }
    for (int k = 2; k < (int)tasks.size(); k++)
      if (ran[k] != 1) return fail(MK_EINVAL, "task graph sanity check: task %d ran %d times", k, ran[k]);
    for (int e = 2; e < end_ev; e++)
      if (fired[e] != 1) return fail(MK_EINVAL, "task graph sanity check: event %d fired %d times", e, fired[e]);
    if (!g->tasks.empty() && fired[end_ev] != 1) return fail(MK_EINVAL, "task graph sanity check: END_OF_TASK_GRAPH fired %d times", fired[end_ev]);
  }
  // variant ids: the reference registers one code variant per distinct instantiation of a task type (task_register.cc:
  // same constants -> same variant); restated here as: tasks of one type with the same name, per-block operand shapes and
  // params share a variant, numbered in order of first appearance
  std::vector<int> variant(g->tasks.size(), 0);
  {
    std::map<int, std::vector<std::string>> seen;  // task type -> signatures
    for (size_t oi = 0; oi < g->tasks.size(); oi++) {
      const Task &t = g->tasks[oi];
      std::string sig = t.name;
      for (size_t a = 0; a < t.ops.size(); a++) {
        sig += "|";
        if (t.ops[a] < 0) continue;
        const Tensor &tn = g->tensors[t.ops[a]];
        int part[4];
        partition_of(t, (int)a, part);
        for (int d = 0; d < tn.ndims; d++) sig += fmt("%lld,", (long long)(tn.dims[d] / std::gcd((long long)tn.dims[d], (long long)part[d])));
      }
      for (int v : t.params) sig += fmt(";%d", v);
      auto &lst = seen[task_type_id(t.name)];
      size_t k = 0;
      while (k < lst.size() && lst[k] != sig) k++;
      if (k == lst.size()) lst.push_back(sig);
      variant[oi] = (int)k;
    }
  }
  // JSON
  std::string &j = g->json;
  j.clear();
  j += "{\n \"all_tasks\": [\n";
  // one operand of one block: the slice the block's grid indices select (runtime.cc:1215-1414).  A shuffled (fused) tensor
  // is resolved to the source tensor and row the slice starts in (:1229-1283).
  auto operand_json = [&](const Task &t, size_t a, const int bid[3]) -> std::string {
    if (t.ops[a] < 0) return "{\"base_ptr\": \"nullptr\", \"offset\": 0, \"data_type\": 999, \"dims\": [], \"strides\": []}";
    const Tensor &tn = g->tensors[t.ops[a]];
    int part[4];
    partition_of(t, (int)a, part);
    long long dims[4];
    for (int d = 0; d < tn.ndims; d++) dims[d] = tn.dims[d] / std::gcd((long long)tn.dims[d], (long long)part[d]);
    const Tensor *base = &tn;
    long long off = 0;
    if (tn.kind == T_SHUFFLED) {
      const int groups = tn.interleave ? tn.num_groups : 1;
      std::vector<long long> gs;
      long long group_rows = 0;
      for (int sid : tn.sources) {
        gs.push_back(g->tensors[sid].dims[0] / groups);
        group_rows += gs.back();
      }
      long long row = 0;
      for (int ax = 0; ax < 3; ax++)
        if (t.maps[a][ax] == 0) row = tn.dims[0] / t.grid[ax] * bid[ax];
      long long in_group = row % group_rows;
      size_t si = 0;
      while (si + 1 < gs.size() && in_group >= gs[si]) in_group -= gs[si++];
      base = &g->tensors[tn.sources[si]];
      const long long sub_row = row / group_rows * gs[si] + in_group;
      for (int ax = 0; ax < 3; ax++) {
        const int d = t.maps[a][ax];
        if (d > 0 && d < base->ndims) off += base->dims[d] / t.grid[ax] * bid[ax] * base->strides[d];
        else if (d == 0) off += sub_row * base->strides[0];
      }
    } else {
      for (int ax = 0; ax < 3; ax++) {
        const int d = t.maps[a][ax];
        if (d >= 0 && d < tn.ndims) off += tn.dims[d] / t.grid[ax] * bid[ax] * tn.strides[d];
      }
    }
    std::string e = fmt("{\"base_ptr\": \"%s\", \"offset\": %lld, \"data_type\": %d, \"dims\": [", base->name.c_str(), off * (long long)dtype_size(base->dtype), tn.dtype);
    for (int d = 0; d < tn.ndims; d++) e += fmt(d ? ", %lld" : "%lld", dims[d]);
    e += "], \"strides\": [";
    for (int d = 0; d < tn.ndims; d++) e += fmt(d ? ", %lld" : "%lld", (long long)base->strides[d]);
    e += "]}";
    return e;
  };
  for (size_t k = 0; k < tasks.size(); k++) {
    const RefTask &rt = tasks[k];
    const int type = k == 0 ? 0 /*TASK_TERMINATE*/ : (k == 1 ? 10 /*TASK_BEGIN_TASK_GRAPH*/ : task_type_id(g->tasks[rt.op_index].name));
    j += fmt("  {\"task_type\": %d, \"variant_id\": %d, \"inputs\": [", type, rt.op_index >= 0 ? variant[rt.op_index] : 0);
    std::string outs;
    unsigned long long meta = ~0ull;
    if (rt.op_index >= 0) {
      const Task &t = g->tasks[rt.op_index];
      const int n_in = (int)t.ops.size() - num_outputs(t);
      for (size_t a = 0; a < t.ops.size(); a++) {
        const std::string e = operand_json(t, a, rt.bid);
        if ((int)a < n_in) j += ((int)a ? ", " : "") + e;
        else outs += ((int)a > n_in ? ", " : "") + e;
      }
      meta = ref_task_metadata(t, rt.bid);
    }
    j += "], \"outputs\": [" + outs + "], ";
    j += fmt("\"trigger_event\": %llu, \"dependent_event\": %llu, \"request_id\": %d, \"expert_offset\": %d, \"kv_idx\": %d, "
             "\"merge_task_offset\": %d, \"n_tile_start\": %d, \"n_tile_count\": %d}%s\n",
             rt.trigger_event, rt.dependent_event, k < 2 ? -1 : (int)(int16_t)(meta & 0xffff), k < 2 ? -1 : (int)(int32_t)(meta & 0xffffffffu),
             k < 2 ? -1 : (int)((meta >> 16) & 0xffff), k < 2 ? -1 : (int)(int32_t)(meta >> 32), k < 2 ? 0 : (int)(meta & 0xffff),
             k < 2 ? 0 : (int)((meta >> 16) & 0xffff), k + 1 < tasks.size() ? "," : "");
  }
  j += " ],\n \"all_events\": [\n";
  for (size_t e = 0; e < events.size(); e++)
    j += fmt("  {\"event_type\": %d, \"num_triggers\": %d, \"first_task_id\": %d, \"last_task_id\": %d}%s\n", events[e].type, events[e].num_triggers,
             events[e].first_task, events[e].last_task, e + 1 < events.size() ? "," : "");
  j += " ],\n \"first_tasks\": [";
  for (size_t k = 0; k < first_tasks.size(); k++) j += fmt(k ? ", %d" : "%d", first_tasks[k]);
  j += "]\n}\n";
  return MK_OK;
}

int upload_runtime(mk_graph *g) {
  HIP_TRY(hipMemcpy(g->d_rt, &g->h_rt, sizeof(MkRuntime), hipMemcpyHostToDevice));
  return MK_OK;
}

// `rt` is the runtime block the kernel receives by value; `cleared_by_caller`: its barrier state has been zeroed already
// graphs that never run more than one token per iteration use the kernel instantiated for exactly that
static const void *kernel_of(const mk_graph *g) {
  return g->cfg.max_num_batched_tokens == 1 ? (const void *)mk_persistent_kernel_m1 : (const void *)mk_persistent_kernel;
}

int do_launch(mk_graph *g, hipStream_t stream, int max_iters, int run_scheduler, const MkRuntime *rt = nullptr, bool cleared_by_caller = false) {
  if (!g->compiled) return fail(MK_ESTATE, "mk_compile has not been called");
  if (g->launch_pending) return fail(MK_ESTATE, "a launch is still pending: call mk_wait first");
  HIP_TRY(hipSetDevice(g->cfg.device));
  if (!rt) rt = &g->h_rt;
  if (!cleared_by_caller) HIP_TRY(hipMemsetAsync(rt->sync, 0, sizeof(MkSync), stream));
  const MkRuntime *rtp = g->d_rt;
  void *args[] = {(void *)rt, (void *)&rtp, (void *)&max_iters, (void *)&run_scheduler};
  HIP_TRY(hipEventRecord(g->ev0, stream));
  HIP_TRY(hipLaunchCooperativeKernel(kernel_of(g), dim3(g->G), dim3(MK_THREADS), args, MK_LDS_BYTES, stream));
  HIP_TRY(hipEventRecord(g->ev1, stream));
  g->launch_pending = true;
  g->pending_sync = rt->sync;
  return MK_OK;
}

int do_wait(mk_graph *g, hipStream_t stream, int *finished_out) {
  if (!g->launch_pending) return fail(MK_ESTATE, "no launch pending");
  HIP_TRY(hipStreamSynchronize(stream));
  g->launch_pending = false;
  float ms = 0.f;
  HIP_TRY(hipEventElapsedTime(&ms, g->ev0, g->ev1));
  g->last_ms = ms;
  MkSync hs;
  HIP_TRY(hipMemcpy(&hs, g->pending_sync ? g->pending_sync : g->d_sync, sizeof(MkSync), hipMemcpyDeviceToHost));
  int nx = 0;
  for (int i = 0; i < MK_MAX_XCD; i++) nx += hs.xcd_count[i] > 0;
  g->last_nxcd = nx;
  g->last_aborted = hs.abort_flag != 0;
  MkSched sc;
  HIP_TRY(hipMemcpy(&sc, g->d_sched, sizeof(MkSched), hipMemcpyDeviceToHost));
  if (finished_out) *finished_out = sc.finished;
  if (hs.abort_flag) {
    // workgroups that unwound mid-stage may have left the split-K and split-KV arrival counters mid-count (their last
    // arriver resets them); the next launch on this handle must not inherit that
    HIP_TRY(hipMemset(g->h_rt.attn_cnt, 0, sizeof(unsigned) * g->attn_cnt_n));
    HIP_TRY(hipMemset(g->h_rt.splitk_cnt, 0, sizeof(unsigned) * 32 * (size_t)g->G));
    return fail(MK_EABORT, "kernel watchdog fired (barrier epoch %u): a workgroup waited longer than the spin limit", hs.abort_where);
  }
  if (sc.bad_batch) {
    static const char *why[] = {"", "rows outside [0, max_num_batched_tokens), overlapping, or with gaps", "more rows for one request than max_tokens_per_request",
                                "a sequence shorter than its new rows, longer than max_seq_length, or without pages"};
    return fail(MK_EINVAL, "the batch described in qo_indptr / paged_kv_* was rejected and nothing was run: %s", why[sc.bad_batch > 0 && sc.bad_batch <= 3 ? sc.bad_batch : 1]);
  }
  return MK_OK;
}

// ---- launch scratch that no call allocates -------------------------------------------------------------------
// mk_enqueue_steps_static runs a compiled graph with every piece of launch scratch -- the grid barrier's counters, the
// K-split partial tiles and their arrival counters, the attention stages' split-KV partials and counters, the
// sampling stages' per-workgroup partials -- taken from this file-scope device array instead of from the buffers
// mk_compile allocated.  Each GPU the library runs on holds its own copy of the array until the process ends.
// Sizes are for the largest launch the entry point accepts (256 workgroups, 64 tokens x 8 kv heads, 8 q heads per kv head).
constexpr size_t align256(size_t n) { return (n + 255) / 256 * 256; }
constexpr int MK_STATIC_MAX_WG = 256;
constexpr int MK_STATIC_MAX_ITEMS = MK_MAX_TOKENS * 8;  // (token, kv head) pairs
constexpr int MK_STATIC_MAX_QPK = 8;
constexpr size_t SS_SYNC = 0;
constexpr size_t SS_SPLITK_CNT = SS_SYNC + align256(sizeof(MkSync));
constexpr size_t SS_ATTN_CNT = SS_SPLITK_CNT + align256((size_t)MK_STATIC_MAX_WG * 32 * sizeof(unsigned));
constexpr size_t SS_CLEARED_END = SS_ATTN_CNT + align256((size_t)MK_STATIC_MAX_ITEMS * 32 * sizeof(unsigned));  // [0, here) starts every call at zero
constexpr size_t SS_ARGMAX_PV = SS_CLEARED_END;
constexpr size_t SS_ARGMAX_PI = SS_ARGMAX_PV + align256((size_t)MK_MAX_TOKENS * MK_STATIC_MAX_WG * sizeof(float));
constexpr size_t SS_ATTN_PART = SS_ARGMAX_PI + align256((size_t)MK_MAX_TOKENS * MK_STATIC_MAX_WG * sizeof(int));
// q-head partials of the attention stages: at most max(workgroups, (token, kv head) pairs) work units of up to 8 q heads each
constexpr size_t MK_STATIC_ATTN_HEADS = (size_t)std::max(MK_STATIC_MAX_ITEMS, MK_STATIC_MAX_WG) * MK_STATIC_MAX_QPK;
constexpr size_t SS_SPLITK_PART = SS_ATTN_PART + align256(MK_STATIC_ATTN_HEADS * MK_ATTN_PSTRIDE * sizeof(float));
constexpr size_t MK_STATIC_SCRATCH_BYTES = SS_SPLITK_PART + (size_t)MK_STATIC_MAX_WG * 4 * 4 * 4 * 64 * 16;  // about 19.6 MB

static __device__ __align__(256) unsigned char scratch[MK_STATIC_SCRATCH_BYTES];

constexpr int MK_MAX_DEVICES = 64;
unsigned char *g_scratch_ptr[MK_MAX_DEVICES];  // device address of `scratch` on each device, resolved once per device

// `scratch` is a host-side stand-in in host code, not a device address: the address every kernel argument, fill and
// copy uses is the one hipGetSymbolAddress returns, asked for once per device with that device current.
int resolve_scratch(int device) {
  if (device < 0 || device >= MK_MAX_DEVICES) return fail(MK_EINVAL, "device %d outside [0, %d)", device, MK_MAX_DEVICES);
  if (g_scratch_ptr[device]) return MK_OK;
  HIP_TRY(hipSetDevice(device));
  void *p = nullptr;
  HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  if (!p) return fail(MK_EHIP, "hipGetSymbolAddress returned a null address for the launch scratch");
  g_scratch_ptr[device] = (unsigned char *)p;
  return MK_OK;
}

// zero-fill by kernel (a fill node that a caller's graph capture records safely, unlike a memset node)
__global__ void mk_fill_zero_kernel(uint4 *p, size_t n16) {
  const uint4 z = {0u, 0u, 0u, 0u};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) p[i] = z;
}

}  // namespace

// ============================================================================ C ABI
extern "C" {

const char *mk_last_error(void) { return g_err.c_str(); }
const char *mk_version(void) { return "fleet_mk 0.1 (gfx950)"; }

int mk_graph_create(const mk_config *cfg, mk_graph **out) {
  if (!cfg || !out) return fail(MK_EINVAL, "null argument");
  if (cfg->max_num_batched_tokens < 1 || cfg->max_num_batched_tokens > MK_MAX_TOKENS)
    return fail(MK_EINVAL, "max_num_batched_tokens=%d outside [1, %d]", cfg->max_num_batched_tokens, MK_MAX_TOKENS);
  if (cfg->max_num_batched_requests < 1 || cfg->max_num_batched_requests > MK_MAX_TOKENS)
    return fail(MK_EINVAL, "max_num_batched_requests=%d outside [1, %d]", cfg->max_num_batched_requests, MK_MAX_TOKENS);
  if (cfg->mode < MK_MODE_OFFLINE || cfg->mode > MK_MODE_ONEPASS) return fail(MK_EINVAL, "mode=%d is not one of enum mk_mode", cfg->mode);
  if (cfg->max_tokens_per_request < 0 || cfg->max_tokens_per_request > MK_MAX_NEW_PER_REQ)
    return fail(MK_EINVAL, "max_tokens_per_request=%d outside [0, %d]", cfg->max_tokens_per_request, MK_MAX_NEW_PER_REQ);
  if (cfg->page_size < 1 || cfg->max_num_pages < 1 || cfg->max_seq_length < 2) return fail(MK_EINVAL, "bad page_size / max_num_pages / max_seq_length");
  if ((int64_t)cfg->max_num_pages * cfg->page_size < cfg->max_seq_length)
    return fail(MK_EINVAL, "max_num_pages*page_size=%lld cannot hold one sequence of max_seq_length=%d", (long long)cfg->max_num_pages * cfg->page_size,
                cfg->max_seq_length);
  // The next two limits protect state only the on-GPU schedulers keep (MK_MODE_OFFLINE, MK_MODE_ONLINE): their page ring
  // and the LDS snapshot of the page table.  In MK_MODE_ONLINE_NOTOKEN / MK_MODE_ONEPASS the host owns the page table;
  // max_num_pages is then the serving engine's block count, which may be oversubscribed and much larger.
  const bool gpu_pages = cfg->mode == MK_MODE_OFFLINE || cfg->mode == MK_MODE_ONLINE;
  if (gpu_pages) {
    // Every slot can grow to max_seq_length, and the page ring (like the reference's) hands out pages without checking
    // that any are free: with fewer pages than that a page would be given to two requests.
    const int64_t per_req = ((int64_t)cfg->max_seq_length + cfg->page_size - 1) / cfg->page_size;
    if (per_req * cfg->max_num_batched_requests > cfg->max_num_pages)
      return fail(MK_EINVAL, "max_num_pages=%d cannot back %d concurrent requests of up to %lld pages each (max_seq_length=%d, page_size=%d)",
                  cfg->max_num_pages, cfg->max_num_batched_requests, (long long)per_req, cfg->max_seq_length, cfg->page_size);
    if (cfg->max_num_pages > (MK_LDS_BYTES / 8)) return fail(MK_EINVAL, "max_num_pages=%d exceeds the scheduler's LDS snapshot (%d)", cfg->max_num_pages, MK_LDS_BYTES / 8);
  }
  if (((int64_t)cfg->max_seq_length + cfg->page_size - 1) / cfg->page_size > MK_ATTN_MAX_REQ_PAGES)
    return fail(MK_EINVAL, "max_seq_length=%d over page_size=%d is more than %d pages per request (the attention stage keeps a request's page list in LDS)",
                cfg->max_seq_length, cfg->page_size, MK_ATTN_MAX_REQ_PAGES);
  if (cfg->device < 0) {
    mk_graph *g = new mk_graph();
    g->cfg = *cfg;
    if (g->cfg.rms_eps == 0.f) g->cfg.rms_eps = 1e-6f;
    g->host_only = true;
    g->num_cus = 256;
    g->G = cfg->num_workers > 0 ? cfg->num_workers : 256;
    memset(&g->h_rt, 0, sizeof(g->h_rt));
    *out = g;
    return MK_OK;
  }
  int ndev = 0;
  HIP_TRY(hipGetDeviceCount(&ndev));
  if (ndev < 1) return fail(MK_EHIP, "no HIP device visible: the megakernel has no CPU fallback");
  if (cfg->device < 0 || cfg->device >= ndev) return fail(MK_EINVAL, "device %d out of range", cfg->device);
  HIP_TRY(hipSetDevice(cfg->device));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, cfg->device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return fail(MK_EUNSUPPORTED, "device is %s; this library is built for gfx950 only", prop.gcnArchName);
  if (!prop.cooperativeLaunch) return fail(MK_EUNSUPPORTED, "device does not support cooperative launch");
  mk_graph *g = new mk_graph();
  g->cfg = *cfg;
  if (g->cfg.rms_eps == 0.f) g->cfg.rms_eps = 1e-6f;
  g->num_cus = prop.multiProcessorCount;
  g->G = cfg->num_workers > 0 ? cfg->num_workers : g->num_cus;
  if (g->G > g->num_cus) {
    delete g;
    return fail(MK_EINVAL, "num_workers=%d exceeds the %d CUs that can be co-resident", cfg->num_workers, prop.multiProcessorCount);
  }
  memset(&g->h_rt, 0, sizeof(g->h_rt));
  *out = g;
  return MK_OK;
}

int mk_graph_destroy(mk_graph *g) {
  if (!g) return MK_OK;
  if (g->launch_pending) (void)hipDeviceSynchronize();
  for (void *p : g->allocs) (void)hipFree(p);
  for (void *p : g->host_allocs) free(p);
  if (g->ev0) (void)hipEventDestroy(g->ev0);
  if (g->ev1) (void)hipEventDestroy(g->ev1);
  delete g;
  return MK_OK;
}

static int add_tensor(mk_graph *g, Tensor &&t) {
  g->tensors.push_back(std::move(t));
  return (int)g->tensors.size() - 1;
}

int mk_tensor_attach(mk_graph *g, void *device_ptr, int ndims, const int64_t *dims, const int64_t *strides, int dtype, const char *name) {
  if (!g || !dims || !name) return fail(MK_EINVAL, "null argument");
  if (g->compiled) return fail(MK_ESTATE, "graph already compiled");
  if (ndims < 1 || ndims > 4) return fail(MK_EINVAL, "tensor '%s': %d dims (1..4 supported)", name, ndims);
  if (!dtype_size(dtype)) return fail(MK_EINVAL, "tensor '%s': unsupported dtype %d", name, dtype);
  if (!device_ptr) return fail(MK_EINVAL, "tensor '%s': null device pointer", name);
  Tensor t;
  t.name = name;
  t.ndims = ndims;
  t.dtype = dtype;
  t.kind = T_ATTACHED;
  t.ptr = device_ptr;
  int64_t expect = 1;
  for (int i = ndims - 1; i >= 0; i--) {
    t.dims[i] = dims[i];
    t.strides[i] = strides ? strides[i] : expect;
    if (t.strides[i] != expect) return fail(MK_EINVAL, "tensor '%s' is not row-major contiguous (stride[%d]=%lld, expected %lld)", name, i, (long long)t.strides[i], (long long)expect);
    expect *= dims[i];
  }
  return add_tensor(g, std::move(t));
}

int mk_tensor_new(mk_graph *g, int ndims, const int64_t *dims, const int64_t *strides, int dtype, const char *name, int io_category) {
  if (!g || !dims || !name) return fail(MK_EINVAL, "null argument");
  if (g->compiled) return fail(MK_ESTATE, "graph already compiled");
  if (ndims < 1 || ndims > 4) return fail(MK_EINVAL, "tensor '%s': %d dims (1..4 supported)", name, ndims);
  if (!dtype_size(dtype)) return fail(MK_EINVAL, "tensor '%s': unsupported dtype %d", name, dtype);
  if (io_category != MK_IO_DEVICE && io_category != MK_IO_SYMMETRIC) return fail(MK_EINVAL, "Invalid io_category: %d", io_category);
  Tensor t;
  t.name = name;
  t.ndims = ndims;
  t.dtype = dtype;
  t.kind = T_OWNED;
  t.io_category = io_category;
  int64_t expect = 1;
  size_t span = 1;
  for (int i = ndims - 1; i >= 0; i--) {
    t.dims[i] = dims[i];
    t.strides[i] = strides ? strides[i] : expect;
    expect *= dims[i];
    span += (size_t)(dims[i] - 1) * (size_t)t.strides[i];
  }
  // allocate right away so later tasks can capture the address; freed in mk_graph_destroy
  void *p = nullptr;
  int rc = dev_alloc(g, &p, span * dtype_size(dtype));
  if (rc) return rc;
  t.ptr = p;
  return add_tensor(g, std::move(t));
}

int mk_tensor_shuffle(mk_graph *g, const int *ids, int n, int dim, int num_groups, int interleave, const char *name) {
  if (!g || !ids || !name) return fail(MK_EINVAL, "null argument");
  if (dim != 0) return fail(MK_EUNSUPPORTED, "only dimension 0 can be shuffled/fused");
  if (n < 1 || n > MK_MAX_SEGS) return fail(MK_EUNSUPPORTED, "shuffle of %d tensors (1..%d supported)", n, MK_MAX_SEGS);
  if (num_groups < 1) return fail(MK_EINVAL, "num_groups must be positive");
  Tensor t;
  t.name = name;
  t.kind = T_SHUFFLED;
  t.num_groups = num_groups;
  t.interleave = interleave != 0;
  int64_t rows = 0;
  for (int i = 0; i < n; i++) {
    if (ids[i] < 0 || ids[i] >= (int)g->tensors.size()) return fail(MK_EINVAL, "bad tensor id %d", ids[i]);
    const Tensor &s = g->tensors[ids[i]];
    if (s.ndims != 2) return fail(MK_EINVAL, "shuffle source '%s' must be 2-D", s.name.c_str());
    if (i && (s.dims[1] != g->tensors[ids[0]].dims[1] || s.dtype != g->tensors[ids[0]].dtype)) return fail(MK_EINVAL, "shuffle sources disagree on columns/dtype");
    if (s.dims[0] % num_groups) return fail(MK_EINVAL, "source '%s' rows %lld not divisible by num_groups %d", s.name.c_str(), (long long)s.dims[0], num_groups);
    rows += s.dims[0];
    t.sources.push_back(ids[i]);
  }
  t.ndims = 2;
  t.dtype = g->tensors[ids[0]].dtype;
  t.dims[0] = rows;
  t.dims[1] = g->tensors[ids[0]].dims[1];
  t.strides[0] = t.dims[1];
  t.strides[1] = 1;
  return add_tensor(g, std::move(t));
}

int mk_tensor_num_dims(mk_graph *g, int id) {
  if (!g || id < 0 || id >= (int)g->tensors.size()) return fail(MK_EINVAL, "bad tensor id %d", id);
  return g->tensors[id].ndims;
}
int64_t mk_tensor_dim(mk_graph *g, int id, int i) {
  if (!g || id < 0 || id >= (int)g->tensors.size()) return fail(MK_EINVAL, "bad tensor id %d", id);
  if (i < 0 || i >= g->tensors[id].ndims) return fail(MK_EINVAL, "bad dim %d", i);
  return g->tensors[id].dims[i];
}
void *mk_tensor_ptr(mk_graph *g, int id) {
  if (!g || id < 0 || id >= (int)g->tensors.size()) return nullptr;
  return g->tensors[id].ptr;
}

int mk_add_task(mk_graph *g, const char *task_name, const int grid_dim[3], const int block_dim[3], int n_operands, const int *tensor_ids,
                const int *input_maps, const int *forloop_dims, int n_params, const int *params) {
  if (!g || !task_name || !grid_dim || !block_dim || (n_operands > 0 && !tensor_ids)) return fail(MK_EINVAL, "null argument");
  if (g->compiled) return fail(MK_ESTATE, "graph already compiled");
  Task t;
  t.name = task_name;
  for (int i = 0; i < 3; i++) {
    t.grid[i] = grid_dim[i];
    t.block[i] = block_dim[i];
    if (grid_dim[i] < 1) return fail(MK_EINVAL, "task '%s': grid_dim[%d]=%d", task_name, i, grid_dim[i]);
  }
  for (int i = 0; i < n_operands; i++) {
    // id -1 = optional operand that is absent: only the q/k-norm weights and the cos/sin tables of the attention tasks
    const bool optional = (t.name == "gang_attn_split_kv_mi300" || t.name == "kv_cache_update_mi300" || t.name == "paged_attention" ||
                           t.name == "paged_attention_split_kv_mi300" || t.name == "attention" || t.name == "single_batch_extend_attention") && i >= 3 && i <= 6;
    if (tensor_ids[i] >= (int)g->tensors.size() || tensor_ids[i] < (optional ? -1 : 0))
      return fail(MK_EINVAL, "task '%s': bad tensor id %d for operand %d", task_name, tensor_ids[i], i);
    t.ops.push_back(tensor_ids[i]);
    std::array<int, 3> m = {-1, -1, -1};
    if (input_maps) m = {input_maps[3 * i], input_maps[3 * i + 1], input_maps[3 * i + 2]};
    t.maps.push_back(m);
    t.forloop.push_back(forloop_dims ? forloop_dims[i] : -1);
  }
  for (int i = 0; i < n_params; i++) t.params.push_back(params[i]);
  // reject unknown names here, like Graph::register_task (src/kernel/graph.cc:844-847)
  bool a, b;
  int c;
  static const char *known[] = {"embedding", "rmsnorm", "gang_rmsnorm_mi300", "silu_mul", "gang_attn_split_kv_mi300", "kv_cache_update_mi300",
                                "paged_attention_ck_fmha_split_kv_mi300", "argmax_partial", "argmax_reduce", "moe_topk_softmax_mi300", "moe_w13_linear_mi300",
                                "moe_w2_linear_mi300", "gang_moe_w13_linear_mi300", "gang_moe_w2_linear_mi300", "moe_silu_mul", "moe_mul_sum_add_mi300",
                                "paged_attention", "paged_attention_split_kv_mi300", "paged_attention_split_kv_merge_mi300",
                                "paged_attention_ck_fmha_merge_mi300", "gang_attn_merge_mi300", "splitk_reduce_mi300", "silu_mul_linear_with_residual", "rmsnorm_linear", "identity", "argmax", "attention",
                                "find_ngram_partial", "find_ngram_global", "target_verify_greedy", "single_batch_extend_attention"};
  bool ok = linear_kind(t.name, &a, &b, &c);
  for (auto k : known) ok = ok || t.name == k;
  if (!ok) return fail(MK_EUNSUPPORTED, "Unsupported task name: %s", task_name);
  g->tasks.push_back(std::move(t));
  return MK_OK;
}

int mk_generate_task_graph(mk_graph *g, int num_gpus, int my_gpu_id, const char **json_out) {
  if (!g || !json_out) return fail(MK_EINVAL, "null argument");
  if (num_gpus != 1 || my_gpu_id != 0) return fail(MK_EUNSUPPORTED, "this build runs on one GPU (num_gpus=%d, my_gpu_id=%d)", num_gpus, my_gpu_id);
  int rc = build_task_graph_json(g);
  if (rc) return rc;
  *json_out = g->json.c_str();
  return MK_OK;
}

// Matrix-core copies of the linear weights (MkStage::wpack).  A graph that can run more than eight tokens per iteration
// streams its weights through the matrix cores in 16-row tiles; read from a row-major matrix that is 64 bytes from each
// of 16 rows per request, which HBM serves at about three quarters of the rate of one contiguous stream.  So every such
// weight is re-laid once, tile by tile, in a buffer the handle owns (this doubles the weight footprint; single-token
// iterations keep reading the caller's row-major tensors).  FLEET_MK_PACK_WEIGHTS=0 turns the copies off.
// allocate = false re-runs the copy kernels into the existing buffers (the caller changed weights after compiling).
static int pack_weights(mk_graph *g, bool allocate) {
  const char *env = getenv("FLEET_MK_PACK_WEIGHTS");
  if (g->cfg.max_num_batched_tokens < 2 || (env && atoi(env) == 0)) return 0;
  for (auto &st : g->stages) {
    if (st.op != MK_OP_LINEAR || (st.k & 63) || st.k < 64) continue;
    const bool silu = st.flags & MK_F_SILU;
    const int n_out = silu ? st.n / 2 : st.n;
    const long long tiles = (long long)((n_out + 15) / 16) * (silu ? 2 : 1);
    const long long total = tiles * (st.k >> 6) * 128;  // 16-byte operands
    if (allocate) {
      void *p = nullptr;
      if (hipMalloc(&p, (size_t)total * 16) != hipSuccess) {
        (void)hipGetLastError();
        return fail(MK_EHIP, "no device memory for the %.1f MB matrix-core copy of a weight (FLEET_MK_PACK_WEIGHTS=0 runs without the copies)", total * 16 / 1e6);
      }
      g->allocs.push_back(p);
      st.wpack = p;
      g->packed_bytes += total * 16;
    }
    if (!st.wpack) continue;
    hipLaunchKernelGGL(mk_pack_weights_kernel, dim3(2048), dim3(256), 0, 0, st.w, st.n, st.k, silu ? 1 : 0, st.silu_half, (u32x4 *)st.wpack, total);
    HIP_TRY(hipGetLastError());
  }
  HIP_TRY(hipDeviceSynchronize());
  return 0;
}

int mk_repack_weights(mk_graph *g) {
  if (!g) return fail(MK_EINVAL, "null argument");
  if (!g->compiled) return fail(MK_ESTATE, "graph not compiled");
  if (g->single_copy) return fail(MK_ESTATE, "this graph keeps only the tile copies of its weights (MK_CFG_SINGLE_WEIGHT_COPY): the row-major tensors may be gone");
  HIP_TRY(hipSetDevice(g->cfg.device));
  return pack_weights(g, false);
}

int mk_tensor_releasable(mk_graph *g, int id) {
  if (!g || id < 0 || id >= (int)g->tensors.size()) return fail(MK_EINVAL, "bad tensor id %d", id);
  if (!g->compiled || id >= (int)g->releasable.size()) return 0;
  return g->releasable[id] ? 1 : 0;
}

int mk_compile(mk_graph *g) {
  if (!g) return fail(MK_EINVAL, "null argument");
  if (g->compiled) return fail(MK_ESTATE, "graph already compiled");
  if (g->host_only) return fail(MK_ESTATE, "this graph was created without a device (device < 0): it can be lowered and described, not compiled");
  HIP_TRY(hipSetDevice(g->cfg.device));
  const mk_config &c = g->cfg;
  if (!c.step || !c.tokens || !c.input_tokens || !c.output_tokens || !c.prompt_lengths || !c.qo_indptr || !c.paged_kv_indptr || !c.paged_kv_indices ||
      !c.paged_kv_last_page_len)
    return fail(MK_EINVAL, "all meta tensors except num_new_tokens must be non-null device pointers");
  int rc = lower(g);
  if (rc) return rc;
  rc = build_task_graph_json(g);
  if (rc) return rc;
  // co-residency: every workgroup must be resident for the in-kernel barriers to make progress
  HIP_TRY(hipFuncSetAttribute(kernel_of(g), hipFuncAttributeMaxDynamicSharedMemorySize, MK_LDS_BYTES));
  int per_cu = 0;
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel_of(g), MK_THREADS, MK_LDS_BYTES));
  if (per_cu < 1 || g->G > per_cu * g->num_cus) return fail(MK_EINVAL, "grid of %d workgroups cannot be co-resident (%d per CU x %d CUs)", g->G, per_cu, g->num_cus);
  MkRuntime &rt = g->h_rt;
  rt.num_stages = (int)g->stages.size();
  rt.max_tokens = c.max_num_batched_tokens;
  rt.max_requests = c.max_num_batched_requests;
  rt.max_seq = c.max_seq_length;
  rt.page_size = c.page_size;
  rt.max_pages = c.max_num_pages;
  rt.total_requests = c.total_num_requests;
  rt.max_new_per_req = c.max_tokens_per_request > 0 ? c.max_tokens_per_request : 8;
  rt.spec_len = g->spec_len;
  rt.eos_token_id = c.eos_token_id;
  rt.step = c.step;
  rt.tokens = (long long *)c.tokens;
  rt.input_tokens = (long long *)c.input_tokens;
  rt.output_tokens = (long long *)c.output_tokens;
  rt.num_new_tokens = c.num_new_tokens;
  rt.prompt_lengths = c.prompt_lengths;
  rt.qo_indptr = c.qo_indptr;
  rt.kv_indptr = c.paged_kv_indptr;
  rt.kv_indices = c.paged_kv_indices;
  rt.kv_last_page_len = c.paged_kv_last_page_len;
  void *p;
  if ((rc = dev_alloc(g, &p, sizeof(int) * rt.max_requests))) return rc;
  rt.request_ids = (int *)p;
  if ((rc = dev_alloc(g, &p, sizeof(int) * rt.max_pages))) return rc;
  rt.page_queue = (int *)p;
  if ((rc = dev_alloc(g, &p, sizeof(int) * rt.max_tokens))) return rc;
  rt.tok_slot = (int *)p;
  if ((rc = dev_alloc(g, &p, sizeof(int) * rt.max_tokens))) return rc;
  rt.tok_pos = (int *)p;
  if ((rc = dev_alloc(g, &p, sizeof(int) * rt.max_tokens))) return rc;
  rt.tok_first = (int *)p;
  if ((rc = dev_alloc(g, &p, sizeof(MkSched)))) return rc;
  rt.sched = g->d_sched = (MkSched *)p;
  if ((rc = dev_alloc(g, &p, sizeof(MkSync)))) return rc;
  rt.sync = g->d_sync = (MkSync *)p;
  // attention split-KV workspace: one partial (max, sum, 128 values) per q head of every work unit, a buffer of its
  // own for every attention stage (a partial address is then written once per iteration), and two sets of arrival
  // counters (device scope / die-local), one 128-byte line per (token, kv head)
  int max_kv = 1;
  for (auto &s : g->stages)
    if (s.op == MK_OP_ATTN) {
      if (s.num_kv_heads > max_kv) max_kv = s.num_kv_heads;
      g->max_qpk = std::max(g->max_qpk, s.num_q_heads / s.num_kv_heads);
    }
  g->max_kv_heads = max_kv;
  g->attn_cnt_n = (size_t)rt.max_tokens * max_kv * 32 * 2;
  if ((rc = dev_alloc(g, &p, sizeof(unsigned) * g->attn_cnt_n))) return rc;
  rt.attn_cnt = (unsigned *)p;
  rt.attn_part = nullptr;
  for (auto &s : g->stages)
    if (s.op == MK_OP_ATTN) {
      // a work unit is (token, kv head, chunk) with chunks = clamp(G / (tokens * kv heads), 1, MK_ATTN_MAX_CHUNKS): never
      // more than max(G, tokens * kv heads) units, each holding q/kv head partials
      const size_t units = (size_t)std::max(g->G, rt.max_tokens * s.num_kv_heads);
      const int qpk = s.num_q_heads / s.num_kv_heads;
      if ((rc = dev_alloc(g, &p, units * qpk * MK_ATTN_PSTRIDE * sizeof(float), false))) return rc;
      s.aux0 = p;
      s.aux1 = rt.attn_cnt + g->attn_cnt_n / 2;
    }
  if ((rc = pack_weights(g, true))) return rc;
  g->single_copy = (c.flags & MK_CFG_SINGLE_WEIGHT_COPY) && c.max_num_batched_tokens >= 2;
  rt.packed_only = g->single_copy ? 1 : 0;
  g->releasable.assign(g->tensors.size(), 0);
  g->row_major_bytes = 0;
  {
    // which attached tensors does a linear stage read in place, and which do other stages read?
    auto storage_ids = [&](int id, std::vector<int> &out) {
      if (id < 0) return;
      const Tensor &t = g->tensors[id];
      if (t.kind == T_SHUFFLED) out.insert(out.end(), t.sources.begin(), t.sources.end());
      else out.push_back(id);
    };
    std::vector<char> as_linear_weight(g->tensors.size(), 0), otherwise(g->tensors.size(), 0);
    for (size_t si = 0; si < g->stages.size(); si++) {
      if (g->stages[si].op != MK_OP_LINEAR || g->stage_weight[si] < 0) continue;
      // (the forms that stream the tile copy at every token count need whole 64-wide steps per wavefront: k % 256 == 0)
      if (g->single_copy && (!g->stages[si].wpack || (g->stages[si].k & 255)))
        return fail(MK_EUNSUPPORTED, "MK_CFG_SINGLE_WEIGHT_COPY: the weight of stage %zu (%s) cannot be laid out in matrix-core tiles (k=%d is not a multiple of 256)", si,
                    g->stage_desc[si].c_str(), g->stages[si].k);
      std::vector<int> ids;
      storage_ids(g->stage_weight[si], ids);
      for (int id : ids) as_linear_weight[id] = 1;
    }
    // every other use of a tensor: any operand of any task except the weight operand (the second) of a linear task
    for (const Task &t : g->ltasks) {
      bool r_, s_;
      int e_;
      const bool lin = linear_kind(t.name, &r_, &s_, &e_) || t.name == "silu_mul_linear_with_residual";
      for (size_t a = 0; a < t.ops.size(); a++) {
        if (t.ops[a] < 0 || (lin && a == 1)) continue;
        std::vector<int> ids;
        storage_ids(t.ops[a], ids);
        for (int k : ids) otherwise[k] = 1;
      }
    }
    // the same memory attached under two ids (tied embedding / LM head) is in use as long as one of them is
    for (size_t a = 0; a < g->tensors.size(); a++)
      for (size_t b = 0; b < g->tensors.size(); b++)
        if (a != b && g->tensors[a].ptr && g->tensors[a].ptr == g->tensors[b].ptr && otherwise[b]) otherwise[a] = 1;
    for (size_t id = 0; id < g->tensors.size(); id++) {
      const Tensor &t = g->tensors[id];
      if (!as_linear_weight[id] || t.kind != T_ATTACHED) continue;
      if (g->single_copy && !otherwise[id]) g->releasable[id] = 1;
      else g->row_major_bytes += (int64_t)t.elems() * (int64_t)dtype_size(t.dtype);
    }
  }
  if ((rc = dev_alloc(g, &p, sizeof(MkStage) * (g->stages.size() + 1)))) return rc;
  g->d_stages = (MkStage *)p;
  rt.stages = g->d_stages;
  if (!g->stages.empty()) HIP_TRY(hipMemcpy(g->d_stages, g->stages.data(), sizeof(MkStage) * g->stages.size(), hipMemcpyHostToDevice));
  if ((rc = dev_alloc(g, &p, (size_t)g->G * 4 * 4 * 4 * 64 * 16, false))) return rc;
  rt.splitk_part = p;
  if ((rc = dev_alloc(g, &p, (size_t)g->G * 32 * sizeof(unsigned)))) return rc;
  rt.splitk_cnt = (unsigned *)p;
  g->timing_cap = 8192;
  if ((rc = dev_alloc(g, &p, sizeof(long long) * (g->timing_cap + 2)))) return rc;
  rt.timing = g->d_timing = (long long *)p;
  rt.timing_cap = g->timing_cap;
  if ((rc = dev_alloc(g, &p, sizeof(long long) * MK_PROF_TICKS * (g->stages.size() + 1) * g->G))) return rc;
  rt.stage_prof = (long long *)p;
  if ((rc = dev_alloc(g, &p, sizeof(unsigned) * (size_t)g->G))) return rc;
  rt.profiler_count = (unsigned *)p;
  rt.profiler = (unsigned long long *)g->profiler_ptr;
  rt.profiler_cap = g->profiler_cap;
  if ((rc = dev_alloc(g, &p, sizeof(MkRuntime)))) return rc;
  g->d_rt = (MkRuntime *)p;
  if ((rc = upload_runtime(g))) return rc;
  HIP_TRY(hipEventCreate(&g->ev0));
  HIP_TRY(hipEventCreate(&g->ev1));
  if ((rc = resolve_scratch(g->cfg.device))) return rc;  // set-up is where the static launch scratch's address is looked up
  g->compiled = true;
  return mk_init_requests(g);
}

int mk_init_requests(mk_graph *g) {
  if (!g || !g->compiled) return fail(MK_ESTATE, "mk_compile has not been called");
  if (g->launch_pending) return fail(MK_ESTATE, "a launch is still pending");
  HIP_TRY(hipSetDevice(g->cfg.device));
  const MkRuntime &rt = g->h_rt;
  HIP_TRY(hipDeviceSynchronize());
  HIP_TRY(hipMemset(rt.step, 0, sizeof(int) * rt.total_requests));
  HIP_TRY(hipMemset(rt.request_ids, 0xFF, sizeof(int) * rt.max_requests));
  HIP_TRY(hipMemset(rt.qo_indptr, 0, sizeof(int) * (rt.max_requests + 1)));
  HIP_TRY(hipMemset(rt.kv_indptr, 0, sizeof(int) * (rt.max_requests + 1)));
  std::vector<int> pq(rt.max_pages);
  for (int i = 0; i < rt.max_pages; i++) pq[i] = i;
  HIP_TRY(hipMemcpy(rt.page_queue, pq.data(), sizeof(int) * rt.max_pages, hipMemcpyHostToDevice));
  MkSched sc;
  memset(&sc, 0, sizeof(sc));
  sc.page_queue_head = 0;
  sc.page_queue_tail = rt.max_pages;
  HIP_TRY(hipMemcpy(g->d_sched, &sc, sizeof(sc), hipMemcpyHostToDevice));
  HIP_TRY(hipMemset(rt.attn_cnt, 0, sizeof(unsigned) * g->attn_cnt_n));
  HIP_TRY(hipMemset(rt.splitk_cnt, 0, sizeof(unsigned) * 32 * (size_t)g->G));
  HIP_TRY(hipMemset(rt.profiler_count, 0, sizeof(unsigned) * (size_t)g->G));
  if (rt.profiler) HIP_TRY(hipMemset(rt.profiler, 0, sizeof(unsigned long long) * (size_t)rt.profiler_cap));
  return MK_OK;
}

int mk_set_profiler(mk_graph *g, void *device_u64, int64_t num_entries) {
  if (!g) return fail(MK_EINVAL, "null argument");
  if (g->launch_pending) return fail(MK_ESTATE, "a launch is still pending");
  if (device_u64 && num_entries < 2) return fail(MK_EINVAL, "a profiler tensor needs at least two entries");
  g->profiler_ptr = device_u64;
  g->profiler_cap = device_u64 ? num_entries : 0;
  if (g->compiled) {
    HIP_TRY(hipSetDevice(g->cfg.device));
    g->h_rt.profiler = (unsigned long long *)device_u64;
    g->h_rt.profiler_cap = g->profiler_cap;
    HIP_TRY(hipMemset(g->h_rt.profiler_count, 0, sizeof(unsigned) * (size_t)g->G));
    if (device_u64) HIP_TRY(hipMemset(device_u64, 0, sizeof(unsigned long long) * (size_t)num_entries));
    return upload_runtime(g);
  }
  return MK_OK;
}

int mk_enqueue_steps(mk_graph *g, void *stream, int max_iterations) {
  if (!g) return fail(MK_EINVAL, "null argument");
  if (max_iterations < 1) return fail(MK_EINVAL, "max_iterations must be positive");
  switch (g->cfg.mode) {
    case MK_MODE_OFFLINE: return do_launch(g, (hipStream_t)stream, max_iterations, MK_SCHED_OFFLINE);
    case MK_MODE_ONLINE: return do_launch(g, (hipStream_t)stream, max_iterations, MK_SCHED_ONLINE);
    default: return do_launch(g, (hipStream_t)stream, 1, MK_SCHED_FROM_META);  // the host's batch is run once
  }
}

int mk_enqueue_steps_static(mk_graph *g, void *stream, int max_iterations) {
  if (!g) return fail(MK_EINVAL, "null argument");
  if (!g->compiled) return fail(MK_ESTATE, "mk_compile has not been called");
  if (max_iterations < 1) return fail(MK_EINVAL, "max_iterations must be positive");
  if (g->G > MK_STATIC_MAX_WG) return fail(MK_EINVAL, "the static launch scratch holds %d workgroups, this graph runs %d", MK_STATIC_MAX_WG, g->G);
  if (g->h_rt.max_tokens * g->max_kv_heads > MK_STATIC_MAX_ITEMS || g->max_qpk > MK_STATIC_MAX_QPK)
    return fail(MK_EINVAL, "the static launch scratch holds %d (token, kv head) pairs of up to %d q heads each; this graph needs %d x %d",
                MK_STATIC_MAX_ITEMS, MK_STATIC_MAX_QPK, g->h_rt.max_tokens * g->max_kv_heads, g->max_qpk);
  int rc = resolve_scratch(g->cfg.device);  // already resolved by mk_compile on this device; no allocation either way
  if (rc) return rc;
  if (g->launch_pending) return fail(MK_ESTATE, "a launch is still pending: call mk_wait first");
  HIP_TRY(hipSetDevice(g->cfg.device));
  unsigned char *base = g_scratch_ptr[g->cfg.device];
  MkRuntime rt = g->h_rt;
  rt.sync = (MkSync *)(base + SS_SYNC);
  rt.splitk_cnt = (unsigned *)(base + SS_SPLITK_CNT);
  rt.attn_cnt = (unsigned *)(base + SS_ATTN_CNT);
  rt.argmax_pv = (float *)(base + SS_ARGMAX_PV);
  rt.argmax_pi = (int *)(base + SS_ARGMAX_PI);
  rt.attn_part = (float *)(base + SS_ATTN_PART);
  rt.splitk_part = base + SS_SPLITK_PART;
  rt.stage_prof = nullptr;  // per-stage timing is library-allocated scratch too: not recorded by this entry point
  rt.timing = nullptr;
  // the array keeps what the previous call left: barrier state and arrival counters must start at zero
  hipLaunchKernelGGL(mk_fill_zero_kernel, dim3(16), dim3(256), 0, (hipStream_t)stream, (uint4 *)base, SS_CLEARED_END / 16);
  HIP_TRY(hipGetLastError());
  const int sched = g->cfg.mode == MK_MODE_OFFLINE ? MK_SCHED_OFFLINE : (g->cfg.mode == MK_MODE_ONLINE ? MK_SCHED_ONLINE : MK_SCHED_FROM_META);
  return do_launch(g, (hipStream_t)stream, sched == MK_SCHED_FROM_META ? 1 : max_iterations, sched, &rt, true);
}

int mk_wait(mk_graph *g, void *stream, int *finished_out) {
  if (!g) return fail(MK_EINVAL, "null argument");
  return do_wait(g, (hipStream_t)stream, finished_out);
}

int mk_launch_steps(mk_graph *g, void *stream, int max_iterations, int *finished_out) {
  int rc = mk_enqueue_steps(g, stream, max_iterations);
  if (rc) return rc;
  return mk_wait(g, stream, finished_out);
}

int mk_launch(mk_graph *g, void *stream) {
  int finished = 0;
  int rc = mk_launch_steps(g, stream, 0x7fffffff, &finished);
  if (rc) return rc;
  const bool runs_to_completion = g->cfg.mode == MK_MODE_OFFLINE || g->cfg.mode == MK_MODE_ONLINE;
  if (runs_to_completion && !finished) return fail(MK_EABORT, "kernel returned before all requests finished");
  return MK_OK;
}

int mk_run_once(mk_graph *g, void *stream, int num_tokens, const int32_t *tok_slot, const int32_t *tok_pos, const int32_t *tok_first) {
  if (!g || !g->compiled) return fail(MK_ESTATE, "mk_compile has not been called");
  const MkRuntime &rt = g->h_rt;
  if (num_tokens < 1 || num_tokens > rt.max_tokens) return fail(MK_EINVAL, "num_tokens=%d outside [1, %d]", num_tokens, rt.max_tokens);
  if (!tok_slot || !tok_pos || !tok_first) return fail(MK_EINVAL, "null argument");
  for (int t = 0; t < num_tokens; t++) {
    if (tok_slot[t] < 0 || tok_slot[t] >= rt.max_requests) return fail(MK_EINVAL, "tok_slot[%d]=%d out of range", t, tok_slot[t]);
    if (tok_pos[t] < 0 || tok_pos[t] >= rt.max_seq) return fail(MK_EINVAL, "tok_pos[%d]=%d outside [0, max_seq_length)", t, tok_pos[t]);
    if (tok_first[t] < 0 || tok_first[t] > t || tok_slot[tok_first[t]] != tok_slot[t] || tok_pos[t] - tok_pos[tok_first[t]] != t - tok_first[t] ||
        t - tok_first[t] >= rt.max_new_per_req)
      return fail(MK_EINVAL, "tok_first[%d]=%d is not the first row of a contiguous run of <= %d tokens of the same request", t, tok_first[t], rt.max_new_per_req);
  }
  HIP_TRY(hipSetDevice(g->cfg.device));
  hipStream_t s = (hipStream_t)stream;
  HIP_TRY(hipStreamSynchronize(s));
  HIP_TRY(hipMemcpy(rt.tok_slot, tok_slot, sizeof(int) * num_tokens, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(rt.tok_pos, tok_pos, sizeof(int) * num_tokens, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(rt.tok_first, tok_first, sizeof(int) * num_tokens, hipMemcpyHostToDevice));
  MkSched sc;
  HIP_TRY(hipMemcpy(&sc, g->d_sched, sizeof(sc), hipMemcpyDeviceToHost));
  sc.num_tokens = num_tokens;
  sc.bad_batch = 0;
  HIP_TRY(hipMemcpy(g->d_sched, &sc, sizeof(sc), hipMemcpyHostToDevice));
  int rc = do_launch(g, s, 1, MK_SCHED_HOST_ARRAYS);
  if (rc) return rc;
  return do_wait(g, s, nullptr);
}

int mk_get_stats(mk_graph *g, mk_stats *out) {
  if (!g || !out) return fail(MK_EINVAL, "null argument");
  memset(out, 0, sizeof(*out));
  out->num_workgroups = g->G;
  out->num_stages = (int)g->stages.size();
  out->num_tasks = g->num_ref_tasks;
  out->num_events = g->num_ref_events;
  out->num_xcds = g->last_nxcd;
  out->aborted = g->last_aborted;
  out->weight_bytes = g->weight_bytes;
  out->packed_weight_bytes = g->packed_bytes;
  out->row_major_weight_bytes = g->row_major_bytes;
  out->last_launch_ms = g->last_ms;
  if (g->compiled && !g->launch_pending) {
    MkSched sc;
    HIP_TRY(hipMemcpy(&sc, g->d_sched, sizeof(sc), hipMemcpyDeviceToHost));
    out->iterations = sc.iterations;
  }
  return MK_OK;
}

// ticks [first, first + 4) of the stage records of one workgroup, scheduler record last
static int copy_stage_ticks(mk_graph *g, int workgroup, int first, int64_t *ticks_out, int max_stages) {
  if (!g || !ticks_out) return fail(MK_EINVAL, "null argument");
  if (!g->compiled || g->launch_pending) return fail(MK_ESTATE, "no finished launch to report");
  if (workgroup < 0 || workgroup >= g->G) return fail(MK_EINVAL, "workgroup %d outside [0, %d)", workgroup, g->G);
  const int recs = (int)g->stages.size() + 1;
  const int n = std::min<int>(max_stages, recs);
  if (n <= 0) return 0;
  std::vector<long long> buf((size_t)MK_PROF_TICKS * recs);
  HIP_TRY(hipMemcpy(buf.data(), g->h_rt.stage_prof + (size_t)MK_PROF_TICKS * workgroup * recs, sizeof(long long) * buf.size(), hipMemcpyDeviceToHost));
  for (int s = 0; s < n; s++)
    for (int k = 0; k < 4; k++) ticks_out[4 * s + k] = buf[(size_t)MK_PROF_TICKS * s + first + k];
  return n;
}

int mk_get_stage_profile(mk_graph *g, int workgroup, int64_t *ticks_out, int max_stages) { return copy_stage_ticks(g, workgroup, 0, ticks_out, max_stages); }

int mk_get_stage_marks(mk_graph *g, int workgroup, int64_t *ticks_out, int max_stages) { return copy_stage_ticks(g, workgroup, 4, ticks_out, max_stages); }

int mk_describe_program(mk_graph *g, const char **text_out) {
  if (!g || !text_out) return fail(MK_EINVAL, "null argument");
  if (!g->compiled) {
    int rc = lower(g);
    if (rc) return rc;
  }
  *text_out = g->program_text.c_str();
  return MK_OK;
}

}  // extern "C"
