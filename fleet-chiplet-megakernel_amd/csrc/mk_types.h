// Descriptors shared between the host lowering (mk_host.cpp) and the persistent
// decode megakernel (mk_kernel.hip).  Everything here is plain-old-data that is
// copied to HBM once at compile() time; the kernel is data-driven and never
// recompiled per model.
//
// Role in the reference: these structs take the place of TaskDesc / EventDesc /
// RuntimeConfig (include/mirage/persistent_kernel/runtime_header.h:200-375), but
// describe a *stage program* (one entry per fused operator, statically tiled
// over the workgroups of the 8 XCDs) instead of per-tile tasks in queues.
#pragma once
#include <stdint.h>

#define MK_THREADS 256        // threads per workgroup (4 wavefronts of 64)
#define MK_WAVES 4
#define MK_MAX_XCD 16
#define MK_MAX_SEGS 3         // a shuffled weight has at most 3 sources (q,k,v)
#define MK_MAX_TOKENS 64      // max tokens per iteration supported by the kernels
#define MK_ATTN_MAX_CHUNKS 32 // split-KV fan-out limit per (token, kv head)
#define MK_ATTN_PSTRIDE 160   // floats per (work unit, q head) split-KV partial: 128 values + one 128-byte line of (max, sum)
#define MK_MAX_NEW_PER_REQ 64 // most prompt tokens one request may ingest per iteration (the attention stage keeps their K/V rows in LDS); the
#define MK_ATTN_MAX_REQ_PAGES 8192  // page-table entries of one request the attention stage keeps in LDS: max_seq_length / page_size may not exceed it
                              // configured value defaults to the reference's 8 (MPK_MAX_TOKENS_PER_REQUEST, persistent_kernel.cuh:115-124)
// LDS map of one workgroup (dynamic, > 80 KB pins one workgroup per CU):
//   [0, 24 KB)      input row(s) of the running stage / attention scratch (attention may run on beyond 32 KB)
//   [24 KB, 25 KB)  reduction scratch
//   [25 KB, 32 KB)  outputs of a single-token linear, collected before they are written out
//   [32 KB, 128 KB) routing lists of the mixture-of-experts stages, matrix-core reduction scratch
//   the matrix-core linear that keeps its token rows resident uses [0, 128 KB) for them and the words above for its flags
// (gfx950 gives a workgroup up to 160 KB; 156 KB dynamic + the kernel's static arrays stay below that)
#define MK_RED_OFFSET (24 * 1024)
#define MK_OUT_OFFSET (25 * 1024)   // [25 KB, 32 KB): outputs of a single-token linear collected before they are written out
#define MK_MOE_OFFSET (32 * 1024)
#define MK_MOE_X_OFFSET (40 * 1024)  // [40 KB, 128 KB): input rows of a multi-token MoE linear's (token, slot) pairs
#define MK_LDS_BYTES (156 * 1024)
#define MK_PROF_TICKS 8

enum MkOp {
  MK_OP_NONE = 0,
  MK_OP_EMBED = 1,
  MK_OP_NORM = 2,
  MK_OP_LINEAR = 3,
  MK_OP_SILU_MUL = 4,
  MK_OP_ATTN = 5,
  MK_OP_ARGMAX_PARTIAL = 6,
  MK_OP_ARGMAX_REDUCE = 7,
  MK_OP_MOE_TOPK = 8,     // router softmax -> top-k -> renormalise, one wavefront per token
  MK_OP_MOE_LINEAR = 9,   // per-expert linear over the active experts (W13 with optional SwiGLU, W2)
  MK_OP_MOE_COMBINE = 10, // out = res + sum_k w[t,k] * x[t,k,:]
  MK_OP_COPY = 11,        // out[t, :] = in[t, :], n 16-bit units per token row
  // prompt-lookup speculative decoding (integer stages; tasks/speculative_decoding/prompt_lookup.cuh, target_verify.cuh)
  MK_OP_NGRAM_PARTIAL = 12,  // out[slot, task] = earliest position among the task's share where the request's last k tokens occurred before
  MK_OP_NGRAM_GLOBAL = 13,   // out[row] = this iteration's token ids: the scheduler's, and for a decoding request the tokens after that position
  MK_OP_VERIFY = 14,         // num_new_tokens[request] = 1 + leading candidates the sampled tokens agree with
};

enum MkStageFlags {
  MK_F_NORM = 1,         // LINEAR: RMSNorm(in, norm_w) is applied to the input rows
  MK_F_RES = 2,          // LINEAR: out = acc + res
  MK_F_SILU = 4,         // LINEAR: weight rows interleave [gate ; up]; out = silu(gate)*up
  MK_F_QK_NORM = 8,      // ATTN: per-head RMSNorm on q and k
  MK_F_ROPE = 16,        // ATTN: rotate-half RoPE on q and k
  MK_F_ONLY_MULTI = 32,  // stage runs only when the iteration has more than one token
  MK_F_EMBED_FROM_TOKENS = 64,  // EMBED: ids come from tokens[req, step+j] instead of input_tokens
  MK_F_MOE_INLINE_TOPK = 128,   // MOE_LINEAR: a single-token iteration routes inside this stage (the MOE_TOPK stage before it is multi-token only)
  MK_F_MOE_COMBINE = 256,       // MOE_LINEAR: a single-token iteration also forms res + sum_k w_k * y_k (the MOE_COMBINE stage after it is multi-token only)
  MK_F_DEFER_SUM = 512,  // LINEAR: the next stage is a full-row NORM over this stage's output, which may be handed the K-slice partials to sum
};

#define MK_MOE_MAX_EXPERTS 256  // one thread per expert when the routing lists are built
#define MK_MOE_MAX_TOPK 16

// A (possibly shuffled) weight matrix [rows, k] bf16.  Virtual row r of a shuffled
// tensor lives in source `seg` at a row computed from the group structure, so no
// interleaved copy is ever made (the reference materialises one,
// src/kernel/runtime.cc:904-943).
struct MkWeight {
  const void *seg[MK_MAX_SEGS];
  int seg_rows[MK_MAX_SEGS];  // rows each source contributes to one group
  int nseg;
  int group_rows;  // sum of seg_rows (== total rows when nseg == 1)
  int pad0, pad1;
};

struct MkStage {
  int op;
  int flags;
  int n;  // LINEAR: virtual weight rows; ARGMAX: vocabulary; SILU_MUL: output columns
  int k;  // LINEAR: reduction length; NORM / EMBED: row length
  int ld_in, ld_out, ld_res, silu_half;  // leading dimensions in elements; silu_half = rows of gate per group
  float eps;
  int groups;  // SILU_MUL: number of [gate;up] groups
  const void *in;
  void *out;
  const void *res;
  const void *norm_w;
  void *norm_out;
  MkWeight w;
  // LINEAR: the same weights re-laid for the matrix cores (null: none), in 16-row tiles -- plain stages tile t = rows
  // [16 t, 16 t + 16), SwiGLU stages tile 2j = gate rows of outputs [16 j, 16 j + 16) and tile 2j + 1 their up rows --
  // as [tile][k / 64][2][64 lanes] 16-byte operands: lane l of (tile, step, h) holds k = 64 step + 32 h + 8 (l / 16) ..
  // + 7 of the tile's row l % 16.  A tile is one contiguous stream of 32 k bytes.
  const void *wpack;
  // attention
  void *k_cache, *v_cache;
  const void *q_norm_w, *k_norm_w, *cos_tab, *sin_tab;
  void *q_ws;
  int num_q_heads, num_kv_heads, head_dim, ld_qws;
  int ld_cos, ld_norm;  // ld_norm: leading dimension of norm_out
  float sm_scale_log2;  // log2(e) / sqrt(head_dim)
  int prof_event;       // the reference's task-type number this stage is recorded under in a caller's profiler tensor
  // argmax
  void *aux0, *aux1;
  // mixture of experts.  MOE_LINEAR: x(t,slot) = in + t*ld_in + slot*ld_in_slot, expert e's weights are rows
  // [e*n, (e+1)*n) of w.seg[0], y(t,slot,row) = out + t*ld_out + slot*ld_out_slot + row; with MK_F_SILU rows
  // [0,n/2) are gate and [n/2,n) up, and out2(t,slot,j) receives silu(gate_j)*up_j; with MK_F_MOE_COMBINE out2 is
  // the [tokens, n] result of the weighted sum.
  const void *moe_logits;  // [tokens, num_experts] bf16 router logits (ld_logits)
  float *moe_topk_w;       // [tokens, topk] fp32 renormalised routing weights (ld_topk_w)
  int *moe_routing;        // [num_experts, tokens] int32: 1 + top-k slot of the expert for that token, 0 = not routed
  int *moe_mask;           // [num_experts + 1] int32: ids of the active experts, then their count at [num_experts]
  void *out2;
  int num_experts, topk, ld_logits, ld_topk_w;
  int ld_routing, ld_in_slot, ld_out_slot, ld_out2;
  int ld_out2_slot, pad4, pad5, pad6;
};

// Hierarchical barrier state.  One 128-byte line per counter so that XCD-local
// counters stay in that XCD's L2.
struct MkSync {
  unsigned global_ctr;
  unsigned pad0[31];
  unsigned local_ctr[MK_MAX_XCD][32];
  unsigned local_flag[MK_MAX_XCD][32];
  unsigned xcd_count[MK_MAX_XCD];
  unsigned pad1[32 - MK_MAX_XCD];
  unsigned init_ctr;
  unsigned pad2[31];
  unsigned abort_flag;
  unsigned abort_where;
  unsigned pad3[30];
};

// Barrier completion test.  Arrival counters and their targets (quota x epoch) are 32-bit and only ever grow during a
// launch, so on a long launch both wrap; their difference taken as a signed number stays correct as long as the two
// are less than 2^31 apart, and they are never more than one stage apart.
#ifdef __HIP__
#define MK_HOST_DEVICE __host__ __device__
#else
#define MK_HOST_DEVICE
#endif
MK_HOST_DEVICE inline bool mk_counter_reached(unsigned counter, unsigned target) { return (int)(counter - target) >= 0; }

// Who describes the batch of an iteration (the kernel's `run_scheduler` argument).
enum MkSchedMode {
  MK_SCHED_HOST_ARRAYS = 0,  // the host wrote tok_slot / tok_pos / tok_first (mk_run_once)
  MK_SCHED_OFFLINE = 1,      // on-GPU continuous batching over `tokens` (MODE_OFFLINE)
  MK_SCHED_FROM_META = 2,    // derived on the GPU from the qo / paged-kv meta tensors the host filled (MODE_ONLINE_NOTOKEN, MODE_ONEPASS)
  MK_SCHED_ONLINE = 3,       // one request, host-written tokens consumed num_new_tokens[0] at a time (MODE_ONLINE)
};

// Scheduler state that persists across launches (continuous batching, page ring).
struct MkSched {
  int page_queue_head, page_queue_tail, next_request_id, num_tokens;
  int num_reqs, finished, online_started;
  int bad_batch;          // host-described batch (MK_SCHED_FROM_META) that was rejected instead of run: 0 = fine, else the reason

  long long iterations;   // decode iterations executed so far (all launches)
  long long pad2;
};

struct MkRuntime {
  int num_stages, max_tokens, max_requests, max_seq;
  int page_size, max_pages, total_requests, max_new_per_req;
  int spec_len, pad_spec;  // speculative candidates a decoding request brings into an iteration beside its newest token (0: none)
  long long eos_token_id;
  // meta tensors (persistent_kernel.py:2590-2600 order)
  int *step;
  long long *tokens;
  long long *input_tokens;
  long long *output_tokens;
  int *num_new_tokens;
  int *prompt_lengths;
  int *qo_indptr;
  int *kv_indptr;
  int *kv_indices;
  int *kv_last_page_len;
  // library-owned scheduler memory
  int *request_ids;   // [max_requests] request id per batch slot, -1 = free
  int *page_queue;    // [max_pages] ring of free page ids
  int *tok_slot;      // [max_tokens] batch slot of each token of this iteration
  int *tok_pos;       // [max_tokens] absolute position of each token
  int *tok_first;     // [max_tokens] index of the first token of the same request in this iteration
  MkSched *sched;
  const MkStage *stages;
  MkSync *sync;
  // attention split-KV workspace
  float *attn_part;     // null: every attention stage has a partial buffer of its own (its descriptor's aux0).  Non-null: ONE buffer
                        // [units][q/kv][MK_ATTN_PSTRIDE] shared by all attention stages, handed off at device scope only
  float *argmax_pv;     // non-null: the sampling stages' per-workgroup partials live here ([tokens][workgroups] values / indices)
  int *argmax_pi;       // instead of in the buffers their descriptors name
  unsigned *attn_cnt;   // [max_tokens * num_kv_heads][32]: one 128-byte line per counter
  void *splitk_part;    // [workgroups][4 wavefronts][4 weight tiles][4 token tiles][64 lanes] f32x4: K-slice partials of the split-K linear
  unsigned *splitk_cnt; // [workgroups][32]: arrival counter per split-K group (one 128-byte line each)
  long long *timing;    // [1 + timing_cap] wall-clock ticks (100 MHz) at the start of each iteration; [0] = kernel end
  int timing_cap;
  int packed_only;       // the handle keeps ONLY the matrix-core copies of its linear weights: iterations of one or two tokens run the matrix-core forms too
  // A caller's profiler tensor (null: none): (tag, time) entries of EVERY executed stage of every iteration, in the
  // reference's layout (include/mirage/persistent_kernel/profiler.h:129-180): entry 0 = (workgroups, 1); the k-th entry of
  // workgroup b sits at 1 + b + k * workgroups; low word tag = stage instance << 19 | b << 11 | task type << 2 | (0 begin, 1
  // end), high word = low 32 bits of the time in ns.  Recording stops when the tensor is full.
  unsigned long long *profiler;
  long long profiler_cap;        // entries the tensor holds
  unsigned *profiler_count;      // [workgroups] entries written so far by each workgroup (kept across launches)
  long long *stage_prof; // [workgroups][num_stages + 1][MK_PROF_TICKS] 100 MHz ticks of the last iteration: entry, wait done, exit, arrived, then
                         // four marks a stage may set in a build with MK_TRACE defined; the extra record holds the scheduler step:
                         // [0] previous iteration complete, [1] batch prepared, [2] batch published to every workgroup
};
