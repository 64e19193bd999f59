/* C ABI of the MI355X persistent decode megakernel library (libfleet_mk.so).
 *
 * This is the drop-in boundary for the decode path of mirage's PersistentKernel:
 * the Python front end (fleet-chiplet-megakernel_amd/mirage) binds these entry
 * points twice -- with ctypes (mirage/_capi.py) and with a compiled Cython module
 * (mirage/_cython/core.pyx over fleet_mk.pxd) -- where the reference binds its C++
 * graph through Cython (python/mirage/_cython/core.pyx, CCore.pxd:236-253) and its
 * generated launcher through a CPython module
 * (python/mirage/mpk/persistent_kernel.py:17-130).
 *
 * Conventions: plain pointers and sizes only; every function returns 0 on success
 * or a negative MK_E* code, and mk_last_error() then returns a description (thread
 * local).  Tensor ids are small non-negative ints scoped to one graph handle.
 * Device pointers passed in stay owned by the caller and must outlive the handle;
 * tensors created with mk_tensor_new are owned (and freed) by the library.
 */
#ifndef FLEET_MK_H
#define FLEET_MK_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct mk_graph mk_graph;

enum mk_status {
  MK_OK = 0,
  MK_EINVAL = -1,   /* bad argument / shape / unsupported configuration */
  MK_EHIP = -2,     /* a HIP runtime call failed */
  MK_ESTATE = -3,   /* call out of order (e.g. launch before compile) */
  MK_EABORT = -4,   /* the kernel hit its bounded-spin watchdog and exited early */
  MK_EUNSUPPORTED = -5
};

/* dtype codes: the reference's type::DataType values used by the decode path
 * (include/mirage/type.h:58-73): */
enum mk_dtype {
  MK_DT_F16 = 940,
  MK_DT_BF16 = 941,
  MK_DT_F32 = 950,
  MK_DT_I32 = 955,
  MK_DT_I64 = 965,
  MK_DT_U64 = 966
};

enum mk_io_category { MK_IO_DEVICE = 0 /* "cuda_tensor" */, MK_IO_SYMMETRIC = 1 /* "nvshmem_tensor": single GPU => same */ };

/* PersistentKernel's `mode` (persistent_kernel.py:204-214: -DMODE_OFFLINE / MODE_ONLINE / MODE_ONLINE_NOTOKEN / MODE_ONEPASS).
 *  MK_MODE_OFFLINE         the on-GPU scheduler batches every request of `tokens` to completion (persistent_kernel.cuh:380-536);
 *  MK_MODE_ONLINE          one request whose tokens the host wrote into tokens[0,:]: every pass consumes num_new_tokens[0] of
 *                          them from step[0] on, until max_seq_length or the EOS id is reached (persistent_kernel.cuh:538-568);
 *  MK_MODE_ONLINE_NOTOKEN  one pass per launch over the batch the host described in input_tokens, qo_indptr, paged_kv_indptr,
 *                          paged_kv_indices and paged_kv_last_page_len (persistent_kernel.cuh:570-582): the serving-loop mode;
 *  MK_MODE_ONEPASS         the same single pass (the reference compiles its test graphs in this mode). */
enum mk_mode { MK_MODE_OFFLINE = 0, MK_MODE_ONLINE = 1, MK_MODE_ONLINE_NOTOKEN = 2, MK_MODE_ONEPASS = 3 };

/* mk_config.flags.  No counterpart in the reference (its kernels read the attached weights in place and its drivers keep an
 * interleaved second copy of the QKV and gate/up weights, src/kernel/runtime.cc:904-943).
 *  MK_CFG_SINGLE_WEIGHT_COPY  a graph with max_num_batched_tokens >= 2 normally holds every linear weight twice -- the
 *      caller's row-major tensor (streamed by iterations of one or two tokens) and a matrix-core tile copy (streamed by larger
 *      iterations).  With this flag the tile copy is the ONLY one the handle reads after mk_compile: iterations of one and
 *      two tokens run the matrix-core forms as well (a single-token iteration then costs about what a four-token one
 *      does), and every tensor for which mk_tensor_releasable() returns 1 may be freed by the caller.  mk_compile fails
 *      with MK_EUNSUPPORTED if a linear weight cannot be tiled (reduction length not a multiple of 256). */
enum mk_config_flags { MK_CFG_SINGLE_WEIGHT_COPY = 1 };

/* Constructor arguments of PersistentKernel (persistent_kernel.py:368-387) plus the
 * ten meta tensors in the order the reference hands them to init_func
 * (persistent_kernel.py:2590-2600).  All meta pointers are device pointers. */
typedef struct mk_config {
  int num_workers;              /* workgroups of the persistent grid; 0 = one per CU */
  int max_seq_length;
  int max_num_batched_requests;
  int max_num_batched_tokens;
  int max_num_pages;
  int page_size;
  int total_num_requests;       /* rows of `tokens` */
  int device;                   /* HIP device ordinal; < 0 = host-only graph (record / validate / lower / emit the task
                                   graph without a GPU; mk_compile and the launch calls then fail with MK_ESTATE) */
  int64_t eos_token_id;
  float rms_eps;                /* 0 => 1e-6, the constant baked into the reference kernels */
  int mode;                     /* enum mk_mode: who prepares the batch of an iteration */
  int max_tokens_per_request;   /* prompt tokens one request may ingest per iteration; 0 => 8, the reference's default for
                                   AMD (MPK_MAX_TOKENS_PER_REQUEST, persistent_kernel.cuh:115-124); at most 64 */
  int flags;                    /* enum mk_config_flags, or'ed */
  int32_t *step;                /* [total_num_requests] */
  int64_t *tokens;              /* [total_num_requests, max_seq_length] */
  int64_t *input_tokens;        /* [max_num_batched_tokens] */
  int64_t *output_tokens;       /* [max_num_batched_tokens] */
  int32_t *num_new_tokens;      /* [total_num_requests] */
  int32_t *prompt_lengths;      /* [total_num_requests] */
  int32_t *qo_indptr;           /* [max_num_batched_requests + 1] */
  int32_t *paged_kv_indptr;     /* [max_num_batched_requests + 1] */
  int32_t *paged_kv_indices;    /* [max_num_pages] */
  int32_t *paged_kv_last_page_len; /* [max_num_batched_requests] */
} mk_config;

/* Replaces CyKNGraph(disable_fingerprint=True) + the PersistentKernel ctor
 * (persistent_kernel.py:404; src/kernel/graph.cc Graph::Graph). */
int mk_graph_create(const mk_config *cfg, mk_graph **out);
/* Replaces finalize_persistent_kernel (persistent_kernel.cuh:2331) and frees library-owned tensors. */
int mk_graph_destroy(mk_graph *g);

/* Replaces KNGraph.new_input + attach_torch_tensor (python/mirage/_cython/core.pyx:718,944;
 * src/kernel/graph.cc:338-344).  Row-major only, like the reference (persistent_kernel.py:473-474).
 * Returns the tensor id (>= 0) or a negative status. */
int mk_tensor_attach(mk_graph *g, void *device_ptr, int ndims, const int64_t *dims, const int64_t *strides, int dtype,
                     const char *name);
/* Replaces new_input + attach_cuda_tensor / attach_nvshmem_tensor (core.pyx:951-965): the library allocates
 * zero-filled device memory right away (later tasks capture its address) and frees it in mk_graph_destroy. */
int mk_tensor_new(mk_graph *g, int ndims, const int64_t *dims, const int64_t *strides, int dtype, const char *name,
                  int io_category);
/* Replaces Graph::shuffle_tensors / fuse_tensors (src/kernel/graph.cc:398-437).  The result is a *view*:
 * row r of the shuffled tensor is resolved to its source at run time; no interleaved copy is made.
 * interleave != 0: groups of [src0 rows ; src1 rows ; ...] (shuffle_tensors); 0: plain concatenation (fuse_tensors
 * with one group). */
int mk_tensor_shuffle(mk_graph *g, const int *ids, int n, int dim, int num_groups, int interleave, const char *name);
/* DTensor.num_dims / DTensor.dim(i) (core.pyx:431-482). */
int mk_tensor_num_dims(mk_graph *g, int id);
int64_t mk_tensor_dim(mk_graph *g, int id, int i);
/* Device address of a tensor after mk_compile (library-owned tensors included); NULL for shuffled views. */
void *mk_tensor_ptr(mk_graph *g, int id);

/* Replaces TBGraph.new_input per operand + KNGraph.customized + Graph::register_task(name, params)
 * (core.pyx:1023-1059,817,1011; src/kernel/graph.cc:439-848).  Operands are given inputs first, outputs last,
 * in the order the reference layer builders use; `input_maps` holds 3 ints per operand, `forloop_dims` one. */
int mk_add_task(mk_graph *g, const char *task_name, const int grid_dim[3], const int block_dim[3], int n_operands,
                const int *tensor_ids, const int *input_maps, const int *forloop_dims, int n_params, const int *params);

/* Replaces Graph::generate_task_graph (src/kernel/runtime.cc:1652-1685): returns the task/event graph as JSON in
 * the reference's task_graph.json schema (runtime.cc:948-1437).  The string is owned by the handle and stays valid
 * until the next call or mk_graph_destroy.  The persistent kernel is precompiled, so there is no generated source. */
int mk_generate_task_graph(mk_graph *g, int num_gpus, int my_gpu_id, const char **json_out);

/* Replaces PersistentKernel.compile's hipcc step + init_persistent_kernel (persistent_kernel.py:2404-2618;
 * persistent_kernel.cuh:1966-2256): lowers the recorded tasks to the stage program, allocates library-owned
 * tensors and runtime state, uploads descriptors, and resets the request scheduler. */
int mk_compile(mk_graph *g);
/* Replaces init_request_resources (persistent_kernel.cuh:1960): resets step[], the page ring and batch slots so the
 * same handle can serve `tokens` again. */
int mk_init_requests(mk_graph *g);
/* Replaces launch_persistent_kernel (persistent_kernel.cuh:2260-2329): one cooperative launch that runs until all
 * requests are finished (offline / online modes) or over the one batch the host described (online_notoken / onepass).
 * Blocks until the kernel has drained, like the reference. `stream` is a hipStream_t (may be 0). */
int mk_launch(mk_graph *g, void *stream);
/* Same kernel, but returns after at most `max_iterations` decode iterations; scheduler state persists in HBM so the
 * next call continues where this one stopped (the reference has no counterpart: its TPOT is an average over one whole
 * launch, demo/qwen3/demo.py:1303-1328).  *finished_out (optional) is set to 1 when no request is left. */
int mk_launch_steps(mk_graph *g, void *stream, int max_iterations, int *finished_out);
/* Non-blocking variant of mk_launch_steps used for timing with events on the caller's stream: enqueues the
 * launch and returns; mk_wait() synchronises and reports watchdog aborts. */
int mk_enqueue_steps(mk_graph *g, void *stream, int max_iterations);
int mk_wait(mk_graph *g, void *stream, int *finished_out);
/* mk_enqueue_steps for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc); it has no counterpart in the reference.  The call allocates and frees nothing, and every piece
 * of scratch its launch uses -- barrier counters, K-split partial tiles and counters, attention split-KV partials and
 * counters, sampling partials -- lives in one file-scope device array of about 19.6 MB per GPU (held until the process
 * ends) instead of in the buffers mk_compile allocated; it is cleared by a fill kernel on `stream`, not by a memset.
 * Limits (MK_EINVAL beyond them): at most 256 workgroups, max_num_batched_tokens x kv heads <= 512, at most 8 q heads
 * per kv head.  All calls on one GPU share that array: calls that overlap on one GPU race, whatever their handles or
 * streams.  Results are bit-identical to mk_enqueue_steps; per-stage timing is not recorded.  Pair with mk_wait. */
int mk_enqueue_steps_static(mk_graph *g, void *stream, int max_iterations);
/* No counterpart in the reference (its kernels read the attached weights in place, persistent_kernel.cuh:1966-2256).
 * A graph with max_num_batched_tokens > 8 keeps, from mk_compile on, a second copy of every linear weight laid out in
 * 16-row matrix-core tiles (iterations of more than eight tokens stream that copy: one contiguous stream per tile is
 * served by HBM about a third faster than 64-byte pieces of 16 rows; single-token iterations read the attached
 * tensors).  A caller that overwrites attached weights after mk_compile calls this to refresh the copies.  Blocking.
 * The environment variable FLEET_MK_PACK_WEIGHTS=0 (read by mk_compile) runs without copies. */
int mk_repack_weights(mk_graph *g);
/* After mk_compile of a graph created with MK_CFG_SINGLE_WEIGHT_COPY: 1 if attached tensor `id` is never read again by this
 * handle (it is a linear weight, or a source of a shuffled linear weight, that now lives in its tile copy and is used by
 * nothing else), 0 if it must stay alive, negative status on a bad id.  Always 0 without the flag.  A released tensor makes
 * mk_repack_weights fail with MK_ESTATE. */
int mk_tensor_releasable(mk_graph *g, int id);
/* Host-driven single pass (the reference's MODE_ONEPASS / online modes, persistent_kernel.cuh:538-582): the caller
 * supplies the batch -- for each of `num_tokens` rows its batch slot, absolute position and the index of the first
 * row of the same request -- and has filled input_tokens / paged_kv_* itself.  Runs the stage program once. */
int mk_run_once(mk_graph *g, void *stream, int num_tokens, const int32_t *tok_slot, const int32_t *tok_pos,
                const int32_t *tok_first);

/* Introspection. */
typedef struct mk_stats {
  int num_workgroups;      /* persistent grid size */
  int num_stages;          /* stages of the lowered program */
  int num_tasks;           /* reference-style tasks in the task graph */
  int num_events;
  int num_xcds;            /* dies that received workgroups in the last launch */
  int aborted;             /* watchdog fired in the last launch */
  int64_t iterations;      /* decode iterations executed since mk_init_requests */
  int64_t weight_bytes;    /* bytes of weight matrices streamed by one iteration */
  double last_launch_ms;   /* HIP-event time of the last launch's kernel, on the stream it ran on */
  int64_t packed_weight_bytes; /* device memory the handle holds for matrix-core copies of the weights (0: none) */
  int64_t row_major_weight_bytes; /* bytes of attached linear weights the handle still reads in place (0 with
                                     MK_CFG_SINGLE_WEIGHT_COPY: every linear weight lives in its tile copy only) */
} mk_stats;
int mk_get_stats(mk_graph *g, mk_stats *out);
/* Device-side stage timing of the LAST decode iteration, as seen by virtual workgroup `workgroup`: for each stage four
 * 100 MHz wall-clock ticks {entered, previous stage's barrier satisfied, work done, arrival posted}.  Returns the number
 * of stages written (<= max_stages).  One record more than there are stages may be asked for: the last one times the
 * scheduler step of that iteration {previous iteration complete, batch prepared (workgroup 0 only), batch published to
 * this workgroup, 0}.  Counterpart of the reference's MPK_ENABLE_EVENT_TIMING ring
 * (persistent_kernel.cuh:1299-1307,2412-2429). */
int mk_get_stage_profile(mk_graph *g, int workgroup, int64_t *ticks_out, int max_stages);
/* Same layout, four further ticks per stage: marks that stage code sets inside its work in a library built with
 * -DMK_TRACE (zero in a regular build).  Used to see where a stage's time goes. */
int mk_get_stage_marks(mk_graph *g, int workgroup, int64_t *ticks_out, int max_stages);
/* Counterpart of the reference's profiler buffer (include/mirage/persistent_kernel/profiler.h:129-180; handed to
 * init_func as profiler_ptr, python/mirage/mpk/persistent_kernel.py:2590-2600): a caller-owned device tensor of
 * `num_entries` uint64 that receives a (tag, time) pair for the begin and the end of EVERY stage every workgroup executes,
 * iteration after iteration, until it is full.  Entry 0 = (workgroups, 1 group); the k-th entry of workgroup b is entry
 * 1 + b + k * workgroups; low 32 bits tag = stage instance << 19 | b << 11 | task type << 2 | (0 begin / 1 end), high 32
 * bits = low word of the device time in ns.  The tensor is cleared here and by mk_init_requests; NULL stops recording. */
int mk_set_profiler(mk_graph *g, void *device_u64, int64_t num_entries);
/* Stage listing (one line per stage) for debugging and tests; owned by the handle. */
int mk_describe_program(mk_graph *g, const char **text_out);

const char *mk_last_error(void);
const char *mk_version(void);

#ifdef __cplusplus
}
#endif
#endif
