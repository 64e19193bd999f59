# Declarations of include/fleet_mk.h for Cython (the reference declares its C++ graph the same way in
# python/mirage/_cython/CCore.pxd:236-253).
from libc.stdint cimport int32_t, int64_t

cdef extern from "fleet_mk.h" nogil:
    ctypedef struct mk_graph:
        pass

    ctypedef struct mk_config:
        int num_workers
        int max_seq_length
        int max_num_batched_requests
        int max_num_batched_tokens
        int max_num_pages
        int page_size
        int total_num_requests
        int device
        int64_t eos_token_id
        float rms_eps
        int mode
        int max_tokens_per_request
        int flags
        int32_t *step
        int64_t *tokens
        int64_t *input_tokens
        int64_t *output_tokens
        int32_t *num_new_tokens
        int32_t *prompt_lengths
        int32_t *qo_indptr
        int32_t *paged_kv_indptr
        int32_t *paged_kv_indices
        int32_t *paged_kv_last_page_len

    ctypedef struct mk_stats:
        int num_workgroups
        int num_stages
        int num_tasks
        int num_events
        int num_xcds
        int aborted
        int64_t iterations
        int64_t weight_bytes
        double last_launch_ms
        int64_t packed_weight_bytes
        int64_t row_major_weight_bytes

    int mk_graph_create(const mk_config *cfg, mk_graph **out)
    int mk_graph_destroy(mk_graph *g)
    int mk_tensor_attach(mk_graph *g, void *device_ptr, int ndims, const int64_t *dims, const int64_t *strides, int dtype, const char *name)
    int mk_tensor_new(mk_graph *g, int ndims, const int64_t *dims, const int64_t *strides, int dtype, const char *name, int io_category)
    int mk_tensor_shuffle(mk_graph *g, const int *ids, int n, int dim, int num_groups, int interleave, const char *name)
    void *mk_tensor_ptr(mk_graph *g, int id)
    int mk_tensor_releasable(mk_graph *g, int id)
    int mk_add_task(mk_graph *g, const char *task_name, const int *grid_dim, const int *block_dim, int n_operands,
                    const int *tensor_ids, const int *input_maps, const int *forloop_dims, int n_params, const int *params)
    int mk_generate_task_graph(mk_graph *g, int num_gpus, int my_gpu_id, const char **json_out)
    int mk_compile(mk_graph *g)
    int mk_init_requests(mk_graph *g)
    int mk_launch(mk_graph *g, void *stream)
    int mk_launch_steps(mk_graph *g, void *stream, int max_iterations, int *finished_out)
    int mk_enqueue_steps(mk_graph *g, void *stream, int max_iterations)
    int mk_enqueue_steps_static(mk_graph *g, void *stream, int max_iterations)
    int mk_wait(mk_graph *g, void *stream, int *finished_out)
    int mk_run_once(mk_graph *g, void *stream, int num_tokens, const int32_t *tok_slot, const int32_t *tok_pos, const int32_t *tok_first)
    int mk_repack_weights(mk_graph *g)
    int mk_get_stats(mk_graph *g, mk_stats *out)
    int mk_get_stage_profile(mk_graph *g, int workgroup, int64_t *ticks_out, int max_stages)
    int mk_get_stage_marks(mk_graph *g, int workgroup, int64_t *ticks_out, int max_stages)
    int mk_set_profiler(mk_graph *g, void *device_u64, int64_t num_entries)
    int mk_describe_program(mk_graph *g, const char **text_out)
    const char *mk_last_error()
    const char *mk_version()
