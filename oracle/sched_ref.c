/* CPU oracle for the offline-serving batch scheduler -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the reference's on-GPU continuous batching step, MODE_OFFLINE
 * prepare_next_batch (include/mirage/persistent_kernel/persistent_kernel.cuh:380-536) and of the state
 * reset done by init_kernel (:268-296).  The HIP kernel's scheduler must leave the ten meta tensors in
 * exactly the state this function leaves them in (integer work: bit-exact).
 *
 * Pinning: tests/test_scheduler_oracle.py checks it against a hand-simulated schedule (3 requests with
 * prompts 5/9/2, 4 tokens per iteration, 4-token pages) and against invariants that any correct
 * scheduler satisfies (every prompt token fed exactly once and in order, one decode token per running
 * request per iteration, no page owned twice, all pages returned at the end).
 *
 * Nothing in the product links or loads this file.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
  /* configuration */
  int max_requests;      /* MPK_MAX_NUM_BATCHED_REQUESTS */
  int max_tokens;        /* MPK_MAX_NUM_BATCHED_TOKENS */
  int max_pages;         /* MPK_MAX_NUM_PAGES */
  int page_size;         /* MPK_PAGE_SIZE */
  int max_seq;           /* MPK_MAX_SEQ_LENGTH == config.max_seq_length */
  int max_new_per_req;   /* MPK_MAX_TOKENS_PER_REQUEST (8 on AMD, persistent_kernel.cuh:115-124) */
  int total_requests;
  int64_t eos_token_id;
  /* meta tensors */
  int32_t *step;              /* [total_requests] */
  int64_t *tokens;            /* [total_requests, max_seq] */
  int64_t *input_tokens;      /* [max_tokens] */
  int64_t *output_tokens;     /* [max_tokens] */
  int32_t *prompt_lengths;    /* [total_requests] */
  int32_t *qo_indptr;         /* [max_requests + 1] */
  int32_t *kv_indptr;         /* [max_requests + 1] */
  int32_t *kv_indices;        /* [max_pages] */
  int32_t *kv_last_page_len;  /* [max_requests] */
  /* scheduler-private state */
  int32_t *request_ids;       /* [max_requests] */
  int32_t *page_queue;        /* [max_pages] */
  int32_t page_queue_head, page_queue_tail, next_request_id;
} sched_state;

/* init_kernel (persistent_kernel.cuh:268-296) */
void sched_ref_reset(sched_state *s) {
  for (int i = 0; i < s->total_requests; i++) s->step[i] = 0;
  s->next_request_id = 0;
  for (int i = 0; i < s->max_requests; i++) s->request_ids[i] = -1;
  for (int i = 0; i <= s->max_requests; i++) {
    s->qo_indptr[i] = 0;
    s->kv_indptr[i] = 0;
  }
  s->page_queue_head = 0;
  s->page_queue_tail = s->max_pages;
  for (int i = 0; i < s->max_pages; i++) s->page_queue[i] = i;
}

static int imin(int a, int b) { return a < b ? a : b; }

/* Returns the number of tokens scheduled for the next iteration (0 = nothing left to do). */
int sched_ref_prepare_next_batch(sched_state *s) {
  const int R = s->max_requests, B = s->max_tokens, PS = s->page_size, NP = s->max_pages;
  int head = s->page_queue_head, tail = s->page_queue_tail;
  int32_t *saved = (int32_t *)malloc(sizeof(int32_t) * (size_t)(NP > 0 ? NP : 1));
  /* step 1 (:386-424): commit the previous iteration's outputs; retire finished requests, free their pages */
  for (int i = 0; i < R; i++) {
    int req = s->request_ids[i];
    if (req == -1) continue;
    int st = s->step[req];
    int q0 = s->qo_indptr[i];
    int n = s->qo_indptr[i + 1] - q0;
    int plen = s->prompt_lengths[req];
    for (int j = 0; j < n; j++)
      if (st + j + 1 >= plen && st + j + 1 < s->max_seq) s->tokens[(int64_t)req * s->max_seq + st + j + 1] = s->output_tokens[q0 + j];
    s->step[req] = st + n;
    if ((st + n + 1 >= s->max_seq) || ((s->tokens[(int64_t)req * s->max_seq + st + n] == s->eos_token_id) && (st + n >= plen))) {
      s->request_ids[i] = -1;
      int k0 = s->kv_indptr[i];
      int np = s->kv_indptr[i + 1] - k0;
      for (int j = 0; j < np; j++) {
        s->page_queue[tail % NP] = s->kv_indices[k0 + j];
        tail++;
      }
    }
  }
  /* step 2 (:427-430): snapshot the page table */
  int old_pages = s->kv_indptr[R];
  for (int i = 0; i < old_pages; i++) saved[i] = s->kv_indices[i];
  /* step 3 (:433-482): running requests, compacted */
  int nreq = 0, ntok = 0, npages = 0;
  for (int i = 0; i < R; i++) {
    int req = s->request_ids[i];
    if (req == -1) continue;
    int k0 = s->kv_indptr[i];
    int had = s->kv_indptr[i + 1] - k0;
    s->request_ids[nreq] = req;
    s->qo_indptr[nreq] = ntok;
    s->kv_indptr[nreq] = npages;
    int st = s->step[req];
    int n = s->prompt_lengths[req] - st;
    if (n > 0) n = imin(n, imin(s->max_new_per_req, B - ntok));
    else n = imin(1, B - ntok);
    for (int j = 0; j < n; j++) s->input_tokens[ntok + j] = s->tokens[(int64_t)req * s->max_seq + st + j];
    int need = (st + n + PS - 1) / PS;
    int last = (st + n) % PS;
    s->kv_last_page_len[nreq] = last == 0 ? PS : last;
    for (int j = 0; j < had; j++) s->kv_indices[npages + j] = saved[k0 + j];
    for (int j = had; j < need; j++) {
      s->kv_indices[npages + j] = s->page_queue[head % NP];
      head++;
    }
    npages += need;
    ntok += n;
    nreq++;
  }
  /* step 3b (:485-517): admit new requests */
  while (nreq < R && ntok < B) {
    int req = s->next_request_id;
    if (req >= s->total_requests) break;
    s->request_ids[nreq] = req;
    s->qo_indptr[nreq] = ntok;
    s->kv_indptr[nreq] = npages;
    int n = imin(s->prompt_lengths[req], imin(s->max_new_per_req, B - ntok));
    for (int j = 0; j < n; j++) s->input_tokens[ntok + j] = s->tokens[(int64_t)req * s->max_seq + j];
    int need = (n + PS - 1) / PS;
    int last = n % PS;
    s->kv_last_page_len[nreq] = last == 0 ? PS : last;
    for (int j = 0; j < need; j++) {
      s->kv_indices[npages + j] = s->page_queue[head % NP];
      head++;
    }
    ntok += n;
    npages += need;
    nreq++;
    s->next_request_id = req + 1;
  }
  /* step 4 (:520-526) */
  for (int i = nreq; i < R; i++) s->request_ids[i] = -1;
  for (int i = nreq; i <= R; i++) {
    s->qo_indptr[i] = ntok;
    s->kv_indptr[i] = npages;
  }
  /* step 5 (:529-530) */
  s->page_queue_head = head;
  s->page_queue_tail = tail;
  free(saved);
  return ntok;
}
