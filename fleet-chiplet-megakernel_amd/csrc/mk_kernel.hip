// Persistent decode megakernel for gfx950 (MI355X): one cooperative launch runs
// every decode iteration of every request.  Each iteration walks a static stage
// program; every stage is tiled over all workgroups, with workgroups ordered
// by the XCD they run on so that one die streams one contiguous chunk of a
// weight matrix and shares activations through its own L2.
//
// Replaces, for the decode path, the reference's device runtime
// (include/mirage/persistent_kernel/persistent_kernel.cuh:693-1907: execute_worker,
// execute_scheduler, prepare_next_batch) and its MI300 task kernels
// (include/mirage/persistent_kernel/tasks/mi300/*.cuh).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "mk_types.h"

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Stage descriptors are written once by the host before the first launch and never by the kernel: reading them
// through the constant address space makes every field a scalar load, so shapes, pointers and everything derived
// from them stay in scalar registers and branches on them are scalar branches.
typedef const __attribute__((address_space(4))) MkStage CStage;
typedef const __attribute__((address_space(4))) MkWeight CWeight;

#define MK_SPIN_LIMIT (1u << 24)
#ifndef MK_TUNE_POLL_SLEEP
#define MK_TUNE_POLL_SLEEP 1
#endif

// weight rows in flight per wavefront of the single-token linear (K = 4096 with SwiGLU / K = 4096 plain / K = 12288)
// (a shallow window and more rows parked in LDS across the barrier beat a deep window: whatever a CU has in flight sits in
// front of the control wavefront's barrier poll and input-row loads)
#ifndef MK_TUNE_R8
#define MK_TUNE_R8 2
#endif
#ifndef MK_TUNE_R8N
#define MK_TUNE_R8N 2
#endif
#ifndef MK_TUNE_R4
#define MK_TUNE_R4 2  // K = 2048
#endif
#ifndef MK_TUNE_MOE_M1_R13
#define MK_TUNE_MOE_M1_R13 2  // single-token expert W13: [gate ; up] row pairs in flight per wavefront (K = 2048)
#endif
#ifndef MK_TUNE_MOE_M1_R2
#define MK_TUNE_MOE_M1_R2 1   // single-token expert W2: output rows (x 8 experts) in flight per wavefront
#endif
// multi-token expert linears: cost of a unit's row load relative to one token's reduction (W13 / W2)
#ifndef MK_TUNE_MOE_ROWCOST13
#define MK_TUNE_MOE_ROWCOST13 4
#endif
#ifndef MK_TUNE_MOE_ROWCOST2
#define MK_TUNE_MOE_ROWCOST2 3
#endif
#ifndef MK_TUNE_MOE_M1_PARK
#define MK_TUNE_MOE_M1_PARK 2 // ... and parked in LDS per wavefront while the barrier is awaited
#endif
// units per group of the multi-token expert linears (W13 / W2)
#ifndef MK_TUNE_MOE_R13
#define MK_TUNE_MOE_R13 4
#endif
#ifndef MK_TUNE_MOE_R2
#define MK_TUNE_MOE_R2 16
#endif
#ifndef MK_TUNE_NL
#define MK_TUNE_NL 3
#endif
#ifndef MK_TUNE_W0_KL
#define MK_TUNE_W0_KL 8  // single-token linears with rows of at least this many KB arrive without a workgroup barrier
#endif
#ifndef MK_TUNE_R24
#define MK_TUNE_R24 2
#endif

struct Ctx {
  int vid;   // virtual workgroup id: xcd-major, so vids [x*quota, (x+1)*quota) share an L2
  int G;     // workgroups in the grid
  int xcd;   // XCC_ID of the CU this workgroup landed on
  int quota; // workgroups on this XCD
  int nxcd;  // XCDs that received at least one workgroup
  unsigned quotas[8];  // workgroups on each of the first 8 XCD ids (0 = unused)
  int xi;     // index of this XCD among the XCDs in use
  int rank;   // rank of this workgroup inside its XCD
  unsigned epoch;
  bool pending;  // an arrive has been posted that no wait has consumed yet
  bool dead;     // the watchdog fired somewhere: unwind
  long long t_wait;  // (profiling) tick at which the last barrier_wait completed
  int *sh_dead;
  MkSync *sync;
  const int *sh_tok;  // LDS copy of this iteration's token metadata: [0] position, [1] batch slot, [2] first token of the request, [3] first page-table entry
  bool even_xcds;     // every die in use runs the same number of workgroups, so die index = vid / quota
  int *sh_ticket;     // two LDS work counters, used alternately by consecutive executed stages; [2] = seq of the single-token
                      // MoE stage that last filled the workgroup's expert list (kept outside the stages' scratch LDS)
  int seq;            // stages executed so far by this workgroup
  unsigned prof_n;    // entries this workgroup has written into the caller's profiler tensor
  bool wrote_through; // the stage that just ran wrote all its outputs with write-through stores: no L2 write-back at its barrier
  bool arrive_w0;     // ... and all of them from wavefront 0, after a workgroup barrier, having reset the next stage's work
                      // counter itself: the arrival then needs no workgroup barrier of its own (see barrier_arrive)
  // A split-K linear whose consumer is a full-row norm leaves its K-slice partials unsummed: the norm stage, which reads
  // every row anyway, sums them (slice order, then the residual, then one rounding: the same arithmetic).
  int defer_S;            // slices left unsummed by the stage that just ran (0: none)
  int defer_rows;         // token rows per slice in the partial buffer
  int defer_n;            // row length of the partial buffer (the producing linear's outputs)
  const float *defer_part;  // [slice][row][n] fp32
  const void *defer_res;  // residual rows of that linear (null: none)
  int defer_ld_res;
#ifdef MK_TRACE
  long long mark[4];  // (tracing builds) wall-clock marks the running stage sets, stored next to its stage timing
#endif
};
#ifdef MK_TRACE
#define MK_MARK(c, i) ((c).mark[i] = (long long)wall_clock64())
#else
#define MK_MARK(c, i) ((void)0)
#endif

// ----------------------------------------------------------------------------- small helpers
__device__ __forceinline__ float bf_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
// round-to-nearest-even float -> bf16 (hardware v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t f2bf(float f) { return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ uint32_t pack2(float a, float b) { return f2bf(a) | (f2bf(b) << 16); }
__device__ __forceinline__ float bfround(float f) { return __uint_as_float(f2bf(f) << 16); }

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b, float c) {
  c = dot2(a.x, b.x, c);
  c = dot2(a.y, b.y, c);
  c = dot2(a.z, b.z, c);
  c = dot2(a.w, b.w, c);
  return c;
}
// Cross-lane reductions on the DPP path (one VALU instruction per step) instead of LDS-crossbar shuffles: a
// 16-lane row is all-reduced with rotations by 8, 4, 2, 1 (every lane ends with the row total), the four rows of a
// wavefront are then combined through scalar lane reads.  Callers run with whole rows / whole wavefronts active.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float group16_sum(float v) {
  v += dpp_f32<0x128>(v);  // row_ror:8
  v += dpp_f32<0x124>(v);  // row_ror:4
  v += dpp_f32<0x122>(v);  // row_ror:2
  v += dpp_f32<0x121>(v);  // row_ror:1
  return v;
}
__device__ __forceinline__ float lane_f32(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = group16_sum(v);
  return (lane_f32(v, 0) + lane_f32(v, 16)) + (lane_f32(v, 32) + lane_f32(v, 48));
}
// Transposing wavefront reduction: every lane holds partial sums of NV values (NV a power of two <= 16); on return lane
// l holds the wavefront total of value l & (NV - 1).  Stage b pairs the values up and exchanges one of each pair with
// the lane whose bit b differs (one DPP move per pair), so 16 values cost about 50 instructions instead of 16 full
// reductions; the four 16-lane rows are combined with two cross-row permutes at the end.
template <int NV>
__device__ __forceinline__ float transpose_sum(float (&v)[NV], int lane) {
  static_assert(NV == 1 || NV == 2 || NV == 4 || NV == 8 || NV == 16, "power of two");
  if constexpr (NV >= 2) {
    const bool b = lane & 1;
#pragma unroll
    for (int j = 0; j < NV / 2; j++) v[j] = (b ? v[2 * j + 1] : v[2 * j]) + dpp_f32<0xB1>(b ? v[2 * j] : v[2 * j + 1]);  // quad_perm [1,0,3,2]
  }
  if constexpr (NV >= 4) {
    const bool b = lane & 2;
#pragma unroll
    for (int j = 0; j < NV / 4; j++) v[j] = (b ? v[2 * j + 1] : v[2 * j]) + dpp_f32<0x4E>(b ? v[2 * j] : v[2 * j + 1]);  // quad_perm [2,3,0,1]
  }
  if constexpr (NV >= 8) {
    const bool b = lane & 4;
#pragma unroll
    for (int j = 0; j < NV / 8; j++) {
      const float give = b ? v[2 * j] : v[2 * j + 1];
      const float up = dpp_f32<0x104>(give), down = dpp_f32<0x114>(give);  // row_shl:4 (from lane + 4), row_shr:4 (from lane - 4)
      v[j] = (b ? v[2 * j + 1] : v[2 * j]) + (b ? down : up);
    }
  }
  if constexpr (NV >= 16) {
    const bool b = lane & 8;
    v[0] = (b ? v[1] : v[0]) + dpp_f32<0x128>(b ? v[0] : v[1]);  // row_ror:8
  }
  float r = v[0];
  if (NV < 16) r += dpp_f32<0x128>(r);
  if (NV < 8) r += dpp_f32<0x124>(r);
  if (NV < 4) r += dpp_f32<0x122>(r);
  if (NV < 2) r += dpp_f32<0x121>(r);
  r += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, r)));
  r += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, r)));
  return r;
}
__device__ __forceinline__ unsigned xcc_id() {
  // HW_REG_XCC_ID (id 20), bits [3:0]
  return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 7u;  // MI355X: 8 XCDs
}
__device__ __forceinline__ u32x4 ldg_stream(const u32x4 *p) { return __builtin_nontemporal_load(p); }

// Loads of data another workgroup produced earlier in this launch.  The per-XCD L2s are write-back and
// not coherent with each other, and the CU's vector L1 is not coherent with anything: producers write back
// their L2 at the barrier (release by the XCD's last arriver), consumers read with device-scope loads
// (sc1: miss the L1, coherent in L2), so no cache invalidate is ever issued.
// (the pointers are cast to the global address space explicitly: an atomic through a generic pointer becomes a flat
// access, which is counted against the LDS queue as well and waits for it)
#define MK_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ uint32_t ldc_u32(const void *p) {
  return __hip_atomic_load((const MK_GLOBAL uint32_t *)(unsigned long long)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int ldc_i32(const int *p) { return (int)ldc_u32(p); }
__device__ __forceinline__ float ldc_f32(const float *p) { return __uint_as_float(ldc_u32(p)); }
__device__ __forceinline__ unsigned long long ldc_u64(const void *p) {
  return __hip_atomic_load((const MK_GLOBAL unsigned long long *)(unsigned long long)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u32x4 ldc_16B(const u32x4 *p) {
  const unsigned long long a = ldc_u64(p), b = ldc_u64((const unsigned long long *)p + 1);
  u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
  return r;
}
// Stores that are written through to memory (device scope), for outputs of stages that skip the L2 write-back at
// their barrier.
__device__ __forceinline__ void stc_u16(uint16_t *p, uint16_t v) {
  __hip_atomic_store((__attribute__((address_space(1))) uint16_t *)(unsigned long long)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc_f32(float *p, float v) {
  __hip_atomic_store((__attribute__((address_space(1))) unsigned *)(unsigned long long)p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc_u64(void *p, unsigned long long v) {
  __hip_atomic_store((__attribute__((address_space(1))) unsigned long long *)(unsigned long long)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc_i32(int *p, int v) {
  __hip_atomic_store((__attribute__((address_space(1))) int *)(unsigned long long)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void stc_16B(u32x4 *p, u32x4 v) {
  __attribute__((address_space(1))) unsigned long long *q = (__attribute__((address_space(1))) unsigned long long *)(unsigned long long)p;
  __hip_atomic_store(q, (unsigned long long)v.x | ((unsigned long long)v.y << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(q + 1, (unsigned long long)v.z | ((unsigned long long)v.w << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// four consecutive bf16 outputs of one token row, written through: one 8-byte store when the run is whole and aligned
__device__ __forceinline__ void stc_bf16x4(uint16_t *row, int n0, int n_out, const float (&r)[4]) {
  uint16_t *p = row + n0;
  if (n0 + 3 < n_out && (((unsigned long long)p) & 7) == 0) {
    const unsigned long long v = (unsigned long long)pack2(r[0], r[1]) | ((unsigned long long)pack2(r[2], r[3]) << 32);
    __hip_atomic_store((__attribute__((address_space(1))) unsigned long long *)(unsigned long long)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++)
      if (n0 + i < n_out) stc_u16(p + i, (uint16_t)f2bf(r[i]));
  }
}
__device__ __forceinline__ uint16_t ldc_u16(const uint16_t *p) {
  const uintptr_t a = (uintptr_t)p;
  const uint32_t w = ldc_u32((const void *)(a & ~(uintptr_t)3));
  return (uint16_t)((a & 2) ? (w >> 16) : (w & 0xffffu));
}

// ----------------------------------------------------------------------------- grid barrier
// Stage barrier with one arrival counter per XCD (each in its own 128-byte line, so a die's arrivals meet in that
// die's L2 and only completed lines travel between dies).  Replaces the reference's per-event two-level counters
// (persistent_kernel.cuh:1214-1284).
__device__ __forceinline__ bool spin_ok(MkSync *s, unsigned &spins, unsigned where) {
  ++spins;
  if ((spins & 1023u) == 0) {
    if (__hip_atomic_load(&s->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return false;
    if (spins >= MK_SPIN_LIMIT) {
      __hip_atomic_store(&s->abort_where, where, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&s->abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
  }
  return true;
}

// arrive: this workgroup's outputs of the current stage are complete: write them back (agent-scope release) and
// count the arrival in the counter of this workgroup's XCD (one 128-byte line per die, so the 32 arrivals of a die meet
// in that die's L2).  Nothing is returned, so nobody waits on the atomic.
__device__ __forceinline__ void barrier_arrive(Ctx &c) {
  MkSync *s = c.sync;
  if (c.arrive_w0) {
    // Only wavefront 0 has stores outstanding: it waits for them and posts the arrival; the other wavefronts go straight
    // on to the next stage, whose weight prefetch is then in flight while those stores are still being acknowledged
    // (about a microsecond per stage in which the CU otherwise requests nothing).
    c.arrive_w0 = false;
    if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    c.seq++;
    c.epoch++;
    if (threadIdx.x == 0) __hip_atomic_fetch_add(&s->local_ctr[c.xcd][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    c.wrote_through = false;
    c.pending = true;
    return;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  c.seq++;
  if (threadIdx.x == 0) c.sh_ticket[c.seq & 1] = 0;  // the counter of the stage that starts now (last used two stages ago)
  __syncthreads();
  c.epoch++;
  if (threadIdx.x == 0) {
    if (c.wrote_through) __hip_atomic_fetch_add(&s->local_ctr[c.xcd][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
      __hip_atomic_fetch_add(&s->local_ctr[c.xcd][0], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
  }
  c.wrote_through = false;
  c.pending = true;
}

// poll (thread 0 only): the barrier is complete when every die's counter has reached quota x epoch.  The eight
// counters are read with independent device-scope loads (one round trip per poll), so completion is seen two hops
// after the last arrival (atomic -> load) instead of going through a leader and a broadcast flag.
__device__ __forceinline__ void barrier_poll(Ctx &c) {
  MkSync *s = c.sync;
  const unsigned epoch = c.epoch;
  unsigned spins = 0;
  unsigned va[8];
  auto issue = [&](unsigned (&v)[8]) {
#pragma unroll
    for (int x = 0; x < 8; x++) v[x] = __hip_atomic_load(&s->local_ctr[x][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  auto done = [&](const unsigned (&v)[8]) -> bool {
    bool ok = true;
#pragma unroll
    for (int x = 0; x < 8; x++) ok = ok && mk_counter_reached(v[x], c.quotas[x] * epoch);
    return ok;
  };
  while (true) {
    issue(va);
    if (done(va) || !spin_ok(s, spins, epoch)) break;
    __builtin_amdgcn_s_sleep(MK_TUNE_POLL_SLEEP);
  }
  *c.sh_dead = (spins >= 1024u) ? (int)__hip_atomic_load(&s->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
}

// bookkeeping after the workgroup barrier that follows barrier_poll
__device__ __forceinline__ void barrier_done(Ctx &c) {
  c.pending = false;
  c.dead = c.dead || (__builtin_amdgcn_readfirstlane(*c.sh_dead) != 0);
  c.t_wait = (long long)wall_clock64();
}

__device__ __forceinline__ void barrier_wait(Ctx &c) {
  if (!c.pending) return;
  if (threadIdx.x == 0) barrier_poll(c);
  __syncthreads();
  barrier_done(c);
}

// ----------------------------------------------------------------------------- scheduler
// On-GPU continuous batching for offline serving: commit the tokens produced by the previous
// iteration, retire finished requests and recycle their pages, then build the next batch
// (running requests first, then new prefills).  Same observable behaviour on the ten meta
// tensors as the reference's MODE_OFFLINE prepare_next_batch (persistent_kernel.cuh:380-536).
// Runs on one thread.  Returns the number of tokens scheduled.
__device__ __attribute__((noinline)) int mk_prepare_next_batch(const MkRuntime &rt, int *scratch_pages) {
  MkSched *sc = rt.sched;
  const int R = rt.max_requests, B = rt.max_tokens, PS = rt.page_size, NP = rt.max_pages;
  int head = sc->page_queue_head, tail = sc->page_queue_tail;
  // 1. commit outputs of the previous iteration, retire finished requests
  for (int i = 0; i < R; i++) {
    const int req = rt.request_ids[i];
    if (req < 0) continue;
    const int st = rt.step[req];
    const int q0 = rt.qo_indptr[i];
    const int n = rt.qo_indptr[i + 1] - q0;
    const int plen = rt.prompt_lengths[req];
    // a decoding request of a speculating graph keeps what its verify stage accepted: the sampled token of its first
    // row, and one more for every candidate row in front that turned out right (persistent_kernel.cuh:541-552)
    int nc = n;
    if (rt.spec_len > 0 && st >= plen && n > 0) nc = max(1, min(n, ldc_i32(&rt.num_new_tokens[req])));
    for (int j = 0; j < nc; j++) {
      const int pos = st + j + 1;
      if (pos >= plen && pos < rt.max_seq) rt.tokens[(long long)req * rt.max_seq + pos] = rt.output_tokens[q0 + j];
    }
    const int ns = st + nc;
    rt.step[req] = ns;
    const bool full = ns + 1 >= rt.max_seq;
    const bool eos = ns >= plen && rt.tokens[(long long)req * rt.max_seq + ns] == rt.eos_token_id;
    if (full || eos) {
      rt.request_ids[i] = -1;
      const int k0 = rt.kv_indptr[i], k1 = rt.kv_indptr[i + 1];
      for (int j = k0; j < k1; j++) {
        rt.page_queue[tail % NP] = rt.kv_indices[j];
        tail++;
      }
    }
  }
  // 2. snapshot the page table (it is compacted in place below)
  const int old_pages = rt.kv_indptr[R];
  for (int i = 0; i < old_pages; i++) scratch_pages[i] = rt.kv_indices[i];
  // 3. running requests keep their slot order; compact over retired slots
  int nreq = 0, ntok = 0, npage = 0;
  for (int i = 0; i < R; i++) {
    const int req = rt.request_ids[i];
    if (req < 0) continue;
    const int k0 = rt.kv_indptr[i];
    const int had = rt.kv_indptr[i + 1] - k0;
    rt.request_ids[nreq] = req;
    rt.qo_indptr[nreq] = ntok;
    rt.kv_indptr[nreq] = npage;
    const int st = rt.step[req];
    int n = rt.prompt_lengths[req] - st;
    if (n > 0) n = min(n, min(rt.max_new_per_req, B - ntok));  // prefill chunk
    else n = min(1 + min(rt.spec_len, min(rt.max_new_per_req - 1, rt.max_seq - 2 - st)), B - ntok);  // decode: the newest token (+ candidate rows,
                                                                                                      // whose ids the n-gram stage fills in)
    for (int j = 0; j < n; j++) {
      rt.input_tokens[ntok + j] = rt.tokens[(long long)req * rt.max_seq + st + j];
      rt.tok_slot[ntok + j] = nreq;
      rt.tok_pos[ntok + j] = st + j;
      rt.tok_first[ntok + j] = ntok;
    }
    const int need = (st + n + PS - 1) / PS;
    const int last = (st + n) % PS;
    rt.kv_last_page_len[nreq] = last == 0 ? PS : last;
    for (int j = 0; j < had; j++) rt.kv_indices[npage + j] = scratch_pages[k0 + j];
    for (int j = had; j < need; j++) {
      rt.kv_indices[npage + j] = rt.page_queue[head % NP];
      head++;
    }
    npage += need;
    ntok += n;
    nreq++;
  }
  // 4. admit new requests while there is room
  while (nreq < R && ntok < B) {
    const int req = sc->next_request_id;
    if (req >= rt.total_requests) break;
    rt.request_ids[nreq] = req;
    rt.qo_indptr[nreq] = ntok;
    rt.kv_indptr[nreq] = npage;
    const int n = min(rt.prompt_lengths[req], min(rt.max_new_per_req, B - ntok));
    for (int j = 0; j < n; j++) {
      rt.input_tokens[ntok + j] = rt.tokens[(long long)req * rt.max_seq + j];
      rt.tok_slot[ntok + j] = nreq;
      rt.tok_pos[ntok + j] = j;
      rt.tok_first[ntok + j] = ntok;
    }
    const int need = (n + PS - 1) / PS;
    const int last = n % PS;
    rt.kv_last_page_len[nreq] = last == 0 ? PS : last;
    for (int j = 0; j < need; j++) {
      rt.kv_indices[npage + j] = rt.page_queue[head % NP];
      head++;
    }
    ntok += n;
    npage += need;
    nreq++;
    sc->next_request_id = req + 1;
  }
  // 5. clear unused slots
  for (int i = nreq; i < R; i++) rt.request_ids[i] = -1;
  for (int i = nreq; i <= R; i++) {
    rt.qo_indptr[i] = ntok;
    rt.kv_indptr[i] = npage;
  }
  sc->page_queue_head = head;
  sc->page_queue_tail = tail;
  sc->num_tokens = ntok;
  sc->num_reqs = nreq;
  return ntok;
}

// The same step on one wavefront: lane i owns batch slot i (at most 64 slots) in the phases that walk the old batch, and
// candidate request next_request_id + i when new requests are admitted.  What the sequential version carries from slot
// to slot are running sums -- tokens scheduled so far (saturating at the iteration's token budget), pages in the
// compacted table, pages taken from / returned to the ring -- and those are wavefront prefix sums:
//   tokens before slot i = min(sum of the earlier slots' wishes, B)   (a saturating sum of non-negative terms)
// so every lane derives exactly the values the sequential loop would have reached at its slot; the result is identical
// entry for entry (checked against the C restatement after every iteration by the GPU scheduler tests).
// Each lane's dependent loads (request id -> step -> token row) then overlap with the other lanes', which is what the
// sequential version spends its time on (about 1.8 us per occupied slot).  `lds` holds the page-table snapshot
// ([0, NP)) and the pages retired in this step in ring order ([NP, 2 NP)): a page returned by one lane and handed out
// again by another in the same step goes through LDS, never through a store and a load of different lanes.
__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int u = __builtin_amdgcn_ds_bpermute(((lane - o) & 63) << 2, v);
    if (lane >= o) v += u;
  }
  return v;
}
__device__ __forceinline__ int wave_bcast(int v, int src) { return __builtin_amdgcn_readlane(v, src); }

__device__ __attribute__((noinline)) int mk_prepare_next_batch_wave(const MkRuntime &rt, int *lds, int lane) {
  MkSched *sc = rt.sched;
  const int R = rt.max_requests, B = rt.max_tokens, PS = rt.page_size, NP = rt.max_pages;
  int *snap = lds, *freed = lds + NP;
  const int head0 = sc->page_queue_head, tail0 = sc->page_queue_tail;
  const int old_pages = rt.kv_indptr[R];
  // 1. commit the previous iteration's outputs, find the requests that retire
  const bool slot = lane < R;
  int req = slot ? rt.request_ids[lane] : -1;
  int st = 0, plen = 0, k0 = 0, k1 = 0;
  bool retire = false;
  if (req >= 0) {
    st = rt.step[req];
    const int q0 = rt.qo_indptr[lane];
    const int n = rt.qo_indptr[lane + 1] - q0;
    plen = rt.prompt_lengths[req];
    k0 = rt.kv_indptr[lane];
    k1 = rt.kv_indptr[lane + 1];
    for (int j = 0; j < n; j++) {
      const int pos = st + j + 1;
      if (pos >= plen && pos < rt.max_seq) rt.tokens[(long long)req * rt.max_seq + pos] = rt.output_tokens[q0 + j];
    }
    st += n;
    rt.step[req] = st;
    const bool full = st + 1 >= rt.max_seq;
    const bool eos = st >= plen && rt.tokens[(long long)req * rt.max_seq + st] == rt.eos_token_id;
    retire = full || eos;
  }
  // 2. snapshot the page table; retired pages go back to the ring in slot order
  for (int i = lane; i < old_pages; i += 64) snap[i] = rt.kv_indices[i];
  const int rp = retire ? k1 - k0 : 0;
  const int rp_incl = wave_incl_scan(rp, lane);
  const int n_freed = wave_bcast(rp_incl, 63);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  for (int j = 0; j < rp; j++) {
    const int pg = snap[k0 + j], at = rp_incl - rp + j;
    freed[at] = pg;
    rt.page_queue[(tail0 + at) % NP] = pg;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  const int avail0 = tail0 - head0;  // pages the ring held before this step
  auto ring_page = [&](int a) -> int {  // the a-th page handed out in this step
    return a < avail0 ? rt.page_queue[(head0 + a) % NP] : freed[a - avail0];
  };
  // 3. running requests keep their slot order, compacted over retired slots
  const bool alive = req >= 0 && !retire;
  const unsigned long long alive_mask = __ballot(alive);
  const int rank = __popcll(alive_mask & ((1ull << lane) - 1ull));
  const int nrun = __popcll(alive_mask);
  const int wish = alive ? (plen - st > 0 ? min(plen - st, rt.max_new_per_req) : 1) : 0;
  const int wish_incl = wave_incl_scan(wish, lane);
  const int tok0 = min(wish_incl - wish, B), n = min(wish_incl, B) - tok0;
  const int had = alive ? k1 - k0 : 0;
  const int need = alive ? (st + n + PS - 1) / PS : 0;
  const int need_incl = wave_incl_scan(need, lane);
  const int fresh = need > had ? need - had : 0;
  const int fresh_incl = wave_incl_scan(fresh, lane);
  if (alive) {
    const int page0 = need_incl - need, a0 = fresh_incl - fresh;
    rt.request_ids[rank] = req;
    rt.qo_indptr[rank] = tok0;
    rt.kv_indptr[rank] = page0;
    for (int j = 0; j < n; j++) {
      rt.input_tokens[tok0 + j] = rt.tokens[(long long)req * rt.max_seq + st + j];
      rt.tok_slot[tok0 + j] = rank;
      rt.tok_pos[tok0 + j] = st + j;
      rt.tok_first[tok0 + j] = tok0;
    }
    const int last = (st + n) % PS;
    rt.kv_last_page_len[rank] = last == 0 ? PS : last;
    for (int j = 0; j < had && j < need; j++) rt.kv_indices[page0 + j] = snap[k0 + j];
    for (int j = had; j < need; j++) rt.kv_indices[page0 + j] = ring_page(a0 + j - had);
  }
  int ntok = min(wave_bcast(wish_incl, 63), B);
  int npage = wave_bcast(need_incl, 63);
  int taken = wave_bcast(fresh_incl, 63);
  int nreq = nrun;
  // 4. admit new requests while there is room: lane k looks at request next_request_id + k
  {
    const int next = sc->next_request_id;
    const int cand = next + lane;
    const bool valid = nreq + lane < R && cand < rt.total_requests;
    const int cplen = valid ? rt.prompt_lengths[cand] : 0;
    const int cwish = valid ? min(cplen, rt.max_new_per_req) : 0;
    const int cw_incl = wave_incl_scan(cwish, lane);
    // the sequential loop reaches candidate k only while the budget is not exhausted, and stops at the first request
    // that does not exist; candidates are valid in a prefix of the lanes, so "admitted" is a prefix too
    const bool admit = valid && ntok + (cw_incl - cwish) < B;
    const int cn = admit ? min(cwish, B - (ntok + cw_incl - cwish)) : 0;
    const int cneed = admit ? (cn + PS - 1) / PS : 0;
    const int cneed_incl = wave_incl_scan(cneed, lane);
    const int n_admit = __popcll(__ballot(admit));
    if (admit) {
      const int s_ = nreq + lane, tok0c = ntok + cw_incl - cwish, page0 = npage + cneed_incl - cneed, a0 = taken + cneed_incl - cneed;
      rt.request_ids[s_] = cand;
      rt.qo_indptr[s_] = tok0c;
      rt.kv_indptr[s_] = page0;
      for (int j = 0; j < cn; j++) {
        rt.input_tokens[tok0c + j] = rt.tokens[(long long)cand * rt.max_seq + j];
        rt.tok_slot[tok0c + j] = s_;
        rt.tok_pos[tok0c + j] = j;
        rt.tok_first[tok0c + j] = tok0c;
      }
      const int last = cn % PS;
      rt.kv_last_page_len[s_] = last == 0 ? PS : last;
      for (int j = 0; j < cneed; j++) rt.kv_indices[page0 + j] = ring_page(a0 + j);
    }
    const int cn_incl = wave_incl_scan(cn, lane);
    ntok += wave_bcast(cn_incl, 63);
    npage += wave_bcast(cneed_incl, 63);
    taken += wave_bcast(cneed_incl, 63);
    nreq += n_admit;
    if (lane == 0) sc->next_request_id = next + n_admit;
  }
  // 5. clear unused slots
  for (int i = nreq + lane; i < R; i += 64) rt.request_ids[i] = -1;
  for (int i = nreq + lane; i <= R; i += 64) {
    rt.qo_indptr[i] = ntok;
    rt.kv_indptr[i] = npage;
  }
  if (lane == 0) {
    sc->page_queue_head = head0 + taken;
    sc->page_queue_tail = tail0 + n_freed;
    sc->num_tokens = ntok;
    sc->num_reqs = nreq;
  }
  return ntok;
}

// Batch description for a launch whose batch the HOST prepared (the reference's MODE_ONLINE_NOTOKEN, one pass per launch,
// persistent_kernel.cuh:570-582, and MODE_ONEPASS): the caller has filled input_tokens, qo_indptr, paged_kv_indptr,
// paged_kv_indices and paged_kv_last_page_len the way the reference's attention tasks read them -- request slot i owns
// rows [qo_indptr[i], qo_indptr[i+1]) and its sequence, new tokens included, is (pages - 1) * page_size + last_page_len
// long, so its rows sit at the last positions of that sequence.  Derives the per-row slot / position / first-row arrays
// on the device (no host round trip, so a serving loop can enqueue launches back to back).  Runs on one thread.
__device__ __attribute__((noinline)) int mk_batch_from_meta(const MkRuntime &rt) {
  const int R = rt.max_requests, B = rt.max_tokens;
  // A batch the stages cannot run as described is not run at all: truncating a request's rows would leave the rest with
  // the slot / position an earlier launch gave them, and they would append K/V rows to some other request's cache.
  // bad: 1 = rows outside [0, max tokens), overlapping, or with gaps; 2 = more rows for one request than
  // max_tokens_per_request; 3 = a sequence shorter than its new rows, longer than max_seq_length, or without pages.
  int ntok = 0, bad = 0;
  unsigned long long covered = 0ull;
  for (int i = 0; i < R && !bad; i++) {
    const int q0 = rt.qo_indptr[i], n = rt.qo_indptr[i + 1] - q0;
    if (n <= 0) continue;  // an unused slot (hosts that fill only the first entries leave zeros behind them)
    if (q0 < 0 || q0 + n > B) {
      bad = 1;
      break;
    }
    if (n > rt.max_new_per_req) {
      bad = 2;
      break;
    }
    const unsigned long long rows = (n >= 64 ? ~0ull : ((1ull << n) - 1ull)) << q0;
    if (covered & rows) {
      bad = 1;
      break;
    }
    covered |= rows;
    const int pages = rt.kv_indptr[i + 1] - rt.kv_indptr[i];
    const int len = (pages - 1) * rt.page_size + rt.kv_last_page_len[i];
    if (pages < 1 || len < n || len > rt.max_seq) {
      bad = 3;
      break;
    }
    for (int j = 0; j < n; j++) {
      rt.tok_slot[q0 + j] = i;
      rt.tok_pos[q0 + j] = len - n + j;
      rt.tok_first[q0 + j] = q0;
    }
    if (q0 + n > ntok) ntok = q0 + n;
  }
  if (!bad && covered != (ntok >= 64 ? ~0ull : ((1ull << ntok) - 1ull))) bad = 1;
  if (bad) ntok = 0;
  rt.sched->bad_batch = bad;
  rt.sched->num_tokens = ntok;
  return ntok;
}

// The reference's MODE_ONLINE step (persistent_kernel.cuh:538-568): one request (slot 0, request 0) whose tokens the
// host has written into tokens[0, :]; every pass consumes num_new_tokens[0] of them starting at step[0].  After a pass
// step[0] advances by what the pass consumed, and the run ends when the position it started from is within two of
// max_seq_length or the token after it is the EOS id -- the reference's test, on the step value from before the
// advance.  What the reference leaves to the host and is done here instead: the page table of the one request
// (identity: page j of the ring is page j of the sequence) and the qo / kv index arrays.  Runs on one thread.
__device__ __attribute__((noinline)) int mk_online_next_batch(const MkRuntime &rt) {
  MkSched *sc = rt.sched;
  const int PS = rt.page_size;
  int step = rt.step[0];
  if (sc->online_started) {
    const int consumed = sc->num_tokens;
    rt.step[0] = step + consumed;
    const bool stop = (step + 2 >= rt.max_seq) || (rt.tokens[step + 1] == rt.eos_token_id);
    step += consumed;
    if (stop) {
      sc->num_tokens = 0;
      return 0;
    }
  }
  sc->online_started = 1;
  int n = rt.num_new_tokens ? rt.num_new_tokens[0] : 1;
  n = n < 1 ? 1 : n;
  n = min(n, min(rt.max_new_per_req, rt.max_tokens));
  n = min(n, rt.max_seq - 1 - step);
  if (n <= 0) {
    sc->num_tokens = 0;
    return 0;
  }
  for (int j = 0; j < n; j++) {
    rt.input_tokens[j] = rt.tokens[step + j];
    rt.tok_slot[j] = 0;
    rt.tok_pos[j] = step + j;
    rt.tok_first[j] = 0;
  }
  const int need = (step + n + PS - 1) / PS, last = (step + n) % PS;
  rt.request_ids[0] = 0;
  rt.kv_last_page_len[0] = last == 0 ? PS : last;
  for (int j = 0; j < need && j < rt.max_pages; j++) rt.kv_indices[j] = j;
  rt.qo_indptr[0] = 0;
  rt.kv_indptr[0] = 0;
  for (int i = 1; i <= rt.max_requests; i++) {
    rt.qo_indptr[i] = n;
    rt.kv_indptr[i] = need;
  }
  sc->num_tokens = n;
  sc->num_reqs = 1;
  return n;
}

// ----------------------------------------------------------------------------- weights
__device__ __forceinline__ const u32x4 *weight_row(CWeight &w, int r, int k8) {
  if (w.nseg == 1) return (const u32x4 *)w.seg[0] + (size_t)r * k8;
  const int g = r / w.group_rows;
  int o = r - g * w.group_rows;
  int s = 0;
  if (o >= w.seg_rows[0]) {
    o -= w.seg_rows[0];
    s = 1;
    if (w.nseg > 2 && o >= w.seg_rows[1]) {
      o -= w.seg_rows[1];
      s = 2;
    }
  }
  return (const u32x4 *)w.seg[s] + (size_t)(g * w.seg_rows[s] + o) * k8;
}

// Re-lays the weights of one linear stage in matrix-core tile order (MkStage::wpack); one thread per 16-byte operand.
// Rows past the last output repeat it (their products are never stored).
extern "C" __global__ __launch_bounds__(256) void mk_pack_weights_kernel(const MkWeight w, int n, int k, int silu, int half, u32x4 *dst, long long total) {
  const int k8 = k / 8, nsteps = k >> 6;
  const int n_out = silu ? n / 2 : n;
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256) {
    const int lane = (int)(idx & 63);
    long long r = idx >> 6;
    const int h = (int)(r & 1);
    r >>= 1;
    const int step = (int)(r % nsteps), ti = (int)(r / nsteps);
    const int lr = lane & 15, lg = lane >> 4;
    int vr;
    if (silu) {
      const int o = min((ti >> 1) * 16 + lr, n_out - 1), gi = o / half;
      vr = gi * 2 * half + (o - gi * half) + ((ti & 1) ? half : 0);
    } else {
      vr = min(ti * 16 + lr, n_out - 1);
    }
    const u32x4 *row;
    if (w.nseg == 1) {
      row = (const u32x4 *)w.seg[0] + (size_t)vr * k8;
    } else {
      const int g = vr / w.group_rows;
      int o = vr - g * w.group_rows, sg = 0;
      while (sg + 1 < w.nseg && o >= w.seg_rows[sg]) o -= w.seg_rows[sg++];
      row = (const u32x4 *)w.seg[sg] + (size_t)(g * w.seg_rows[sg] + o) * k8;
    }
    dst[idx] = row[step * 8 + h * 4 + lg];
  }
}

// ----------------------------------------------------------------------------- stages
// Every stage function posts barrier_wait(c) itself, after any work that does not depend on the previous
// stage (weight prefetch), and the main loop posts barrier_arrive(c) when the function returns.

// Gather embedding rows.  Reference task: tasks/ampere/embedding.cuh:42-72.
__device__ __forceinline__ void stage_embed(CStage &st, Ctx &c, const MkRuntime &rt, int M) {
  barrier_wait(c);
  const int k8 = st.k / 8;
  for (int t = c.vid; t < M; t += c.G) {
    long long id;
    if (st.flags & MK_F_EMBED_FROM_TOKENS) {
      const int req = ldc_i32(&rt.request_ids[ldc_i32(&rt.tok_slot[t])]);
      id = (long long)ldc_u64(&rt.tokens[(long long)req * rt.max_seq + ldc_i32(&rt.tok_pos[t])]);
    } else {
      id = (long long)ldc_u64((const long long *)st.in + t);
    }
    const u32x4 *src = (const u32x4 *)st.w.seg[0] + (size_t)(id < 0 ? 0 : id) * k8;
    u32x4 *dst = (u32x4 *)st.out + (size_t)t * (st.ld_out / 8);
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int i = threadIdx.x; i < k8; i += MK_THREADS) dst[i] = id < 0 ? zero : src[i];
  }
}

// Block-wide sum of one float per thread.
__device__ __forceinline__ float block_sum(float v, float *red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// RMSNorm of full rows, one workgroup per token row (used when an iteration has several tokens;
// single-token iterations fuse the norm into the consuming linear).  y = bf16((x * r) * w) with
// r = rsqrt(mean(x^2) + eps) in fp32.  Reference task: tasks/mi300/rmsnorm_mi300.cuh:37-188.
__device__ __forceinline__ void stage_norm(CStage &st, Ctx &c, int M, char *smem) {
  const int k8 = st.k / 8;
  if ((st.k & 7) == 0 && k8 <= 6 * MK_THREADS && (st.ld_in & 7) == 0 && (st.ld_out & 7) == 0) {
    // Row per workgroup, up to six 16-byte segments per thread: the norm weights are requested before the barrier is
    // awaited, the row is read with device-scope loads and written through, so the arrival needs no L2 write-back.
    constexpr int NS = 6;
    const int tid = threadIdx.x;
    float *red = (float *)smem;
    const u32x4 *w4 = (const u32x4 *)st.norm_w;
    u32x4 g[NS], v[NS];
#pragma unroll
    for (int j = 0; j < NS; j++)
      if (j * MK_THREADS < k8) g[j] = w4[min(tid + j * MK_THREADS, k8 - 1)];
    barrier_wait(c);
    const int dS = c.defer_S;
    c.defer_S = 0;
    // rows are dealt round-robin over the dies, so a handful of rows does not funnel through one die's memory path
    const int t0 = c.even_xcds ? c.rank * c.nxcd + c.xi : c.vid;
    for (int t = t0; t < M; t += c.G) {
      const u32x4 *x = (const u32x4 *)((const uint16_t *)st.in + (size_t)t * st.ld_in);
      u32x4 *y = (u32x4 *)((uint16_t *)st.out + (size_t)t * st.ld_out);
      float ss = 0.f;
      if (dS) {
        // the rows are still K-slice partials: finish the producing linear (sum, residual, rounding), store its output
        // row where it belongs, and normalise the rounded values
        const u32x4 *r4 = (const u32x4 *)((const uint16_t *)c.defer_res + (size_t)t * c.defer_ld_res);
#pragma unroll
        for (int j = 0; j < NS; j++)
          if (j * MK_THREADS < k8) {
            const int seg = min(tid + j * MK_THREADS, k8 - 1);
            float a[8];
#pragma unroll
            for (int e = 0; e < 8; e++) a[e] = 0.f;
            const u32x4 rv = ldc_16B(c.defer_res ? r4 + seg : (const u32x4 *)c.defer_part);  // requested ahead of the partials it is added to
            auto sum_slices = [&](auto ns) {  // all slices requested at once, summed in slice order
              constexpr int Q = decltype(ns)::value;
              u32x4 pv[Q][2];
#pragma unroll
              for (int q = 0; q < Q; q++) {
                const u32x4 *p = (const u32x4 *)(c.defer_part + ((size_t)q * c.defer_rows + t) * st.k) + seg * 2;
                pv[q][0] = ldc_16B(p);
                pv[q][1] = ldc_16B(p + 1);
              }
#pragma unroll
              for (int q = 0; q < Q; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                  a[e] += __uint_as_float(pv[q][0][e]);
                  a[4 + e] += __uint_as_float(pv[q][1][e]);
                }
            };
            if (dS == 2) sum_slices(std::integral_constant<int, 2>{});
            else if (dS == 4) sum_slices(std::integral_constant<int, 4>{});
            else sum_slices(std::integral_constant<int, 8>{});
            if (c.defer_res) {
#pragma unroll
              for (int e = 0; e < 4; e++) {
                a[2 * e] += bf_lo(rv[e]);
                a[2 * e + 1] += bf_hi(rv[e]);
              }
            }
#pragma unroll
            for (int e = 0; e < 4; e++) v[j][e] = pack2(a[2 * e], a[2 * e + 1]);
          }
#pragma unroll
        for (int j = 0; j < NS; j++)  // stores after all the loads: neither is moved across the other
          if (tid + j * MK_THREADS < k8) stc_16B((u32x4 *)x + tid + j * MK_THREADS, v[j]);
      }
#pragma unroll
      for (int j = 0; j < NS; j++)
        if (j * MK_THREADS < k8) {
          const bool ok = tid + j * MK_THREADS < k8;
          if (!dS) v[j] = ldc_16B(x + min(tid + j * MK_THREADS, k8 - 1));
#pragma unroll
          for (int e = 0; e < 4; e++) ss += ok ? bf_lo(v[j][e]) * bf_lo(v[j][e]) + bf_hi(v[j][e]) * bf_hi(v[j][e]) : 0.f;
        }
      ss = block_sum(ss, red);
      const float r = rsqrtf(ss / (float)st.k + st.eps);
#pragma unroll
      for (int j = 0; j < NS; j++)
        if (tid + j * MK_THREADS < k8) {
          u32x4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) o[e] = pack2((bf_lo(v[j][e]) * r) * bf_lo(g[j][e]), (bf_hi(v[j][e]) * r) * bf_hi(g[j][e]));
          stc_16B(y + tid + j * MK_THREADS, o);
        }
      __syncthreads();
    }
    c.wrote_through = true;
    return;
  }
  barrier_wait(c);
  float *red = (float *)smem;
  uint32_t *xs = (uint32_t *)(smem + 1024);
  const int k2 = st.k / 2;
  for (int t = c.vid; t < M; t += c.G) {
    const uint32_t *x = (const uint32_t *)st.in + (size_t)t * (st.ld_in / 2);
    const uint32_t *w = (const uint32_t *)st.norm_w;
    uint32_t *y = (uint32_t *)st.out + (size_t)t * (st.ld_out / 2);
    float ss = 0.f;
    for (int i = threadIdx.x; i < k2; i += MK_THREADS) {
      const uint32_t u = ldc_u32(x + i);
      xs[i] = u;
      ss += bf_lo(u) * bf_lo(u) + bf_hi(u) * bf_hi(u);
    }
    ss = block_sum(ss, red);
    const float r = rsqrtf(ss / (float)st.k + st.eps);
    for (int i = threadIdx.x; i < k2; i += MK_THREADS) {
      const uint32_t u = xs[i], g = w[i];
      y[i] = pack2((bf_lo(u) * r) * bf_lo(g), (bf_hi(u) * r) * bf_hi(g));
    }
    __syncthreads();
  }
}

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.f + __expf(-g)) * u; }

// Stage the single input row of a one-token linear in LDS as packed bf16, applying the fused RMSNorm when the
// stage asks for it (virtual workgroup 0 also stores the normalised row, which is the norm task's output tensor).
__device__ __forceinline__ void stage_x_m1(CStage &st, const Ctx &c, uint32_t *xs, float *red) {
  const int tid = threadIdx.x, k4 = st.k / 4;
  const unsigned long long *xin = (const unsigned long long *)st.in;
  unsigned long long *xs2 = (unsigned long long *)xs;
  if (st.flags & MK_F_NORM) {
    float ss = 0.f;
    for (int i = tid; i < k4; i += MK_THREADS) {
      const unsigned long long u = ldc_u64(xin + i);
      xs2[i] = u;
      const uint32_t a = (uint32_t)u, b = (uint32_t)(u >> 32);
      ss += bf_lo(a) * bf_lo(a) + bf_hi(a) * bf_hi(a) + bf_lo(b) * bf_lo(b) + bf_hi(b) * bf_hi(b);
    }
    ss = block_sum(ss, red);
    const float r = rsqrtf(ss / (float)st.k + st.eps);
    const uint32_t *nw = (const uint32_t *)st.norm_w;
    uint32_t *no = (c.vid == 0) ? (uint32_t *)st.norm_out : nullptr;
    for (int i = tid; i < st.k / 2; i += MK_THREADS) {
      const uint32_t u = xs[i], g = nw[i];
      const uint32_t y = pack2((bf_lo(u) * r) * bf_lo(g), (bf_hi(u) * r) * bf_hi(g));
      xs[i] = y;
      if (no) no[i] = y;
    }
  } else {
    for (int i = tid; i < k4; i += MK_THREADS) xs2[i] = ldc_u64(xin + i);
  }
  __syncthreads();
}

// Same staging done by ONE wavefront (the control wavefront of a tuned single-token linear): lane l owns the
// 16-byte segments l, l+64, ... of the row, the sum of squares is a wavefront reduction, no workgroup barrier inside.
template <int KL>
__device__ __forceinline__ void stage_x_m1_wave(CStage &st, const Ctx &c, uint32_t *xs, int lane, const u32x4 (&nwv)[KL]) {
  const u32x4 *xin = (const u32x4 *)st.in;
  u32x4 *xs4 = (u32x4 *)xs;
  u32x4 v[KL];
#pragma unroll
  for (int kc = 0; kc < KL; kc++) v[kc] = ldc_16B(xin + kc * 64 + lane);
  if (st.flags & MK_F_NORM) {
    float ss = 0.f;
#pragma unroll
    for (int kc = 0; kc < KL; kc++) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t u = v[kc][e];
        ss += bf_lo(u) * bf_lo(u) + bf_hi(u) * bf_hi(u);
      }
    }
    ss = wave_sum(ss);
    const float r = rsqrtf(ss / (float)(KL * 512) + st.eps);
    u32x4 *no = (c.vid == 0) ? (u32x4 *)st.norm_out : nullptr;
#pragma unroll
    for (int kc = 0; kc < KL; kc++) {
      const u32x4 g = nwv[kc];  // norm weights were requested before the barrier was awaited
      u32x4 y;
#pragma unroll
      for (int e = 0; e < 4; e++) y[e] = pack2((bf_lo(v[kc][e]) * r) * bf_lo(g[e]), (bf_hi(v[kc][e]) * r) * bf_hi(g[e]));
      xs4[kc * 64 + lane] = y;
      if (no) stc_16B(no + kc * 64 + lane, y);
    }
  } else {
#pragma unroll
    for (int kc = 0; kc < KL; kc++) xs4[kc * 64 + lane] = v[kc];
  }
}

// Single-token linear: out[n] = bf16(sum_k W[n,k] * x[k] (+ res[n])), optionally with the RMSNorm of x
// fused in front and with the SwiGLU epilogue fused behind.  The weight matrix is streamed from HBM
// exactly once with 128-bit loads, one 1 KB row segment per wavefront instruction; x lives in LDS as
// packed bf16 and the products run on v_dot2_f32_bf16 with fp32 accumulation.
//
// Wavefront roles: wavefront 0 is the control wavefront -- it polls the grid barrier, then loads, normalises and
// publishes x, and only then joins the streaming -- while wavefronts 1..3 stream weight rows from the start.  A
// wavefront's vector loads return in order, so a wavefront that has weight loads in flight cannot observe the
// barrier before they land; keeping the poll on a wavefront without weight loads lets the weight prefetch and the
// barrier overlap.
// KL = K/512 row segments per lane.  Every worker keeps U outputs' rows in flight in registers; the first U are
// requested BEFORE the previous stage is known to be complete (weights do not depend on it), so the HBM pipe stays
// busy across the grid barrier, and a slot is refilled from the workgroup's ticket counter as soon as it is consumed.
// Reference tasks: linear_kernel_ck (tasks/mi300/linear_ck_mi300.cuh:289-619), gang_linear_silu_kernel
// (tasks/mi300/gang_linear_mi300.cuh:359-576).
template <int KL, int R, bool SILU, bool W0OK>
__device__ __forceinline__ void stage_linear_m1_t(CStage &st, Ctx &c, char *smem) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int K8 = KL * 64;
  constexpr int NROW = SILU ? 2 : 1;  // weight rows per output ([gate ; up] pair)
  constexpr int U = R / NROW;         // outputs in flight per worker wavefront
  uint32_t *xs = (uint32_t *)smem;
  const bool ctrl = wave == 0;
  const int n_out = SILU ? st.n / 2 : st.n;
  // The workgroup owns a contiguous range of outputs; its three worker wavefronts draw them one at a time from an LDS
  // ticket counter, so all three stream until the range is exhausted however the CU's memory pipeline favours them.
  const int oq = n_out / c.G, orem = n_out - oq * c.G;
  const int o_begin = c.vid * oq + min(c.vid, orem), o_end = o_begin + oq + (c.vid < orem ? 1 : 0);
  int *ticket = c.sh_ticket + (c.seq & 1);
  const int half = st.silu_half;
  auto take = [&]() -> int {  // next output index of this workgroup, or -1
    int t = 0;
    if (lane == 0) t = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    t = __builtin_amdgcn_readfirstlane(t) + o_begin;
    return t < o_end ? t : -1;
  };
  auto load_unit = [&](int o, u32x4 (&b)[NROW][KL]) {
    int vr = o;
    if (SILU) {
      const int g = o / half;
      vr = g * 2 * half + (o - g * half);
    }
#pragma unroll
    for (int h = 0; h < NROW; h++) {
      const u32x4 *p = weight_row(st.w, vr + h * half, K8) + lane;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) b[h][kc] = ldg_stream(p + kc * 64);
    }
  };
  u32x4 buf[U][NROW][KL];
  int uo[U];
  // LDS side of the prefetch: NL further outputs per worker wavefront whose rows are parked in the LDS window above
  // MK_MOE_OFFSET while the barrier is awaited (the registers alone hold about 3.5 us of streaming, the barrier and the
  // staging of the input row take longer).  They are reduced from LDS right after the barrier.
  constexpr int NLFIT = 32 / (KL * NROW);  // rows of KL KB that fit a wavefront's 32 KB share of the window
  constexpr int NL = NLFIT < MK_TUNE_NL ? NLFIT : MK_TUNE_NL;
  u32x4 *lrows = (u32x4 *)(smem + MK_MOE_OFFSET) + (size_t)(wave > 0 ? wave - 1 : 0) * (NL > 0 ? NL : 1) * NROW * K8;
  int lo_[NL > 0 ? NL : 1];
  if (!ctrl) {
    // weights do not depend on the previous stage: the first outputs' rows are requested before its barrier completes
    if (NL > 0) {
      // A rolling window of U outputs: output i goes to register slot i % U; from the U-th on, the slot's previous
      // output has landed by then and is parked in LDS first.  The first NL outputs end up parked, the last U stay in the
      // register slots, and never more than U outputs per wavefront are in flight -- a load the control wavefront issues
      // (the barrier poll, then the input row) queues behind whatever the CU has in flight, so it must not be the whole
      // prefetch.  Every load is unconditional (an exhausted ticket re-reads a valid row), so the waits count exactly.
#pragma unroll
      for (int i = 0; i < NL + U; i++) {
        const int sl = i % U;
        if (i >= U) {
#pragma unroll
          for (int h = 0; h < NROW; h++)
#pragma unroll
            for (int kc = 0; kc < KL; kc++) lrows[(((i - U) * NROW + h) * KL + kc) * 64 + lane] = buf[sl][h][kc];
          lo_[i - U] = uo[sl];
        }
        uo[sl] = take();
        load_unit(uo[sl] >= 0 ? uo[sl] : min(o_begin, n_out - 1), buf[sl]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < U; j++) {
        uo[j] = take();
        if (uo[j] >= 0) load_unit(uo[j], buf[j]);
      }
    }
  } else {
    u32x4 nwv[KL];
    if (st.flags & MK_F_NORM) {
#pragma unroll
      for (int kc = 0; kc < KL; kc++) nwv[kc] = ((const u32x4 *)st.norm_w)[kc * 64 + lane];
    }
    if (c.pending && tid == 0) barrier_poll(c);
    stage_x_m1_wave<KL>(st, c, xs, lane, nwv);
  }
  __syncthreads();
  barrier_done(c);
  // Outputs are collected in LDS and written out together once every worker is done: one write-through request per
  // 128-byte line instead of one 2-byte write per output.
  uint16_t *so = (uint16_t *)(smem + MK_OUT_OFFSET);
  // Rows of 8 KB and more: wavefront 0 alone writes the outputs out, so that the arrival needs no workgroup barrier and
  // the other wavefronts go straight on to the next stage's prefetch (barrier_arrive).  With shorter rows (stages of a
  // few microseconds) the earlier prefetch gains less than it costs wavefront 0's arrival and next poll, which then
  // queue behind it.
  // (only in the kernel instantiation for single-token graphs: W0OK)
  constexpr bool W0 = W0OK && KL >= MK_TUNE_W0_KL;
  auto flush = [&]() {
    if (W0 && tid == 0) c.sh_ticket[(c.seq + 1) & 1] = 0;  // the next stage's work counter (idle since the previous stage)
    __syncthreads();
    uint16_t *dst = (uint16_t *)st.out + o_begin;
    if (W0) {
      if (wave == 0) {
        for (int i = lane; i < o_end - o_begin; i += 64) stc_u16(dst + i, so[i]);
      }
    } else {
      for (int i = tid; i < o_end - o_begin; i += MK_THREADS) stc_u16(dst + i, so[i]);
    }
    c.wrote_through = true;
    c.arrive_w0 = W0;
  };
  if (ctrl) {  // the control wavefront has done its part: it now streams rows like the others
#pragma unroll
    for (int j = 0; j < U; j++) {
      uo[j] = take();
      if (uo[j] >= 0) load_unit(uo[j], buf[j]);
    }
  }
  const bool has_res = st.flags & MK_F_RES;
  const uint16_t *res = (const uint16_t *)st.res;
  float ures[U];
#pragma unroll
  for (int j = 0; j < U; j++) ures[j] = (has_res && uo[j] >= 0) ? bf2f(ldc_u16(res + uo[j])) : 0.f;
  // (the residual values of the parked outputs too: requested together here, not one round trip per parked output)
  float lres[NL > 0 ? NL : 1];
#pragma unroll
  for (int i = 0; i < (NL > 0 ? NL : 1); i++) lres[i] = (NL > 0 && has_res && !ctrl && lo_[i] >= 0) ? bf2f(ldc_u16(res + lo_[i])) : 0.f;
  const u32x4 *xs4 = (const u32x4 *)xs;
  u32x4 xr[KL <= 8 ? KL : 1];
  if (KL <= 8) {
#pragma unroll
    for (int kc = 0; kc < (KL <= 8 ? KL : 1); kc++) xr[kc] = xs4[kc * 64 + lane];
  }
  if (NL > 0 && !ctrl) {  // the parked rows first: no memory traffic, the register slots keep landing meanwhile
#pragma unroll
    for (int i = 0; i < NL; i++) {
      if (lo_[i] >= 0) {
        float a[NROW];
#pragma unroll
        for (int h = 0; h < NROW; h++) {
          a[h] = 0.f;
#pragma unroll
          for (int kc = 0; kc < KL; kc++) a[h] = dot8(lrows[((i * NROW + h) * KL + kc) * 64 + lane], KL <= 8 ? xr[KL <= 8 ? kc : 0] : xs4[kc * 64 + lane], a[h]);
        }
#pragma unroll
        for (int h = 0; h < NROW; h++) a[h] = wave_sum(a[h]);
        const float v = SILU ? silu_mul(a[0], a[NROW - 1]) : a[0] + lres[i];
        if (lane == 0) so[lo_[i] - o_begin] = (uint16_t)f2bf(v);
      }
    }
  }
  while (true) {
    bool any = false;
#pragma unroll
    for (int j = 0; j < U; j++) {
      if (uo[j] >= 0) {
        any = true;
        float a[NROW];
#pragma unroll
        for (int h = 0; h < NROW; h++) {
          a[h] = 0.f;
#pragma unroll
          for (int kc = 0; kc < KL; kc++) a[h] = dot8(buf[j][h][kc], KL <= 8 ? xr[KL <= 8 ? kc : 0] : xs4[kc * 64 + lane], a[h]);
        }
        const int o = uo[j];
        const float r = ures[j];
        uo[j] = take();
        if (uo[j] >= 0) {
          load_unit(uo[j], buf[j]);
          if (has_res) ures[j] = bf2f(ldc_u16(res + uo[j]));
        }
#pragma unroll
        for (int h = 0; h < NROW; h++) a[h] = wave_sum(a[h]);
        const float v = SILU ? silu_mul(a[0], a[NROW - 1]) : a[0] + r;
        if (lane == 0) so[o - o_begin] = (uint16_t)f2bf(v);
      }
    }
    if (!any) break;
  }
  flush();
}

// Generic single-token linear for reduction lengths that are not a multiple of 512 or have no tuned
// instantiation: same arithmetic, no cross-barrier prefetch.
__device__ __forceinline__ void stage_linear_m1_generic(CStage &st, Ctx &c, char *smem) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = st.k, k8 = K / 8;
  uint32_t *xs = (uint32_t *)smem;
  float *red = (float *)(smem + MK_RED_OFFSET);
  barrier_wait(c);
  stage_x_m1(st, c, xs, red);
  const bool silu = st.flags & MK_F_SILU;
  const int n_out = silu ? st.n / 2 : st.n;
  const int nwaves = c.G * MK_WAVES;
  const int rpw = (n_out + nwaves - 1) / nwaves;
  const int r0 = (c.vid * MK_WAVES + wave) * rpw;
  const int r1 = min(n_out, r0 + rpw);
  const u32x4 *xs4 = (const u32x4 *)xs;
  uint16_t *out = (uint16_t *)st.out;
  const uint16_t *res = (const uint16_t *)st.res;
  for (int r = r0; r < r1; r++) {
    float v;
    if (silu) {
      const int half = st.silu_half;
      const int vr = (r / half) * 2 * half + (r % half);
      const u32x4 *wg = weight_row(st.w, vr, k8);
      const u32x4 *wu = weight_row(st.w, vr + half, k8);
      float ag = 0.f, au = 0.f;
#pragma unroll 4
      for (int kc = lane; kc < k8; kc += 64) {
        const u32x4 x = xs4[kc];
        ag = dot8(ldg_stream(wg + kc), x, ag);
        au = dot8(ldg_stream(wu + kc), x, au);
      }
      v = silu_mul(wave_sum(ag), wave_sum(au));
    } else {
      const u32x4 *w0 = weight_row(st.w, r, k8);
      float a0 = 0.f;
#pragma unroll 4
      for (int kc = lane; kc < k8; kc += 64) a0 = dot8(ldg_stream(w0 + kc), xs4[kc], a0);
      v = wave_sum(a0);
      if (st.flags & MK_F_RES) v += bf2f(ldc_u16(res + r));
    }
    if (lane == 0) out[r] = (uint16_t)f2bf(v);
  }
}

template <bool W0OK>
__device__ __forceinline__ void stage_linear_m1(CStage &st, Ctx &c, char *smem) {
  const bool silu = st.flags & MK_F_SILU;
  // the tuned forms collect a workgroup's outputs in the LDS window [MK_OUT_OFFSET, MK_MOE_OFFSET)
  const bool fits = ((silu ? st.n / 2 : st.n) / c.G + 1) * 2 <= MK_MOE_OFFSET - MK_OUT_OFFSET;
  if (!fits) {
    stage_linear_m1_generic(st, c, smem);
  } else if (st.k == 4096) {
    if (silu) stage_linear_m1_t<8, MK_TUNE_R8, true, W0OK>(st, c, smem);
    else stage_linear_m1_t<8, MK_TUNE_R8N, false, W0OK>(st, c, smem);
  } else if (st.k == 12288 && !silu) {
    stage_linear_m1_t<24, MK_TUNE_R24, false, W0OK>(st, c, smem);
  } else if (st.k == 2048) {
    if (silu) stage_linear_m1_t<4, 4, true, W0OK>(st, c, smem);
    else stage_linear_m1_t<4, MK_TUNE_R4, false, W0OK>(st, c, smem);
  } else if (st.k == 1024 && !silu) {
    stage_linear_m1_t<2, 4, false, W0OK>(st, c, smem);
  } else {
    stage_linear_m1_generic(st, c, smem);
  }
}


// Few-token linear (2..MB tokens): the single-token structure with the token rows in LDS.  Every weight row is still
// read once and dotted against all token rows (v_dot2, fp32); up to 8 tokens this stays under the streaming time, so
// small batches cost little more than one token, where the matrix-core path (16-row tiles, one tile per workgroup
// on the narrow stages) is bound by latency.  A stage that carries MK_F_NORM normalises the rows itself while staging
// them (the standalone NORM stage in front is skipped for these batch sizes).  Outputs are collected in LDS
// [token][output] and written through.
template <int KL, int R, bool SILU, int MB>
__device__ __forceinline__ void stage_linear_small(CStage &st, Ctx &c, int M, char *smem) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int K8 = KL * 64;
  constexpr int NROW = SILU ? 2 : 1;
  constexpr int U = R / NROW;
  const bool ctrl = wave == 0;
  const int n_out = SILU ? st.n / 2 : st.n;
  const int oq = n_out / c.G, orem = n_out - oq * c.G;
  const int o_begin = c.vid * oq + min(c.vid, orem), o_end = o_begin + oq + (c.vid < orem ? 1 : 0);
  const int n_loc = o_end - o_begin;
  int *ticket = c.sh_ticket + (c.seq & 1);
  const int half = st.silu_half;
  // Plain rows are drawn and reduced two at a time: a token-row segment read from LDS is used for both weight rows
  // (half the LDS reads per output); a [gate ; up] pair already shares the segment.
  constexpr int Q = SILU ? 1 : 2;  // outputs per ticket
  static_assert(U == 2 * Q, "two groups of rows in flight");
  auto take = [&]() -> int {  // first output of the next group of this workgroup (may lie at or beyond o_end)
    int t = 0;
    if (lane == 0) t = __hip_atomic_fetch_add(ticket, Q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return __builtin_amdgcn_readfirstlane(t) + o_begin;
  };
  auto load_unit = [&](int o, u32x4 (&b)[NROW][KL]) {
    int vr = o;
    if (SILU) {
      const int g = o / half;
      vr = g * 2 * half + (o - g * half);
    }
#pragma unroll
    for (int h = 0; h < NROW; h++) {
      const u32x4 *p = weight_row(st.w, vr + h * half, K8) + lane;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) b[h][kc] = ldg_stream(p + kc * 64);
    }
  };
  // Every load is unconditional: a group at or beyond the end of the range re-reads the range's last row and its
  // results are dropped.  (A load under a branch would turn every wait for one group into a drain of the other too.)
  // The residual values of a group travel with its rows: lane (q * MB + m) loads the one of output q, token m (stages
  // without a residual read a valid dummy location instead, so that this load is unconditional too).
  const bool has_res = st.flags & MK_F_RES;
  const uint16_t *rbase = has_res ? (const uint16_t *)st.res + (size_t)min(lane & (MB - 1), M - 1) * st.ld_res : (const uint16_t *)st.in;
  auto load_group = [&](int o, u32x4 (&b)[Q][NROW][KL], uint16_t &r) {
#pragma unroll
    for (int q = 0; q < Q; q++) load_unit(max(min(o + q, o_end - 1), 0), b[q]);
    r = rbase[has_res ? max(min(o + ((lane / MB) & (Q - 1)), o_end - 1), 0) : 0];
  };
  u32x4 bufA[Q][NROW][KL], bufB[Q][NROW][KL];
  uint16_t rA = 0, rB = 0;
  int gA = 0, gB = 0;
  if (!ctrl) {
    gA = take();
    load_group(gA, bufA, rA);
    gB = take();
    load_group(gB, bufB, rB);
  } else {
    if (c.pending && tid == 0) barrier_poll(c);
    // the token rows come from other workgroups: one acquire, then ordinary loads that share them through the die's L2
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  __syncthreads();
  barrier_done(c);
  // all four wavefronts stage the token rows (the workers' requests queue behind their weight rows, which were issued
  // long before)
  const uint16_t *x = (const uint16_t *)st.in;
  const int ldx = st.ld_in;
  u32x4 *xs4 = (u32x4 *)(smem + MK_MOE_X_OFFSET);  // [token][K8]
  if (st.flags & MK_F_NORM) {
    // Fused RMSNorm (the standalone NORM stage in front is skipped for these batch sizes): every workgroup normalises
    // all rows itself, a wavefront per row, exactly as the single-token form does; virtual workgroup 0 also stores the
    // normalised rows, which are the norm task's output tensor.
    const u32x4 *nw4 = (const u32x4 *)st.norm_w;
    for (int m = wave; m < M; m += MK_WAVES) {
      const u32x4 *xr = (const u32x4 *)(x + (size_t)m * ldx);
      u32x4 v[KL];
#pragma unroll
      for (int kc = 0; kc < KL; kc++) v[kc] = xr[kc * 64 + lane];
      float ss = 0.f;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const uint32_t u = v[kc][e];
          ss += bf_lo(u) * bf_lo(u) + bf_hi(u) * bf_hi(u);
        }
      }
      ss = wave_sum(ss);
      const float r = rsqrtf(ss / (float)(KL * 512) + st.eps);
      u32x4 *no = (c.vid == 0) ? (u32x4 *)((uint16_t *)st.norm_out + (size_t)m * st.ld_norm) : nullptr;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) {
        const u32x4 g = nw4[kc * 64 + lane];
        u32x4 y;
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = pack2((bf_lo(v[kc][e]) * r) * bf_lo(g[e]), (bf_hi(v[kc][e]) * r) * bf_hi(g[e]));
        xs4[m * K8 + kc * 64 + lane] = y;
        if (no) stc_16B(no + kc * 64 + lane, y);
      }
    }
  } else {
    constexpr int NCH = MB * KL / MK_WAVES;  // 16-byte segments per lane
    u32x4 xv[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      const int ci = (i * MK_WAVES + wave) * 64 + lane, m = ci / K8, o = ci - m * K8;
      if (m < M) xv[i] = ((const u32x4 *)(x + (size_t)m * ldx))[o];
    }
#pragma unroll
    for (int i = 0; i < NCH; i++) {
      const int ci = (i * MK_WAVES + wave) * 64 + lane;
      if (ci / K8 < M) xs4[ci] = xv[i];
    }
  }
  __syncthreads();
  if (ctrl) {
    gA = take();
    load_group(gA, bufA, rA);
    gB = take();
    load_group(gB, bufB, rB);
  }
  uint16_t *so = (uint16_t *)smem;  // [token][output - o_begin]
  auto reduce_group = [&](const u32x4 (&b)[Q][NROW][KL], uint16_t r, int o) {
    const float rf = has_res ? bf2f(r) : 0.f;
    // the LDS addresses of the token rows are rebuilt from the lane index in every call: hoisted out of the loop they
    // would be long-lived registers that get spilled, and a spill reload in this loop is a vector-memory wait
    int lo = lane;
    asm volatile("" : "+v"(lo));
    float a[Q][NROW][MB];
    // the segments of token m + 1 are read from LDS while token m is reduced (rows beyond M re-read row M - 1)
    u32x4 xk[2][KL];
#pragma unroll
    for (int kc = 0; kc < KL; kc++) xk[0][kc] = xs4[kc * 64 + lo];
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
      for (int q = 0; q < Q; q++)
#pragma unroll
        for (int h = 0; h < NROW; h++) a[q][h][m] = 0.f;
      if (m + 1 < MB) {
        const int mn = min(m + 1, M - 1);
#pragma unroll
        for (int kc = 0; kc < KL; kc++) xk[(m + 1) & 1][kc] = xs4[mn * K8 + kc * 64 + lo];
      }
      __builtin_amdgcn_sched_barrier(0);
      if (m < M) {
#pragma unroll
        for (int kc = 0; kc < KL; kc++) {
#pragma unroll
          for (int q = 0; q < Q; q++)
#pragma unroll
            for (int h = 0; h < NROW; h++) a[q][h][m] = dot8(b[q][h][kc], xk[m & 1][kc], a[q][h][m]);
        }
      }
    }
    // all Q * NROW * MB sums are reduced together; lane q * MB + m (plain) / h * MB + m ([gate ; up]) gets the total
    constexpr int NV = Q * NROW * MB;
    float vv[NV];
#pragma unroll
    for (int q = 0; q < Q; q++)
#pragma unroll
      for (int h = 0; h < NROW; h++)
#pragma unroll
        for (int m = 0; m < MB; m++) vv[(q * NROW + h) * MB + m] = a[q][h][m];
    const float tot = transpose_sum<NV>(vv, lane);
    const int m = lane & (MB - 1), q = SILU ? 0 : lane / MB;
    float v;
    if (SILU) v = silu_mul(tot, dpp_f32<0x100 + MB>(tot));  // row_shl:MB: the up sum sits MB lanes above the gate sum
    else v = tot + rf;
    if (lane < Q * MB && m < M && o + q < o_end) so[m * n_loc + (o + q - o_begin)] = (uint16_t)f2bf(v);
  };
  // two groups in flight: while one is reduced the other one's rows are landing; tickets only grow, so the first
  // group found beyond the range ends the loop
  while (gA < o_end) {
    reduce_group(bufA, rA, gA);
    gA = take();
    load_group(gA, bufA, rA);
    if (gB >= o_end) break;
    reduce_group(bufB, rB, gB);
    gB = take();
    load_group(gB, bufB, rB);
  }
  __syncthreads();
  uint16_t *dst = (uint16_t *)st.out + o_begin;
  for (int i = tid; i < M * n_loc; i += MK_THREADS) {
    const int m = i / n_loc, r = i - m * n_loc;
    stc_u16(dst + (size_t)m * st.ld_out + r, so[i]);
  }
  c.wrote_through = true;
}

// Whether the few-token form can run this stage: reduction length with a tuned instantiation, token rows within the
// LDS window above MK_MOE_X_OFFSET, collected outputs within the window below MK_MOE_OFFSET.
#ifndef MK_TUNE_SMALL_MAX
#define MK_TUNE_SMALL_MAX 2
#endif
__device__ __forceinline__ bool linear_small_ok(CStage &st, const Ctx &c, int M) {
  if (M > MK_TUNE_SMALL_MAX || (st.k != 4096 && st.k != 2048)) return false;
  const int n_out = (st.flags & MK_F_SILU) ? st.n / 2 : st.n;
  return (size_t)M * st.k * 2 <= (size_t)(MK_LDS_BYTES - MK_MOE_X_OFFSET) && (size_t)M * (n_out / c.G + 1) * 2 <= (size_t)MK_MOE_OFFSET;
}

template <int MB>
__device__ __forceinline__ void stage_linear_small_dispatch(CStage &st, Ctx &c, int M, char *smem) {
  const bool silu = st.flags & MK_F_SILU;
  if (st.k == 4096) {
    if (silu) stage_linear_small<8, 4, true, MB>(st, c, M, smem);
    else stage_linear_small<8, 4, false, MB>(st, c, M, smem);
  } else {
    if (silu) stage_linear_small<4, 4, true, MB>(st, c, M, smem);
    else stage_linear_small<4, 4, false, MB>(st, c, M, smem);
  }
}

// Matrix-core linear for several tokens.  A workgroup owns a range of 16-row weight tiles and one K slice (S slices
// per range when a stage has too few tiles to fill the machine, S = 1 otherwise).  The range is worked off in sweeps:
// every wavefront holds TW tiles of the sweep over the whole slice, and all four share the token rows of the slice,
// which one pass stages per 64-wide step in LDS (double-buffered, in matrix-core operand order, so the reads are linear
// in the lane index).  Token-row traffic per weight byte is M / (64 TW); weight steps sit NB deep in registers.
//
// Every load is unconditional and the step loop has a fixed trip structure (slices are multiples of NB steps; slots
// past the range re-read its last tile): a load under a branch makes the compiler's wait counts drain everything
// younger, which costs the whole prefetch depth.  Loads return in issue order, so token rows are prefetched exactly as
// deep as the weights.
//
// With S > 1 the partial tiles go through a write-through buffer; the last workgroup of a group to arrive sums them in
// slice order (deterministic), applies SwiGLU / residual and stores bf16.  SwiGLU stages number their weight tiles
// gate, up, gate, up ... so that a pair always sits in one wavefront.
// Reference tasks: linear / linear_with_residual / splitk_linear (tasks/mi300/linear_ck_mi300.cuh), silu_mul_linear.
#ifndef MK_TUNE_SPLITK_MAXS
#define MK_TUNE_SPLITK_MAXS 8
#endif
#ifndef MK_TUNE_TPU
#define MK_TUNE_TPU 4  // tiles per workgroup a split stage aims for
#endif
#ifndef MK_TUNE_NB1
#define MK_TUNE_NB1 8
#endif
#ifndef MK_TUNE_NB2
#define MK_TUNE_NB2 4
#endif
#ifndef MK_TUNE_NB4
#define MK_TUNE_NB4 2
#endif
#ifndef MK_TUNE_TILES_MIN_TPW
#define MK_TUNE_TILES_MIN_TPW 16
#endif
#define MK_TILES_NB 4  // a K slice is a multiple of 64 * 2 * MK_TILES_NB (the deepest instantiation's ring)

struct TilePlan {
  int S;       // K slices per tile range (0: this form cannot run the stage)
  int groups;  // tile ranges
  int wt;      // weight tiles of the stage
};
__device__ __forceinline__ TilePlan linear_tiles_plan(CStage &st, const Ctx &c) {
  TilePlan p;
  const bool silu = st.flags & MK_F_SILU;
  const int n_out = silu ? st.n / 2 : st.n;
  const int unit = silu ? 2 : 1;                      // ranges are made of whole gate/up pairs
  p.wt = ((n_out + 15) / 16) * unit;
  p.S = 0;
  p.groups = 0;
  if (st.k % (64 * 2 * MK_TILES_NB) != 0) return p;
  const int tpw = (p.wt + c.G - 1) / c.G;            // tiles per workgroup without a K split
  int S = 1;
  while (S < MK_TUNE_SPLITK_MAXS && tpw * S < MK_TUNE_TPU && 2 * S <= c.G && st.k % (S * 2 * 64 * 2 * MK_TILES_NB) == 0) S *= 2;
  const int gs = c.G / S;                             // ranges the grid can hold: S adjacent workgroups each
  int tpu = (p.wt + gs - 1) / gs;                     // tiles per range
  tpu = (tpu + unit - 1) / unit * unit;
  if (S > 1 && tpu > 16) return p;                    // a split range is a single sweep
  if (S == 1 && tpw < MK_TUNE_TILES_MIN_TPW) return p;  // a few tiles per workgroup without a K split: the form that splits K inside the workgroup
  p.groups = (p.wt + tpu - 1) / tpu;
  p.S = S;
  return p;
}

template <int MT>
__device__ __forceinline__ void stage_linear_mfma_tiles(CStage &st, Ctx &c, const MkRuntime &rt, int M, const TilePlan plan, char *smem) {
  barrier_wait(c);
  c.wrote_through = true;  // partial tiles and outputs are all written through: no L2 write-back at this stage's arrival
  if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  __syncthreads();
  MK_MARK(c, 0);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const bool silu = st.flags & MK_F_SILU;
  const int K = st.k, k8 = K / 8;
  const int n_out = silu ? st.n / 2 : st.n;
  const int half = st.silu_half;
  const int S = plan.S, unit = silu ? 2 : 1;
  const int g = c.vid / S, sl = c.vid - g * S;
  if (g >= plan.groups) return;  // workgroups beyond the last range have nothing to do in this stage
  // balanced ranges of whole units
  const int nun = plan.wt / unit;
  const int tb = (int)(((long long)g * nun) / plan.groups) * unit, te = (int)(((long long)(g + 1) * nun) / plan.groups) * unit;
  const int kslice = K / S, kbeg = sl * kslice, nsteps = kslice >> 6;
  const uint16_t *x = (st.flags & MK_F_NORM) ? (const uint16_t *)st.norm_out : (const uint16_t *)st.in;
  const int ldx = (st.flags & MK_F_NORM) ? st.ld_norm : st.ld_in;
  u32x4 *xl = (u32x4 *)smem;  // two buffers of [MT][2][64] 16-byte operands
  int *sflag = (int *)(smem + 2 * MT * 2048);
  // token rows: wavefront w stages token tile w, every lane the same 32 contiguous bytes it would feed the matrix core
  // with, stored at its own lane slot of the operand block (consecutive 16-byte slots: no bank conflicts either way)
  const uint16_t *xsrc = x + (size_t)min(min(wave, MT - 1) * 16 + lr, M - 1) * ldx + kbeg + lg * 16;
  const int xdst = min(wave, MT - 1) * 128 + lane;
  // first weight row of weight tile ti for this lane
  auto tile_row = [&](int ti) -> const uint16_t * {
    int o, vr;
    if (silu) {
      o = min((ti >> 1) * 16 + lr, n_out - 1);
      const int gi = o / half;
      vr = gi * 2 * half + (o - gi * half) + ((ti & 1) ? half : 0);
    } else {
      o = min(ti * 16 + lr, n_out - 1);
      vr = o;
    }
    return (const uint16_t *)weight_row(st.w, vr, k8) + kbeg + lg * 16;
  };
  u32x4 *part = (u32x4 *)rt.splitk_part;

  auto sweep = [&](int t0, auto twc) {
    constexpr int TW = decltype(twc)::value;
    constexpr int NB = TW == 1 ? MK_TUNE_NB1 : (TW == 2 ? MK_TUNE_NB2 : MK_TUNE_NB4);
    const int tw0 = t0 + wave * TW;           // this wavefront's first tile
    const bool has_tile = tw0 < te;           // wavefronts without one only stage token rows and keep the barriers
    const uint16_t *wrow[TW];
#pragma unroll
    for (int t = 0; t < TW; t++) wrow[t] = tile_row(min(tw0 + t, te - 1));
    bf16x8 a[NB][TW][2];
    u32x4 xq[NB][2];
    auto w_load = [&](int step, bf16x8 (&aa)[TW][2]) {
#pragma unroll
      for (int t = 0; t < TW; t++) {
        aa[t][0] = __builtin_nontemporal_load((const bf16x8 *)(wrow[t] + (step << 6)));
        aa[t][1] = __builtin_nontemporal_load((const bf16x8 *)(wrow[t] + (step << 6) + 8));
      }
    };
    auto x_load = [&](int step, u32x4 (&q)[2]) {
      q[0] = *(const u32x4 *)(xsrc + (step << 6));
      q[1] = *(const u32x4 *)(xsrc + (step << 6) + 8);
    };
    auto x_store = [&](int buf, const u32x4 (&q)[2]) {
      if (wave < MT) {
        xl[buf * MT * 128 + xdst] = q[0];
        xl[buf * MT * 128 + xdst + 64] = q[1];
      }
    };
    f32x4 acc[TW][MT];
#pragma unroll
    for (int t = 0; t < TW; t++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) acc[t][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // Copies of the step loop for wavefronts with / without tiles and with / without a token tile to stage: a branch
    // around loads inside one copy would spoil its wait counts.  All copies execute the same barriers.
    auto pipeline = [&](auto htc, auto xlc) {
      constexpr bool HT = decltype(htc)::value;
      constexpr bool XL = decltype(xlc)::value;  // this wavefront stages a token tile (wavefront index < MT)
      __syncthreads();  // the previous sweep has finished with the LDS buffers
#pragma unroll
      for (int j = 0; j < NB; j++) {
        if (HT) w_load(j, a[j]);
        if (XL) x_load(j, xq[j]);
      }
      if (XL) x_store(0, xq[0]);
      __syncthreads();
      auto block = [&](int s0, auto refill) {
        constexpr bool REFILL = decltype(refill)::value;
#pragma unroll
        for (int j = 0; j < NB; j++) {
          const int step = s0 + j;
          if (XL && (REFILL || j + 1 < NB)) x_store((step + 1) & 1, xq[(j + 1) % NB]);  // that buffer was last read before the previous barrier
          if (HT) {
            const u32x4 *xb = xl + (step & 1) * MT * 128;
            u32x4 b[2][MT];
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
              for (int mt = 0; mt < MT; mt++) b[h][mt] = xb[(mt * 2 + h) * 64 + lane];
            __builtin_amdgcn_sched_barrier(0);  // all operand reads in flight before the first matrix instruction waits
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
              for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int t = 0; t < TW; t++)
                  acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j][t][h], __builtin_bit_cast(bf16x8, b[h][mt]), acc[t][mt], 0, 0, 0);
          }
          if (REFILL) {
            if (HT) w_load(step + NB, a[j]);
            if (XL) x_load(step + NB, xq[j]);
          }
          __syncthreads();
        }
      };
      int s0 = 0;
      for (; s0 + NB < nsteps; s0 += NB) block(s0, std::true_type{});
      block(s0, std::false_type{});
    };
    const bool stages_x = wave < MT;
    if (MT == MK_WAVES || stages_x) {
      if (has_tile) pipeline(std::true_type{}, std::true_type{});
      else pipeline(std::false_type{}, std::true_type{});
    } else {
      if (has_tile) pipeline(std::true_type{}, std::false_type{});
      else pipeline(std::false_type{}, std::false_type{});
    }

    MK_MARK(c, 1);
    // ---- combine the S slices (a split range is a single sweep, so slots are indexed by wavefront and tile only)
    if (S > 1) {
      if (has_tile) {
#pragma unroll
        for (int t = 0; t < TW; t++)
#pragma unroll
          for (int mt = 0; mt < MT; mt++)
            stc_16B(part + ((((size_t)c.vid * 4 + wave) * 4 + t) * 4 + mt) * 64 + lane, __builtin_bit_cast(u32x4, acc[t][mt]));
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0) {
        unsigned *cnt = rt.splitk_cnt + (size_t)g * 32;
        const int last = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(S - 1);
        if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *sflag = last;
      }
      __syncthreads();
      MK_MARK(c, 2);
      if (!*sflag || !has_tile) return;
#pragma unroll
      for (int t = 0; t < TW; t++) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[t][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
        for (int q0 = 0; q0 < S; q0 += 4) {  // four slices requested at once; summed in slice order
          u32x4 pv[4][MT];
#pragma unroll
          for (int q = 0; q < 4; q++)
            if (q0 + q < S) {
#pragma unroll
              for (int mt = 0; mt < MT; mt++) pv[q][mt] = ldc_16B(part + ((((size_t)(g * S + q0 + q) * 4 + wave) * 4 + t) * 4 + mt) * 64 + lane);
            }
#pragma unroll
          for (int q = 0; q < 4; q++)
            if (q0 + q < S) {
#pragma unroll
              for (int mt = 0; mt < MT; mt++) acc[t][mt] += __builtin_bit_cast(f32x4, pv[q][mt]);
            }
        }
      }
    }
    MK_MARK(c, 3);
    if (!has_tile) return;
    // ---- epilogue: lane l holds token m = mt * 16 + (l & 15), output columns tile * 16 + (l >> 4) * 4 .. + 3
    constexpr int OT = TW >= 2 ? TW / 2 : 1;
#pragma unroll
    for (int u = 0; u < (TW >= 2 ? TW : 1); u++) {
      if (silu && u >= OT) break;
      const int ti = silu ? tw0 + 2 * u : tw0 + u;
      if (ti >= te) break;
      const int otile = silu ? (ti >> 1) : ti;
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int m = mt * 16 + lr;
        if (m < M) {
          uint16_t *orow = (uint16_t *)st.out + (size_t)m * st.ld_out;
          const uint16_t *rrow = (const uint16_t *)st.res + (size_t)m * st.ld_res;
          float rr[4];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int n = otile * 16 + lg * 4 + i;
            float r;
            if (silu) r = TW >= 2 ? silu_mul(acc[(2 * u) % TW][mt][i], acc[(2 * u + 1) % TW][mt][i]) : 0.f;
            else r = acc[u][mt][i];
            if ((st.flags & MK_F_RES) && n < n_out) r += bf2f(rrow[n]);
            rr[i] = r;
          }
          stc_bf16x4(orow, otile * 16 + lg * 4, n_out, rr);
        }
      }
    }
  };

  for (int t0 = tb; t0 < te;) {
    const int r = te - t0;
    if (r > 8) {
      sweep(t0, std::integral_constant<int, 4>{});
      t0 += 16;
    } else if (r > 4 || silu) {
      sweep(t0, std::integral_constant<int, 2>{});
      t0 += 8;
    } else {
      sweep(t0, std::integral_constant<int, 1>{});
      t0 += 4;
    }
  }
}

// Matrix-core linear with the token rows staged through LDS by wavefronts of their own.  A workgroup owns a range of 4..6
// weight tiles and one K slice, which it works off in passes of 8 steps (512 k).  Wavefronts 0 and 1 hold two or three
// tiles each and do nothing but stream weights (a ring of NB = 8 steps, 32 or 48 KB per wavefront, which runs on across
// the passes without ever draining) and feed the matrix cores from LDS; wavefronts 2 and 3 stage the token rows of the
// NEXT pass -- all rows, 64 KB for 64 tokens, in matrix-core operand order, with loads that write LDS directly (no
// registers) -- into the other half of a double buffer.  Loads return in issue order per wavefront, and a token-row
// load queues behind the weight stream in the memory system like any other request, so in a wavefront that also
// streams weights every batch of row loads stalls the weight ring for a full memory latency; on wavefronts of their
// own they cost the streaming wavefronts nothing.  (One staging wavefront is not enough: with at most 63 requests
// outstanding it needs two memory latencies for the 128 requests of a pass, and the pass cannot be shorter than that.)
// One workgroup barrier per pass hands a buffer over.  The first NB weight steps are requested before the previous
// stage's barrier is awaited; the rows of the first pass are staged by all four wavefronts.  The S workgroups that
// share a tile range exchange their partial tiles as the streaming form does (write-through buffer, last arriver sums
// in slice order), or leave the sum to a norm stage that follows.  Used for the QKV, o, gate/up and down projections at
// 9..64 tokens.  SwiGLU stages number their weight tiles gate, up, gate, up ...; with three tiles per wavefront the
// middle pair straddles the two streaming wavefronts and is joined through LDS in the epilogue.
#define MK_XRES_STEPS 8  // steps per pass
#ifndef MK_TUNE_XRES_PRE
#define MK_TUNE_XRES_PRE 6  // ring steps requested before the previous stage's barrier is awaited
#endif
struct XresPlan {
  int S;       // K slices per tile range (0: this form cannot run the stage)
  int groups;  // tile ranges
  int wt;      // weight tiles of the stage
  int tpu;     // most tiles a range holds (decides tiles per wavefront and prefetch depth for every workgroup alike)
};
__device__ __forceinline__ XresPlan linear_xres_plan(CStage &st, const Ctx &c) {
  XresPlan p;
  p.S = 0;
  p.groups = 0;
  p.tpu = 0;
  const bool silu = st.flags & MK_F_SILU;
  const int n_out = silu ? st.n / 2 : st.n, unit = silu ? 2 : 1;
  p.wt = ((n_out + 15) / 16) * unit;
  for (int S = 1; S <= 8; S *= 2) {
    if (c.G % S || st.k % (S * 64 * MK_XRES_STEPS)) break;
    const int gs = c.G / S;
    int tpu = (p.wt + gs - 1) / gs;  // tiles per range
    tpu = (tpu + unit - 1) / unit * unit;
    if (tpu > 6) break;              // two streaming wavefronts with three tiles each
    if (tpu < 4) continue;           // too few tiles to occupy them: split K further
    p.S = S;
    p.tpu = tpu;
    p.groups = (p.wt / unit + tpu / unit - 1) / (tpu / unit);
    return p;
  }
  return p;
}

template <int MT, int TW>
__device__ __forceinline__ void stage_linear_mfma_xres(CStage &st, Ctx &c, const MkRuntime &rt, int M, const XresPlan plan, char *smem) {
  c.wrote_through = true;  // partial tiles and outputs are all written through: no L2 write-back at this stage's arrival
  constexpr int NSP = MK_XRES_STEPS;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const bool silu = st.flags & MK_F_SILU;
  const int K = st.k, k8 = K / 8;
  const int n_out = silu ? st.n / 2 : st.n, unit = silu ? 2 : 1;
  const int half = st.silu_half;
  const int S = plan.S;
  const int g = c.vid / S, sl = c.vid - g * S;
  const bool active = g < plan.groups;  // workgroups beyond the last range only keep the barriers
  const int nun = plan.wt / unit;       // balanced ranges of whole units
  const int tb = active ? (int)(((long long)g * nun) / plan.groups) * unit : 0, te = active ? (int)(((long long)(g + 1) * nun) / plan.groups) * unit : 0;
  const int kslice = K / S, kbeg = sl * kslice, nsteps = kslice >> 6, npass = nsteps / NSP;
  const uint16_t *x = (st.flags & MK_F_NORM) ? (const uint16_t *)st.norm_out : (const uint16_t *)st.in;
  const int ldx = (st.flags & MK_F_NORM) ? st.ld_norm : st.ld_in;
  u32x4 *xl = (u32x4 *)smem;  // two buffers of [step of the pass][token tile][2][64 lanes] 16-byte operands
  constexpr int XBUF = NSP * MT * 128;  // 16-byte operands per buffer
  int *sflag = (int *)(smem + 2 * XBUF * 16);
  u32x4 *part = (u32x4 *)rt.splitk_part;
  // hand the K-slice sum to the norm stage that follows, if there is one and the rows fit the partial buffer
  const bool defer = (st.flags & MK_F_DEFER_SUM) && S > 1 && (size_t)S * (MT * 16) * st.n * 4 <= (size_t)c.G * 65536;
  if (defer) {
    c.defer_S = S;
    c.defer_rows = MT * 16;
    c.defer_n = st.n;
    c.defer_part = (const float *)rt.splitk_part;
    c.defer_res = (st.flags & MK_F_RES) ? st.res : nullptr;
    c.defer_ld_res = st.ld_res;
  }
  // this lane's first operand of weight tile ti, and the distance (in 16-byte operands) between steps and between the two
  // halves of a step: the re-laid copy streams contiguously, the row-major original reads 64 bytes of each of 16 rows
  const bool packed = st.wpack != nullptr;
  const int step_stride = packed ? 128 : 8, half_stride = packed ? 64 : 4;
  auto tile_base = [&](int ti) -> const u32x4 * {
    if (packed) return (const u32x4 *)st.wpack + ((size_t)ti * (K >> 6) + (kbeg >> 6)) * 128 + lane;
    int o, vr;
    if (silu) {
      o = min((ti >> 1) * 16 + lr, n_out - 1);
      const int gi = o / half;
      vr = gi * 2 * half + (o - gi * half) + ((ti & 1) ? half : 0);
    } else {
      o = min(ti * 16 + lr, n_out - 1);
      vr = o;
    }
    return weight_row(st.w, vr, k8) + (kbeg >> 3) + lg;
  };
  // stage the token rows of one pass: item i = (step, token tile), two 1 KB requests each, straight into LDS (lane l's 16
  // bytes land at l * 16 behind the request's LDS base, which is the operand order).  `nw` wavefronts share the items:
  // wavefront `w` of them takes items w, w + nw, ...
  auto stage_pass = [&](int pass, int w, int nw) {
    const uint16_t *base = x + kbeg + pass * (NSP * 64) + lg * 8;
    u32x4 *buf = xl + (pass & 1) * XBUF;
    for (int i = w; i < MT * NSP; i += nw) {
      const int step = i / MT, mt = i - step * MT;
      const uint16_t *src = base + (size_t)min(mt * 16 + lr, M - 1) * ldx + (step << 6);
      __attribute__((address_space(3))) char *dst = (__attribute__((address_space(3))) char *)(buf + (size_t)i * 128);
      __builtin_amdgcn_global_load_lds((const MK_GLOBAL void *)(unsigned long long)src, (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
      __builtin_amdgcn_global_load_lds((const MK_GLOBAL void *)(unsigned long long)(src + 32), (__attribute__((address_space(3))) void *)(dst + 1024), 16, 0, 0);
    }
  };

  {
    constexpr int NB = 8, NSW = 2;    // ring depth in steps; streaming wavefronts
    const bool loader = wave >= NSW;  // stages token rows, holds no tiles
    const int tw0 = tb + wave * TW;   // a streaming wavefront's first tile
    const bool has_tile = active && !loader && tw0 < te;
    const u32x4 *wrow[TW];
#pragma unroll
    for (int t = 0; t < TW; t++) wrow[t] = tile_base(max(min(tw0 + t, te - 1), 0));
    bf16x8 a[NB][TW][2];
    auto w_load = [&](int step, bf16x8 (&aa)[TW][2]) {
#pragma unroll
      for (int t = 0; t < TW; t++) {
        aa[t][0] = __builtin_nontemporal_load((const bf16x8 *)(wrow[t] + step * step_stride));
        aa[t][1] = __builtin_nontemporal_load((const bf16x8 *)(wrow[t] + step * step_stride + half_stride));
      }
    };
    // weights do not depend on the previous stage: the first NBP steps are requested before its barrier is awaited, the
    // rest of the ring right after the first pass's token rows (what a CU has in flight sits in front of the barrier
    // poll and of the row requests)
    constexpr int NBP = MK_TUNE_XRES_PRE < NB ? MK_TUNE_XRES_PRE : NB;
    if (has_tile) {
#pragma unroll
      for (int j = 0; j < NBP; j++) w_load(j, a[j]);
    }
    // Token rows come from other workgroups and are read with cached loads, so what this die's caches hold of them must
    // go first.  The invalidate is issued BEFORE the barrier is awaited: nothing on this die reads the stage's input
    // buffers between the stage that last consumed them (barriers ago) and this barrier, so no stale line can come
    // back in between, and the invalidate's latency is off the path from the last arrival to the first row request.
    // The poll runs on the first row-staging wavefront, which has no weight loads in flight: loads return in order, so
    // on a streaming wavefront the poll's answer would wait behind the NB steps just requested -- two to four
    // microseconds for exactly the workgroups that enter last (those that did the norm stage's rows, or everybody after
    // an attention stage), which are the ones the stage then waits for.
    constexpr int POLL_TID = NSW * 64;
    if (tid == POLL_TID) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (c.pending && tid == POLL_TID) barrier_poll(c);
    __syncthreads();
    barrier_done(c);
    MK_MARK(c, 0);
    f32x4 acc[TW][MT];
#pragma unroll
    for (int t = 0; t < TW; t++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) acc[t][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const u32x4 *xb, const bf16x8 (&aa)[TW][2]) {
      u32x4 b[2][MT];
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) b[h][mt] = xb[(mt * 2 + h) * 64 + lane];
      __builtin_amdgcn_sched_barrier(0);  // all operand reads in flight before the first matrix instruction waits
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int t = 0; t < TW; t++) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aa[t][h], __builtin_bit_cast(bf16x8, b[h][mt]), acc[t][mt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    };
    // Passes [0, n_refill) refill the ring as they go, the last one only consumes it.  Every pass starts with a workgroup
    // barrier: its rows have landed (whoever requested them has waited for them) and everybody is done with the other
    // buffer, into which the loader then requests the next pass's rows.
    const int n_refill = npass - 1;
    auto do_pass = [&](int pass, auto refill_c) {
      constexpr bool REFILL = decltype(refill_c)::value;
      if (pass == 0 && has_tile && NBP < NB) {
        // the token rows of pass 0 have landed once nothing but the ring steps requested after them is outstanding
        static_assert((NB - NBP) * TW * 2 <= 63, "vmcnt range");
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NB - NBP) * TW * 2) : "memory");
      } else if (pass == 0 || loader) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
      if (pass == 0) MK_MARK(c, 1);
      if (loader && active && pass + 1 < npass) stage_pass(pass + 1, wave - NSW, MK_WAVES - NSW);
      __builtin_amdgcn_sched_barrier(0);
      if (has_tile) {
        const u32x4 *xb = xl + (pass & 1) * XBUF;
#pragma unroll
        for (int j = 0; j < NSP; j++) {
          compute(xb + j * MT * 128, a[j]);
          if (REFILL) w_load(pass * NSP + j + NB, a[j]);
        }
      }
    };
    if (active) stage_pass(0, wave, MK_WAVES);
    __builtin_amdgcn_sched_barrier(0);
    if (has_tile) {
#pragma unroll
      for (int j = NBP; j < NB; j++) w_load(j, a[j]);
    }
    __builtin_amdgcn_sched_barrier(0);
    int pass = 0;
    for (; pass < n_refill; pass++) do_pass(pass, std::true_type{});
    MK_MARK(c, 2);
    do_pass(pass, std::false_type{});
    MK_MARK(c, 3);
    if (defer) {
      // the consumer sums the slices: leave them as [slice][token][n] fp32 rows
      if (has_tile) {
        float *prow = (float *)rt.splitk_part + (size_t)sl * (MT * 16) * st.n;
#pragma unroll
        for (int t = 0; t < TW; t++)
          if (tw0 + t < te) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
              stc_16B((u32x4 *)(prow + (size_t)(mt * 16 + lr) * st.n + (tw0 + t) * 16 + lg * 4), __builtin_bit_cast(u32x4, acc[t][mt]));
          }
      }
      return;
    }
    // ---- combine the S slices: partial tiles through the write-through buffer, summed by the last workgroup to arrive
    if (S > 1) {
      if (has_tile) {
#pragma unroll
        for (int t = 0; t < TW; t++)
#pragma unroll
          for (int mt = 0; mt < MT; mt++)
            stc_16B(part + ((((size_t)c.vid * 4 + wave) * 4 + t) * 4 + mt) * 64 + lane, __builtin_bit_cast(u32x4, acc[t][mt]));
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0) {
        int last = 0;
        if (active) {
          unsigned *cnt = rt.splitk_cnt + (size_t)g * 32;
          last = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(S - 1);
          if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        *sflag = last;
      }
      __syncthreads();
      if (!*sflag) return;  // (the whole workgroup)
#pragma unroll
      for (int t = 0; t < TW; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[t][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
      for (int q0 = 0; has_tile && q0 < S; q0 += 4) {  // four slices of both tiles requested at once; summed in slice order
        u32x4 pv[4][TW][MT];
#pragma unroll
        for (int q = 0; q < 4; q++)
          if (q0 + q < S) {
#pragma unroll
            for (int t = 0; t < TW; t++)
#pragma unroll
              for (int mt = 0; mt < MT; mt++) pv[q][t][mt] = ldc_16B(part + ((((size_t)(g * S + q0 + q) * 4 + wave) * 4 + t) * 4 + mt) * 64 + lane);
          }
#pragma unroll
        for (int q = 0; q < 4; q++)
          if (q0 + q < S) {
#pragma unroll
            for (int t = 0; t < TW; t++)
#pragma unroll
              for (int mt = 0; mt < MT; mt++) acc[t][mt] += __builtin_bit_cast(f32x4, pv[q][t][mt]);
          }
      }
    }
    // ---- epilogue: lane l holds token m = mt * 16 + (l & 15), output columns tile * 16 + (l >> 4) * 4 .. + 3
    if (silu && (TW & 1)) {
      // an odd tile count per wavefront leaves the middle gate/up pair split: wavefront 1 hands its first tile (an up
      // tile) to wavefront 0, which holds the gate tile, through LDS
      __syncthreads();  // everybody is done with the row buffers
      if (wave == 1 && has_tile) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) xl[mt * 64 + lane] = __builtin_bit_cast(u32x4, acc[0][mt]);
      }
      __syncthreads();
    }
    if (!has_tile) return;
    auto store_tile = [&](int otile, const f32x4 (&v)[MT]) {
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int m = mt * 16 + lr;
        if (m < M) {
          uint16_t *orow = (uint16_t *)st.out + (size_t)m * st.ld_out;
          const uint16_t *rrow = (const uint16_t *)st.res + (size_t)m * st.ld_res;
          float rr[4];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const int n = otile * 16 + lg * 4 + i;
            float r = v[mt][i];
            if ((st.flags & MK_F_RES) && n < n_out) r += bf2f(rrow[n]);
            rr[i] = r;
          }
          stc_bf16x4(orow, otile * 16 + lg * 4, n_out, rr);
        }
      }
    };
    if (!silu) {
#pragma unroll
      for (int t = 0; t < TW; t++)
        if (tw0 + t < te) store_tile(tw0 + t, acc[t]);
    } else {
      // tile index relative to the range start is even for gate tiles (ranges hold whole pairs)
#pragma unroll
      for (int t = 0; t < TW; t++) {
        const int ti = tw0 + t;
        if (ti >= te || ((ti - tb) & 1)) continue;  // pairs are stored by the holder of their gate tile
        f32x4 v[MT];
        if (t + 1 < TW) {
#pragma unroll
          for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < 4; i++) v[mt][i] = silu_mul(acc[t][mt][i], acc[(t + 1) % TW][mt][i]);
        } else {
#pragma unroll
          for (int mt = 0; mt < MT; mt++) {
            const f32x4 up = __builtin_bit_cast(f32x4, xl[mt * 64 + lane]);
#pragma unroll
            for (int i = 0; i < 4; i++) v[mt][i] = silu_mul(acc[t][mt][i], up[i]);
          }
        }
        store_tile(ti >> 1, v);
      }
    }
  }
}

#ifndef MK_TUNE_NBN
#define MK_TUNE_NBN 4
#endif
// Multi-token linear on the matrix cores, K split inside the workgroup: out[m, n] = bf16(sum_k x[m,k] * W[n,k] (+ res[m,n])) for 2..64 token rows,
// optional SwiGLU epilogue.  A workgroup owns a contiguous range of 16-row weight tiles and ALL token rows, so every
// weight byte is still read from HBM exactly once; its four wavefronts split K and are reduced through LDS.  One
// v_mfma_f32_16x16x32_bf16 consumes a 16(n) x 32(k) weight fragment (one 16-byte load per lane, 64 contiguous bytes per
// weight row) against a 32(k) x 16(m) activation fragment that comes from the L2-resident activation rows.
// Reference tasks: linear_kernel_ck tile tiers (tasks/mi300/linear_ck_mi300.cuh:306-332), gang_linear_kernel
// (tasks/mi300/gang_linear_mi300.cuh:47-108), gang_linear_silu_kernel (:359-576).
// TG = weight tiles per K sweep, NB = 64-wide k steps in flight per wavefront.  Two shapes are instantiated: wide
// stages (several tiles per workgroup) run <6, 2>; narrow ones (one or two weight tiles per workgroup, e.g. N = 4096
// on 256 workgroups) spend the registers on depth instead: <2, MK_TUNE_NBN>.
template <int MT, int TG, int NB>
__device__ __forceinline__ void stage_linear_mfma(CStage &st, Ctx &c, int M, char *smem) {
  // activations were produced by other workgroups: drop what this die's caches hold of them once, then use cached loads
  // so the rows are shared through the die's L2.  (Issued before the barrier is awaited: nothing on this die reads
  // the stage's input buffers between their previous consumer and this barrier.)
  if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  barrier_wait(c);
  c.wrote_through = true;  // outputs are written through: no L2 write-back at this stage's arrival
  MK_MARK(c, 0);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const bool silu = st.flags & MK_F_SILU;
  const int K = st.k, k8 = K / 8;
  const int n_out = silu ? st.n / 2 : st.n;
  const int ntiles = (n_out + 15) / 16;  // output tiles of 16 columns
  const int t_begin = (int)(((long long)c.vid * ntiles) / c.G), t_end = (int)(((long long)(c.vid + 1) * ntiles) / c.G);
  const uint16_t *x = (st.flags & MK_F_NORM) ? (const uint16_t *)st.norm_out : (const uint16_t *)st.in;
  const int ldx = (st.flags & MK_F_NORM) ? st.ld_norm : st.ld_in;
  const bool pipe = (K & 255) == 0;  // every wavefront's K slice is a whole number of 64-wide steps
  const int lgw = pipe ? 16 : 8;     // k elements a lane group owns per step
  const int kq = ((K / 32 + MK_WAVES - 1) / MK_WAVES) * 32;  // K slice per wavefront, multiple of 32
  const int kbeg = min(K, wave * kq), kend = min(K, kbeg + kq);
  const int half = st.silu_half;
  const int otg = silu ? TG / 2 : TG;  // output tiles per sweep
  f32x4 *red = (f32x4 *)smem;           // [waves][TG][MT][64]
  // With a tile-ordered weight copy the step's two operands hold k = 64 s + 8 lg .. and 64 s + 32 + 8 lg .. (the copy's
  // order) and a tile streams contiguously; read from the row-major weights they are the 32 contiguous bytes at
  // k = 64 s + 16 lg.  The token rows follow the same order.
  const bool packed = pipe && st.wpack != nullptr;
  const int wstep = packed ? 128 : 8, whalf = packed ? 64 : 1;  // 16-byte operands between steps / between the halves
  const int xhalf = packed ? 32 : 8;                           // elements between the halves of a token-row step
  const uint16_t *xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) xrow[mt] = x + (size_t)min(mt * 16 + lr, M - 1) * ldx + (packed ? lg * 8 : lg * lgw);

  for (int ot0 = t_begin; ot0 < t_end; ot0 += otg) {
    const int not_ = min(otg, t_end - ot0);       // output tiles in this sweep
    const int nt = silu ? 2 * not_ : not_;        // weight tiles in this sweep
    const uint16_t *wrow[TG];
#pragma unroll
    for (int t = 0; t < TG; t++) {
      const int ot = ot0 + (silu ? (t >> 1) : t);
      int o = min(ot * 16 + lr, n_out - 1);       // output column owned by this lane's weight row
      int vr = o;
      if (silu) {
        const int g = o / half;
        vr = g * 2 * half + (o - g * half) + ((t & 1) ? half : 0);
      }
      wrow[t] = packed ? (const uint16_t *)((const u32x4 *)st.wpack + (size_t)(silu ? 2 * ot + (t & 1) : ot) * (K >> 6) * 128 + lane)
                       : (const uint16_t *)weight_row(st.w, vr, k8) + lg * lgw;
    }
    f32x4 acc[TG][MT];
#pragma unroll
    for (int t = 0; t < TG; t++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) acc[t][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (pipe) {
      // 64 k per step: a lane owns 32 contiguous bytes of its weight row and of its token row (two matrix-core
      // operands), so the four lane groups of a row cover one whole 128-byte line; NB steps are kept in flight.
      const int nsteps = (kend - kbeg) >> 6;
      bf16x8 a[NB][TG][2], b[NB][MT][2];
      auto load_step = [&](int s_, bf16x8 (&aa)[TG][2], bf16x8 (&bb)[MT][2]) {
        const int k = kbeg + (s_ << 6);
#pragma unroll
        for (int t = 0; t < TG; t++)
          if (t < nt) {
            const bf16x8 *wp = (const bf16x8 *)wrow[t] + (k >> 6) * wstep;
            aa[t][0] = __builtin_nontemporal_load(wp);
            aa[t][1] = __builtin_nontemporal_load(wp + whalf);
          }
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
          bb[mt][0] = *(const bf16x8 *)(xrow[mt] + k);
          bb[mt][1] = *(const bf16x8 *)(xrow[mt] + k + xhalf);
        }
      };
#pragma unroll
      for (int j = 0; j < NB; j++)
        if (j < nsteps) load_step(j, a[j], b[j]);
      for (int s0 = 0; s0 < nsteps; s0 += NB) {
#pragma unroll
        for (int j = 0; j < NB; j++) {
          if (s0 + j < nsteps) {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
              for (int t = 0; t < TG; t++)
                if (t < nt) {
#pragma unroll
                  for (int mt = 0; mt < MT; mt++) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j][t][h], b[j][mt][h], acc[t][mt], 0, 0, 0);
                }
            if (s0 + j + NB < nsteps) load_step(s0 + j + NB, a[j], b[j]);
          }
        }
      }
    } else {
#pragma unroll 2
      for (int k = kbeg; k < kend; k += 32) {
        bf16x8 a[TG], b[MT];
#pragma unroll
        for (int t = 0; t < TG; t++)
          if (t < nt) a[t] = __builtin_nontemporal_load((const bf16x8 *)(wrow[t] + k));
#pragma unroll
        for (int mt = 0; mt < MT; mt++) b[mt] = *(const bf16x8 *)(xrow[mt] + k);
#pragma unroll
        for (int t = 0; t < TG; t++)
          if (t < nt) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], b[mt], acc[t][mt], 0, 0, 0);
          }
      }
    }
    MK_MARK(c, 1);
    __syncthreads();  // previous sweep's epilogue has finished reading LDS
#pragma unroll
    for (int t = 0; t < TG; t++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) red[((wave * TG + t) * MT + mt) * 64 + lane] = acc[t][mt];
    __syncthreads();
    MK_MARK(c, 2);
    // epilogue: entry (output tile u, token tile mt, lane slot l) -> 4 consecutive output columns of one token row
    const int entries = not_ * MT * 64;
    for (int e = tid; e < entries; e += MK_THREADS) {
      const int l = e & 63, mt = (e >> 6) % MT, u = (e >> 6) / MT;
      const int m = mt * 16 + (l & 15);
      const int n0 = (ot0 + u) * 16 + (l >> 4) * 4;
      f32x4 v, v2;
      if (silu) {
        v = red[((0 * TG + 2 * u) * MT + mt) * 64 + l];
        v2 = red[((0 * TG + 2 * u + 1) * MT + mt) * 64 + l];
#pragma unroll
        for (int w = 1; w < MK_WAVES; w++) {
          v += red[((w * TG + 2 * u) * MT + mt) * 64 + l];
          v2 += red[((w * TG + 2 * u + 1) * MT + mt) * 64 + l];
        }
      } else {
        v = red[((0 * TG + u) * MT + mt) * 64 + l];
#pragma unroll
        for (int w = 1; w < MK_WAVES; w++) v += red[((w * TG + u) * MT + mt) * 64 + l];
      }
      if (m < M) {
        uint16_t *orow = (uint16_t *)st.out + (size_t)m * st.ld_out;
        const uint16_t *rrow = (const uint16_t *)st.res + (size_t)m * st.ld_res;
        float rr[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int n = n0 + i;
          float r = silu ? silu_mul(v[i], v2[i]) : v[i];
          if ((st.flags & MK_F_RES) && n < n_out) r += bf2f(rrow[n]);
          rr[i] = r;
        }
        stc_bf16x4(orow, n0, n_out, rr);
      }
    }
  }
}

// Standalone SwiGLU over interleaved [gate ; up] groups (used when the graph keeps the
// gate/up linear and the activation apart).  Reference task: tasks/mi300/silu_mul_mi300.cuh:42-184.
__device__ __forceinline__ void stage_silu_mul(CStage &st, Ctx &c, int M) {
  barrier_wait(c);
  const int n = st.n, half = st.silu_half;
  const uint16_t *in = (const uint16_t *)st.in;
  uint16_t *out = (uint16_t *)st.out;
  const int total = M * (st.topk > 0 ? st.topk : 1) * n;  // MoE: topk rows per token, contiguous
  for (int i = c.vid * MK_THREADS + threadIdx.x; i < total; i += c.G * MK_THREADS) {
    const int t = i / n, j = i - t * n;
    const int g = j / half, jj = j - g * half;
    const uint16_t *row = in + (size_t)t * st.ld_in + (size_t)g * 2 * half;
    out[(size_t)t * st.ld_out + j] = (uint16_t)f2bf(silu_mul(bf2f(ldc_u16(row + jj)), bf2f(ldc_u16(row + half + jj))));
  }
}

// Row copy.  Reference task: identity_task_impl (tasks/ampere/identity.cuh:24-37).
__device__ __forceinline__ void stage_copy(CStage &st, Ctx &c, int M) {
  barrier_wait(c);
  const uint16_t *in = (const uint16_t *)st.in;
  uint16_t *out = (uint16_t *)st.out;
  const long long total = (long long)M * st.n;
  for (long long i = (long long)c.vid * MK_THREADS + threadIdx.x; i < total; i += (long long)c.G * MK_THREADS) stc_u16(out + i, ldc_u16(in + i));
  c.wrote_through = true;
}

// ----------------------------------------------------------------------------- mixture of experts
// Routing lists of one workgroup, kept in the LDS region above MK_MOE_OFFSET.
struct MoeLds {
  int r[MK_MOE_MAX_EXPERTS];          // single-token routing: 1 + slot per expert
  int act_e[MK_MOE_MAX_EXPERTS];      // expert id of each active expert
  int pair_off[MK_MOE_MAX_EXPERTS + 4];  // first (token, slot) pair of each active expert; [n_act] = number of pairs
  int pair_ts[MK_MAX_TOKENS * MK_MOE_MAX_TOPK];  // token | slot << 8
  int n_act;
  int wtot[2][MK_WAVES];
  float w[MK_MOE_MAX_TOPK];           // single-token routing weights by slot
};

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f32<0x128>(v));
  v = fmaxf(v, dpp_f32<0x124>(v));
  v = fmaxf(v, dpp_f32<0x122>(v));
  v = fmaxf(v, dpp_f32<0x121>(v));
  return fmaxf(fmaxf(lane_f32(v, 0), lane_f32(v, 16)), fmaxf(lane_f32(v, 32), lane_f32(v, 48)));
}

// Arg-max of (value, index) pairs over the wavefront; equal values go to the lower index.  Every lane returns the winner.
__device__ __forceinline__ void wave_argmax(float &bv, int &be) {
#define MK_ARGMAX_STEP(CTRL)                                                 \
  {                                                                          \
    const float ov = dpp_f32<CTRL>(bv);                                      \
    const int oe = __builtin_amdgcn_update_dpp(0, be, CTRL, 0xF, 0xF, true); \
    if (ov > bv || (ov == bv && oe < be)) {                                  \
      bv = ov;                                                               \
      be = oe;                                                               \
    }                                                                        \
  }
  MK_ARGMAX_STEP(0x128)
  MK_ARGMAX_STEP(0x124)
  MK_ARGMAX_STEP(0x122)
  MK_ARGMAX_STEP(0x121)
#undef MK_ARGMAX_STEP
  float rv = lane_f32(bv, 0);
  int re = __builtin_amdgcn_readlane(be, 0);
#pragma unroll
  for (int r = 16; r < 64; r += 16) {
    const float ov = lane_f32(bv, r);
    const int oe = __builtin_amdgcn_readlane(be, r);
    if (ov > rv || (ov == rv && oe < re)) {
      rv = ov;
      re = oe;
    }
  }
  bv = rv;
  be = re;
}

// Route one token with one wavefront: fp32 softmax over all experts, `topk` rounds of arg-max (equal probabilities
// go to the lower expert id), weights renormalised by the sum of the selected probabilities.  Lane l owns experts
// l, l+64, ...: sel[j] becomes 1 + slot for a selected expert l + 64 j, 0 otherwise; lane s < topk returns the weight
// and expert of slot s.  Reference task: tasks/mi300/moe_topk_softmax_mi300.cuh:100-213.
__device__ __forceinline__ void moe_route_wave(const uint16_t *logits, int E, int topk, int lane, int sel[4], float &w_slot, int &e_slot) {
  float p[4];
  float mx = -3.0e38f;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int e = j * 64 + lane;
    p[j] = e < E ? bf2f(ldc_u16(logits + e)) : -3.0e38f;
    mx = fmaxf(mx, p[j]);
    sel[j] = 0;
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    p[j] = (j * 64 + lane < E) ? expf(p[j] - mx) : 0.f;
    sum += p[j];
  }
  const float inv = 1.f / wave_sum(sum);
#pragma unroll
  for (int j = 0; j < 4; j++) p[j] = (j * 64 + lane < E) ? p[j] * inv : -1.f;
  float tot = 0.f;
  w_slot = 0.f;
  e_slot = 0;
  for (int s = 0; s < topk; s++) {
    float bv = p[0];
    int be = lane;
#pragma unroll
    for (int j = 1; j < 4; j++)
      if (p[j] > bv) {
        bv = p[j];
        be = j * 64 + lane;
      }
    wave_argmax(bv, be);
    tot += bv;
    if (lane == s) {
      w_slot = bv;
      e_slot = be;
    }
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (j * 64 + lane == be) {
        sel[j] = s + 1;
        p[j] = -10000.f;
      }
  }
  w_slot *= 1.f / tot;
}

// Router stage for multi-token iterations: one wavefront per token writes the routing weights and the token's
// column of the routing table.  Columns of tokens that are not part of the iteration are left alone.
__device__ __forceinline__ void stage_moe_topk(CStage &st, Ctx &c, int M) {
  barrier_wait(c);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int E = st.num_experts;
  for (int t = c.vid * MK_WAVES + wave; t < M; t += c.G * MK_WAVES) {
    int sel[4];
    float w;
    int e;
    moe_route_wave((const uint16_t *)st.moe_logits + (size_t)t * st.ld_logits, E, st.topk, lane, sel, w, e);
    if (lane < st.topk) __hip_atomic_store(st.moe_topk_w + (size_t)t * st.ld_topk_w + lane, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (j * 64 + lane < E) __hip_atomic_store(st.moe_routing + (size_t)(j * 64 + lane) * st.ld_routing + t, sel[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  c.wrote_through = true;  // written through: no L2 write-back at this stage's arrival
}

// Build the active-expert list and the (token, slot) pairs of every active expert from the routing table.
// Single-token iterations keep slot order (active expert s is the expert of slot s); multi-token iterations list
// experts in ascending id with their tokens in ascending order.
__device__ __forceinline__ void moe_build_lists(CStage &st, MoeLds *L, int M, bool r_in_lds) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int E = st.num_experts;
  if (M == 1) {
    if (tid <= st.topk) {  // slot s is "active expert" s; a slot no expert claims (caller-written table) stays empty
      L->act_e[tid] = -1;
      L->pair_off[tid] = tid;
      L->pair_ts[tid] = tid << 8;
    }
    if (tid == 0) L->n_act = st.topk;
    __syncthreads();
    if (tid < E) {
      const int r = r_in_lds ? L->r[tid] : ldc_i32(st.moe_routing + (size_t)tid * st.ld_routing);
      if (r > 0 && r <= st.topk) L->act_e[r - 1] = tid;
    }
    __syncthreads();
    return;
  }
  // the expert's row of the routing table, all requested at once (the multi-token callers have done their acquire,
  // but the table is tiny: device-scope loads keep this correct for any caller)
  int rv[MK_MAX_TOKENS];
  int cnt = 0;
  if (tid < E) {
#pragma unroll
    for (int t = 0; t < MK_MAX_TOKENS; t++)
      if (t < M) rv[t] = ldc_i32(st.moe_routing + (size_t)tid * st.ld_routing + t);
#pragma unroll
    for (int t = 0; t < MK_MAX_TOKENS; t++)
      if (t < M) cnt += rv[t] > 0 && rv[t] <= st.topk;
  }
  int sc = cnt, sa = cnt > 0;  // inclusive scans inside the wavefront
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int vc = __shfl_up(sc, o, 64), va = __shfl_up(sa, o, 64);
    if (lane >= o) {
      sc += vc;
      sa += va;
    }
  }
  if (lane == 63) {
    L->wtot[0][wave] = sc;
    L->wtot[1][wave] = sa;
  }
  __syncthreads();
  int bc = 0, ba = 0;
  for (int w = 0; w < wave; w++) {
    bc += L->wtot[0][w];
    ba += L->wtot[1][w];
  }
  const int off = bc + sc - cnt, ai = ba + sa - (cnt > 0);
  if (cnt > 0) {
    L->act_e[ai] = tid;
    L->pair_off[ai] = off;
    int i = off;
#pragma unroll
    for (int t = 0; t < MK_MAX_TOKENS; t++)
      if (t < M) {
        const int r = rv[t];
        if (r > 0 && r <= st.topk && i < MK_MAX_TOKENS * MK_MOE_MAX_TOPK) L->pair_ts[i++] = t | ((r - 1) << 8);
      }
  }
  if (tid == MK_THREADS - 1) {
    L->n_act = ba + sa;
    L->pair_off[ba + sa] = bc + sc;
  }
  __syncthreads();
}

// Per-expert linear over the active experts: y[t, slot, :] = W[e(t,slot)] x(t, slot), one weight row (or one
// [gate ; up] row pair) per wavefront step, each row read once and applied to every token routed to its expert.
// Work units (active expert, row) are dealt out in contiguous runs per wavefront; the rows of the next R units are
// in flight in registers while a unit is reduced.  Optional epilogues: SwiGLU (gate and up rounded to bf16 first, as
// the separate activation task of the reference sees them) and, for a single token, the weighted sum over the
// slots plus residual, accumulated in slot order in fp32 from the bf16-rounded expert outputs.
// KL = 16-byte row segments per lane (K <= 512 KL).
// Reference tasks: moe_linear_kernel_mi300 (tasks/mi300/moe_linear_mi300.cuh:53-295), silu_mul_task_impl,
// mul_sum_add_mi300_task_impl (tasks/mi300/moe_mul_sum_add_mi300.cuh:31-55).
template <int KL, int R, bool SILU>
__device__ __forceinline__ void stage_moe_linear_t(CStage &st, Ctx &c, int M, char *smem) {
  constexpr int NROW = SILU ? 2 : 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  MoeLds *L = (MoeLds *)(smem + MK_MOE_OFFSET);
  const int k8 = st.k / 8;
  const bool combine = !SILU && (st.flags & MK_F_MOE_COMBINE) && M == 1;
  const bool inline_topk = (st.flags & MK_F_MOE_INLINE_TOPK) && M == 1;
  barrier_wait(c);
  if (M > 1) {  // activation rows are read with cached loads below: drop stale lines of this CU's L1 first
    if (tid == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    __syncthreads();
  }
  if (inline_topk) {
    if (wave == 0) {
      int sel[4];
      float w;
      int e;
      moe_route_wave((const uint16_t *)st.moe_logits, st.num_experts, st.topk, lane, sel, w, e);
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (j * 64 + lane < st.num_experts) {
          L->r[j * 64 + lane] = sel[j];
          if (c.vid == 0) st.moe_routing[(size_t)(j * 64 + lane) * st.ld_routing] = sel[j];
        }
      if (lane < st.topk) {
        L->w[lane] = w;
        if (c.vid == 0) st.moe_topk_w[lane] = w;
      }
    }
    __syncthreads();
  } else if (combine && tid < st.topk) {
    L->w[tid] = ldc_f32(st.moe_topk_w + tid);
  }
  moe_build_lists(st, L, M, inline_topk);
  const int n_act = L->n_act;
  if (c.vid == 0 && st.moe_mask) {  // publish the active-expert list (its order is unspecified in the reference)
    for (int i = tid; i < st.num_experts; i += MK_THREADS) st.moe_mask[i] = i < n_act ? L->act_e[i] : -1;
    if (tid == 0) st.moe_mask[st.num_experts] = n_act;
  }
  // single token: stage the input row(s) in LDS (one row, or one row per slot)
  const int nslot_in = st.ld_in_slot ? st.topk : 1;
  const bool x_lds = M == 1 && (size_t)nslot_in * st.k * 2 <= (size_t)MK_RED_OFFSET;
  u32x4 *xs4 = (u32x4 *)smem;
  if (x_lds) {
    for (int i = tid; i < nslot_in * k8; i += MK_THREADS) {
      const int s = i / k8, o = i - s * k8;
      xs4[i] = ldc_16B((const u32x4 *)((const uint16_t *)st.in + (size_t)s * st.ld_in_slot) + o);
    }
    __syncthreads();
  }
  const int NR = SILU ? st.n / 2 : st.n;  // units per expert
  const int nwaves = c.G * MK_WAVES, gw = c.vid * MK_WAVES + wave;
  int U, upw;
  if (combine) {  // token-major: the n_act units of one output row are consecutive and stay in one wavefront
    U = NR * n_act;
    upw = ((NR + nwaves - 1) / nwaves) * n_act;
  } else {
    U = n_act * NR;
    upw = (U + nwaves - 1) / nwaves;
  }
  const int u0 = min(U, gw * upw), u1 = min(U, u0 + upw);
  const u32x4 *W = (const u32x4 *)st.w.seg[0];
  const u32x4 zero = {0u, 0u, 0u, 0u};
  u32x4 buf[R][NROW][KL];
  auto load_unit = [&](int u, u32x4 (&b)[NROW][KL]) {
    int a, j;
    if (combine) {
      j = u / n_act;
      a = u - j * n_act;
    } else {
      a = u / NR;
      j = u - a * NR;
    }
    const int ei = L->act_e[a];
    const size_t e = (size_t)max(ei, 0);
#pragma unroll
    for (int h = 0; h < NROW; h++) {
      const u32x4 *p = W + (e * st.n + (size_t)(j + h * NR)) * k8;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) b[h][kc] = (ei >= 0 && kc * 64 + lane < k8) ? ldg_stream(p + kc * 64 + lane) : zero;
    }
  };
#pragma unroll
  for (int jj = 0; jj < R; jj++)
    if (u0 + jj < u1) load_unit(u0 + jj, buf[jj]);
  uint16_t *out = (uint16_t *)st.out, *out2 = (uint16_t *)st.out2;
  float comb = 0.f;
  for (int i = u0; i < u1; i += R) {
#pragma unroll
    for (int jj = 0; jj < R; jj++) {
      const int u = i + jj;
      if (u < u1) {
        int a, j;
        if (combine) {
          j = u / n_act;
          a = u - j * n_act;
        } else {
          a = u / NR;
          j = u - a * NR;
        }
        const int p0 = L->pair_off[a], p1 = L->act_e[a] >= 0 ? L->pair_off[a + 1] : p0;
        if (combine && a == 0) comb = bf2f(ldc_u16((const uint16_t *)st.res + j));
        for (int p = p0; p < p1; p++) {
          const int ts = L->pair_ts[p], tok = ts & 255, slot = ts >> 8;
          const u32x4 *x = x_lds ? xs4 + (st.ld_in_slot ? slot * k8 : 0)
                                 : (const u32x4 *)((const uint16_t *)st.in + (size_t)tok * st.ld_in + (size_t)slot * st.ld_in_slot);
          float acc[NROW];
#pragma unroll
          for (int h = 0; h < NROW; h++) acc[h] = 0.f;
#pragma unroll
          for (int kc = 0; kc < KL; kc++) {
            u32x4 xv = zero;
            if (kc * 64 + lane < k8) xv = (x_lds || M > 1) ? x[kc * 64 + lane] : ldc_16B(x + kc * 64 + lane);
#pragma unroll
            for (int h = 0; h < NROW; h++) acc[h] = dot8(buf[jj][h][kc], xv, acc[h]);
          }
#pragma unroll
          for (int h = 0; h < NROW; h++) acc[h] = wave_sum(acc[h]);
          uint16_t *y = out + (size_t)tok * st.ld_out + (size_t)slot * st.ld_out_slot;
          if (SILU) {
            const uint32_t g = f2bf(acc[0]), up = f2bf(acc[NROW - 1]);
            if (lane == 0) {
              y[j] = (uint16_t)g;
              y[j + NR] = (uint16_t)up;
              out2[(size_t)tok * st.ld_out2 + (size_t)slot * st.ld_out2_slot + j] = (uint16_t)f2bf(silu_mul(bf2f((uint16_t)g), bf2f((uint16_t)up)));
            }
          } else {
            const uint32_t v = f2bf(acc[0]);
            if (lane == 0) y[j] = (uint16_t)v;
            if (combine) comb = fmaf(bf2f((uint16_t)v), L->w[slot], comb);
          }
        }
        if (combine && a == n_act - 1 && lane == 0) out2[j] = (uint16_t)f2bf(comb);
        if (u + R < u1) load_unit(u + R, buf[jj]);
      }
    }
  }
}

// Single-token per-expert linear, tuned like the dense single-token linear: wavefront 0 polls the barrier, routes
// (or reads the routing of the stage before), stages the input row(s) and publishes the routing outputs; wavefronts
// 1..3 draw work from the workgroup's LDS ticket counter with R tickets of weight rows in flight each.  A ticket is
// one [gate ; up] row pair of one slot's expert (SILU) or, for the W2 + weighted-sum form, output row j of ALL TK
// slots' experts, so the combine stays inside one wavefront.  When the stage directly before was the W13 stage of the
// same token its expert list is still in LDS: the first tickets' rows are then requested before the barrier.  All
// outputs are written through.
template <int KL, int R, bool SILU>
__device__ __forceinline__ void stage_moe_linear_m1(CStage &st, Ctx &c, char *smem) {
  constexpr int TK = 8;
  constexpr int NSUB = SILU ? 2 : TK;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  MoeLds *L = (MoeLds *)(smem + MK_MOE_OFFSET);
  const int k8 = st.k / 8, topk = st.topk, E = st.num_experts;
  const bool ctrl = wave == 0;
  const bool inline_topk = st.flags & MK_F_MOE_INLINE_TOPK;
  const int NR = SILU ? st.n / 2 : st.n;
  const int n_tk = SILU ? topk * NR : NR;
  const int tq = n_tk / c.G, trem = n_tk - tq * c.G;
  const int t_begin = c.vid * tq + min(c.vid, trem), t_end = t_begin + tq + (c.vid < trem ? 1 : 0);
  int *ticket = c.sh_ticket + (c.seq & 1);
  const bool reuse = !inline_topk && __builtin_amdgcn_readfirstlane(c.sh_ticket[2]) == c.seq - 1;
  const u32x4 *W = (const u32x4 *)st.w.seg[0];
  u32x4 *xs4 = (u32x4 *)smem;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  auto take = [&]() -> int {
    int t = 0;
    if (lane == 0) t = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    t = __builtin_amdgcn_readfirstlane(t) + t_begin;
    return t < t_end ? t : -1;
  };
  // W2 form: the weight base of every slot's expert, fixed for the whole stage (set once the expert list is known)
  const u32x4 *eb[SILU ? 1 : TK];
  bool ev[SILU ? 1 : TK];
  auto set_bases = [&]() {
    if (!SILU) {
#pragma unroll
      for (int h = 0; h < (SILU ? 1 : TK); h++) {
        const int ei = __builtin_amdgcn_readfirstlane(L->act_e[h]);
        ev[h] = ei >= 0;
        eb[h] = W + (size_t)max(ei, 0) * st.n * k8 + lane;
      }
    }
  };
  auto load_ticket = [&](int tk, u32x4 (&b)[NSUB][KL]) {
    if (SILU) {
      const int a = tk / NR, j = tk - a * NR;
      const int ei = __builtin_amdgcn_readfirstlane(L->act_e[a]);
#pragma unroll
      for (int h = 0; h < NSUB; h++) {
        const u32x4 *p = W + ((size_t)max(ei, 0) * st.n + (size_t)(j + h * NR)) * k8;
#pragma unroll
        for (int kc = 0; kc < KL; kc++) b[h][kc] = (ei >= 0 && kc * 64 + lane < k8) ? ldg_stream(p + kc * 64 + lane) : zero;
      }
    } else {
#pragma unroll
      for (int h = 0; h < NSUB; h++) {
        const u32x4 *p = eb[SILU ? 0 : h] + (size_t)tk * k8;
#pragma unroll
        for (int kc = 0; kc < KL; kc++) b[h][kc] = (ev[SILU ? 0 : h] && kc * 64 + lane < k8) ? ldg_stream(p + kc * 64) : zero;
      }
    }
  };
  u32x4 buf[R][NSUB][KL];
  int ut[R];
#pragma unroll
  for (int j = 0; j < R; j++) ut[j] = -1;
  // W2 form after the W13 stage of the same token: the experts are known before the barrier, and a workgroup's whole
  // share of the weights (a few tickets of TK rows) fits the idle LDS above the routing lists.  Each worker wavefront
  // keeps its R tickets in flight as a rolling window: a ticket that has landed is parked in LDS and its slot refilled,
  // NLP tickets per wavefront; they are reduced from LDS once the input rows are there.
  constexpr int NLP = SILU ? 0 : MK_TUNE_MOE_M1_PARK;
  constexpr int PARK_OFF = MK_MOE_OFFSET + 8192;
  static_assert(sizeof(MoeLds) <= 8192, "routing lists overlap the parked rows");
  static_assert(PARK_OFF + (MK_WAVES - 1) * NLP * NSUB * KL * 1024 <= MK_LDS_BYTES, "parked rows exceed the LDS window");
  u32x4 *lrows = (u32x4 *)(smem + PARK_OFF) + (size_t)(wave > 0 ? wave - 1 : 0) * (NLP > 0 ? NLP : 1) * NSUB * KL * 64;
  int lo_[NLP > 0 ? NLP : 1];
#pragma unroll
  for (int i = 0; i < (NLP > 0 ? NLP : 1); i++) lo_[i] = -1;
  if (!ctrl) {
    if (reuse) {
      set_bases();
#pragma unroll
      for (int i = 0; i < NLP + R; i++) {
        const int sl = i % R;
        if (i >= R) {
#pragma unroll
          for (int h = 0; h < NSUB; h++)
#pragma unroll
            for (int kc = 0; kc < KL; kc++) lrows[(((i - R) * NSUB + h) * KL + kc) * 64 + lane] = buf[sl][h][kc];
          lo_[i - R] = ut[sl];
        }
        ut[sl] = take();
        if (ut[sl] >= 0) load_ticket(ut[sl], buf[sl]);
      }
    }
  } else {
    if (c.pending && tid == 0) barrier_poll(c);
    // input row(s): one row, or one row per slot (at most 12 16-byte segments per lane)
    const int nx = (st.ld_in_slot ? topk : 1) * k8;
    u32x4 xv[12];
#pragma unroll
    for (int i = 0; i < 12; i++) {
      const int ci = i * 64 + lane;
      if (ci < nx) {
        const int sl = ci / k8, o = ci - sl * k8;
        xv[i] = ldc_16B((const u32x4 *)((const uint16_t *)st.in + (size_t)sl * st.ld_in_slot) + o);
      }
    }
    if (inline_topk) {
      int sel[4];
      float w;
      int e;
      moe_route_wave((const uint16_t *)st.moe_logits, E, topk, lane, sel, w, e);
      if (lane < topk) {
        L->act_e[lane] = e;
        L->w[lane] = w;
        if (c.vid == 0) __hip_atomic_store(st.moe_topk_w + lane, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (c.vid == 0) {
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (j * 64 + lane < E) __hip_atomic_store(st.moe_routing + (size_t)(j * 64 + lane) * st.ld_routing, sel[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    } else if (!reuse) {
      if (lane < topk) L->act_e[lane] = -1;
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (j * 64 + lane < E) {
          const int r = ldc_i32(st.moe_routing + (size_t)(j * 64 + lane) * st.ld_routing);
          if (r > 0 && r <= topk) L->act_e[r - 1] = j * 64 + lane;
        }
      if (!SILU && lane < topk) L->w[lane] = ldc_f32(st.moe_topk_w + lane);
    }
#pragma unroll
    for (int i = 0; i < 12; i++)
      if (i * 64 + lane < nx) xs4[i * 64 + lane] = xv[i];
    if (lane == 0) c.sh_ticket[2] = c.seq;
  }
  __syncthreads();
  barrier_done(c);
  // outputs are collected in LDS ([array][ticket - t_begin]) and written out together once every worker is done
  uint16_t *so = (uint16_t *)(smem + MK_OUT_OFFSET);
  const int n_loc = t_end - t_begin;
  constexpr int NARR = SILU ? 3 : TK + 1;
  auto flush = [&]() {
    __syncthreads();
    uint16_t *o1 = (uint16_t *)st.out, *o2 = (uint16_t *)st.out2;
    for (int i = tid; i < NARR * n_loc; i += MK_THREADS) {
      const int arr = i / n_loc, tk = t_begin + (i - arr * n_loc);
      uint16_t *dst;
      if (SILU) {
        const int a = tk / NR, row = tk - a * NR;
        dst = arr == 2 ? o2 + (size_t)a * st.ld_out2_slot + row : o1 + (size_t)a * st.ld_out_slot + row + arr * NR;
      } else {
        if (arr < TK && L->act_e[arr] < 0) continue;
        dst = arr == TK ? o2 + tk : o1 + (size_t)arr * st.ld_out_slot + tk;
      }
      stc_u16(dst, so[i]);
    }
    c.wrote_through = true;
  };
  if (ctrl) {
    if (c.vid == 0 && st.moe_mask) {  // active-expert list (its order is unspecified in the reference) and count
      for (int i = lane; i < E; i += 64) __hip_atomic_store(st.moe_mask + i, i < topk ? L->act_e[i] : -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (lane == 0) __hip_atomic_store(st.moe_mask + E, topk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (!reuse || ctrl) set_bases();
  // the staged input row(s) stay in registers for the whole stage
  u32x4 xr[SILU ? 1 : TK][KL];
#pragma unroll
  for (int h = 0; h < (SILU ? 1 : TK); h++)
#pragma unroll
    for (int kc = 0; kc < KL; kc++) xr[h][kc] = (kc * 64 + lane < k8) ? xs4[(st.ld_in_slot ? h * k8 : 0) + kc * 64 + lane] : zero;
  float ures[R];
#pragma unroll
  for (int j = 0; j < R; j++) {
    if (!reuse || ctrl) {  // the control wavefront joins the streaming once its part is done
      ut[j] = take();
      if (ut[j] >= 0) load_ticket(ut[j], buf[j]);
    }
    ures[j] = (!SILU && ut[j] >= 0) ? bf2f(ldc_u16((const uint16_t *)st.res + ut[j])) : 0.f;
  }
  if constexpr (NLP > 0) {
    // the parked tickets first: no memory traffic, the register slots keep landing meanwhile
    float lres[NLP];
#pragma unroll
    for (int i = 0; i < NLP; i++) lres[i] = lo_[i] >= 0 ? bf2f(ldc_u16((const uint16_t *)st.res + lo_[i])) : 0.f;
#pragma unroll
    for (int i = 0; i < NLP; i++) {
      if (lo_[i] >= 0) {
        const int tk = lo_[i];
        float acc[NSUB];
#pragma unroll
        for (int h = 0; h < NSUB; h++) {
          acc[h] = 0.f;
#pragma unroll
          for (int kc = 0; kc < KL; kc++) acc[h] = dot8(lrows[((i * NSUB + h) * KL + kc) * 64 + lane], xr[SILU ? 0 : h][kc], acc[h]);
        }
#pragma unroll
        for (int h = 0; h < NSUB; h++) acc[h] = wave_sum(acc[h]);
        float comb = lres[i];
#pragma unroll
        for (int h = 0; h < NSUB; h++) {
          const uint32_t v = f2bf(acc[h]);
          if (lane == 0) so[h * n_loc + tk - t_begin] = (uint16_t)v;
          comb = fmaf(bf2f((uint16_t)v), L->w[SILU ? 0 : h], comb);
        }
        if (lane == 0) so[TK * n_loc + tk - t_begin] = (uint16_t)f2bf(comb);
      }
    }
  }
  while (true) {
    bool any = false;
#pragma unroll
    for (int j = 0; j < R; j++) {
      if (ut[j] >= 0) {
        any = true;
        const int tk = ut[j];
        int a = 0, row = tk;
        if (SILU) {
          a = tk / NR;
          row = tk - a * NR;
        }
        float acc[NSUB];
#pragma unroll
        for (int h = 0; h < NSUB; h++) {
          acc[h] = 0.f;
#pragma unroll
          for (int kc = 0; kc < KL; kc++) {
            acc[h] = dot8(buf[j][h][kc], xr[SILU ? 0 : h][kc], acc[h]);
          }
        }
        const float r0 = ures[j];
        ut[j] = take();
        if (ut[j] >= 0) {
          load_ticket(ut[j], buf[j]);
          if (!SILU) ures[j] = bf2f(ldc_u16((const uint16_t *)st.res + ut[j]));
        }
#pragma unroll
        for (int h = 0; h < NSUB; h++) acc[h] = wave_sum(acc[h]);
        if (SILU) {
          const uint32_t g = f2bf(acc[0]), up = f2bf(acc[1]);
          if (lane == 0) {
            so[tk - t_begin] = (uint16_t)g;
            so[n_loc + tk - t_begin] = (uint16_t)up;
            so[2 * n_loc + tk - t_begin] = (uint16_t)f2bf(silu_mul(bf2f((uint16_t)g), bf2f((uint16_t)up)));
          }
        } else {
          float comb = r0;
#pragma unroll
          for (int h = 0; h < NSUB; h++) {
            const uint32_t v = f2bf(acc[h]);
            if (lane == 0) so[h * n_loc + tk - t_begin] = (uint16_t)v;
            comb = fmaf(bf2f((uint16_t)v), L->w[h], comb);
          }
          if (lane == 0) so[TK * n_loc + tk - t_begin] = (uint16_t)f2bf(comb);
        }
      }
    }
    if (!any) break;
  }
  flush();
}

// Multi-token per-expert linear.  Work units (active expert, row) in expert-major order are split over the workgroups
// by cost (a workgroup then touches one or two experts) and drawn from the LDS ticket counter by all four wavefronts.
// The input rows of the tokens routed to the workgroup's experts are staged in LDS once and the outputs are collected
// in an LDS tile, so the loop over an expert's tokens contains NO vector-memory instruction: the compiler can then
// count the weight-row loads in flight exactly, and R units' rows really stay in flight (with a store inside that
// loop every unit waited for all outstanding loads).  The tile is written out at the end, one contiguous run of
// rows per (token, slot).  A workgroup whose tile or staged rows do not fit runs a plain loop over the same units.
template <int KL, int R, bool SILU>
__device__ __forceinline__ void stage_moe_linear_multi(CStage &st, Ctx &c, int M, char *smem) {
  constexpr int NROW = SILU ? 2 : 1;
  constexpr int NARR = SILU ? 3 : 1;
  const int tid = threadIdx.x, lane = tid & 63;
  MoeLds *L = (MoeLds *)(smem + MK_MOE_OFFSET);
  const int k8 = st.k / 8;
  const int n_act = L->n_act;
  const int NR = SILU ? st.n / 2 : st.n;  // units per expert
  const int n_units = n_act * NR;
  // A unit of expert a costs one row load (RC, in units of one reduction) plus one reduction per token routed to a: split
  // the units so that every workgroup gets the same cost.  With w_a = tokens(a) + RC the cost before expert a is
  // NR * (pair_off[a] + RC * a).
  constexpr int RC = SILU ? MK_TUNE_MOE_ROWCOST13 : MK_TUNE_MOE_ROWCOST2;
  int *bnd = L->wtot[0];  // reused: the scans of the list building are done
  if (tid < 2) bnd[tid] = 0;
  __syncthreads();
  const long long total = (long long)NR * (L->pair_off[n_act] + RC * n_act);
  const long long tgt0 = total * c.vid / c.G, tgt1 = total * (c.vid + 1) / c.G;
  if (tid < n_act) {
    const long long before = (long long)NR * (L->pair_off[tid] + RC * tid);
    if (before <= tgt0) __hip_atomic_fetch_max(&bnd[0], tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (before <= tgt1) __hip_atomic_fetch_max(&bnd[1], tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  __syncthreads();
  auto unit_at = [&](long long tgt, int a) -> int {
    if (n_act == 0) return 0;
    const long long before = (long long)NR * (L->pair_off[a] + RC * a);
    const int w = L->pair_off[a + 1] - L->pair_off[a] + RC;
    return a * NR + min(NR, (int)((tgt - before) / w));
  };
  const int u_begin = __builtin_amdgcn_readfirstlane(unit_at(tgt0, bnd[0]));
  const int u_end = __builtin_amdgcn_readfirstlane(c.vid == c.G - 1 ? n_units : unit_at(tgt1, bnd[1]));
  const int nu = u_end - u_begin;
  int p_base = 0, n_pairs = 0, maxp = 0;
  if (nu > 0) {
    const int a0 = u_begin / NR, a1 = (u_end - 1) / NR;
    p_base = L->pair_off[a0];
    n_pairs = L->pair_off[a1 + 1] - p_base;
    for (int a = a0; a <= a1; a++) maxp = max(maxp, L->pair_off[a + 1] - L->pair_off[a]);
  }
  // the decision below is per workgroup (uniform within it); either form covers exactly [u_begin, u_end)
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const u32x4 *W = (const u32x4 *)st.w.seg[0];
  if ((size_t)n_pairs * k8 * 16 > (size_t)(MK_LDS_BYTES - MK_MOE_X_OFFSET) || (size_t)NARR * maxp * nu * 2 > (size_t)MK_MOE_OFFSET) {
    // too many tokens on this workgroup's experts for the LDS windows: plain form over the same unit range
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint16_t *out = (uint16_t *)st.out, *out2 = (uint16_t *)st.out2;
    for (int u = u_begin + wv; u < u_end; u += MK_WAVES) {
      const int a = u / NR, j = u - a * NR;
      const size_t e = (size_t)L->act_e[a];
      for (int p = L->pair_off[a]; p < L->pair_off[a + 1]; p++) {
        const int ts = L->pair_ts[p], tok = ts & 255, slot = ts >> 8;
        const u32x4 *x = (const u32x4 *)((const uint16_t *)st.in + (size_t)tok * st.ld_in + (size_t)slot * st.ld_in_slot);
        float acc[NROW];
#pragma unroll
        for (int h = 0; h < NROW; h++) {
          acc[h] = 0.f;
          const u32x4 *wr = W + (e * st.n + (size_t)(j + h * NR)) * k8;
          for (int kc = lane; kc < k8; kc += 64) acc[h] = dot8(wr[kc], x[kc], acc[h]);
          acc[h] = wave_sum(acc[h]);
        }
        uint16_t *y = out + (size_t)tok * st.ld_out + (size_t)slot * st.ld_out_slot;
        if (SILU) {
          const uint32_t g = f2bf(acc[0]), up = f2bf(acc[NROW - 1]);
          if (lane == 0) {
            y[j] = (uint16_t)g;
            y[j + NR] = (uint16_t)up;
            out2[(size_t)tok * st.ld_out2 + (size_t)slot * st.ld_out2_slot + j] = (uint16_t)f2bf(silu_mul(bf2f((uint16_t)g), bf2f((uint16_t)up)));
          }
        } else if (lane == 0) {
          y[j] = (uint16_t)f2bf(acc[0]);
        }
      }
    }
    return;
  }
  // stage the input rows of the (token, slot) pairs of this workgroup's experts
  u32x4 *xs4 = (u32x4 *)(smem + MK_MOE_X_OFFSET);
  uint16_t *so = (uint16_t *)smem;  // [array][pair of the expert][unit - u_begin]
  for (int i = tid; i < n_pairs * k8; i += MK_THREADS) {
    const int p = i / k8, o = i - p * k8;
    const int ts = L->pair_ts[p_base + p], tok = ts & 255, slot = ts >> 8;
    xs4[i] = ((const u32x4 *)((const uint16_t *)st.in + (size_t)tok * st.ld_in + (size_t)slot * st.ld_in_slot))[o];
  }
  __syncthreads();
  int *ticket = c.sh_ticket + (c.seq & 1);
  auto take = [&](int n) -> int {  // first of the next n units of this workgroup (may lie at or beyond u_end)
    int t = 0;
    if (lane == 0) t = __hip_atomic_fetch_add(ticket, n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return __builtin_amdgcn_readfirstlane(t) + u_begin;
  };
  // Every row load is unconditional: a unit at or beyond the end of the range re-reads the range's last unit and is
  // not reduced.  (With the loads under a branch every wait for one unit's rows drained the other units' loads too.)
  auto load_unit = [&](int u_, u32x4 (&b)[NROW][KL]) {
    const int u = min(u_, u_end - 1);
    const int a = u / NR, j = u - a * NR;
    const size_t e = (size_t)__builtin_amdgcn_readfirstlane(L->act_e[a]);
#pragma unroll
    for (int h = 0; h < NROW; h++) {
      const u32x4 *p = W + (e * st.n + (size_t)(j + h * NR)) * k8;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) b[h][kc] = ldg_stream(p + min(kc * 64 + lane, k8 - 1));  // lanes past the row re-read its last segment; their products are dropped below
    }
  };
  auto reduce_unit = [&](const u32x4 (&b)[NROW][KL], int u) {
    const int a = u / NR;
    const int p0 = __builtin_amdgcn_readfirstlane(L->pair_off[a]), p1 = __builtin_amdgcn_readfirstlane(L->pair_off[a + 1]);
    for (int p = p0; p < p1; p++) {  // LDS only in here
      const u32x4 *x = xs4 + (p - p_base) * k8;
      float acc[NROW];
#pragma unroll
      for (int h = 0; h < NROW; h++) acc[h] = 0.f;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) {
        const u32x4 xv = (kc * 64 + lane < k8) ? x[kc * 64 + lane] : zero;
#pragma unroll
        for (int h = 0; h < NROW; h++) acc[h] = dot8(b[h][kc], xv, acc[h]);
      }
#pragma unroll
      for (int h = 0; h < NROW; h++) acc[h] = wave_sum(acc[h]);
      uint16_t *t0 = so + (size_t)(p - p0) * nu + (u - u_begin);
      if (SILU) {
        const uint32_t g = f2bf(acc[0]), up = f2bf(acc[NROW - 1]);
        if (lane == 0) {
          t0[0] = (uint16_t)g;
          t0[(size_t)maxp * nu] = (uint16_t)up;
          t0[(size_t)2 * maxp * nu] = (uint16_t)f2bf(silu_mul(bf2f((uint16_t)g), bf2f((uint16_t)up)));
        }
      } else if (lane == 0) {
        t0[0] = (uint16_t)f2bf(acc[0]);
      }
    }
  };
  // The units of a group are consecutive rows, nearly always of one expert: they are then reduced jointly per (token,
  // slot) pair -- the pair's input segments are read from LDS once for all of them and their sums are reduced together
  // (transposing reduction, lane q * NROW + h gets unit q's sum h).  A group that straddles two experts takes the
  // unit-by-unit form.
  auto reduce_group = [&](auto &bufs, int g, auto nqc) {
    constexpr int NQ = decltype(nqc)::value;
    constexpr int NVAL = NQ * NROW;
    constexpr int NV = NVAL <= 1 ? 1 : (NVAL <= 2 ? 2 : (NVAL <= 4 ? 4 : (NVAL <= 8 ? 8 : 16)));
    static_assert(NVAL <= 16, "group size");
    const int nvalid = min(NQ, u_end - g);
    const int a = g / NR;
    if ((g + nvalid - 1) / NR != a) {
#pragma unroll
      for (int q = 0; q < NQ; q++)
        if (q < nvalid) reduce_unit(bufs[q], g + q);
      return;
    }
    const int p0 = __builtin_amdgcn_readfirstlane(L->pair_off[a]), p1 = __builtin_amdgcn_readfirstlane(L->pair_off[a + 1]);
    for (int p = p0; p < p1; p++) {  // LDS only in here
      const u32x4 *x = xs4 + (p - p_base) * k8;
      float vv[NV];
#pragma unroll
      for (int i = 0; i < NV; i++) vv[i] = 0.f;
#pragma unroll
      for (int kc = 0; kc < KL; kc++) {
        const u32x4 xv = (kc * 64 + lane < k8) ? x[kc * 64 + lane] : zero;
#pragma unroll
        for (int q = 0; q < NQ; q++)
#pragma unroll
          for (int h = 0; h < NROW; h++) vv[q * NROW + h] = dot8(bufs[q][h][kc], xv, vv[q * NROW + h]);
      }
      const float tot = transpose_sum<NV>(vv, lane);
      const int q = lane / NROW;
      uint16_t *t0 = so + (size_t)(p - p0) * nu + (g + q - u_begin);
      if (SILU) {
        const float upv = dpp_f32<0x101>(tot);  // row_shl:1: the up sum sits one lane above the gate sum
        const uint32_t gb = f2bf(tot), ub = f2bf(upv);
        if (lane < NVAL && (lane & 1) == 0 && q < nvalid) {
          t0[0] = (uint16_t)gb;
          t0[(size_t)maxp * nu] = (uint16_t)ub;
          t0[(size_t)2 * maxp * nu] = (uint16_t)f2bf(silu_mul(bf2f((uint16_t)gb), bf2f((uint16_t)ub)));
        }
      } else if (lane < NVAL && q < nvalid) {
        t0[0] = (uint16_t)f2bf(tot);
      }
    }
  };
  // two groups of units in flight: while one is reduced the other one's rows are landing; tickets only grow, so the
  // first group found beyond the range ends the loop
  constexpr int QA = (R + 1) / 2, QB = R / 2;
  if (nu > 0) {
    u32x4 bufA[QA][NROW][KL], bufB[QB > 0 ? QB : 1][NROW][KL];
    int gA = take(QA), gB = u_end;
#pragma unroll
    for (int q = 0; q < QA; q++) load_unit(gA + q, bufA[q]);
    if (QB > 0) {
      gB = take(QB);
#pragma unroll
      for (int q = 0; q < QB; q++) load_unit(gB + q, bufB[q]);
    }
    while (gA < u_end) {
      reduce_group(bufA, gA, std::integral_constant<int, QA>{});
      gA = take(QA);
#pragma unroll
      for (int q = 0; q < QA; q++) load_unit(gA + q, bufA[q]);
      if (QB > 0) {
        if (gB >= u_end) break;
        reduce_group(bufB, gB, std::integral_constant<int, (QB > 0 ? QB : 1)>{});
        gB = take(QB);
#pragma unroll
        for (int q = 0; q < QB; q++) load_unit(gB + q, bufB[q]);
      }
    }
  }
  __syncthreads();
  // write the tile out: consecutive threads take consecutive rows of one (token, slot)
  uint16_t *out = (uint16_t *)st.out, *out2 = (uint16_t *)st.out2;
  for (int i = tid; i < NARR * maxp * nu; i += MK_THREADS) {
    const int arr = i / (maxp * nu), r = i - arr * maxp * nu, pi = r / nu, ui = r - pi * nu;
    const int u = u_begin + ui, a = u / NR, j = u - a * NR;
    const int p = L->pair_off[a] + pi;
    if (p >= L->pair_off[a + 1]) continue;
    const int ts = L->pair_ts[p], tok = ts & 255, slot = ts >> 8;
    if (SILU && arr == 2) stc_u16(out2 + (size_t)tok * st.ld_out2 + (size_t)slot * st.ld_out2_slot + j, so[i]);
    else stc_u16(out + (size_t)tok * st.ld_out + (size_t)slot * st.ld_out_slot + j + (arr == 1 ? NR : 0), so[i]);
  }
  c.wrote_through = true;  // (the plain form above returns before this and keeps the write-back)
}

__device__ __forceinline__ void stage_moe_linear(CStage &st, Ctx &c, int M, char *smem) {
  const bool silu = st.flags & MK_F_SILU;
  if (M == 1) {
    // tuned single-token forms: W13 + SwiGLU (one input row), W2 + weighted sum over exactly 8 slots
    const int nx = (st.ld_in_slot ? st.topk : 1) * (st.k / 8);
    const int n_loc = (silu ? st.topk * (st.n / 2) : st.n) / c.G + 1;
    if ((silu ? 3 : 9) * n_loc * 2 > MK_MOE_OFFSET - MK_OUT_OFFSET) {
      // outputs of one workgroup do not fit the LDS collection window: generic form below
    } else if (silu && !st.ld_in_slot && nx <= 768) {
      if (st.k <= 1024) return stage_moe_linear_m1<2, 4, true>(st, c, smem);
      if (st.k <= 2048) return stage_moe_linear_m1<4, MK_TUNE_MOE_M1_R13, true>(st, c, smem);
    } else if (!silu && (st.flags & MK_F_MOE_COMBINE) && st.ld_in_slot && st.topk == 8 && nx <= 768) {
      if (st.k <= 1024) return stage_moe_linear_m1<2, MK_TUNE_MOE_M1_R2, false>(st, c, smem);
    }
  }
  if (M > 1) {
    // common front: wait for the previous stage, one acquire (activation rows are read with cached loads), routing lists
    MoeLds *L = (MoeLds *)(smem + MK_MOE_OFFSET);
    barrier_wait(c);
    if (threadIdx.x == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    __syncthreads();
    moe_build_lists(st, L, M, false);
    if (c.vid == 0 && st.moe_mask) {  // publish the active-expert list (its order is unspecified in the reference)
      const int n_act = L->n_act;
      for (int i = threadIdx.x; i < st.num_experts; i += MK_THREADS) st.moe_mask[i] = i < n_act ? L->act_e[i] : -1;
      if (threadIdx.x == 0) st.moe_mask[st.num_experts] = n_act;
    }
    if (st.k <= 1024) {
      if (silu) stage_moe_linear_multi<2, 4, true>(st, c, M, smem);
      else stage_moe_linear_multi<2, MK_TUNE_MOE_R2, false>(st, c, M, smem);
    } else if (st.k <= 2048) {
      if (silu) stage_moe_linear_multi<4, MK_TUNE_MOE_R13, true>(st, c, M, smem);
      else stage_moe_linear_multi<4, 4, false>(st, c, M, smem);
    } else {
      if (silu) stage_moe_linear_multi<8, 1, true>(st, c, M, smem);
      else stage_moe_linear_multi<8, 2, false>(st, c, M, smem);
    }
    return;
  }
  if (st.k <= 1024) {
    if (silu) stage_moe_linear_t<2, 4, true>(st, c, M, smem);
    else stage_moe_linear_t<2, 6, false>(st, c, M, smem);
  } else if (st.k <= 2048) {
    if (silu) stage_moe_linear_t<4, 3, true>(st, c, M, smem);
    else stage_moe_linear_t<4, 4, false>(st, c, M, smem);
  } else {
    if (silu) stage_moe_linear_t<8, 1, true>(st, c, M, smem);
    else stage_moe_linear_t<8, 2, false>(st, c, M, smem);
  }
}

// Weighted sum of the expert outputs plus residual for multi-token iterations:
// out[t, :] = bf16(res[t, :] + sum_k w[t, k] * y[t, k, :]), fp32, slots in order.
// Reference task: mul_sum_add_mi300_task_impl (tasks/mi300/moe_mul_sum_add_mi300.cuh:31-55).
__device__ __forceinline__ void stage_moe_combine(CStage &st, Ctx &c, int M) {
  barrier_wait(c);
  const int n = st.n, total = M * n;
  const uint16_t *in = (const uint16_t *)st.in, *res = (const uint16_t *)st.res;
  uint16_t *out = (uint16_t *)st.out;
  for (int i = c.vid * MK_THREADS + threadIdx.x; i < total; i += c.G * MK_THREADS) {
    const int t = i / n, j = i - t * n;
    float s = bf2f(ldc_u16(res + (size_t)t * st.ld_res + j));
    for (int k = 0; k < st.topk; k++)
      s = fmaf(bf2f(ldc_u16(in + (size_t)t * st.ld_in + (size_t)k * st.ld_in_slot + j)), ldc_f32(st.moe_topk_w + (size_t)t * st.ld_topk_w + k), s);
    stc_u16(out + (size_t)t * st.ld_out + j, (uint16_t)f2bf(s));
  }
  c.wrote_through = true;
}

// Per-head RMSNorm + rotate-half RoPE of one 128-wide head row by one wavefront (lane l owns elements
// l and l+64, the two halves of a rotation pair).  The normalised value is rounded to bf16 before the
// rotation, as in the reference (tasks/mi300/kv_cache_update_mi300.cuh:129-182).  Split in a load half and a
// compute half so that a wavefront can have the loads of several rows in flight.
__device__ __forceinline__ void head_row_load(const uint16_t *src, int lane, float &x0, float &x1) {
  x0 = bf2f(ldc_u16(src + lane));
  x1 = bf2f(ldc_u16(src + lane + 64));
}
// The same two elements when the producing linear left its K-slice partials unsummed: sum of the NS slices in slice
// order, rounded to bf16 (what that linear would have stored).  `p` points at slice 0's element l of the row.
template <int NS>
__device__ __forceinline__ void head_row_load_slices(const float *p, size_t slice_stride, int lane, float &x0, float &x1) {
  float a[NS], b[NS];
#pragma unroll
  for (int q = 0; q < NS; q++) {
    a[q] = ldc_f32(p + q * slice_stride + lane);
    b[q] = ldc_f32(p + q * slice_stride + lane + 64);
  }
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int q = 0; q < NS; q++) {
    s0 += a[q];
    s1 += b[q];
  }
  x0 = bfround(s0);
  x1 = bfround(s1);
}
__device__ __forceinline__ void head_row_finish(float x0, float x1, uint16_t *dst, const uint16_t *nw, const uint16_t *cos_row, const uint16_t *sin_row,
                                                int flags, float eps, int lane) {
  if (flags & MK_F_QK_NORM) {
    const float ss = wave_sum(x0 * x0 + x1 * x1);
    const float r = rsqrtf(ss * (1.f / 128.f) + eps);
    x0 = bfround((x0 * r) * bf2f(nw[lane]));
    x1 = bfround((x1 * r) * bf2f(nw[lane + 64]));
  }
  if (flags & MK_F_ROPE) {
    const float cs = bf2f(cos_row[lane]), sn = bf2f(sin_row[lane]);
    const float y0 = x0 * cs - x1 * sn;
    const float y1 = x0 * sn + x1 * cs;
    x0 = y0;
    x1 = y1;
  }
  dst[lane] = (uint16_t)f2bf(x0);
  dst[lane + 64] = (uint16_t)f2bf(x1);
}

#ifndef MK_TUNE_ATTN_TILES
#define MK_TUNE_ATTN_TILES 2
#endif
#ifndef MK_TUNE_NPRE
#define MK_TUNE_NPRE 4
#endif
struct AttnUnit {
  int t, h, cidx, C, start, end, p, p0, t0, new_lo, n_new, cend;
  const int *pages;
};

// GQA decode attention with the q/k-norm, RoPE and KV append fused in front.  Work unit =
// (token, kv head, KV chunk); chunks of one (token, kv head) are adjacent virtual workgroups so a
// kv head stays on one XCD.  Inside a workgroup, sixteen 16-lane groups each walk every 16th
// position of the chunk with their own online-softmax state (fp32 running max / sum, exp2 with
// log2e folded into the scale); each lane owns 8 of the 128 head dims.  Groups are merged through
// LDS, chunks through an HBM workspace by the last workgroup to arrive.
//
// The cached K/V rows of a chunk do not depend on the running iteration (positions below the request's first new
// token were appended by earlier iterations), so the first unit's rows are requested BEFORE the grid barrier of the
// previous stage is awaited, like the weight rows of a linear.  They are read with ordinary loads: every iteration
// starts with a cache invalidate, rows are line-aligned per (position, head), and a row is never read in the
// iteration that writes it (the new positions come from LDS).
// Reference tasks: kv_cache_update_impl (tasks/mi300/kv_cache_update_mi300.cuh:41-327),
// paged_attention_minimal_decode (tasks/mi300/paged_attention_decode_minimal_mi300.cuh:100-371),
// gang_attention_split_kv_kernel (tasks/mi300/gang_attention_mi300.cuh:49-153).
template <int QPK, bool MF>
__device__ __forceinline__ void stage_attn(CStage &st, Ctx &c, const MkRuntime &rt, int M, char *smem) {
  constexpr int D = 128;
  constexpr int NPRE = MK_TUNE_NPRE;          // positions per lane group requested ahead
  constexpr int DPT = QPK * D / MK_THREADS;   // merged outputs per thread (all of one head)
  constexpr int TPH = D / DPT;                // threads per head in the merges
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j16 = lane & 15, gg = wave * 4 + (lane >> 4);
  const int nkv = st.num_kv_heads;
  // LDS: q rows, then the K and V rows of this iteration's new positions (a request ingests up to MK_MAX_NEW_PER_REQ prompt
  // tokens per iteration), then the per-group partial results
  uint16_t *qs = (uint16_t *)smem;                                        // [QPK][128]
  int *sflag = (int *)(smem + 2048);
  uint16_t *knew = (uint16_t *)(smem + 4096);                             // [MK_MAX_NEW_PER_REQ][128]
  uint16_t *vnew = knew + MK_MAX_NEW_PER_REQ * D;                         // [MK_MAX_NEW_PER_REQ][128]
  // MF (iterations of many tokens): the cached positions go through the matrix cores, one wavefront per 16-position
  // tile, and leave four more partial results (one per wavefront) next to the sixteen lane groups'; each wavefront has
  // two private 4 KB buffers for the V tiles it transposes through LDS.  The page list of the running unit aliases the
  // partial-result area (used before the partials are written).
  constexpr int NG = MF ? 20 : 16;
  // A K or V tile in LDS: 16 rows of 256 bytes as four groups of four rows, one direct-to-LDS request per group (each
  // lane 16 bytes: four whole rows, 1 KB contiguous in LDS), the groups GS bytes apart (+64: the transposed V reads of
  // the four groups then fall into different banks).  With four q heads per kv head there is room to stage K this way
  // as well (whole rows per request instead of 64 bytes of each of 16 rows); otherwise K goes to registers.
  constexpr int GS = 1088, TS = 4 * GS;
  constexpr bool KLDS = QPK == 4;
  constexpr int SLOT = KLDS ? 2 * TS : TS;  // bytes per tile in flight
  constexpr int PART_OFF = 4096 + 2 * MK_MAX_NEW_PER_REQ * D * 2, VBUF_OFF = PART_OFF + NG * QPK * 132 * 4;
  float *part = (float *)(smem + PART_OFF);  // [NG][QPK][132]
  int *spg = (int *)(smem + PART_OFF);
  constexpr int RB = QPK == 4 ? MK_TUNE_ATTN_TILES : 2;  // (MF) tiles a wavefront keeps in flight, as LDS allows
  static_assert(VBUF_OFF + (MF ? MK_WAVES * RB * SLOT : 0) <= MK_LDS_BYTES, "attention scratch exceeds the LDS window");
  static_assert(MK_ATTN_MAX_REQ_PAGES * 4 <= NG * QPK * 132 * 4, "page list exceeds the area it aliases");
  const int n_items = M * nkv;
  int cmax = c.G / n_items;
  cmax = cmax < 1 ? 1 : (cmax > MK_ATTN_MAX_CHUNKS ? MK_ATTN_MAX_CHUNKS : cmax);
  const int n_units = n_items * cmax;
  const int ps = rt.page_size;
  const u32x4 *kc = (const u32x4 *)st.k_cache;
  const u32x4 *vc = (const u32x4 *)st.v_cache;

  auto decode = [&](int u, AttnUnit &a) -> bool {
    const int item = u / cmax;
    a.cidx = u - item * cmax;
    a.t = item / nkv;
    a.h = item - a.t * nkv;
    a.p = __builtin_amdgcn_readfirstlane(c.sh_tok[a.t]);
    const int L = a.p + 1;
    a.t0 = __builtin_amdgcn_readfirstlane(c.sh_tok[2 * MK_MAX_TOKENS + a.t]);
    a.p0 = __builtin_amdgcn_readfirstlane(c.sh_tok[a.t0]);
    const int Lc = min(a.p0, L);  // cached positions this token sees
    // Up to 64 cached positions (4 per lane group: one block) per chunk.  While workgroups are plenty, one more chunk
    // takes this iteration's new positions and nothing else: that chunk also prepares their K/V rows and appends the
    // newest one, which would otherwise make it the last to finish.
    const int Cd = (Lc + 63) / 64 + 1;
    const bool own_chunk = L > 64 && Cd <= cmax;
    int C = own_chunk ? Cd : (L + 63) / 64;
    a.C = C > cmax ? cmax : C;
    if (a.cidx >= a.C) return false;
    if (own_chunk) {
      const int nc = a.C - 1;
      a.start = a.cidx < nc ? (int)(((long long)Lc * a.cidx) / nc) : Lc;
      a.end = a.cidx < nc ? (int)(((long long)Lc * (a.cidx + 1)) / nc) : L;
    } else {
      a.start = (int)(((long long)L * a.cidx) / a.C);
      a.end = (int)(((long long)L * (a.cidx + 1)) / a.C);
    }
    a.pages = rt.kv_indices + __builtin_amdgcn_readfirstlane(c.sh_tok[3 * MK_MAX_TOKENS + a.t]);
    a.new_lo = max(a.start, a.p0);  // new positions handled here: [new_lo, end)
    a.n_new = a.end > a.new_lo ? a.end - a.new_lo : 0;
    a.cend = min(a.end, a.p0);      // cached positions handled here: [start, cend)
    return true;
  };
  auto kvoff = [&](const AttnUnit &a, int pos) -> size_t {
    const int pg = pos / ps;
    const size_t row = (size_t)a.pages[pg] * ps + (pos - pg * ps);
    return (row * nkv + a.h) * (D / 8) + j16;
  };

  // ---- before the barrier: the first unit's cached rows
  AttnUnit a0;
  const bool have0 = c.vid < n_units && decode(c.vid, a0);
  u32x4 pk[NPRE], pv[NPRE];
  auto prefetch0 = [&]() {
#pragma unroll
    for (int i = 0; i < NPRE; i++) {
      const int pos = a0.start + gg + 16 * i;
      if (pos < a0.cend) {
        const size_t off = kvoff(a0, pos);
        pk[i] = kc[off];
        pv[i] = vc[off];
      }
    }
  };
  // the polling wavefront keeps its memory queue empty until the barrier is through (its loads would delay the poll
  // results behind them); its rows are requested right after and land while the q rows are being fetched
  if (!MF && have0 && wave != 0) prefetch0();
  barrier_wait(c);
  if (!MF && have0 && wave == 0) prefetch0();
  // the q/k/v rows: stored by the producing linear, or -- when it left its K-slice partials to this stage -- summed here
  const int dS = c.defer_S;
  c.defer_S = 0;
  const float *dpart = c.defer_part;
  const size_t dn = (size_t)c.defer_n, dslice = (size_t)c.defer_rows * dn;
  auto fetch = [&](int tok, int off, float &y0, float &y1) {
    if (dS == 0) {
      head_row_load((const uint16_t *)st.in + (size_t)tok * st.ld_in + off, lane, y0, y1);
    } else {
      const float *pp = dpart + (size_t)tok * dn + off;
      if (dS == 2) head_row_load_slices<2>(pp, dslice, lane, y0, y1);
      else if (dS == 4) head_row_load_slices<4>(pp, dslice, lane, y0, y1);
      else head_row_load_slices<8>(pp, dslice, lane, y0, y1);
    }
  };

  for (int uu = c.vid; uu < n_units; uu += c.G) {
    AttnUnit a;
    const bool first = uu == c.vid;
    // More (token, kv head) pairs than workgroups: every other round deals them in reverse order, so a workgroup that
    // drew a long context in one round draws from the other end of the batch in the next (requests that entered the
    // batch together sit next to each other and are about equally far along).
    int u = uu;
    if (cmax == 1 && ((uu / c.G) & 1)) {
      const int r0 = (uu / c.G) * c.G, rn = min(c.G, n_units - r0);
      u = r0 + rn - 1 - (uu - r0);
    }
    if (first) {
      if (!have0) continue;
      a = a0;
    } else if (!decode(u, a)) {
      continue;
    }
    const int t = a.t, h = a.h, p = a.p, C = a.C;
    __syncthreads();  // LDS reuse across units
    // (MF) this unit's page-table entries: requested here, stored to LDS after the row requests below are out -- an LDS
    // store waits for its load, and loads return in order
    const int pg_lo = a.start / ps;
    const int npg = (MF && a.cend > a.start) ? (a.cend - 1) / ps - pg_lo + 1 : 0;
    const int pg_first = tid < npg ? a.pages[pg_lo + tid] : 0;
    // ---- phase A: prepare q heads and the new K/V rows of this chunk, two rows per wavefront in flight
    const int n_rows = QPK + a.n_new;
    for (int row0 = wave; row0 < n_rows; row0 += 2 * MK_WAVES) {
      float x0[2], x1[2], v0[2], v1[2];
      int tok[2], off[2];
#pragma unroll
      for (int r = 0; r < 2; r++) {
        const int row = row0 + r * MK_WAVES;
        if (row < n_rows) {
          const bool isq = row < QPK;
          tok[r] = isq ? t : a.t0 + (a.new_lo + (row - QPK) - a.p0);
          off[r] = h * (QPK + 2) * D + (isq ? row : QPK) * D;
          fetch(tok[r], off[r], x0[r], x1[r]);
          if (!isq) fetch(tok[r], off[r] + D, v0[r], v1[r]);  // (a V row is copied as it is)
        }
      }
      if (MF && row0 == wave) {
        if (tid < npg) spg[tid] = pg_first;
        for (int i = tid + MK_THREADS; i < npg; i += MK_THREADS) spg[i] = a.pages[pg_lo + i];
      }
#pragma unroll
      for (int r = 0; r < 2; r++) {
        const int row = row0 + r * MK_WAVES;
        if (row < n_rows) {
          const bool isq = row < QPK;
          const int pos = isq ? p : a.new_lo + (row - QPK);
          if (!isq) {
            vnew[(row - QPK) * D + lane] = (uint16_t)f2bf(v0[r]);
            vnew[(row - QPK) * D + lane + 64] = (uint16_t)f2bf(v1[r]);
          }
          if (dS && a.cidx == C - 1 && tok[r] == t) {
            // the producing linear left these rows unsummed: the chunk that owns the token's newest position also
            // stores the token's own q/k/v rows where that linear would have
            uint16_t *dst = (uint16_t *)st.in + (size_t)t * st.ld_in + off[r];
            dst[lane] = (uint16_t)f2bf(x0[r]);
            dst[lane + 64] = (uint16_t)f2bf(x1[r]);
            if (!isq) {
              dst[D + lane] = (uint16_t)f2bf(v0[r]);
              dst[D + lane + 64] = (uint16_t)f2bf(v1[r]);
            }
          }
          head_row_finish(x0[r], x1[r], isq ? qs + row * D : knew + (row - QPK) * D, (const uint16_t *)(isq ? st.q_norm_w : st.k_norm_w),
                          (const uint16_t *)st.cos_tab + (size_t)pos * st.ld_cos, (const uint16_t *)st.sin_tab + (size_t)pos * st.ld_cos, st.flags, st.eps,
                          lane);
        }
      }
    }
    __syncthreads();
    // the chunk that owns the newest position appends this token's K/V and publishes q (MF: after the tile loop, whose
    // request counting must not see other vector-memory traffic)
    auto append = [&]() {
      if (a.cidx != C - 1) return;
      const int j = p - a.new_lo;
      const size_t rowi = (size_t)a.pages[p / ps] * ps + (p % ps);
      uint32_t *kd = (uint32_t *)st.k_cache + (rowi * nkv + h) * (D / 2);
      uint32_t *vd = (uint32_t *)st.v_cache + (rowi * nkv + h) * (D / 2);
      if (tid < 64) kd[tid] = ((const uint32_t *)(knew + j * D))[tid];
      else if (tid < 128) vd[tid - 64] = ((const uint32_t *)(vnew + j * D))[tid - 64];
      if (st.q_ws) {
        uint32_t *qd = (uint32_t *)st.q_ws + ((size_t)t * st.ld_qws + (size_t)h * QPK * D) / 2;
        for (int i = tid; i < QPK * D / 2; i += MK_THREADS) qd[i] = ((const uint32_t *)qs)[i];
      }
    };
    if (!MF) append();
    MK_MARK(c, first ? 0 : 2);
    // ---- phase B: online softmax over the chunk
    u32x4 qv[QPK];
#pragma unroll
    for (int hh = 0; hh < QPK; hh++) qv[hh] = ((const u32x4 *)qs)[hh * 16 + j16];
    float m[QPK], l[QPK], acc[QPK][8];
#pragma unroll
    for (int hh = 0; hh < QPK; hh++) {
      m[hh] = -INFINITY;
      l[hh] = 0.f;
#pragma unroll
      for (int d = 0; d < 8; d++) acc[hh][d] = 0.f;
    }
    auto process = [&](const u32x4 kv, const u32x4 vv) {
      float v[8] = {bf_lo(vv.x), bf_hi(vv.x), bf_lo(vv.y), bf_hi(vv.y), bf_lo(vv.z), bf_hi(vv.z), bf_lo(vv.w), bf_hi(vv.w)};
#pragma unroll
      for (int hh = 0; hh < QPK; hh++) {
        float s = group16_sum(dot8(kv, qv[hh], 0.f)) * st.sm_scale_log2;
        const float mn = fmaxf(m[hh], s);
        const float alpha = __builtin_amdgcn_exp2f(m[hh] - mn);
        const float pr = __builtin_amdgcn_exp2f(s - mn);
        l[hh] = l[hh] * alpha + pr;
#pragma unroll
        for (int d = 0; d < 8; d++) acc[hh][d] = acc[hh][d] * alpha + pr * v[d];
        m[hh] = mn;
      }
    };
    // NPRE positions at a time: all scores first (independent reductions), then ONE rescale of the running state.
    // Entries at or beyond cend hold whatever the registers held; their scores are forced to -inf (weight 0).
    auto process_block = [&](const u32x4 (&kk)[NPRE], const u32x4 (&vv)[NPRE], int pos0) {
      float sc[NPRE][QPK];  // scores, then softmax weights
#pragma unroll
      for (int i = 0; i < NPRE; i++) {
        const bool ok = pos0 + 16 * i < a.cend;
#pragma unroll
        for (int hh = 0; hh < QPK; hh++) {
          const float d = group16_sum(dot8(kk[i], qv[hh], 0.f)) * st.sm_scale_log2;
          sc[i][hh] = ok ? d : -INFINITY;
        }
      }
#pragma unroll
      for (int hh = 0; hh < QPK; hh++) {
        float mn = m[hh];
#pragma unroll
        for (int i = 0; i < NPRE; i++) mn = fmaxf(mn, sc[i][hh]);
        const float alpha = __builtin_amdgcn_exp2f(m[hh] - mn);
        float ps_ = 0.f;
#pragma unroll
        for (int i = 0; i < NPRE; i++) {
          sc[i][hh] = __builtin_amdgcn_exp2f(sc[i][hh] - mn);
          ps_ += sc[i][hh];
        }
        l[hh] = l[hh] * alpha + ps_;
        m[hh] = mn;
#pragma unroll
        for (int d = 0; d < 8; d++) acc[hh][d] *= alpha;
      }
#pragma unroll
      for (int i = 0; i < NPRE; i++) {
        const bool ok = pos0 + 16 * i < a.cend;
        const u32x4 w = vv[i];
        float v[8] = {bf_lo(w.x), bf_hi(w.x), bf_lo(w.y), bf_hi(w.y), bf_lo(w.z), bf_hi(w.z), bf_lo(w.w), bf_hi(w.w)};
#pragma unroll
        for (int d = 0; d < 8; d++) v[d] = ok ? v[d] : 0.f;  // 0 * NaN from an unloaded register would poison the sum
#pragma unroll
        for (int hh = 0; hh < QPK; hh++) {
#pragma unroll
          for (int d = 0; d < 8; d++) acc[hh][d] += sc[i][hh] * v[d];
        }
      }
    };
    if constexpr (MF) {
      // ---- cached positions on the matrix cores.  Tile = 16 positions, one wavefront per tile.  Scores: A = the K tile
      // (lane (i, g): row of position i; step s contracts dims 32 s + 8 g ..; read from the K tile in LDS, or -- eight q
      // heads per kv head -- requested straight into registers, 64 bytes of each of 16 rows per request), B = q (lane
      // (j, g): head j, same dims; heads past QPK are zero) -> lane (j, g) holds the scores of head j at
      // positions 4 g .. 4 g + 3.  Those four weights, as bf16 (value and rounding remainder: two operands), are already
      // the A operand of a 16x16x16 step over positions; its B operand -- four consecutive positions of one dim --
      // is read out of the V tile that direct-to-LDS loads put into this wavefront's buffer.  The running maximum is
      // kept per head for the whole wavefront (the products of a step are summed across its lanes, so they must share
      // their reference), the running sum per lane.
      typedef short s16x4 __attribute__((ext_vector_type(4)));
      const int lr = lane & 15, lg = lane >> 4;
      char *vb0 = smem + VBUF_OFF + wave * (RB * SLOT);
      bf16x8 qb[4];
#pragma unroll
      for (int s_ = 0; s_ < 4; s_++) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        qb[s_] = __builtin_bit_cast(bf16x8, lr < QPK ? *(const u32x4 *)(qs + lr * D + s_ * 32 + lg * 8) : z);
      }
      f32x4 o[8];
#pragma unroll
      for (int dt = 0; dt < 8; dt++) o[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
      float mrun = -INFINITY, lsum = 0.f;
      const int nt = a.cend > a.start ? (a.cend - a.start + 15) >> 4 : 0;
      auto row_base = [&](int pos) -> size_t {  // first 16-byte operand of the (position, head) row
        const int pc = min(pos, a.cend - 1), pg = pc / ps;
        return (((size_t)spg[pg - pg_lo] * ps + (pc - pg * ps)) * nkv + h) * (D / 8);
      };
      auto load_tile = [&](int tt, bf16x8 (&kk)[4], char *vbuf) {
        const int p0 = a.start + min(tt, nt - 1) * 16;
        if (!KLDS) {  // K to registers: lane (row, g), request s reads bytes 64 s + 16 g of its row
          const size_t base = row_base(p0 + lr) + lg;
#pragma unroll
          for (int s_ = 0; s_ < 4; s_++) kk[s_] = __builtin_nontemporal_load((const bf16x8 *)(kc + base + s_ * 4));
        }
        // to LDS: request s brings rows 4 s .. 4 s + 3 whole (lane (row in group, 16-byte piece))
        // (streaming requests -- the cache-policy bit the nontemporal loads of the other paths carry: a cached K/V row is
        // read once per iteration and need not displace the activations the linears share through the L2)
        constexpr int KV_NT = 2;
        size_t gb[4];
#pragma unroll
        for (int s_ = 0; s_ < 4; s_++) gb[s_] = row_base(p0 + 4 * s_ + lg) + lr;
        if (KLDS) {
#pragma unroll
          for (int s_ = 0; s_ < 4; s_++)
            __builtin_amdgcn_global_load_lds((const MK_GLOBAL void *)(unsigned long long)(kc + gb[s_]),
                                             (__attribute__((address_space(3))) void *)(__attribute__((address_space(3))) char *)(vbuf + TS + s_ * GS), 16, 0, KV_NT);
        }
#pragma unroll
        for (int s_ = 0; s_ < 4; s_++)
          __builtin_amdgcn_global_load_lds((const MK_GLOBAL void *)(unsigned long long)(vc + gb[s_]),
                                           (__attribute__((address_space(3))) void *)(__attribute__((address_space(3))) char *)(vbuf + s_ * GS), 16, 0, KV_NT);
      };
      const int vlane = lg * GS + lr * 2;
      const int klane = (lr >> 2) * GS + (lr & 3) * 256 + lg * 16;
      auto compute_tile = [&](int t_, const bf16x8 (&kk)[4], const char *vbuf) {
        f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s_ = 0; s_ < 4; s_++) {
          const bf16x8 ko = KLDS ? __builtin_bit_cast(bf16x8, *(const u32x4 *)(vbuf + TS + klane + s_ * 64)) : kk[s_];
          s4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ko, qb[s_], s4, 0, 0, 0);
        }
        const int pbase = a.start + t_ * 16 + lg * 4;
        float sc[4];
#pragma unroll
        for (int r = 0; r < 4; r++) sc[r] = pbase + r < a.cend ? s4[r] * st.sm_scale_log2 : -INFINITY;
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, mx))));
        mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, mx))));
        const float mn = fmaxf(mrun, mx);
        const float alpha = __builtin_amdgcn_exp2f(mrun - mn);
        float pw[4];
#pragma unroll
        for (int r = 0; r < 4; r++) pw[r] = __builtin_amdgcn_exp2f(sc[r] - mn);
        lsum = lsum * alpha + ((pw[0] + pw[1]) + (pw[2] + pw[3]));
        mrun = mn;
        if (__ballot(lr < QPK && alpha != 1.f)) {  // (uniform) some head's maximum moved: rescale what has been summed
          float ar[4];
#pragma unroll
          for (int r = 0; r < 4; r++) ar[r] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lg * 4 + r) << 2, __builtin_bit_cast(int, alpha)));
#pragma unroll
          for (int dt = 0; dt < 8; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++) o[dt][r] *= ar[r];
        }
        float ph[4];
#pragma unroll
        for (int r = 0; r < 4; r++) ph[r] = bfround(pw[r]);
        const unsigned h01 = pack2(ph[0], ph[1]), h23 = pack2(ph[2], ph[3]);
        const unsigned l01 = pack2(pw[0] - ph[0], pw[1] - ph[1]), l23 = pack2(pw[2] - ph[2], pw[3] - ph[3]);
        const s16x4 a_hi = __builtin_bit_cast(s16x4, (unsigned long long)h01 | ((unsigned long long)h23 << 32));
        const s16x4 a_lo = __builtin_bit_cast(s16x4, (unsigned long long)l01 | ((unsigned long long)l23 << 32));
        const char *vb = vbuf + vlane;
#pragma unroll
        for (int dt = 0; dt < 8; dt++) {
          const char *q_ = vb + dt * 32;
          const unsigned v0 = *(const uint16_t *)(q_), v1 = *(const uint16_t *)(q_ + 256), v2 = *(const uint16_t *)(q_ + 512), v3 = *(const uint16_t *)(q_ + 768);
          const s16x4 bv = __builtin_bit_cast(s16x4, (unsigned long long)(v0 | (v1 << 16)) | ((unsigned long long)(v2 | (v3 << 16)) << 32));
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_hi, bv, o[dt], 0, 0, 0);
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_lo, bv, o[dt], 0, 0, 0);
        }
      };
      // RB tiles in flight per wavefront: every request is issued unconditionally (a tile index past the end re-reads the
      // last tile; it is never computed), and the wait before a tile counts the 8 (RB - 1) requests of the tiles after it
      int t_ = wave;
      if (t_ < nt) {
        bf16x8 kr[RB][4];
#pragma unroll
        for (int b_ = 0; b_ < RB - 1; b_++) load_tile(t_ + b_ * MK_WAVES, kr[b_], vb0 + b_ * SLOT);
        bool more = true;
        while (more) {
#pragma unroll
          for (int b_ = 0; b_ < RB; b_++) {
            // slot (b_ + RB - 1) % RB was computed in the previous round: refill it with the tile RB - 1 ahead
            load_tile(t_ + (RB - 1) * MK_WAVES, kr[(b_ + RB - 1) % RB], vb0 + ((b_ + RB - 1) % RB) * SLOT);
            if (RB == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else if (RB == 3) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
            if (more) {
              compute_tile(t_, kr[b_], vb0 + b_ * SLOT);
              t_ += MK_WAVES;
              more = t_ < nt;
            }
          }
        }
      }
      MK_MARK(c, first ? 1 : 3);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the direct-to-LDS requests of the tile that was not computed)
      append();
      __syncthreads();  // every wavefront is done with the page list: the partial results may overwrite it
      float lt = lsum;
      lt += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) << 2, __builtin_bit_cast(int, lt)));
      lt += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, lt)));
      const int gm = 16 + wave;
      if (lg == 0 && lr < QPK) {
        part[(gm * QPK + lr) * 132 + 128] = mrun;
        part[(gm * QPK + lr) * 132 + 129] = lt;
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int head = lg * 4 + r;
        if (head < QPK) {
#pragma unroll
          for (int dt = 0; dt < 8; dt++) part[(gm * QPK + head) * 132 + dt * 16 + lr] = o[dt][r];
        }
      }
    } else {
    int pos = a.start + gg;
    if (first) {
      if (pos < a.cend) process_block(pk, pv, pos);
      pos += 16 * NPRE;
    }
    // later blocks: the next block's rows are in flight while the current one is reduced
    // Every load is issued unconditionally (positions beyond the chunk re-read its last row and are masked in
    // process_block): a load under a branch would turn the wait for the current block into a wait for the next one too.
    auto load_block = [&](int p0, u32x4 (&kk)[NPRE], u32x4 (&vv)[NPRE]) {
#pragma unroll
      for (int i = 0; i < NPRE; i++) {
        const size_t off = kvoff(a, min(p0 + 16 * i, a.cend - 1));
        kk[i] = kc[off];
        vv[i] = vc[off];
      }
    };
    if (pos < a.cend) {
      u32x4 ka[NPRE], va[NPRE], kb[NPRE], vb[NPRE];
      load_block(pos, ka, va);
      while (true) {
        load_block(pos + 16 * NPRE, kb, vb);
        process_block(ka, va, pos);
        pos += 16 * NPRE;
        if (pos >= a.cend) break;
        load_block(pos + 16 * NPRE, ka, va);
        process_block(kb, vb, pos);
        pos += 16 * NPRE;
        if (pos >= a.cend) break;
      }
    }
    }
    for (int j = gg; j < a.n_new; j += 16) process(((const u32x4 *)(knew + j * D))[j16], ((const u32x4 *)(vnew + j * D))[j16]);
    // ---- phase C: merge the 16 groups through LDS
#pragma unroll
    for (int hh = 0; hh < QPK; hh++) {
      float *pp = part + (gg * QPK + hh) * 132;
#pragma unroll
      for (int d = 0; d < 8; d++) pp[j16 * 8 + d] = acc[hh][d];
      if (j16 == 0) {
        pp[128] = m[hh];
        pp[129] = l[hh];
      }
    }
    __syncthreads();
    // When every chunk of this (token, kv head) runs on one die, the partials and the arrival counter never leave that
    // die's L2: workgroup-scope atomic, ordinary stores and loads (each stage has its own partial buffer and the L1 is
    // invalidated once per iteration, so a partial is never read from a stale line).  Otherwise device scope.
    const int item = u / cmax;
    // (a launch whose attention stages all share one partial buffer -- rt.attn_part -- always takes the device-scope
    // path: a buffer that is rewritten several times per iteration must not be read through lines an earlier stage left
    // in the L1)
    const bool local = !rt.attn_part && c.even_xcds && (item * cmax) / c.quota == (item * cmax + C - 1) / c.quota;
    float *part_base = rt.attn_part ? rt.attn_part : (float *)st.aux0;
    float *gpart = part_base + (size_t)u * QPK * MK_ATTN_PSTRIDE;
    uint16_t *orow = (uint16_t *)st.out + (size_t)t * st.ld_out + (size_t)h * QPK * D;
    const int mh = tid / TPH, md = (tid - mh * TPH) * DPT;  // this thread merges dims [md, md+DPT) of head mh
    {
      float mx = -INFINITY;
#pragma unroll
      for (int g = 0; g < NG; g++) mx = fmaxf(mx, part[(g * QPK + mh) * 132 + 128]);
      float ls = 0.f, os[DPT];
#pragma unroll
      for (int d = 0; d < DPT; d++) os[d] = 0.f;
#pragma unroll
      for (int g = 0; g < NG; g++) {
        const float *pp = part + (g * QPK + mh) * 132;
        const float wgt = __builtin_amdgcn_exp2f(pp[128] - mx);
        ls += pp[129] * wgt;
#pragma unroll
        for (int d = 0; d < DPT; d++) os[d] += pp[md + d] * wgt;
      }
      if (C == 1) {
#pragma unroll
        for (int d = 0; d < DPT; d += 2)  // written through: the stage's barrier skips the L2 write-back
          __hip_atomic_store((uint32_t *)(orow + mh * D + md + d), pack2(os[d] / ls, os[d + 1] / ls), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        // 8-byte stores that together cover whole 128-byte lines (the running max and sum fill a line of their own, 16
        // copies), so that the merging workgroup never reads a line that is only partly valid in the L2
#pragma unroll
        for (int d = 0; d < DPT; d += 2) *(float2 *)(gpart + mh * MK_ATTN_PSTRIDE + md + d) = make_float2(os[d], os[d + 1]);
        if (md < 16 * DPT) *(float2 *)(gpart + mh * MK_ATTN_PSTRIDE + D + 2 * (md / DPT)) = make_float2(mx, ls);
      }
    }
    if (C > 1) {
      // ---- phase D: the last chunk to finish merges all chunks of this (token, kv head)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0) {
        int last;
        if (local) {
          unsigned *cnt = (unsigned *)st.aux1 + (size_t)item * 32;
          last = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP) == (unsigned)(C - 1);
          if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
          unsigned *cnt = &rt.attn_cnt[(size_t)item * 32];
          last = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(C - 1);
          if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        *sflag = last;
      }
      __syncthreads();
      if (*sflag) {
        // every chunk partial is read with independent loads (8 bytes each), sixteen chunks in flight per thread
        const float *ip = part_base + (size_t)item * cmax * QPK * MK_ATTN_PSTRIDE;
        float mx = -INFINITY, ls = 0.f, os[DPT];
#pragma unroll
        for (int d = 0; d < DPT; d++) os[d] = 0.f;
        auto merge16 = [&](int c0, auto load8) {
          float2 ml[16], ov[16][DPT / 2];
#pragma unroll
          for (int j = 0; j < 16; j++) {
            if (c0 + j < C) {
              const float *pp = ip + ((size_t)(c0 + j) * QPK + mh) * MK_ATTN_PSTRIDE;
              ml[j] = load8(pp + D);
#pragma unroll
              for (int d = 0; d < DPT / 2; d++) ov[j][d] = load8(pp + md + 2 * d);
            }
          }
#pragma unroll
          for (int j = 0; j < 16; j++)
            if (c0 + j < C) {
              const float mn = fmaxf(mx, ml[j].x);
              const float sa = __builtin_amdgcn_exp2f(mx - mn), sb = __builtin_amdgcn_exp2f(ml[j].x - mn);
              ls = ls * sa + ml[j].y * sb;
#pragma unroll
              for (int d = 0; d < DPT / 2; d++) {
                os[2 * d] = os[2 * d] * sa + ov[j][d].x * sb;
                os[2 * d + 1] = os[2 * d + 1] * sa + ov[j][d].y * sb;
              }
              mx = mn;
            }
        };
        if (local) {
          for (int c0 = 0; c0 < C; c0 += 16) merge16(c0, [](const float *q) { return *(const float2 *)q; });
        } else {
          for (int c0 = 0; c0 < C; c0 += 16)
            merge16(c0, [](const float *q) {
              const unsigned long long u = ldc_u64(q);
              return make_float2(__uint_as_float((uint32_t)u), __uint_as_float((uint32_t)(u >> 32)));
            });
        }
#pragma unroll
        for (int d = 0; d < DPT; d += 2)  // written through: the stage's barrier skips the L2 write-back
          __hip_atomic_store((uint32_t *)(orow + mh * D + md + d), pack2(os[d] / ls, os[d + 1] / ls), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  // The attention outputs went through to memory.  The appended K/V rows and the published q rows stay in this die's
  // L2 until a later barrier of this iteration writes it back (the sampling stages and the scheduler step always do);
  // nothing reads them before the next iteration.
  c.wrote_through = true;
}

// Greedy sampling, stage 1: every workgroup scans a contiguous slice of each token's logits and keeps
// (max, lowest index attaining it).  Reference task: tasks/mi300/argmax_mi300.cuh:78-127.
__device__ __forceinline__ void stage_argmax_partial(CStage &st, Ctx &c, const MkRuntime &rt, int M, char *smem) {
  barrier_wait(c);
  const int n = st.n;
  int per = (n + c.G - 1) / c.G;
  per = (per + 1) & ~1;  // even, so slices start on a dword
  const int c0 = c.vid * per, c1 = min(n, c0 + per);
  float *pv = rt.argmax_pv ? rt.argmax_pv : (float *)st.aux0;
  int *pi = rt.argmax_pv ? rt.argmax_pi : (int *)st.aux1;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int NDW = 5, TB = 4;  // dwords per lane per token, tokens in flight per wavefront
  const int nd = (c1 - c0 + 1) / 2;
  // one wavefront per token, TB tokens' slices requested together; slices longer than NDW * 64 dwords loop
  for (int t0 = wave * TB; t0 < M; t0 += MK_WAVES * TB) {
    uint32_t w[TB][NDW];
#pragma unroll
    for (int k = 0; k < TB; k++)
#pragma unroll
      for (int j = 0; j < NDW; j++)
        if (t0 + k < M && j * 64 + lane < nd) w[k][j] = ldc_u32((const uint16_t *)st.in + (size_t)(t0 + k) * st.ld_in + c0 + 2 * (j * 64 + lane));
#pragma unroll
    for (int k = 0; k < TB; k++) {
      if (t0 + k >= M) break;
      const uint16_t *row = (const uint16_t *)st.in + (size_t)(t0 + k) * st.ld_in;
      float best = -INFINITY;
      int bi = 0x7fffffff;
      auto consider = [&](uint32_t u, int i) {
        const float v0 = bf_lo(u), v1 = bf_hi(u);
        if (v0 > best) {
          best = v0;
          bi = i;
        }
        if (i + 1 < c1 && v1 > best) {
          best = v1;
          bi = i + 1;
        }
      };
#pragma unroll
      for (int j = 0; j < NDW; j++)
        if (j * 64 + lane < nd) consider(w[k][j], c0 + 2 * (j * 64 + lane));
      for (int d = NDW * 64 + lane; d < nd; d += 64) consider(ldc_u32(row + c0 + 2 * d), c0 + 2 * d);
      wave_argmax(best, bi);
      if (lane == 0) {
        pv[(t0 + k) * c.G + c.vid] = best;
        pi[(t0 + k) * c.G + c.vid] = bi;
      }
    }
  }
}

// Greedy sampling, stage 2: one wavefront per token reduces the per-workgroup partials.
// Reference task: tasks/mi300/argmax_mi300.cuh:129-158.
__device__ __forceinline__ void stage_argmax_reduce(CStage &st, Ctx &c, const MkRuntime &rt, int M) {
  barrier_wait(c);
  const float *pv = rt.argmax_pv ? rt.argmax_pv : (const float *)st.aux0;
  const int *pi = rt.argmax_pv ? rt.argmax_pi : (const int *)st.aux1;
  long long *out = (long long *)st.out;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int t = c.vid * MK_WAVES + wave; t < M; t += c.G * MK_WAVES) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < c.G; i += 64) {
      const float v = ldc_f32(&pv[t * c.G + i]);
      const int ix = ldc_i32(&pi[t * c.G + i]);
      if (v > best || (v == best && ix < bi)) {
        best = v;
        bi = ix;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) {
        best = ov;
        bi = oi;
      }
    }
    if (lane == 0) out[t] = (long long)bi;
  }
}

// ----------------------------------------------------------------------------- the kernel
// One pass over the stage program for the M tokens of this iteration.
// ----------------------------------------------------------------------------- prompt-lookup speculative decoding
// A decoding request of a speculating graph brings n = 1 + (up to spec_len) rows into an iteration (the scheduler sizes
// the group): row 0 is its newest token at position s, rows 1.. are guesses -- the tokens that followed the EARLIEST
// earlier occurrence of its last N tokens (reference tasks find_ngram_partial_kernel / find_ngram_global_kernel,
// tasks/speculative_decoding/prompt_lookup.cuh:22-140, called with input_token_num = step + 1 and step,
// src/kernel/task_register.cc:1713-1752).  All rows run through the model as a chunk of the same request (causal
// attention inside the chunk, K/V appended at s .. s + n - 1); the verify stage then keeps the sampled token of row 0
// and one more for every guess in front that the model agrees with (target_verify_greedy_kernel,
// tasks/speculative_decoding/target_verify.cuh:21-62), and the next scheduler step advances the request by that many
// positions.  K/V rows of rejected guesses are rewritten before anything reads them.  These three stages are plain
// integer work on a few kilobytes; they are kept out of line so that the stage loop's register allocation does not see
// them.
//
// The search space of a request with T = s + 1 known tokens is idx in [0, T - N); position idx belongs to task
// (idx / 128) % P, as in the reference (128 threads per task, P tasks round-robin).  A match compares the real tokens
// idx .. idx + N - 1; the reference compares against a shared-memory window whose last N - 1 entries it leaves unset
// when they lie at or beyond T - N (prompt_lookup.cuh:62-72), so for the few idx > T - 2 N it reads unset memory.
__device__ __attribute__((noinline)) void mk_ngram_partial(int stage, const MkRuntime *rtp, int vid, int G, int *lds) {
  const MkStage *stp = rtp->stages + stage;
  const int P = stp->n, N = stp->k, ld = stp->ld_out;
  long long *part = (long long *)stp->out;
  const int R = rtp->max_requests, tid = threadIdx.x;
  for (int u = vid; u < R * P; u += G) {
    const int slot = u / P, k = u - slot * P;
    const int q0 = ldc_i32(&rtp->qo_indptr[slot]), n = ldc_i32(&rtp->qo_indptr[slot + 1]) - q0;
    const int req = ldc_i32(&rtp->request_ids[slot]);
    __syncthreads();
    if (tid == 0) lds[0] = 0x7fffffff;
    __syncthreads();
    if (req >= 0 && n > 1) {
      const int s = ldc_i32(&rtp->tok_pos[q0]);
      if (s >= rtp->prompt_lengths[req]) {  // decoding
        const long long *tok = rtp->tokens + (long long)req * rtp->max_seq;
        const int T = s + 1, total = T - N;
        for (int it = tid >> 7;; it += 2) {  // the reference's 128-thread block, two of its rounds at a time
          const long long base = ((long long)it * P + k) * 128;
          if (base >= total) break;
          const int idx = (int)base + (tid & 127);
          if (idx < total) {
            bool eq = true;
            for (int i = 0; i < N; i++) eq = eq && ldc_u64(&tok[idx + i]) == ldc_u64(&tok[T - N + i]);
            if (eq) {
              atomicMin(&lds[0], idx);
              break;  // this thread's later rounds only hold larger positions
            }
          }
        }
      }
    }
    __syncthreads();
    if (tid == 0) {
      const int m = lds[0];
      stc_u64(part + (size_t)slot * ld + k, m == 0x7fffffff ? 0x7fffffffffffffffull : (unsigned long long)m);
    }
  }
}

__device__ __attribute__((noinline)) void mk_ngram_global(int stage, const MkRuntime *rtp, int vid, int G, int *lds) {
  const MkStage *stp = rtp->stages + stage;
  const int P = stp->n, N = stp->k, ld = stp->ld_in;
  const long long *part = (const long long *)stp->in;
  long long *spec = (long long *)stp->out;
  const int R = rtp->max_requests, tid = threadIdx.x;
  for (int slot = vid; slot < R; slot += G) {
    const int q0 = ldc_i32(&rtp->qo_indptr[slot]), n = ldc_i32(&rtp->qo_indptr[slot + 1]) - q0;
    const int req = ldc_i32(&rtp->request_ids[slot]);
    if (req < 0 || n <= 0) continue;  // (uniform)
    const int s = ldc_i32(&rtp->tok_pos[q0]);
    const bool guess = n > 1 && s >= rtp->prompt_lengths[req];
    __syncthreads();
    if (tid == 0) lds[0] = 0x7fffffff;
    __syncthreads();
    if (guess) {
      for (int k = tid; k < P; k += MK_THREADS) {
        const unsigned long long v = ldc_u64(part + (size_t)slot * ld + k);
        if (v < 0x7fffffffull) atomicMin(&lds[0], (int)v);
      }
    }
    __syncthreads();
    const int first = lds[0];
    const long long *tok = rtp->tokens + (long long)req * rtp->max_seq;
    for (int j = tid; j < n; j += MK_THREADS) {
      long long v;
      if (!guess || j == 0) {
        v = (long long)ldc_u64(&rtp->input_tokens[q0 + j]);  // the scheduler's token (prompt chunk, or the newest token)
      } else {
        const long long ci = (long long)first + N + (j - 1);
        v = (first != 0x7fffffff && ci <= s) ? (long long)ldc_u64(&tok[ci]) : -1;
      }
      stc_u64(spec + q0 + j, (unsigned long long)v);
    }
  }
}

__device__ __attribute__((noinline)) void mk_verify_greedy(int stage, const MkRuntime *rtp, int vid, int G) {
  const MkStage *stp = rtp->stages + stage;
  const long long *spec = (const long long *)stp->in, *target = (const long long *)stp->aux0;
  const int R = rtp->max_requests;
  for (int slot = vid * MK_THREADS + threadIdx.x; slot < R; slot += G * MK_THREADS) {
    const int q0 = ldc_i32(&rtp->qo_indptr[slot]), n = ldc_i32(&rtp->qo_indptr[slot + 1]) - q0;
    const int req = ldc_i32(&rtp->request_ids[slot]);
    if (req < 0 || n <= 0) continue;
    int nc = n;
    if (ldc_i32(&rtp->tok_pos[q0]) >= rtp->prompt_lengths[req]) {
      // token j of this iteration is what the model sampled on row j; it counts while every guess before it was right
      // (guess j + 1 is the input of row j + 1) and nothing before it ended the request
      nc = 1;
      for (int j = 0; j + 1 < n; j++) {
        const long long tj = (long long)ldc_u64(&target[q0 + j]);
        if (tj == rtp->eos_token_id || (long long)ldc_u64(&spec[q0 + j + 1]) != tj) break;
        nc = j + 2;
      }
    }
    stc_i32(&rtp->num_new_tokens[req], nc);
    if (slot == 0 && stp->out) stc_u64(stp->out, (unsigned long long)nc);
  }
}

template <int MAXM>
__device__ __forceinline__ void run_stage_program(const MkRuntime &rt, const MkRuntime *rtp, Ctx &c, const int M, char *smem) {
    for (int s = 0; s < rt.num_stages && !c.dead; s++) {
      CStage &st = ((CStage *)(unsigned long long)rt.stages)[s];
      const int op = st.op, flags = st.flags;
      // (a handle that holds only the matrix-core copies of its weights runs every linear in a matrix-core form, which
      // reads normalised rows from the NORM stage's output: that stage then runs for one and two tokens as well)
      const bool packed_only = MAXM > 1 && rt.packed_only;
      if ((flags & MK_F_ONLY_MULTI) && M == 1 && !(packed_only && op == MK_OP_NORM)) continue;
      if ((flags & MK_F_ONLY_MULTI) && op == MK_OP_NORM && s + 1 < rt.num_stages && !packed_only) {
        // the few-token linear normalises its rows itself
        CStage &nx = ((CStage *)(unsigned long long)rt.stages)[s + 1];
        if (nx.op == MK_OP_LINEAR && (nx.flags & MK_F_NORM) && nx.in == st.in && linear_small_ok(nx, c, M)) continue;
      }
      const long long t_in = (long long)wall_clock64();
      switch (op) {
        case MK_OP_EMBED: stage_embed(st, c, rt, M); break;
        case MK_OP_NORM: stage_norm(st, c, M, smem); break;
        case MK_OP_LINEAR:
          if constexpr (MAXM == 1) stage_linear_m1<true>(st, c, smem);
          else if (M == 1 && !(packed_only && st.wpack)) stage_linear_m1<false>(st, c, smem);
          else if (linear_small_ok(st, c, M) && !(packed_only && st.wpack)) {
            if (M <= 2) stage_linear_small_dispatch<2>(st, c, M, smem);
            else if (M <= 4) stage_linear_small_dispatch<4>(st, c, M, smem);
            else stage_linear_small_dispatch<8>(st, c, M, smem);
          } else {
            const int wt = (((flags & MK_F_SILU) ? st.n / 2 : st.n) + 15) / 16;  // output tiles of the stage
            const bool narrow = ((wt + c.G - 1) / c.G) * ((flags & MK_F_SILU) ? 2 : 1) <= 2;
            const TilePlan plan = linear_tiles_plan(st, c);
            const XresPlan xp = linear_xres_plan(st, c);
            if (xp.S >= 1 && (M > MK_TUNE_SMALL_MAX || packed_only)) {
              if (M <= 32) {
                if (xp.tpu <= 4) stage_linear_mfma_xres<2, 2>(st, c, rt, M, xp, smem);
                else stage_linear_mfma_xres<2, 3>(st, c, rt, M, xp, smem);
              } else {
                if (xp.tpu <= 4) stage_linear_mfma_xres<4, 2>(st, c, rt, M, xp, smem);
                else stage_linear_mfma_xres<4, 3>(st, c, rt, M, xp, smem);
              }
            } else if (plan.S >= 1 && !(packed_only && st.wpack)) {  // (this form reads the row-major weights)
              if (M <= 16) stage_linear_mfma_tiles<1>(st, c, rt, M, plan, smem);
              else if (M <= 32) stage_linear_mfma_tiles<2>(st, c, rt, M, plan, smem);
              else if (M <= 48) stage_linear_mfma_tiles<3>(st, c, rt, M, plan, smem);
              else stage_linear_mfma_tiles<4>(st, c, rt, M, plan, smem);
            } else if (narrow) {
              if (M <= 16) stage_linear_mfma<1, 2, 2 * MK_TUNE_NBN>(st, c, M, smem);
              else if (M <= 32) stage_linear_mfma<2, 2, MK_TUNE_NBN + MK_TUNE_NBN / 2>(st, c, M, smem);
              else if (M <= 48) stage_linear_mfma<3, 2, MK_TUNE_NBN>(st, c, M, smem);
              else stage_linear_mfma<4, 2, MK_TUNE_NBN>(st, c, M, smem);
            } else {
              if (M <= 16) stage_linear_mfma<1, 6, 2>(st, c, M, smem);
              else if (M <= 32) stage_linear_mfma<2, 6, 2>(st, c, M, smem);
              else if (M <= 48) stage_linear_mfma<3, 6, 2>(st, c, M, smem);
              else stage_linear_mfma<4, 6, 2>(st, c, M, smem);
            }
          }
          break;
        case MK_OP_SILU_MUL: stage_silu_mul(st, c, M); break;
        case MK_OP_COPY: stage_copy(st, c, M); break;
        case MK_OP_NGRAM_PARTIAL:
        case MK_OP_NGRAM_GLOBAL:
        case MK_OP_VERIFY:
          barrier_wait(c);
          if constexpr (MAXM > 1) {  // (a graph of one token per iteration has no room for guesses)
            if (st.op == MK_OP_NGRAM_PARTIAL) mk_ngram_partial(s, rtp, c.vid, c.G, (int *)smem);
            else if (st.op == MK_OP_NGRAM_GLOBAL) mk_ngram_global(s, rtp, c.vid, c.G, (int *)smem);
            else mk_verify_greedy(s, rtp, c.vid, c.G);
            c.wrote_through = true;
          }
          break;
        case MK_OP_ATTN:
          if constexpr (MAXM == 1) {
            if (st.num_q_heads == 4 * st.num_kv_heads) stage_attn<4, false>(st, c, rt, M, smem);
            else if (st.num_q_heads == 8 * st.num_kv_heads) stage_attn<8, false>(st, c, rt, M, smem);
            else barrier_wait(c);
          } else {
            // many (token, kv head) pairs per workgroup-chunk: cached positions on the matrix cores
            const bool mf = 2 * M * st.num_kv_heads >= c.G;
            if (st.num_q_heads == 4 * st.num_kv_heads) {
              if (mf) stage_attn<4, true>(st, c, rt, M, smem);
              else stage_attn<4, false>(st, c, rt, M, smem);
            } else if (st.num_q_heads == 8 * st.num_kv_heads) {
              if (mf) stage_attn<8, true>(st, c, rt, M, smem);
              else stage_attn<8, false>(st, c, rt, M, smem);
            } else {
              barrier_wait(c);
            }
          }
          break;
        case MK_OP_MOE_TOPK: stage_moe_topk(st, c, M); break;
        case MK_OP_MOE_LINEAR: stage_moe_linear(st, c, M, smem); break;
        case MK_OP_MOE_COMBINE: stage_moe_combine(st, c, M); break;
        case MK_OP_ARGMAX_PARTIAL: stage_argmax_partial(st, c, rt, M, smem); break;
        case MK_OP_ARGMAX_REDUCE: stage_argmax_reduce(st, c, rt, M); break;
        default: barrier_wait(c); break;
      }
      const long long t_out = (long long)wall_clock64();
      barrier_arrive(c);
      if (threadIdx.x == 0 && rt.profiler) {
        // begin = this stage's inputs were complete (the previous stage's barrier seen), end = its outputs were posted
        const long long at = 1 + c.vid + (long long)c.prof_n * c.G;
        if (at + c.G < rt.profiler_cap) {
          const unsigned tag = ((unsigned)(c.seq & 0x1FFF) << 19) | ((unsigned)(c.vid & 0xFF) << 11) | ((unsigned)(st.prof_event & 0x1FF) << 2);
          rt.profiler[at] = (unsigned long long)tag | (((unsigned long long)(c.t_wait * 10) & 0xFFFFFFFFull) << 32);
          rt.profiler[at + c.G] = (unsigned long long)(tag | 1u) | (((unsigned long long)((long long)wall_clock64() * 10) & 0xFFFFFFFFull) << 32);
          c.prof_n += 2;
        }
      }
      if (threadIdx.x == 0 && rt.stage_prof) {
        long long *pr = rt.stage_prof + MK_PROF_TICKS * ((size_t)c.vid * (rt.num_stages + 1) + s);
        pr[0] = t_in;
        pr[1] = c.t_wait;
        pr[2] = t_out;
        pr[3] = (long long)wall_clock64();
#ifdef MK_TRACE
        for (int i = 0; i < 4; i++) {
          pr[4 + i] = c.mark[i];
          c.mark[i] = 0;
        }
#endif
      }
    }
}

// The kernel body, instantiated twice: MAXM = 1 for graphs that never run more than one token per iteration (every
// multi-token stage form is compiled out, so the single-token loops get the register file to themselves), and the
// general one.
template <int MAXM>
__device__ __forceinline__ void mk_kernel_body(const MkRuntime &rt, const MkRuntime *rtp, int max_iters, int run_scheduler) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ int sh_bcast[4];
  __shared__ int sh_quota[10];
  __shared__ int sh_tok[4][MK_MAX_TOKENS];
  __shared__ int sh_ticket[3];
  // rt arrives by value in the kernel-argument segment (scalar loads); rtp is the same structure in device memory
  // for the one non-inlined function that takes its address (the scheduler step)
  Ctx c;
  c.G = gridDim.x;
  c.sync = rt.sync;
  c.xcd = xcc_id();
  c.epoch = 0;
  c.pending = false;
  c.dead = false;
  c.t_wait = 0;
  c.sh_dead = &sh_bcast[3];
  c.sh_tok = &sh_tok[0][0];
  c.sh_ticket = sh_ticket;
  c.seq = 0;
  c.prof_n = 0;
  c.defer_S = 0;
  c.wrote_through = false;
  c.arrive_w0 = false;
  if (threadIdx.x == 0) {
    sh_ticket[0] = sh_ticket[1] = 0;
    sh_ticket[2] = -2;
  }
  // ---- XCD discovery: rank of this workgroup inside its die, dies in use, workgroups per die
  if (threadIdx.x == 0) {
    MkSync *s = rt.sync;
    const unsigned rank = __hip_atomic_fetch_add(&s->xcd_count[c.xcd], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_fetch_add(&s->init_ctr, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    unsigned spins = 0;
    while (__hip_atomic_load(&s->init_ctr, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)c.G && spin_ok(s, spins, 0xFFFF0000u))
      __builtin_amdgcn_s_sleep(1);
    int nx = 0, before = 0, xi = 0;
    for (int i = 0; i < MK_MAX_XCD; i++) {
      const unsigned n = __hip_atomic_load(&s->xcd_count[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      nx += n > 0;
      if (i < c.xcd) {
        before += (int)n;
        xi += n > 0;
      }
    }
    sh_quota[8] = xi;
    sh_quota[9] = (int)rank;
    for (int i = 0; i < 8; i++) sh_quota[i] = (int)__hip_atomic_load(&s->xcd_count[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh_bcast[0] = before + (int)rank;
    sh_bcast[1] = nx;
    sh_bcast[2] = (int)__hip_atomic_load(&s->xcd_count[c.xcd], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh_bcast[3] = (int)__hip_atomic_load(&s->abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  // values read back from LDS are the same in every lane: tell the compiler, so that everything derived from them
  // (tile ranges, loop bounds, guards) lives in scalar registers and branches stay scalar
  c.vid = __builtin_amdgcn_readfirstlane(sh_bcast[0]);
  c.nxcd = __builtin_amdgcn_readfirstlane(sh_bcast[1]);
  c.quota = __builtin_amdgcn_readfirstlane(sh_bcast[2]);
  c.dead = __builtin_amdgcn_readfirstlane(sh_bcast[3]) != 0;
  for (int i = 0; i < 8; i++) c.quotas[i] = (unsigned)__builtin_amdgcn_readfirstlane(sh_quota[i]);
  c.xi = __builtin_amdgcn_readfirstlane(sh_quota[8]);
  c.rank = __builtin_amdgcn_readfirstlane(sh_quota[9]);
  c.even_xcds = true;
  for (int i = 0; i < 8; i++) c.even_xcds = c.even_xcds && (c.quotas[i] == 0 || c.quotas[i] == (unsigned)c.quota);
  __syncthreads();
  if (rt.profiler) {
    c.prof_n = (unsigned)__builtin_amdgcn_readfirstlane((int)ldc_u32(&rt.profiler_count[c.vid]));
    if (c.vid == 0 && threadIdx.x == 0) rt.profiler[0] = (unsigned long long)(unsigned)c.G | (1ull << 32);
  }

  for (int it = 0; it < max_iters && !c.dead; it++) {
    // ---- scheduler step on one thread of virtual workgroup 0, published through the barrier
    long long t_sched0 = 0, t_sched1 = 0;
    if (run_scheduler) {
      barrier_wait(c);  // the previous iteration's sampled tokens are complete
      t_sched0 = (long long)wall_clock64();
      // a handful of slots: one thread walks them; more: a wavefront, one lane per slot
      const bool wave_sched = run_scheduler == MK_SCHED_OFFLINE && rt.max_requests > 2 && rt.spec_len == 0;
      int ntok_w = 0;
      if (c.vid == 0 && threadIdx.x < 64 && wave_sched) ntok_w = mk_prepare_next_batch_wave(*rtp, (int *)smem, threadIdx.x);
      if (c.vid == 0 && threadIdx.x == 0) {
        int ntok;
        if (wave_sched) ntok = ntok_w;
        else if (run_scheduler == MK_SCHED_OFFLINE) ntok = mk_prepare_next_batch(*rtp, (int *)smem);
        else if (run_scheduler == MK_SCHED_ONLINE) ntok = mk_online_next_batch(*rtp);
        else ntok = mk_batch_from_meta(*rtp);
        if (ntok == 0) rt.sched->finished = 1;
        else rt.sched->iterations++;
        if (rt.timing && rt.sched->iterations <= rt.timing_cap) rt.timing[rt.sched->iterations] = (long long)wall_clock64();
        t_sched1 = (long long)wall_clock64();
      }
      barrier_arrive(c);
    }
    barrier_wait(c);
    // one cache invalidate per iteration: whatever this CU's L1 or this die's L2 kept from earlier iterations
    // (KV rows, page tables) is dropped, so this iteration's ordinary loads of such data see what was written back
    if (threadIdx.x == 0) {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      sh_bcast[0] = ldc_i32(&rt.sched->num_tokens);
    }
    __syncthreads();
    const int Mrt = __builtin_amdgcn_readfirstlane(sh_bcast[0]);
    const int M = MAXM == 1 ? (Mrt > 0 ? 1 : 0) : Mrt;
    // token metadata of this iteration, read once (it is on the critical path of every attention stage otherwise)
    if ((int)threadIdx.x < M) {
      const int t = threadIdx.x, slot = ldc_i32(&rt.tok_slot[t]);
      sh_tok[0][t] = ldc_i32(&rt.tok_pos[t]);
      sh_tok[1][t] = slot;
      sh_tok[2][t] = ldc_i32(&rt.tok_first[t]);
      sh_tok[3][t] = ldc_i32(&rt.kv_indptr[slot]);
    }
    __syncthreads();
    if (threadIdx.x == 0 && rt.stage_prof && run_scheduler) {
      long long *pr = rt.stage_prof + MK_PROF_TICKS * ((size_t)c.vid * (rt.num_stages + 1) + rt.num_stages);
      pr[0] = t_sched0;
      pr[1] = t_sched1;
      pr[2] = (long long)wall_clock64();
    }
    if (M == 0 || c.dead) break;
    run_stage_program<MAXM>(rt, rtp, c, MAXM == 1 ? 1 : M, smem);
  }
  barrier_wait(c);  // drain: nobody leaves while another workgroup may still poll
  if (rt.profiler && threadIdx.x == 0) rt.profiler_count[c.vid] = c.prof_n;
  if (c.vid == 0 && threadIdx.x == 0 && rt.timing) rt.timing[0] = (long long)wall_clock64();
}


extern "C" __global__ __launch_bounds__(MK_THREADS, 1) void mk_persistent_kernel(const MkRuntime rt, const MkRuntime *rtp, int max_iters,
                                                                                int run_scheduler) {
  mk_kernel_body<MK_MAX_TOKENS>(rt, rtp, max_iters, run_scheduler);
}
// the same for graphs with max_num_batched_tokens == 1
extern "C" __global__ __launch_bounds__(MK_THREADS, 1) void mk_persistent_kernel_m1(const MkRuntime rt, const MkRuntime *rtp, int max_iters,
                                                                                   int run_scheduler) {
  mk_kernel_body<1>(rt, rtp, max_iters, run_scheduler);
}
