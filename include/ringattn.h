/*
 * ringattn.h -- C ABI of the MI355X (gfx950) ring-attention forward engine.
 *
 * Every entry point is extern "C", takes plain pointers and sizes, and returns an
 * int status (0 = RINGATTN_OK).  Argument validation happens before the first HIP
 * call, so bad arguments are reported on a host without a GPU as well.  Tensors
 * are device-resident and contiguous, the convention of the reference's
 * include/attention_api.cuh:12-18 (CHECK_CUDA / CHECK_CONTIGUOUS).  Where the
 * reference prints and exits on an error (include/attention_api.cuh:20-29,
 * csrc/utils.h:1-11), this library returns a code; ringattn_strerror() names it.
 *
 * Layout: Q, K, V, O are [batch, heads, S, dim] row-major, so each (batch, head)
 * slab is the reference's [seqlen, dim] layout (csrc/ring_attention.cu:422-426).
 * The sequence is split into npes chunks in order; virtual ring rank r owns the
 * h_seqlen[r] rows that follow those of rank r-1.  At ring step s rank r works on KV chunk (r + s) mod npes
 * (csrc/ring_attention.cu:463,531,615) -- by indexing, no data is moved.
 */
#ifndef RINGATTN_H
#define RINGATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RINGATTN_OK 0
#define RINGATTN_ERR_NULL 1        /* a required pointer is NULL */
#define RINGATTN_ERR_NPES 2        /* npes < 1 or above RINGATTN_MAX_NPES */
#define RINGATTN_ERR_DIM 3         /* dim not in {64, 128} */
#define RINGATTN_ERR_DTYPE 4       /* dtype not fp16 / bf16 */
#define RINGATTN_ERR_SEQLEN 5      /* a per-rank length is not positive (or odd, with the zigzag layout), or max_seq is below it */
#define RINGATTN_ERR_SHAPE 6       /* batch or heads < 1, kv_heads does not divide heads, unknown layout, sizes overflow */
#define RINGATTN_ERR_WORKSPACE 7   /* caller workspace missing or too small */
#define RINGATTN_ERR_RANK 8        /* mype / step outside [0, npes) */
#define RINGATTN_ERR_PLAN 9        /* plan handle invalid or already destroyed */
#define RINGATTN_ERR_HIP 10        /* a HIP runtime call failed (see ringattn_last_hip_error) */
#define RINGATTN_ERR_ALLOC 11      /* device or host allocation failed */
#define RINGATTN_ERR_ALIGN 12      /* a tensor pointer is not 16-byte aligned */

#define RINGATTN_DTYPE_FP16 0
#define RINGATTN_DTYPE_BF16 1

#define RINGATTN_MAX_NPES 64
#define RINGATTN_TILE 256          /* query rows per workgroup: per-rank lengths may be any positive number and may differ between
                                      ranks (the tail predication the reference leaves open, csrc/ring_attention.cu:143-145);
                                      multiples of this waste no part of a tile */

#define RINGATTN_FLAG_GRAPH 1      /* capture the launch of a forward (one kernel node) in a hipGraph and replay it */
#define RINGATTN_FLAG_TIMING 2     /* record timing events around every block-attention launch of ringattn_fwd
                                      (read with ringattn_plan_launch_times); ignored together with FLAG_GRAPH */
#define RINGATTN_FLAG_HALF_PARTIALS 4 /* keep the per-step partial O in fp16 instead of fp32 (for either input dtype): halves
                                      the workspace and the bytes the attention kernel writes and the merge reads.  A partial O
                                      row is a weighted mean of V rows, so this needs |V| < 65504, and it adds up to 2^-11
                                      relative error per partial (fp32 partials add none); the partial LSE stays fp32.
                                      Applies wherever partials are written (ringattn_block_fwd, ringattn_rank_step_fwd,
                                      ringattn_fwd with RINGATTN_FLAG_STEP_PARTIALS) */
#define RINGATTN_FLAG_STEP_PARTIALS 8 /* ringattn_fwd keeps the ring steps apart: a normalised partial (O, LSE) per step in
                                      the workspace, merged at the end -- the arithmetic of ringattn_block_fwd +
                                      ringattn_merge_ring, bit for bit, in one launch.  Without the flag (the default)
                                      the softmax state (max, sum, acc-O) runs through all steps in registers, as in the
                                      reference's kernel (csrc/ring_attention.cu:439-443,597), and no workspace is needed */
#define RINGATTN_FLAG_ROW_PARTIALS 16 /* caller-held per-step partials keep a row's steps next to each other:
                                      o_parts [batch*heads*S, npes, dim] and lse_parts [batch*heads*S, npes] instead of
                                      [npes, batch*heads*S, dim] / [npes, batch*heads*S].  ringattn_block_fwd and
                                      ringattn_rank_step_fwd then take the BASE of those buffers for every step and
                                      write entry `step` of each row; ringattn_merge_ring / ringattn_rank_merge read a
                                      row's steps as one contiguous run (the merge of many short steps -- 32 steps of
                                      256-byte fp16 rows -- then streams instead of gathering pieces 4 MB apart).  No
                                      effect on ringattn_fwd */

/*
 * Placement of the sequence on the ranks.  CONTIGUOUS: rank r holds the tokens that follow
 * those of rank r-1 (the reference's split, csrc/ring_attention.cu:753-757).  ZIGZAG: rank r
 * holds two half-chunks back to back, a low one and a high one; in the sequence the low
 * halves of ranks 0..npes-1 come first and then the high halves of ranks npes-1..0, so that
 * under the causal mask every rank has the same amount of work (with CONTIGUOUS rank r has
 * r + 1 visible chunks).  The reference has no causal mask and therefore no such layout; it
 * only matters when `causal` is set.  Per-rank lengths must then be even.
 */
#define RINGATTN_LAYOUT_CONTIGUOUS 0
#define RINGATTN_LAYOUT_ZIGZAG 1

/*
 * Replaces struct Ring_fwd_params (csrc/ring.h:5-19).  npes, h_seqlen, dim and
 * softmax_scale keep their meaning; mype is gone because one call runs every
 * virtual rank; the device copy of seqlen and the k/v staging buffers are gone
 * because nothing is fetched from a peer.  batch, heads, dtype, causal are the
 * generalisations the reference hard-wires (fp16, one head, non-causal:
 * csrc/ring_attention.cu:18,422-426,530).
 */
typedef struct ringattn_params {
  int npes;              /* P: virtual ring ranks */
  const int* h_seqlen;   /* [npes] tokens per rank, may differ per rank like the reference's seqlen[]
                            (csrc/ring_attention.cu:753); host array, read during the call only */
  int dim;               /* head dimension: 64 or 128 */
  float softmax_scale;   /* logit scale; <= 0 selects 1/sqrt(dim) */
  int batch;
  int heads;
  int dtype;             /* RINGATTN_DTYPE_* of Q, K, V and O */
  int causal;            /* 0: every rank sees every chunk; 1: chunks in sequence order, KV chunk j > r skipped, j == r masked */
  int flags;             /* RINGATTN_FLAG_* */
  int kv_heads;          /* heads of K and V (grouped-query attention): 0 or `heads` = one KV head per
                            query head; otherwise it must divide `heads`, and query head h reads KV head
                            h / (heads / kv_heads).  K and V are then [batch, kv_heads, S, dim]. */
  int layout;            /* RINGATTN_LAYOUT_*: which tokens of the sequence the rows of rank r are */
} ringattn_params;

typedef struct ringattn_plan ringattn_plan;

/* Bytes of device workspace a plan needs.  0 unless RINGATTN_FLAG_STEP_PARTIALS is set; then one
 * partial O row and one partial LSE per query row and VISIBLE ring step -- (dim + 1) * 4 bytes
 * each, (2 dim + 4) with RINGATTN_FLAG_HALF_PARTIALS.  Without a mask every row has npes steps;
 * with the causal mask a row of rank r has r + 1 (36 of the 64 (rank, step) pairs at npes = 8);
 * with the zigzag layout the low half of rank r has r + 1 and the high half npes.  Also 0 if the
 * parameters are invalid. */
size_t ringattn_workspace_bytes(const ringattn_params* params);

/*
 * Create a plan: validates the parameters and allocates the workspace (if the plan needs one)
 * ONCE -- the job set_params_fprop (csrc/ring_attention.cu:361-395) does on every call with a
 * cudaMalloc and two nvshmem_mallocs that are never freed (:383-394).
 * If workspace != NULL it is used instead of an internal allocation and must hold
 * at least ringattn_workspace_bytes() bytes (workspace_bytes is checked).
 */
int ringattn_plan_create(const ringattn_params* params, void* workspace, size_t workspace_bytes,
                         ringattn_plan** plan_out);

/* Destroy a plan and free what it allocated.  NULL or an already destroyed plan gives RINGATTN_ERR_PLAN. */
int ringattn_plan_destroy(ringattn_plan* plan);

/*
 * The whole forward for all npes virtual ranks: replaces ring_attention()
 * (csrc/ring_attention.cu:706-722) run on every PE.  ONE block-attention launch: a workgroup
 * owns 256 query rows and walks every ring step of those rows with the running max, sum and
 * acc-O in registers, like the reference's CTA (:439-443,456,597), then writes O = acc / sum
 * (:621-664) and the LSE.  (With RINGATTN_FLAG_STEP_PARTIALS: a partial (O, LSE) per step into
 * the workspace, merged at the end of the workgroup.)
 *   q, k, v : [batch, heads, S, dim] dtype     out : same shape and dtype
 *   lse     : [batch, heads, S] fp32, natural log (the reference never writes it)
 * Asynchronous on `stream` (a hipStream_t, or NULL for the default stream); the
 * reference blocks with cudaDeviceSynchronize (:721) -- callers that want that
 * synchronise the stream.  A plan is used by one host thread at a time.
 */
int ringattn_fwd(ringattn_plan* plan, const void* q, const void* k, const void* v,
                 void* out, float* lse, void* stream);

/*
 * One ring step (the body of the reference's step loop, csrc/ring_attention.cu:456-620,
 * for every active rank at once): rank r attends KV chunk (r + step) mod npes and the
 * normalised partial O [batch, heads, S, dim] (fp32; fp16 on a plan with
 * RINGATTN_FLAG_HALF_PARTIALS) and fp32 partial LSE
 * [batch, heads, S] are written for the rows of the active ranks.  Rows that see no key of
 * the visited chunk (causal: chunk j > r; zigzag: also the low half against j > r) are
 * left untouched.
 */
int ringattn_block_fwd(ringattn_plan* plan, int step, const void* q, const void* k, const void* v,
                       void* o_part, float* lse_part, void* stream);

/*
 * Cross-step merge (no function of its own in the reference: it is the algebra of
 * carrying max / sum / acc-O across steps, csrc/ring_attention.cu:207-245,621-633):
 *   lse = logsumexp_s lse_parts[s];  out = sum_s exp(lse_parts[s] - lse) * o_parts[s]
 * o_parts [n_parts, rows, dim] fp32, lse_parts [n_parts, rows] fp32 (a part with
 * lse = -inf is the identity); out [rows, dim] dtype; lse [rows] fp32.
 */
int ringattn_merge(const float* o_parts, const float* lse_parts, int n_parts, int64_t rows, int dim,
                   int dtype, void* out, float* lse, void* stream);

/*
 * The merge as ringattn_fwd runs it, on caller-held partials: o_parts
 * [npes, batch*heads*S, dim] and lse_parts [npes, batch*heads*S] as written by
 * ringattn_block_fwd for steps 0..npes-1.  With a causal plan, part s of a row is read
 * only if ringattn_block_fwd writes that row in step s (contiguous layout: s == 0 or
 * r + s >= npes for a row of rank r), so parts the step loop never wrote are never touched.  Like ringattn_merge, it has no counterpart
 * function in the reference (csrc/ring_attention.cu:207-245,621-633 pin the algebra).
 */
int ringattn_merge_ring(ringattn_plan* plan, const void* o_parts, const float* lse_parts,
                        void* out, float* lse, void* stream);

/*
 * One ring step of ONE rank on rank-local buffers -- what a process of the reference does in
 * one iteration of its step loop (csrc/ring_attention.cu:456-620) once the K/V chunk of rank
 * (rank + step) mod npes has arrived (:611-619):
 *   q        : [batch, heads, h_seqlen[rank], dim]       the rank's own queries
 *   k_chunk,
 *   v_chunk  : [batch, kv_heads, h_seqlen[j], dim]       the visited chunk, j = (rank + step) mod npes
 *   o_part   : [batch, heads, h_seqlen[rank], dim] fp32 (fp16 with RINGATTN_FLAG_HALF_PARTIALS)
 *   lse_part : [batch, heads, h_seqlen[rank]] fp32
 * Rows that see no key of the visited chunk are left untouched (nothing at all is launched if
 * that holds for the whole rank).  The results are bit-identical to the rows ringattn_block_fwd
 * writes for this rank in this step.  This is the call a one-process-per-GPU ring makes between
 * its K/V exchanges; the exchange itself is the caller's.
 */
int ringattn_rank_step_fwd(ringattn_plan* plan, int rank, int step, const void* q, const void* k_chunk,
                           const void* v_chunk, void* o_part, float* lse_part, void* stream);

/*
 * The merge of one rank's per-step partials: o_parts [npes, batch*heads*h_seqlen[rank], dim] and
 * lse_parts [npes, batch*heads*h_seqlen[rank]], slot s as written by ringattn_rank_step_fwd for
 * step s (slots of steps that left the rows untouched are not read); out / lse hold the rank's
 * rows only.  Bit-identical to the rows ringattn_fwd produces for this rank on a plan with
 * RINGATTN_FLAG_STEP_PARTIALS (without the flag ringattn_fwd rounds differently: it never
 * normalises per step).
 */
int ringattn_rank_merge(ringattn_plan* plan, int rank, const void* o_parts, const float* lse_parts, void* out,
                        float* lse, void* stream);

/*
 * The schedule of a plan, for inspection (host data, no GPU work; the reference has no
 * counterpart: its schedule is the loop `for step in 0..npes-1: kv_pe = (mype + step) % npes`
 * of csrc/ring_attention.cu:456-470,615).  A work item is one block-attention job: the
 * queries [q_start, q_start + q_len) of every head against the keys [kv_start, kv_start +
 * kv_len), rows counted within a head.  diag_off < 0: every key visible; otherwise key kl
 * (local to the KV range) is visible to query ql (local to the query range) iff
 * kl <= ql + diag_off.  The partial result goes to slot `slot` (= the ring step).
 * step in [0, npes): the items ringattn_block_fwd(step) runs; step == -1: all items of
 * ringattn_fwd, row range by row range, in the order a workgroup runs them (a range that is
 * masked differently within a rank, as the two halves of a zigzag rank are, is listed as
 * separate items).  Writes min(n, capacity) items and stores n in *n_out.
 */
typedef struct ringattn_work_item {
  int q_start, q_len, kv_start, kv_len, diag_off, slot;
} ringattn_work_item;

int ringattn_plan_work_items(const ringattn_plan* plan, int step, ringattn_work_item* out, int capacity, int* n_out);

/*
 * Durations in milliseconds of the block-attention launches (one, as things are) of the most
 * recent ringattn_fwd on a plan created with RINGATTN_FLAG_TIMING, from events recorded on the
 * caller's stream right before and after each launch -- the job of the cudaEvent pair around the
 * timed loop of the reference harness (csrc/ring_attention.cu:772-783), per launch.  Blocks until
 * that forward's launches have finished.  Writes min(n, capacity) values and stores n in *n_out;
 * RINGATTN_ERR_PLAN if the plan has no timing flag or has not run a forward yet.
 */
int ringattn_plan_launch_times(ringattn_plan* plan, float* ms, int capacity, int* n_out);

/*
 * Name of the kernel ringattn_fwd launches for this plan, for reading kernel traces: "ring_walk64_kernel" (every KV
 * range a multiple of 32 keys and at least 128; with RINGATTN_FLAG_STEP_PARTIALS only at d = 128 in causal plans with at
 * least 2048 keys per chunk; RINGATTN_WIDE=0, RINGATTN_WIDE_D64=0 and RINGATTN_WIDE_PARTIALS=0 / 1 in the environment
 * override) or "ring_walk_kernel".  Both are restatements of the reference's one
 * kernel (csrc/ring_attention.cu:398-666) with its tiling (csrc/kernel_traits.h:11-177) replaced; they differ in how
 * the 256 query rows of a workgroup are laid out over waves (64 rows per wave at one wave per SIMD, or 32 rows per
 * wave at two).  NULL for an invalid plan.
 */
const char* ringattn_plan_forward_kernel(const ringattn_plan* plan);

/*
 * The row ranges ringattn_merge_ring merges separately: rows [start[i], start[i] + len[i])
 * of every head read the partial slots whose bit is set in active[i].  Writes
 * min(n, capacity) entries and stores n in *n_out.
 */
int ringattn_plan_merge_regions(const ringattn_plan* plan, int* start, int* len, uint64_t* active, int capacity, int* n_out);

/*
 * Reference-shaped convenience entry: the signature of
 *   void ring_attention(FPC* q, FPC* k, FPC* v, float* out, int npes, int mype,
 *                       int* seqlen, int dim, int max_seq)   (csrc/ring_attention.cu:706)
 * for ONE head and ONE rank: q is rank mype's [seqlen[mype], dim] block; k and v hold
 * the chunks of all ranks back to back ([sum seqlen, dim]) -- what the reference
 * reaches through NVSHMEM gets (:612-619); out is [seqlen[mype], dim] in `dtype`
 * (the reference declares float* but stores 16-bit values, :635,763); lse (may be
 * NULL) is [seqlen[mype]] fp32.  max_seq is accepted for signature parity and only
 * checked (>= every seqlen).  Blocks until the result is ready, like the reference (:721).
 */
int ringattn_ring_attention(const void* q, const void* k, const void* v, void* out, float* lse,
                            int npes, int mype, const int* seqlen, int dim, int max_seq,
                            int dtype, int causal, float softmax_scale);

/*
 * ringattn_ring_attention for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose entry allocates on every call, csrc/ring_attention.cu:383-394).  Same
 * arguments and results as ringattn_ring_attention, plus the stream; it calls no hipMalloc,
 * hipFree, memcpy or other allocating routine and does not synchronise: the work (a
 * table-writing kernel, then the attention kernel) is queued on `stream`.  The table of ring steps
 * the attention kernel reads (32 bytes + 32 per visible step), which ringattn_ring_attention keeps
 * in a per-call allocation, lives in a static device array of ringattn_noalloc_scratch_bytes()
 * bytes (4 KiB, held by every GPU the library runs on until the process ends): enough for
 * RINGATTN_MAX_NPES steps, and a ring with more ranks is refused with RINGATTN_ERR_NPES like
 * everywhere else.  All calls on one GPU share that array.  A call's table takes the next slice of it, round
 * robin, and the attention kernel reads its slice for as long as it runs: calls on one stream are ordered by the
 * stream, and calls on several streams or threads may overlap as long as no more of them are in flight on a GPU
 * than slices fit (fourteen with 8-step rings, 288 bytes each; one when a table takes more than half the array).
 * Beyond that a running kernel may find another call's KV ranges in its table and read outside its K and V: do
 * not let that many calls overlap.  Nothing in the array needs clearing between calls.  The first call on a
 * device looks up the array's address (hipGetSymbolAddress): make it outside a stream capture.
 */
int ringattn_ring_attention_noalloc(const void* q, const void* k, const void* v, void* out, float* lse,
                                    int npes, int mype, const int* seqlen, int dim, int max_seq,
                                    int dtype, int causal, float softmax_scale, void* stream);

/* Size in bytes of the static device scratch behind ringattn_ring_attention_noalloc. */
size_t ringattn_noalloc_scratch_bytes(void);

/*
 * Seeded input generator -- the counterpart of fillWithNum / initQKV
 * (csrc/ring_attention.cu:731-748), which fill a host buffer and copy it to the
 * device.  Writes n values of N(0, sigma^2), rounded to nearest-even into `dtype`,
 * to a HOST buffer: element i uses counters 2*(offset+i)+1 and 2*(offset+i)+2 of the
 * splitmix64 stream keyed by `seed` (Box-Muller, cosine branch).  Pure host code.
 */
int ringattn_fill_normal(void* dst_host, int dtype, int64_t n, uint64_t seed, int64_t offset, double sigma);

/* The reference's own deterministic fill h[i*n+j] = i/130 + j/110 + i*j/600
 * (csrc/ring_attention.cu:731-741), rounded into `dtype`, for an [m, n] host matrix. */
int ringattn_fill_reference_pattern(void* dst_host, int dtype, int m, int n);

const char* ringattn_strerror(int code);

/* The hipError_t (as int) of the last failing HIP call seen by this thread, 0 if none. */
int ringattn_last_hip_error(void);

#ifdef __cplusplus
}
#endif
#endif /* RINGATTN_H */
