// Internal launch interface between the C-ABI host layer and the gfx950 kernels.
// Plain structs and pointers only; nothing here is exported from the library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ringattn {

constexpr int kBlockM = 128;  // query rows per workgroup (4 waves x 32 rows)
constexpr int kMaxRanks = 64;

// A batch of (rank, ring step) pairs: rank r at step s works on KV chunk (r + s) mod P --
// the launch-level restatement of the step loop body of the reference kernel
// (csrc/ring_attention.cu:456-470,531-610).  Two ways to name the pairs:
//   pairs == nullptr : one ring step for the ranks rank_base .. rank_base + n_active - 1;
//                      o_part / lse_part point at that step's slot;
//   pairs != nullptr : n_active packed pairs (rank << 16 | step) read from device memory;
//                      o_part / lse_part point at slot 0 and step s is written at
//                      + s * part_stride_rows rows.
struct BlockStepArgs {
  const void* q;       // [BH, S, D] storage dtype
  const void* k;       // [batch * heads / kv_group, S, D]
  const void* v;       // [batch * heads / kv_group, S, D]
  float* o_part;       // [BH, S, D] fp32 partial O of this step (normalised)
  float* lse_part;     // [BH, S]    fp32 partial LSE of this step (natural log)
  int64_t bh_stride;   // elements between heads (= S * D)
  int S;               // tokens per head
  int q_tiles_max;     // kBlockM-row q tiles of the longest rank (grid dimension)
  int P;               // virtual ranks
  const int* pairs;    // device array of packed (rank, step) pairs, or nullptr
  int64_t part_stride_rows;  // rows between the partial slots of consecutive steps
  int step;            // ring step s (pairs == nullptr)
  int rank_base;       // first active rank of this step (pairs == nullptr)
  int n_active;        // active ranks of the step, or number of pairs
  int BH;              // batch * heads
  int heads;           // query heads per batch entry
  int kv_group;        // query heads per KV head (1 = one KV head per query head)
  int causal;          // chunk-level causal ring: j<r full, j==r diagonal mask
  float scale_log2;    // softmax_scale * log2(e)
  // rank r owns rows [rank_start[r], rank_start[r+1]) of every head; lengths are multiples
  // of kBlockM and may differ per rank (the per-PE seqlen[] of csrc/ring_attention.cu:753)
  int rank_start[kMaxRanks + 1];
};

// n-way merge of (O, LSE) partials into the final O (storage dtype) and LSE, for the rows
// [sel_start, sel_start + sel_len) of every head (one virtual rank, or everything).
struct MergeArgs {
  const float* o_parts;   // [n_parts, heads * S, D]
  const float* lse_parts; // [n_parts, heads * S]
  void* out;              // [heads * S, D] storage dtype
  float* lse;             // [heads * S]
  int64_t rows;           // heads * sel_len rows are merged
  int64_t part_stride_rows;  // rows between consecutive parts (>= heads * S)
  int n_parts;
  int first_wrapped;      // active parts: part 0 and parts first_wrapped .. n_parts-1 (1 = all);
                          // inactive parts are never read
  int S;                  // rows per head
  int sel_start, sel_len; // row range within a head
};

// dtype: 0 = fp16, 1 = bf16.  Return hipSuccess or the launch error.
hipError_t launch_block_step(const BlockStepArgs& a, int dtype, int dim, hipStream_t stream);
hipError_t launch_merge(const MergeArgs& a, int dtype, int dim, hipStream_t stream);

}  // namespace ringattn
