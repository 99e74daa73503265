// Internal launch interface between the C-ABI host layer and the gfx950 kernels.
// Plain structs and pointers only; nothing here is exported from the library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ringattn {

constexpr int kBlockM = 128;  // query rows per workgroup (4 waves x 32 rows)

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
  const void* k;       // [BH, S, D]
  const void* v;       // [BH, S, D]
  float* o_part;       // [BH, S, D] fp32 partial O of this step (normalised)
  float* lse_part;     // [BH, S]    fp32 partial LSE of this step (natural log)
  int64_t bh_stride;   // elements between heads (= S * D)
  int S;               // tokens per head
  int chunk;           // tokens per virtual rank
  int P;               // virtual ranks
  const int* pairs;    // device array of packed (rank, step) pairs, or nullptr
  int64_t part_stride_rows;  // rows between the partial slots of consecutive steps
  int step;            // ring step s (pairs == nullptr)
  int rank_base;       // first active rank of this step (pairs == nullptr)
  int n_active;        // active ranks of the step, or number of pairs
  int BH;              // batch * heads
  int causal;          // chunk-level causal ring: j<r full, j==r diagonal mask
  float scale_log2;    // softmax_scale * log2(e)
};

// P-way merge of the per-step partials into the final O (storage dtype) and LSE.
struct MergeArgs {
  const float* o_parts;   // [n_parts, rows, D]
  const float* lse_parts; // [n_parts, rows]
  void* out;              // [rows, D] storage dtype
  float* lse;             // [rows]
  int64_t rows;           // BH * S
  int64_t part_stride_rows;  // rows between consecutive parts (>= rows)
  int n_parts;
  // ring structure: when causal_ring != 0, part s of a row of rank r = (row % S) / chunk
  // is active iff s == 0 or r + s >= P; inactive parts are never read.
  int causal_ring;
  int S, chunk, P;
  // rank_sel >= 0: only the rows of that virtual rank are merged (rows = BH * chunk, row i
  // is row (i / chunk) * S + rank_sel * chunk + i % chunk of the tensors); -1: all rows.
  int rank_sel;
};

// dtype: 0 = fp16, 1 = bf16.  Return hipSuccess or the launch error.
hipError_t launch_block_step(const BlockStepArgs& a, int dtype, int dim, hipStream_t stream);
hipError_t launch_merge(const MergeArgs& a, int dtype, int dim, hipStream_t stream);

}  // namespace ringattn
