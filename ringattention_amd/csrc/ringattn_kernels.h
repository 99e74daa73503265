// Internal launch interface between the C-ABI host layer and the gfx950 kernels.
// Plain structs and pointers only; nothing here is exported from the library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ringattn {

constexpr int kBlockM = 128;  // query rows per workgroup (4 waves x 32 rows)
constexpr int kMaxParts = 64; // partial slots a merge can combine

// One unit of block-attention work: the queries [q_start, q_start + q_len) of every head
// against the keys/values [kv_start, kv_start + kv_len) of the matching KV head -- the body
// of one ring step of one rank (csrc/ring_attention.cu:456-470,531-610: rank r at step s
// works on the KV chunk of rank (r + s) mod P).  Row numbers are local to a head's [S, D]
// slab and need not be multiples of any tile size.  The normalised partial O and the partial LSE
// of the item go to partial slot `slot`, at the rows of its queries.
struct WorkItem {
  int q_start, q_len;
  int kv_start, kv_len;
  int diag_off;  // < 0: every key is visible.  >= 0: key kl (local to the KV range) is visible
                 // to query ql (local to the query range) iff kl <= ql + diag_off; then
                 // diag_off + q_len <= kv_len
  int slot;
  int pad0, pad1;
};
static_assert(sizeof(WorkItem) == 32, "WorkItem is read as two 16-byte scalar loads");

struct BlockStepArgs {
  const void* q;       // [BH, S, D] storage dtype
  const void* k;       // [batch * heads / kv_group, S, D]
  const void* v;       // [batch * heads / kv_group, S, D]
  void* o_part;        // partial slot `slot_bias`: [BH, S, D] partial O (normalised), fp32 or fp16 (half_partials)
  float* lse_part;     // partial slot `slot_bias`: [BH, S] fp32 partial LSE (natural log)
  const WorkItem* items;     // device array
  int64_t bh_stride;   // elements between heads of q (= S * D)
  int64_t kv_bh_stride;      // elements between heads of k and v
  int64_t part_stride_rows;  // rows between consecutive partial slots
  int S;               // rows per head in the partial slots
  int q_tiles_max;     // kBlockM-row q tiles of the longest item (grid dimension)
  int n_items;
  int slot_bias;       // item.slot - slot_bias is the slot index relative to o_part / lse_part
  int BH;              // batch * heads
  int heads;           // query heads per batch entry
  int kv_group;        // query heads per KV head (1 = one KV head per query head)
  float scale_log2;    // softmax_scale * log2(e)
  int half_partials;   // partial O stored as fp16 instead of fp32
};

// Merge of (O, LSE) partials into the final O (storage dtype) and LSE, for the rows
// [sel_start, sel_start + sel_len) of every head.
struct MergeArgs {
  const void* o_parts;    // [slots, heads * S, D] fp32, or fp16 with half_partials
  const float* lse_parts; // [slots, heads * S]
  void* out;              // [heads * S, D] storage dtype
  float* lse;             // [heads * S]
  int64_t rows;           // heads * sel_len rows are merged
  int64_t part_stride_rows;  // rows between consecutive slots (>= heads * S)
  uint64_t active;        // bit s set: slot s holds a partial for these rows; other slots are never read
  int S;                  // rows per head
  int sel_start, sel_len; // row range within a head
  int half_partials;
};

// Up to kMaxParts work items passed BY VALUE to a small kernel that writes them to device
// memory: an item table for callers that may not copy from the host (no allocation, no
// memcpy node: a plain kernel launch).
struct ItemPack {
  WorkItem items[kMaxParts];
};

// dtype: 0 = fp16, 1 = bf16.  Return hipSuccess or the launch error.
hipError_t launch_block_step(const BlockStepArgs& a, int dtype, int dim, hipStream_t stream);
hipError_t launch_merge(const MergeArgs& a, int dtype, int dim, hipStream_t stream);
hipError_t launch_write_items(const ItemPack& pack, int n, WorkItem* dst, hipStream_t stream);

}  // namespace ringattn
