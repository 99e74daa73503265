// Internal launch interface between the C-ABI host layer and the gfx950 kernels.
// Plain structs and pointers only; nothing here is exported from the library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ringattn {

constexpr int kWalkM = 256;   // query rows per workgroup of ring_walk_kernel (8 waves x 32 rows)
constexpr int kMaxParts = 64; // partial slots a merge can combine

// One unit of block-attention work as the host layer lists it: the queries
// [q_start, q_start + q_len) of every head against the keys/values
// [kv_start, kv_start + kv_len) of the matching KV head -- the body of one ring step of one
// rank (csrc/ring_attention.cu:456-470,531-610: rank r at step s works on the KV chunk of rank
// (r + s) mod P).  Row numbers are local to a head's [S, D] slab and need not be multiples of
// any tile size.  The normalised partial O and the partial LSE of the item go to partial slot
// `slot`, at the rows of its queries.
struct WorkItem {
  int q_start, q_len;
  int kv_start, kv_len;
  int diag_off;  // < 0: every key is visible.  >= 0: key kl (local to the KV range) is visible
                 // to query ql (local to the query range) iff kl <= ql + diag_off; then
                 // diag_off + q_len <= kv_len
  int slot;
  int pad0, pad1;
};

// What the attention kernel runs: a SEGMENT is a range of query rows (of every head) together with
// ALL the key ranges it meets -- the ring steps of the reference's step loop
// (csrc/ring_attention.cu:456-620) for those rows.  One workgroup owns kWalkM rows of a segment,
// keeps their Q in registers and walks the segment's items, as the reference's CTA walks the
// ring steps (:439-443,456), emitting one (partial O, partial LSE) per item.
struct SegItem {
  int kv_start, kv_len;
  int diag_off;         // as in WorkItem, relative to the first row of the segment
  int part_bh_stride;   // rows between consecutive heads in this item's partial block
  int64_t part_base;    // row (in the partial buffers) of the segment's first row of head 0
  int slot;             // ring step: the entry of a row's run with row-major partials, else for inspection only
  int part_row_mul;     // 0: the partial of row r lives at row r of the buffers; n > 0: at entry n r + slot (a row's
                        // steps next to each other, n of them)
};
static_assert(sizeof(SegItem) == 32, "SegItem is read as two 16-byte scalar loads");

struct Segment {
  int q_start, q_len;
  int item_begin, item_count;  // slice of the SegItem table, in ascending ring-step order
  int last_item;               // index (within the slice) of the item to run last, -1: table order.
                               // A masked (diagonal) item runs last: its length differs per q tile,
                               // and the q tiles that share a KV chunk in L2 stay in step until then.
  int reverse_tiles;           // the q tiles with the most visible keys are scheduled first
  int pad0, pad1;
};
static_assert(sizeof(Segment) == 32, "Segment is read as two 16-byte scalar loads");

// What a workgroup does with the softmax state (max, sum, acc-O) of its rows between the KV chunks it walks.
enum BlockMode {
  kBlockPartials = 0,        // per chunk: emit the normalised partial (O, LSE), reset the state
  kBlockPartialsMerged = 1,  // the same, and after the last chunk merge the partials of the rows into out / lse
  kBlockCarryState = 2,      // carry the state across the chunks, as the reference's CTA does across its ring
                             // steps (csrc/ring_attention.cu:439-443,597), and write out / lse once: no partials
};

struct BlockArgs {
  const void* q;       // [BH, S, D] storage dtype
  const void* k;       // [batch * heads / kv_group, S, D]
  const void* v;       // [batch * heads / kv_group, S, D]
  void* o_part;        // partial O rows (normalised), fp32 or fp16 (half_partials); indexed by SegItem::part_base
  float* lse_part;     // partial LSE rows (natural log), same row numbering; both unused with kBlockCarryState
  void* out;           // unless kBlockPartials: [BH, S, D] storage dtype
  float* lse;          // unless kBlockPartials: [BH, S]; may be NULL with kBlockCarryState
  const Segment* segs; // device arrays
  const SegItem* items;
  const int2* groups;  // NULL, or [8][groups_per_xcd] (segment, head) pairs: what the workgroups of each XCD run,
                       // in order; segment < 0 marks an unused entry
  int groups_per_xcd;
  int64_t bh_stride;   // elements between heads of q and out (= S * D)
  int64_t kv_bh_stride;      // elements between heads of k and v
  int S;               // rows per head of q, out and lse
  int q_tiles_max;     // kWalkM-row q tiles of the longest segment (grid dimension)
  int n_segs;
  int BH;              // batch * heads
  int heads;           // query heads per batch entry
  int kv_group;        // query heads per KV head (1 = one KV head per query head)
  float scale_log2;    // softmax_scale * log2(e)
  int half_partials;   // partial O stored as fp16 instead of fp32
  int mode;            // BlockMode
};

// Merge of (O, LSE) partials into the final O (storage dtype) and LSE, for row ranges of every
// head: a region covers rows [start, start + len) and reads the slots whose bit is set in `active`.
struct MergeRegion {
  int start, len;
  uint64_t active;
};
static_assert(sizeof(MergeRegion) == 16, "MergeRegion is read as one 16-byte scalar load");

struct MergeArgs {
  const void* o_parts;    // [slots, heads * S, D] fp32, or fp16 with half_partials
  const float* lse_parts; // [slots, heads * S]
  void* out;              // [heads * S, D] storage dtype
  float* lse;             // [heads * S]
  const MergeRegion* regions;  // device array of n_regions entries, one grid row each; NULL: `single`
  MergeRegion single;
  int n_regions;          // 1 with `single`
  int max_len;            // longest region (grid columns)
  int heads;              // batch * heads: every region is merged for each of them
  int S;                  // rows per head
  int64_t part_stride_rows;  // rows between consecutive slots (>= heads * S)
  int half_partials;
  int row_mul;            // 0: slot-major partials as above; n > 0: [heads * S, n, D] / [heads * S, n], a row's slots adjacent
};

// Up to kMaxParts table entries passed BY VALUE to a small kernel that writes them to device
// memory: an item table for callers that may not copy from the host (no allocation, no
// memcpy node: a plain kernel launch).
struct TablePack {
  Segment seg;
  SegItem items[kMaxParts];
};

// dtype: 0 = fp16, 1 = bf16.  Return hipSuccess or the launch error.
hipError_t launch_walk(const BlockArgs& a, int dtype, int dim, hipStream_t stream);  // ring_walk_kernel, any BlockMode
// ring_walk64_kernel: the carried-state forward at d = 128 with 64 query rows per wave; only for tables that
// walk64_takes() accepts
hipError_t launch_walk64(const BlockArgs& a, int dtype, int dim, hipStream_t stream);
hipError_t launch_merge(const MergeArgs& a, int dtype, int dim, hipStream_t stream);
// writes pack.seg to *seg_dst and pack.items[0..n) to item_dst
hipError_t launch_write_table(const TablePack& pack, int n, Segment* seg_dst, SegItem* item_dst, hipStream_t stream);

}  // namespace ringattn
