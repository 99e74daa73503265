// Host side of the C ABI declared in include/ringattn.h: parameter validation, plan and
// workspace lifetime, the ring step loop over P virtual ranks, optional hipGraph replay.
// It replaces the host functions of the reference -- set_params_fprop
// (csrc/ring_attention.cu:361-395), run_ring_fwd (:669-704) and ring_attention (:706-722).
#include "ringattn.h"
#include "ringattn_kernels.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <unordered_set>
#include <vector>

namespace {

// Live plan handles.  A handle is valid only while it is in this set, so a second
// destroy (or a garbage pointer) is reported instead of touching freed memory.
std::mutex g_plans_mu;
std::unordered_set<const void*> g_plans;

thread_local int g_last_hip_error = 0;

inline int hip_fail(hipError_t e) {
  g_last_hip_error = (int)e;
  return RINGATTN_ERR_HIP;
}
#define RA_HIP(expr)                          \
  do {                                        \
    hipError_t e__ = (expr);                  \
    if (e__ != hipSuccess) return hip_fail(e__); \
  } while (0)

constexpr float kLog2e = 1.4426950408889634f;

struct Derived {
  int start[RINGATTN_MAX_NPES + 1] = {};  // rank r owns rows [start[r], start[r+1]) of every head
  int max_len = 0;
  bool zigzag = false;  // causal ring over the zigzag layout (without the mask the layouts coincide)
  int64_t S = 0;
  int64_t BH = 0;
  int64_t kv_BH = 0;
  int64_t rows = 0;  // BH * S
  float scale = 0.f;
};

// All checks that need no GPU.  Mirrors what the reference leaves unchecked: its kernel
// has no tail predication (csrc/ring_attention.cu:143-145) and is instantiated for
// dim 64 only (:707-710); here unsupported shapes are refused instead of mis-computed.
int validate(const ringattn_params* p, Derived* d) {
  if (!p) return RINGATTN_ERR_NULL;
  if (p->npes < 1 || p->npes > RINGATTN_MAX_NPES) return RINGATTN_ERR_NPES;
  if (!p->h_seqlen) return RINGATTN_ERR_NULL;
  if (p->dim != 64 && p->dim != 128) return RINGATTN_ERR_DIM;
  if (p->dtype != RINGATTN_DTYPE_FP16 && p->dtype != RINGATTN_DTYPE_BF16) return RINGATTN_ERR_DTYPE;
  if (p->batch < 1 || p->heads < 1) return RINGATTN_ERR_SHAPE;
  if (p->kv_heads < 0 || (p->kv_heads > 0 && p->heads % p->kv_heads != 0)) return RINGATTN_ERR_SHAPE;
  if (p->layout != RINGATTN_LAYOUT_CONTIGUOUS && p->layout != RINGATTN_LAYOUT_ZIGZAG) return RINGATTN_ERR_SHAPE;
  // any positive length (the zigzag layout halves it, so even there); multiples of
  // RINGATTN_TILE waste no part of a tile
  const int granule = p->layout == RINGATTN_LAYOUT_ZIGZAG ? 2 : 1;
  int64_t S = 0;
  int max_len = 0;
  for (int r = 0; r < p->npes; ++r) {
    const int c = p->h_seqlen[r];
    if (c <= 0 || c % granule != 0) return RINGATTN_ERR_SEQLEN;
    S += c;
    if (c > max_len) max_len = c;
  }
  const int64_t BH = (int64_t)p->batch * p->heads;
  if (S > INT32_MAX / 2 || BH > INT32_MAX / 2) return RINGATTN_ERR_SHAPE;
  if (BH * p->npes * p->npes > (int64_t)INT32_MAX / 64) return RINGATTN_ERR_SHAPE;  // grid size
  if (BH * S > (int64_t)1 << 40) return RINGATTN_ERR_SHAPE;
  if (!std::isfinite(p->softmax_scale)) return RINGATTN_ERR_SHAPE;
  if (d) {
    d->start[0] = 0;
    for (int r = 0; r < p->npes; ++r) d->start[r + 1] = d->start[r] + p->h_seqlen[r];
    d->max_len = max_len;
    d->zigzag = p->layout == RINGATTN_LAYOUT_ZIGZAG && p->causal;
    d->S = S;
    d->BH = BH;
    d->kv_BH = p->kv_heads > 0 ? (int64_t)p->batch * p->kv_heads : BH;
    d->rows = BH * S;
    d->scale = p->softmax_scale > 0.f ? p->softmax_scale : 1.0f / std::sqrt((float)p->dim);
  }
  return RINGATTN_OK;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

inline bool half_partials(const ringattn_params& p) { return (p.flags & RINGATTN_FLAG_HALF_PARTIALS) != 0; }
inline bool step_partials(const ringattn_params& p) { return (p.flags & RINGATTN_FLAG_STEP_PARTIALS) != 0; }
inline bool row_partials(const ringattn_params& p) { return (p.flags & RINGATTN_FLAG_ROW_PARTIALS) != 0; }

inline ringattn::WorkItem make_item(int q_start, int q_len, int kv_start, int kv_len, int diag_off, int slot) {
  ringattn::WorkItem w;
  w.q_start = q_start;
  w.q_len = q_len;
  w.kv_start = kv_start;
  w.kv_len = kv_len;
  w.diag_off = diag_off;
  w.slot = slot;
  w.pad0 = w.pad1 = 0;
  return w;
}

// The work of virtual rank r at ring step s: it visits the KV of rank j = (r + s) mod P
// (csrc/ring_attention.cu:463,531,615).  Partials go to slot s.
//   no mask            : all queries of r against all keys of j;
//   causal, contiguous : j > r nothing, j == r diagonal, j < r everything;
//   causal, zigzag     : rank r holds a low half (sequence position r) and a high half
//       (position 2P-1-r) back to back.  The low queries see the low keys of j <= r; the high
//       queries see every low half and the high halves of j >= r.  So: j < r, all queries of
//       r against the low half of j; j == r, the plain diagonal over the whole chunk (its
//       low half precedes its high half in the sequence too); j > r, the high queries of r
//       against the whole chunk of j.  Every rank does the same amount of work.
void append_items(std::vector<ringattn::WorkItem>& out, const Derived& d, int P, bool causal, int r, int s) {
  const int j = (r + s) % P;
  const int q0 = d.start[r], ql = d.start[r + 1] - q0;
  const int k0 = d.start[j], kl = d.start[j + 1] - k0;
  if (!causal) {
    out.push_back(make_item(q0, ql, k0, kl, -1, s));
  } else if (j == r) {
    out.push_back(make_item(q0, ql, k0, kl, 0, s));
  } else if (!d.zigzag) {
    if (j < r) out.push_back(make_item(q0, ql, k0, kl, -1, s));
  } else {
    if (j < r) out.push_back(make_item(q0, ql, k0, kl / 2, -1, s));
    else out.push_back(make_item(q0 + ql / 2, ql / 2, k0, kl, -1, s));
  }
}

// A SEGMENT: rows of one rank that meet the same ring steps, with those steps' key ranges in
// ascending step order -- what one workgroup of the attention kernel walks (the reference's CTA
// walks the steps of its rows the same way, csrc/ring_attention.cu:456-620).  Contiguous
// layouts have one segment per rank; a zigzag rank has two (its low half sees fewer steps).
struct HostSegment {
  int start = 0, len = 0;
  std::vector<ringattn::WorkItem> items;  // restricted to the segment: q_start = start, q_len = len
  uint64_t active = 0;                    // the steps (partial slots) of the items
  int64_t tile_work = 0;                  // keys the busiest q tile of the segment visits
};

void rank_segments(std::vector<HostSegment>& out, const Derived& d, int P, bool causal, int r) {
  std::vector<ringattn::WorkItem> all;
  for (int s = 0; s < P; ++s) append_items(all, d, P, causal, r, s);
  const int q0 = d.start[r], q1 = d.start[r + 1];
  std::vector<int> cut{q0, q1};
  if (d.zigzag) cut.push_back(q0 + (q1 - q0) / 2);
  for (const auto& w : all) {
    cut.push_back(w.q_start);
    cut.push_back(w.q_start + w.q_len);
  }
  std::sort(cut.begin(), cut.end());
  cut.erase(std::unique(cut.begin(), cut.end()), cut.end());
  for (size_t i = 0; i + 1 < cut.size(); ++i) {
    HostSegment sg;
    sg.start = cut[i];
    sg.len = cut[i + 1] - cut[i];
    for (const auto& w : all) {
      if (w.q_start > sg.start || sg.start + sg.len > w.q_start + w.q_len) continue;
      ringattn::WorkItem x = w;
      x.q_start = sg.start;
      x.q_len = sg.len;
      if (w.diag_off >= 0) x.diag_off = w.diag_off + (sg.start - w.q_start);
      sg.items.push_back(x);
      sg.active |= (uint64_t)1 << w.slot;
      sg.tile_work += x.diag_off >= 0 ? std::min<int64_t>(x.kv_len, (int64_t)x.diag_off + sg.len) : x.kv_len;
    }
    if (!sg.items.empty()) out.push_back(sg);
  }
}

// All segments of a forward, busiest first: the attention kernel's workgroups are dispatched in
// this order, so the launch ends on its shortest ones.
std::vector<HostSegment> forward_segments(const Derived& d, int P, bool causal) {
  std::vector<HostSegment> segs;
  for (int r = 0; r < P; ++r) rank_segments(segs, d, P, causal, r);
  std::stable_sort(segs.begin(), segs.end(),
                   [](const HostSegment& x, const HostSegment& y) { return x.tile_work > y.tile_work; });
  return segs;
}

// Workspace of a forward that keeps per-step partials (RINGATTN_FLAG_STEP_PARTIALS; none
// otherwise): one partial block [batch*heads, len] rows per (segment, item) -- only the
// (rank, step) pairs the mask leaves visible -- partial O of every block first (fp32, or fp16
// with RINGATTN_FLAG_HALF_PARTIALS), then the fp32 partial LSEs.
int64_t partial_rows_of(const std::vector<HostSegment>& segs, const Derived& d) {
  int64_t rows = 0;
  for (const auto& sg : segs) rows += (int64_t)sg.items.size() * d.BH * sg.len;
  return rows;
}

size_t workspace_bytes_of(const ringattn_params* p, const Derived& d) {
  if (!step_partials(*p)) return 0;
  const size_t o_elem = half_partials(*p) ? 2 : 4;
  const int64_t rows = partial_rows_of(forward_segments(d, p->npes, p->causal != 0), d);
  return (size_t)rows * ((size_t)p->dim * o_elem + sizeof(float));
}

}  // namespace

// A slice of the device tables: what one block launch runs.
struct TableSlice {
  int seg_begin = 0, seg_count = 0;
  int q_tiles_max = 0;  // kWalkM-row tiles of the longest segment
  bool wide = false;    // every KV range of the slice suits ring_walk64_kernel
  int min_kv = 0;       // the shortest KV range of the slice
};

// ring_walk64_kernel walks whole 32-key tiles, and past the end of its sequence its load streams go round the first
// four tiles of a head: a KV range must be a multiple of 32 keys and hold at least 128.
static bool walk64_takes(const ringattn::SegItem& it) { return it.kv_len % 32 == 0 && it.kv_len >= 128; }
// RINGATTN_WIDE=0 in the environment keeps every forward on ring_walk_kernel (for comparisons)
static bool walk64_enabled() {
  const char* e = std::getenv("RINGATTN_WIDE");
  return !(e && e[0] == '0');
}
// RINGATTN_WIDE_PARTIALS in the environment: 0 keeps the launches that emit per-step partials on ring_walk_kernel,
// 1 puts them on ring_walk64_kernel whenever the shapes allow (tests); unset, the chunk length decides
// RINGATTN_WIDE_D64=0 keeps the d = 64 forwards (state carried) on ring_walk_kernel
static bool walk64_d64_enabled() {
  const char* e = std::getenv("RINGATTN_WIDE_D64");
  return !(e && e[0] == '0');
}
static int walk64_partials_choice() {
  const char* e = std::getenv("RINGATTN_WIDE_PARTIALS");
  return !e ? -1 : (e[0] == '0' ? 0 : 1);
}

struct ringattn_plan {
  ringattn_params p{};
  int seqlen[RINGATTN_MAX_NPES]{};
  Derived d{};
  void* ws = nullptr;
  size_t ws_bytes = 0;
  bool own_ws = false;
  void* o_parts = nullptr;     // partial O rows, fp32 (fp16 with RINGATTN_FLAG_HALF_PARTIALS)
  float* lse_parts = nullptr;  // partial LSE rows
  // Segment / item tables (host copies + device copies made at the first launch).  Three
  // families of slices: the forward (all ring steps of every rank, one launch, partials in the
  // workspace), one ring step of every rank (ringattn_block_fwd, partials in the caller's
  // [batch*heads, S] slot), one step of one rank on rank-local rows (ringattn_rank_step_fwd).
  std::vector<ringattn::Segment> h_segs;
  std::vector<ringattn::SegItem> h_segitems;
  TableSlice fwd;
  std::vector<TableSlice> step;    // [npes]
  std::vector<TableSlice> local;   // [npes * npes]
  // the same schedule as plain work items, for ringattn_plan_work_items
  std::vector<ringattn::WorkItem> h_items;
  int fwd_items = 0;               // h_items[0, fwd_items): the forward, in run order
  std::vector<int> step_begin;     // [npes + 1] slices of h_items, one per ring step
  // merge regions, rank by rank (global rows), then the same with rank-local rows
  std::vector<ringattn::MergeRegion> regions;
  int n_regions = 0;               // global ones; regions[n_regions + i] is regions[i] in local rows
  std::vector<int> region_rank;    // [n_regions]
  int region_max_len = 0;
  // forward only: per XCD, the (segment, head) pairs its workgroups run, heads dealt round-robin
  std::vector<int2> fwd_groups;
  int fwd_groups_per_xcd = 0;
  int2* d_groups = nullptr;
  ringattn::Segment* d_segs = nullptr;
  ringattn::SegItem* d_segitems = nullptr;
  ringattn::MergeRegion* d_regions = nullptr;
  hipEvent_t ev_t0 = nullptr, ev_t1 = nullptr;  // RINGATTN_FLAG_TIMING: around the block launch
  bool timed_forward = false;                    // a forward has recorded them
  bool tables_ready = false;
  // hipGraph replay (RINGATTN_FLAG_GRAPH): one captured graph per pointer set
  hipStream_t cap_stream = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  const void *gq = nullptr, *gk = nullptr, *gv = nullptr;
  void* gout = nullptr;
  float* glse = nullptr;
};

namespace {

// fields of the launch arguments that depend only on the geometry
void fill_geometry(ringattn::BlockArgs& a, const ringattn_params& p, const Derived& d) {
  std::memset(&a, 0, sizeof(a));
  a.bh_stride = d.S * p.dim;
  a.kv_bh_stride = d.S * p.dim;
  a.S = (int)d.S;
  a.BH = (int)d.BH;
  a.heads = p.heads;
  a.kv_group = p.kv_heads > 0 ? p.heads / p.kv_heads : 1;
  a.scale_log2 = d.scale * kLog2e;
  a.half_partials = half_partials(p) ? 1 : 0;
}

inline int q_tiles_of(int len) { return (len + ringattn::kWalkM - 1) / ringattn::kWalkM; }

// Appends one segment with its items to the tables.  part_base(i) / stride: where item i's
// partial block lives.  A masked (diagonal) item runs last and the q tiles go busiest first.
template <class BaseFn>
void push_segment(ringattn_plan* pl, TableSlice& slice, int q_start, int q_len,
                  const std::vector<ringattn::WorkItem>& items, int kv_shift, BaseFn part_base, int part_bh_stride,
                  int part_row_mul = 0) {
  ringattn::Segment sg;
  std::memset(&sg, 0, sizeof(sg));
  sg.q_start = q_start;
  sg.q_len = q_len;
  sg.item_begin = (int)pl->h_segitems.size();
  sg.item_count = (int)items.size();
  sg.last_item = -1;
  for (size_t i = 0; i < items.size(); ++i) {
    const ringattn::WorkItem& w = items[i];
    ringattn::SegItem it;
    std::memset(&it, 0, sizeof(it));
    it.kv_start = w.kv_start - kv_shift;
    it.kv_len = w.kv_len;
    it.diag_off = w.diag_off;
    it.part_bh_stride = part_bh_stride;
    it.part_base = part_base((int)i);
    it.slot = w.slot;
    it.part_row_mul = part_row_mul;
    if (w.diag_off >= 0) {
      sg.last_item = (int)i;
      sg.reverse_tiles = 1;
    }
    pl->h_segitems.push_back(it);
  }
  if (sg.item_count == 1) sg.last_item = -1;
  pl->h_segs.push_back(sg);
  bool wide = true;
  for (size_t i = 0; i < items.size(); ++i) wide = wide && walk64_takes(pl->h_segitems[(size_t)sg.item_begin + i]);
  slice.wide = slice.seg_count == 0 ? wide : (slice.wide && wide);
  for (size_t i = 0; i < items.size(); ++i) {
    const int kv = pl->h_segitems[(size_t)sg.item_begin + i].kv_len;
    slice.min_kv = (slice.seg_count == 0 && i == 0) ? kv : std::min(slice.min_kv, kv);
  }
  ++slice.seg_count;
  slice.q_tiles_max = std::max(slice.q_tiles_max, q_tiles_of(q_len));
}

// The tables of a plan (host side; nothing here touches the GPU).
void build_schedule(ringattn_plan* pl) {
  const int P = pl->p.npes;
  const Derived& d = pl->d;
  const bool causal = pl->p.causal != 0;

  // ---- the forward: every segment with all its steps; partial blocks packed in the workspace
  const std::vector<HostSegment> segs = forward_segments(d, P, causal);
  pl->fwd.seg_begin = 0;
  int64_t next_row = 0;
  for (const auto& sg : segs) {
    const int64_t block_rows = d.BH * sg.len;
    const int64_t base = next_row;
    push_segment(pl, pl->fwd, sg.start, sg.len, sg.items, 0,
                 [&](int i) { return base + (int64_t)i * block_rows; }, sg.len);
    next_row += (int64_t)sg.items.size() * block_rows;
    // the same items in run order (the masked one last), for inspection
    const ringattn::Segment& t = pl->h_segs.back();
    for (int i = 0; i < t.item_count; ++i) {
      int idx = i;
      if (t.last_item >= 0) idx = (i == t.item_count - 1) ? t.last_item : (i >= t.last_item ? i + 1 : i);
      pl->h_items.push_back(sg.items[(size_t)idx]);
    }
  }
  pl->fwd_items = (int)pl->h_items.size();
  // Workgroup order of the forward.  Heads are dealt to the 8 XCDs round-robin; an XCD runs
  // the segments of one head after the other (busiest first within a head), so the ranks of
  // a head, which read the same K and V, follow each other through that XCD's L2.  Only when
  // the heads divide evenly; otherwise the kernel's arithmetic mapping spreads (segment,
  // head) pairs over the XCDs.
  if (d.BH % 8 == 0) {
    const int heads_per_xcd = (int)(d.BH / 8);
    pl->fwd_groups_per_xcd = heads_per_xcd * pl->fwd.seg_count;
    pl->fwd_groups.assign((size_t)8 * pl->fwd_groups_per_xcd, int2{-1, -1});
    for (int x = 0; x < 8; ++x) {
      size_t pos = (size_t)x * pl->fwd_groups_per_xcd;
      for (int hh = 0; hh < heads_per_xcd; ++hh)
        for (int sgi = 0; sgi < pl->fwd.seg_count; ++sgi) pl->fwd_groups[pos++] = int2{sgi, hh * 8 + x};
    }
  }

  // ---- one ring step of every rank: partials at the rows of the queries in a [BH, S] slot
  for (int s = 0; s < P; ++s) {
    pl->step_begin.push_back((int)pl->h_items.size());
    TableSlice sl;
    sl.seg_begin = (int)pl->h_segs.size();
    std::vector<ringattn::WorkItem> one;
    for (int r = 0; r < P; ++r) {
      one.clear();
      append_items(one, d, P, causal, r, s);
      for (const auto& w : one) {
        pl->h_items.push_back(w);
        const std::vector<ringattn::WorkItem> v1{w};
        push_segment(pl, sl, w.q_start, w.q_len, v1, 0, [&](int) { return (int64_t)w.q_start; }, (int)d.S,
                     row_partials(pl->p) ? P : 0);
      }
    }
    pl->step.push_back(sl);
  }
  pl->step_begin.push_back((int)pl->h_items.size());

  // ---- one step of one rank in rank-local rows (queries from 0, keys from 0 of the visited chunk)
  for (int r = 0; r < P; ++r)
    for (int s = 0; s < P; ++s) {
      TableSlice sl;
      sl.seg_begin = (int)pl->h_segs.size();
      std::vector<ringattn::WorkItem> one;
      append_items(one, d, P, causal, r, s);
      const int q0 = d.start[r], rows = d.start[r + 1] - q0, k0 = d.start[(r + s) % P];
      for (const auto& w : one) {
        const std::vector<ringattn::WorkItem> v1{w};
        push_segment(pl, sl, w.q_start - q0, w.q_len, v1, k0, [&](int) { return (int64_t)(w.q_start - q0); }, rows,
                     row_partials(pl->p) ? P : 0);
      }
      pl->local.push_back(sl);
    }

  // ---- merge regions of caller-held per-step partials, rank by rank
  for (int r = 0; r < P; ++r) {
    std::vector<HostSegment> rs;
    rank_segments(rs, d, P, causal, r);
    for (const auto& sg : rs) {
      pl->regions.push_back(ringattn::MergeRegion{sg.start, sg.len, sg.active});
      pl->region_rank.push_back(r);
      pl->region_max_len = std::max(pl->region_max_len, sg.len);
    }
  }
  pl->n_regions = (int)pl->regions.size();
  for (int i = 0; i < pl->n_regions; ++i) {
    ringattn::MergeRegion m = pl->regions[(size_t)i];
    m.start -= d.start[pl->region_rank[(size_t)i]];
    pl->regions.push_back(m);
  }
}

// Device copies of the tables and the timing events: made at the first launch, outside any capture.
int ensure_tables(ringattn_plan* pl) {
  if (pl->tables_ready) return RINGATTN_OK;
  // a call that failed half way is resumed: nothing is created twice
  const size_t seg_bytes = pl->h_segs.size() * sizeof(ringattn::Segment);
  const size_t item_bytes = pl->h_segitems.size() * sizeof(ringattn::SegItem);
  const size_t reg_bytes = pl->regions.size() * sizeof(ringattn::MergeRegion);
  if (!pl->d_segs) RA_HIP(hipMalloc((void**)&pl->d_segs, seg_bytes));
  if (!pl->d_segitems) RA_HIP(hipMalloc((void**)&pl->d_segitems, item_bytes));
  if (!pl->d_regions) RA_HIP(hipMalloc((void**)&pl->d_regions, reg_bytes));
  if (!pl->fwd_groups.empty()) {
    const size_t grp_bytes = pl->fwd_groups.size() * sizeof(int2);
    if (!pl->d_groups) RA_HIP(hipMalloc((void**)&pl->d_groups, grp_bytes));
    RA_HIP(hipMemcpy(pl->d_groups, pl->fwd_groups.data(), grp_bytes, hipMemcpyHostToDevice));
  }
  RA_HIP(hipMemcpy(pl->d_segs, pl->h_segs.data(), seg_bytes, hipMemcpyHostToDevice));
  RA_HIP(hipMemcpy(pl->d_segitems, pl->h_segitems.data(), item_bytes, hipMemcpyHostToDevice));
  RA_HIP(hipMemcpy(pl->d_regions, pl->regions.data(), reg_bytes, hipMemcpyHostToDevice));
  if (pl->p.flags & RINGATTN_FLAG_TIMING) {
    if (!pl->ev_t0) RA_HIP(hipEventCreate(&pl->ev_t0));
    if (!pl->ev_t1) RA_HIP(hipEventCreate(&pl->ev_t1));
  }
  pl->tables_ready = true;
  return RINGATTN_OK;
}

// ring_walk64_kernel runs the launch of a slice when every KV range suits it and d = 128.  The launches that emit
// partials go by the forward's ranges, so that the forward and the steps run one by one keep giving the same bits.
// A chunk walked on its own costs ring_walk64_kernel a start and a drain of its pipeline, and its four waves move the
// partials (stores, merge) more slowly than the eight of ring_walk_kernel.  It wins where its loop is well ahead --
// causal forwards, whose masked tiles it skips wave by wave -- and the chunks are long; measured with per-step
// partials, ring_walk64_kernel against ring_walk_kernel: cfg4 (causal, 4096 keys per chunk) 1130 against 1050
// TFLOP/s, cfg5 (not causal, 8192) 1060 against 1145, cfg3 (not causal, 512) 590 against 700.
constexpr int kWidePartialsMinKeys = 2048;
bool slice_takes_walk64(const ringattn_plan* pl, const TableSlice& sl, int mode) {
  if (!sl.wide || !walk64_enabled()) return false;
  if (mode != ringattn::kBlockCarryState) {
    const int choice = walk64_partials_choice();
    if (pl->p.dim != 128 || choice == 0 || !pl->fwd.wide) return false;
    if (choice < 0 && !(pl->p.causal && pl->fwd.min_kv >= kWidePartialsMinKeys)) return false;
    return true;
  }
  return pl->p.dim == 128 || (pl->p.dim == 64 && walk64_d64_enabled());
}

// A block launch over a slice of the tables.
int launch_slice(const ringattn_plan* pl, const TableSlice& sl, ringattn::BlockArgs& a, hipStream_t stream) {
  if (sl.seg_count == 0) return RINGATTN_OK;
  a.segs = pl->d_segs + sl.seg_begin;
  a.items = pl->d_segitems;
  a.n_segs = sl.seg_count;
  a.q_tiles_max = sl.q_tiles_max;
  if (slice_takes_walk64(pl, sl, a.mode))
    RA_HIP(ringattn::launch_walk64(a, pl->p.dtype, pl->p.dim, stream));
  else
    RA_HIP(ringattn::launch_walk(a, pl->p.dtype, pl->p.dim, stream));
  return RINGATTN_OK;
}

// The ring step loop (csrc/ring_attention.cu:456-620) and the epilogue (:621-664), ONE launch:
// every workgroup walks the ring steps of its 256 rows with the softmax state carried in
// registers, like the reference's CTA (:439-443,597).  With RINGATTN_FLAG_STEP_PARTIALS it
// writes a partial (O, LSE) per step instead and merges them at the end.
int run_forward(ringattn_plan* pl, const void* q, const void* k, const void* v, void* out,
                float* lse, hipStream_t stream) {
  const bool timing = (pl->p.flags & RINGATTN_FLAG_TIMING) && !(pl->p.flags & RINGATTN_FLAG_GRAPH);
  ringattn::BlockArgs a;
  fill_geometry(a, pl->p, pl->d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.o_part = pl->o_parts;
  a.lse_part = pl->lse_parts;
  a.out = out;
  a.lse = lse;
  a.mode = step_partials(pl->p) ? ringattn::kBlockPartialsMerged : ringattn::kBlockCarryState;
  a.groups = pl->d_groups;
  a.groups_per_xcd = pl->fwd_groups_per_xcd;
  if (timing) RA_HIP(hipEventRecord(pl->ev_t0, stream));
  const int rc = launch_slice(pl, pl->fwd, a, stream);
  if (rc != RINGATTN_OK) return rc;
  if (timing) {
    RA_HIP(hipEventRecord(pl->ev_t1, stream));
    pl->timed_forward = true;
  }
  return RINGATTN_OK;
}

void drop_graph(ringattn_plan* pl) {
  if (pl->exec) (void)hipGraphExecDestroy(pl->exec);
  if (pl->graph) (void)hipGraphDestroy(pl->graph);
  pl->exec = nullptr;
  pl->graph = nullptr;
}

inline bool plan_ok(const ringattn_plan* pl) {
  if (!pl) return false;
  std::lock_guard<std::mutex> lk(g_plans_mu);
  return g_plans.count(pl) != 0;
}

// ---- the reference-shaped call for one rank (ringattn_ring_attention and its variant that
// allocates nothing) ------------------------------------------------------------------------
// Device scratch of one call: the segment + item table the attention kernel reads (the softmax state
// is carried in registers across the ring steps, so there are no partials to park).
struct RankCall {
  ringattn_params p;
  Derived d;
  ringattn::TablePack pack;  // the visible ring steps of the rank in ring order
  int n_parts = 0;
  int c = 0;                // rows of this rank
  size_t scratch_bytes = 0;
};

int prepare_rank_call(RankCall* rc, const void* q, const void* k, const void* v, void* out, int npes, int mype,
                      const int* seqlen, int dim, int max_seq, int dtype, int causal, float softmax_scale) {
  ringattn_params& p = rc->p;
  std::memset(&p, 0, sizeof(p));
  p.npes = npes;
  p.h_seqlen = seqlen;
  p.dim = dim;
  p.softmax_scale = softmax_scale;
  p.batch = 1;
  p.heads = 1;
  p.dtype = dtype;
  p.causal = causal;
  int err = validate(&p, &rc->d);
  if (err != RINGATTN_OK) return err;
  const Derived& d = rc->d;
  if (mype < 0 || mype >= npes) return RINGATTN_ERR_RANK;
  if (max_seq < d.max_len) return RINGATTN_ERR_SEQLEN;
  if (!q || !k || !v || !out) return RINGATTN_ERR_NULL;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return RINGATTN_ERR_ALIGN;
  // the query rows are local to the caller's rank-sized q and out buffers
  const int c = rc->c = d.start[mype + 1] - d.start[mype];
  std::memset(&rc->pack, 0, sizeof(rc->pack));
  ringattn::Segment& sg = rc->pack.seg;
  sg.q_start = 0;
  sg.q_len = c;
  sg.item_begin = 0;
  sg.last_item = -1;
  rc->n_parts = 0;
  for (int s = 0; s < npes; ++s) {
    const int j = (mype + s) % npes;
    if (causal && j > mype) continue;
    ringattn::SegItem& it = rc->pack.items[rc->n_parts];
    it.kv_start = d.start[j];
    it.kv_len = d.start[j + 1] - d.start[j];
    it.diag_off = (causal && j == mype) ? 0 : -1;
    it.part_bh_stride = c;
    it.part_base = (int64_t)rc->n_parts * c;
    it.slot = s;
    if (it.diag_off >= 0) {
      sg.last_item = rc->n_parts;
      sg.reverse_tiles = 1;
    }
    ++rc->n_parts;
  }
  sg.item_count = rc->n_parts;
  if (rc->n_parts == 1) sg.last_item = -1;
  rc->scratch_bytes = sizeof(ringattn::Segment) + (size_t)rc->n_parts * sizeof(ringattn::SegItem);
  return RINGATTN_OK;
}

// The table (written by a kernel from its arguments), then the attention kernel: two launches on
// `stream`, nothing is allocated or copied from the host.
// `scratch`: rc.scratch_bytes of device memory, 32-byte aligned.
int run_rank_call(const RankCall& rc, void* scratch, const void* q, const void* k, const void* v, void* out,
                  float* lse, hipStream_t stream) {
  const int dim = rc.p.dim, c = rc.c, n_parts = rc.n_parts;
  ringattn::Segment* d_seg = (ringattn::Segment*)scratch;
  ringattn::SegItem* d_items = (ringattn::SegItem*)(d_seg + 1);
  RA_HIP(ringattn::launch_write_table(rc.pack, n_parts, d_seg, d_items, stream));
  ringattn::BlockArgs a;
  fill_geometry(a, rc.p, rc.d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.out = out;
  a.lse = lse;  // may be NULL
  a.mode = ringattn::kBlockCarryState;
  a.segs = d_seg;
  a.items = d_items;
  a.n_segs = 1;
  a.q_tiles_max = q_tiles_of(c);
  a.bh_stride = (int64_t)c * dim;  // q and out hold this rank's rows only; k and v the whole sequence
  a.S = c;
  bool wide = (dim == 128 || (dim == 64 && walk64_d64_enabled())) && walk64_enabled();
  for (int i = 0; i < n_parts; ++i) wide = wide && walk64_takes(rc.pack.items[i]);
  if (wide) RA_HIP(ringattn::launch_walk64(a, rc.p.dtype, dim, stream));
  else RA_HIP(ringattn::launch_walk(a, rc.p.dtype, dim, stream));
  return RINGATTN_OK;
}

// Static device scratch of ringattn_ring_attention_noalloc.  In host code the array's name is
// only a handle for hipGetSymbolAddress; the device address is looked up once per device
// (each GPU holds its own copy of the array) and kept.
// A call's table (32 bytes + 32 per visible ring step) takes the next slice of the array, round robin: the walk
// kernel reads its table for as long as it runs, so a later call must not overwrite it while an earlier one is still
// in flight on another stream.  With the tables of an 8-step ring (288 bytes) fourteen calls can be in flight
// before a slice is used again; a call whose table needs more than half the array has it to itself.
constexpr size_t kScratchBytes = 4096;
static_assert(kScratchBytes >= sizeof(ringattn::Segment) + RINGATTN_MAX_NPES * sizeof(ringattn::SegItem),
              "the table of the largest ring fits");
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};
size_t g_scratch_next[kMaxDevices] = {};

int device_scratch(size_t bytes, void** slice) {
  int dev = -1;
  RA_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return RINGATTN_ERR_SHAPE;
  if (bytes > kScratchBytes) return RINGATTN_ERR_WORKSPACE;
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    RA_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return RINGATTN_ERR_HIP;
    g_scratch_ptr[dev] = ptr;
  }
  const size_t need = (bytes + 31) & ~(size_t)31;   // tables are read with 16-byte scalar loads
  if (g_scratch_next[dev] + need > kScratchBytes) g_scratch_next[dev] = 0;
  *slice = (char*)g_scratch_ptr[dev] + g_scratch_next[dev];
  g_scratch_next[dev] += need;
  return RINGATTN_OK;
}

// merge launch over `count` regions of the plan's device table starting at `first`
int launch_regions(const ringattn_plan* pl, int first, int count, int max_len, int rows_per_head, int64_t part_stride_rows,
                   const void* o_parts, const float* lse_parts, void* out, float* lse, hipStream_t stream) {
  ringattn::MergeArgs m;
  std::memset(&m, 0, sizeof(m));
  m.o_parts = o_parts;
  m.lse_parts = lse_parts;
  m.out = out;
  m.lse = lse;
  m.regions = pl->d_regions + first;
  m.n_regions = count;
  m.max_len = max_len;
  m.heads = (int)pl->d.BH;
  m.S = rows_per_head;
  m.part_stride_rows = part_stride_rows;
  m.half_partials = half_partials(pl->p) ? 1 : 0;
  m.row_mul = row_partials(pl->p) ? pl->p.npes : 0;
  RA_HIP(ringattn::launch_merge(m, pl->p.dtype, pl->p.dim, stream));
  return RINGATTN_OK;
}

}  // namespace

extern "C" {

size_t ringattn_workspace_bytes(const ringattn_params* params) {
  Derived d;
  if (validate(params, &d) != RINGATTN_OK) return 0;
  return workspace_bytes_of(params, d);
}

int ringattn_plan_create(const ringattn_params* params, void* workspace, size_t workspace_bytes,
                         ringattn_plan** plan_out) {
  if (!plan_out) return RINGATTN_ERR_NULL;
  *plan_out = nullptr;
  Derived d;
  int rc = validate(params, &d);
  if (rc != RINGATTN_OK) return rc;
  const size_t need = workspace_bytes_of(params, d);
  if (workspace) {
    if (workspace_bytes < need) return RINGATTN_ERR_WORKSPACE;
    if (!aligned16(workspace)) return RINGATTN_ERR_ALIGN;
  }
  ringattn_plan* pl = new (std::nothrow) ringattn_plan();
  if (!pl) return RINGATTN_ERR_ALLOC;
  pl->p = *params;
  std::memcpy(pl->seqlen, params->h_seqlen, sizeof(int) * (size_t)params->npes);
  pl->p.h_seqlen = pl->seqlen;
  pl->d = d;
  pl->ws_bytes = need;
  if (workspace) {
    pl->ws = workspace;
    pl->own_ws = false;
  } else if (need > 0) {
    hipError_t e = hipMalloc(&pl->ws, need);
    if (e != hipSuccess) {
      delete pl;
      g_last_hip_error = (int)e;
      return e == hipErrorOutOfMemory ? RINGATTN_ERR_ALLOC : RINGATTN_ERR_HIP;
    }
    pl->own_ws = true;
  }
  build_schedule(pl);
  const size_t part_rows = need / ((size_t)params->dim * (half_partials(*params) ? 2 : 4) + sizeof(float));
  pl->o_parts = pl->ws;
  pl->lse_parts = (float*)((char*)pl->ws + part_rows * params->dim * (half_partials(*params) ? 2 : 4));
  {
    std::lock_guard<std::mutex> lk(g_plans_mu);
    g_plans.insert(pl);
  }
  *plan_out = pl;
  return RINGATTN_OK;
}

int ringattn_plan_destroy(ringattn_plan* plan) {
  {
    std::lock_guard<std::mutex> lk(g_plans_mu);
    if (!plan || g_plans.erase(plan) == 0) return RINGATTN_ERR_PLAN;
  }
  int rc = RINGATTN_OK;
  drop_graph(plan);
  if (plan->cap_stream) (void)hipStreamDestroy(plan->cap_stream);
  // whatever ensure_tables() got to create, also after a failure half way
  if (plan->ev_t0) (void)hipEventDestroy(plan->ev_t0);
  if (plan->ev_t1) (void)hipEventDestroy(plan->ev_t1);
  if (plan->d_segs) (void)hipFree(plan->d_segs);
  if (plan->d_segitems) (void)hipFree(plan->d_segitems);
  if (plan->d_regions) (void)hipFree(plan->d_regions);
  if (plan->d_groups) (void)hipFree(plan->d_groups);
  if (plan->own_ws && plan->ws) {
    hipError_t e = hipFree(plan->ws);
    if (e != hipSuccess) rc = hip_fail(e);
  }
  delete plan;
  return rc;
}

int ringattn_fwd(ringattn_plan* plan, const void* q, const void* k, const void* v, void* out,
                 float* lse, void* stream_) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!q || !k || !v || !out || !lse) return RINGATTN_ERR_NULL;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || ((uintptr_t)lse & 3u)) return RINGATTN_ERR_ALIGN;
  hipStream_t stream = (hipStream_t)stream_;
  int rc0 = ensure_tables(plan);
  if (rc0 != RINGATTN_OK) return rc0;
  if (!(plan->p.flags & RINGATTN_FLAG_GRAPH)) return run_forward(plan, q, k, v, out, lse, stream);

  // hipGraph replay: the launch of a forward is captured once per pointer set on a private
  // stream (kernel nodes only, no memset nodes) and replayed on the caller's stream.
  if (!plan->exec || plan->gq != q || plan->gk != k || plan->gv != v || plan->gout != out || plan->glse != lse) {
    drop_graph(plan);
    if (!plan->cap_stream) RA_HIP(hipStreamCreateWithFlags(&plan->cap_stream, hipStreamNonBlocking));
    RA_HIP(hipStreamBeginCapture(plan->cap_stream, hipStreamCaptureModeThreadLocal));
    int rc = run_forward(plan, q, k, v, out, lse, plan->cap_stream);
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(plan->cap_stream, &g);
    if (rc != RINGATTN_OK) {
      if (g) (void)hipGraphDestroy(g);
      return rc;
    }
    if (e != hipSuccess) return hip_fail(e);
    plan->graph = g;
    e = hipGraphInstantiate(&plan->exec, plan->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
      drop_graph(plan);
      return hip_fail(e);
    }
    plan->gq = q;
    plan->gk = k;
    plan->gv = v;
    plan->gout = out;
    plan->glse = lse;
  }
  RA_HIP(hipGraphLaunch(plan->exec, stream));
  return RINGATTN_OK;
}

int ringattn_block_fwd(ringattn_plan* plan, int step, const void* q, const void* k, const void* v,
                       void* o_part, float* lse_part, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!q || !k || !v || !o_part || !lse_part) return RINGATTN_ERR_NULL;
  if (step < 0 || step >= plan->p.npes) return RINGATTN_ERR_RANK;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o_part) || ((uintptr_t)lse_part & 3u)) return RINGATTN_ERR_ALIGN;
  int rc = ensure_tables(plan);
  if (rc != RINGATTN_OK) return rc;
  ringattn::BlockArgs a;
  fill_geometry(a, plan->p, plan->d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.o_part = o_part;
  a.lse_part = lse_part;
  return launch_slice(plan, plan->step[(size_t)step], a, (hipStream_t)stream);
}

int ringattn_merge_ring(ringattn_plan* plan, const void* o_parts, const float* lse_parts, void* out,
                        float* lse, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (!aligned16(o_parts) || !aligned16(out) || ((uintptr_t)lse_parts & 3u) || ((uintptr_t)lse & 3u)) return RINGATTN_ERR_ALIGN;
  int rc = ensure_tables(plan);
  if (rc != RINGATTN_OK) return rc;
  // ONE launch: a grid row per region
  return launch_regions(plan, 0, plan->n_regions, plan->region_max_len, (int)plan->d.S, plan->d.rows, o_parts, lse_parts,
                        out, lse, (hipStream_t)stream);
}

int ringattn_rank_step_fwd(ringattn_plan* plan, int rank, int step, const void* q, const void* k_chunk,
                           const void* v_chunk, void* o_part, float* lse_part, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!q || !k_chunk || !v_chunk || !o_part || !lse_part) return RINGATTN_ERR_NULL;
  const int P = plan->p.npes;
  if (rank < 0 || rank >= P || step < 0 || step >= P) return RINGATTN_ERR_RANK;
  if (!aligned16(q) || !aligned16(k_chunk) || !aligned16(v_chunk) || !aligned16(o_part) || ((uintptr_t)lse_part & 3u)) return RINGATTN_ERR_ALIGN;
  int rc = ensure_tables(plan);
  if (rc != RINGATTN_OK) return rc;
  const Derived& d = plan->d;
  const int j = (rank + step) % P;
  const int64_t q_rows = d.start[rank + 1] - d.start[rank], kv_rows = d.start[j + 1] - d.start[j];
  ringattn::BlockArgs a;
  fill_geometry(a, plan->p, d);
  a.q = q;
  a.k = k_chunk;
  a.v = v_chunk;
  a.o_part = o_part;
  a.lse_part = lse_part;
  a.bh_stride = q_rows * plan->p.dim;      // every tensor holds one rank's rows only
  a.kv_bh_stride = kv_rows * plan->p.dim;
  a.S = (int)q_rows;
  // an empty slice: nothing of the visited chunk is visible to this rank
  return launch_slice(plan, plan->local[(size_t)rank * P + step], a, (hipStream_t)stream);
}

int ringattn_rank_merge(ringattn_plan* plan, int rank, const void* o_parts, const float* lse_parts, void* out,
                        float* lse, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (rank < 0 || rank >= plan->p.npes) return RINGATTN_ERR_RANK;
  if (!aligned16(o_parts) || !aligned16(out) || ((uintptr_t)lse_parts & 3u) || ((uintptr_t)lse & 3u)) return RINGATTN_ERR_ALIGN;
  int rc = ensure_tables(plan);
  if (rc != RINGATTN_OK) return rc;
  const Derived& d = plan->d;
  const int rows = d.start[rank + 1] - d.start[rank];
  int first = -1, count = 0, max_len = 0;  // the regions of a rank are consecutive
  for (int i = 0; i < plan->n_regions; ++i)
    if (plan->region_rank[(size_t)i] == rank) {
      if (first < 0) first = i;
      ++count;
      max_len = std::max(max_len, plan->regions[(size_t)i].len);
    }
  if (count == 0) return RINGATTN_OK;
  return launch_regions(plan, plan->n_regions + first, count, max_len, rows, d.BH * (int64_t)rows, o_parts, lse_parts,
                        out, lse, (hipStream_t)stream);
}

int ringattn_plan_work_items(const ringattn_plan* plan, int step, ringattn_work_item* out, int capacity, int* n_out) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!n_out || (capacity > 0 && !out)) return RINGATTN_ERR_NULL;
  if (step < -1 || step >= plan->p.npes) return RINGATTN_ERR_RANK;
  const int begin = step < 0 ? 0 : plan->step_begin[(size_t)step];
  const int end = step < 0 ? plan->fwd_items : plan->step_begin[(size_t)step + 1];
  *n_out = end - begin;
  for (int i = begin; i < end && i - begin < capacity; ++i) {
    const ringattn::WorkItem& w = plan->h_items[(size_t)i];
    out[i - begin] = ringattn_work_item{w.q_start, w.q_len, w.kv_start, w.kv_len, w.diag_off, w.slot};
  }
  return RINGATTN_OK;
}

int ringattn_plan_launch_times(ringattn_plan* plan, float* ms, int capacity, int* n_out) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!n_out || (capacity > 0 && !ms)) return RINGATTN_ERR_NULL;
  if (!plan->timed_forward) return RINGATTN_ERR_PLAN;
  *n_out = 1;
  if (capacity > 0) {
    RA_HIP(hipEventSynchronize(plan->ev_t1));
    RA_HIP(hipEventElapsedTime(&ms[0], plan->ev_t0, plan->ev_t1));
  }
  return RINGATTN_OK;
}

const char* ringattn_plan_forward_kernel(const ringattn_plan* plan) {
  if (!plan_ok(plan)) return nullptr;
  const int mode = step_partials(plan->p) ? ringattn::kBlockPartialsMerged : ringattn::kBlockCarryState;
  return slice_takes_walk64(plan, plan->fwd, mode) ? "ring_walk64_kernel" : "ring_walk_kernel";
}

int ringattn_plan_merge_regions(const ringattn_plan* plan, int* start, int* len, uint64_t* active, int capacity, int* n_out) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!n_out || (capacity > 0 && (!start || !len || !active))) return RINGATTN_ERR_NULL;
  const int n = plan->n_regions;
  *n_out = n;
  for (int i = 0; i < n && i < capacity; ++i) {
    const ringattn::MergeRegion& m = plan->regions[(size_t)i];
    start[i] = m.start;
    len[i] = m.len;
    active[i] = m.active;
  }
  return RINGATTN_OK;
}

int ringattn_merge(const float* o_parts, const float* lse_parts, int n_parts, int64_t rows, int dim,
                   int dtype, void* out, float* lse, void* stream) {
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (n_parts < 1 || n_parts > ringattn::kMaxParts) return RINGATTN_ERR_NPES;
  if (dim != 64 && dim != 128) return RINGATTN_ERR_DIM;
  if (dtype != RINGATTN_DTYPE_FP16 && dtype != RINGATTN_DTYPE_BF16) return RINGATTN_ERR_DTYPE;
  if (rows < 0 || rows > ((int64_t)1 << 40)) return RINGATTN_ERR_SHAPE;
  if (!aligned16(o_parts) || !aligned16(out)) return RINGATTN_ERR_ALIGN;
  // one launch per 2^30 rows (a launch's row count is an int)
  const int64_t kChunk = (int64_t)1 << 30;
  for (int64_t r0 = 0; r0 < rows; r0 += kChunk) {
    const int len = (int)std::min(kChunk, rows - r0);
    ringattn::MergeArgs m;
    std::memset(&m, 0, sizeof(m));
    m.o_parts = o_parts + r0 * dim;
    m.lse_parts = lse_parts + r0;
    m.out = (char*)out + r0 * dim * 2;
    m.lse = lse + r0;
    m.single = ringattn::MergeRegion{0, len, n_parts >= 64 ? ~(uint64_t)0 : (((uint64_t)1 << n_parts) - 1)};
    m.n_regions = 1;
    m.max_len = len;
    m.heads = 1;
    m.S = len;
    m.part_stride_rows = rows;
    RA_HIP(ringattn::launch_merge(m, dtype, dim, (hipStream_t)stream));
  }
  return RINGATTN_OK;
}

int ringattn_ring_attention(const void* q, const void* k, const void* v, void* out, float* lse,
                            int npes, int mype, const int* seqlen, int dim, int max_seq,
                            int dtype, int causal, float softmax_scale) {
  RankCall rc_;
  int rc = prepare_rank_call(&rc_, q, k, v, out, npes, mype, seqlen, dim, max_seq, dtype, causal, softmax_scale);
  if (rc != RINGATTN_OK) return rc;
  // per-call scratch, like the reference's per-call allocations (:383-394) but freed
  void* ws = nullptr;
  RA_HIP(hipMalloc(&ws, rc_.scratch_bytes));
  rc = run_rank_call(rc_, ws, q, k, v, out, lse, nullptr);
  hipError_t e = hipDeviceSynchronize();  // blocking, as csrc/ring_attention.cu:721
  if (rc == RINGATTN_OK && e != hipSuccess) rc = hip_fail(e);
  (void)hipFree(ws);
  return rc;
}

size_t ringattn_noalloc_scratch_bytes(void) { return kScratchBytes; }

int ringattn_ring_attention_noalloc(const void* q, const void* k, const void* v, void* out, float* lse,
                                    int npes, int mype, const int* seqlen, int dim, int max_seq,
                                    int dtype, int causal, float softmax_scale, void* stream) {
  RankCall rc_;
  int rc = prepare_rank_call(&rc_, q, k, v, out, npes, mype, seqlen, dim, max_seq, dtype, causal, softmax_scale);
  if (rc != RINGATTN_OK) return rc;
  void* slice = nullptr;
  rc = device_scratch(rc_.scratch_bytes, &slice);
  if (rc != RINGATTN_OK) return rc;
  return run_rank_call(rc_, slice, q, k, v, out, lse, (hipStream_t)stream);
}

const char* ringattn_strerror(int code) {
  switch (code) {
    case RINGATTN_OK: return "ok";
    case RINGATTN_ERR_NULL: return "a required pointer is NULL";
    case RINGATTN_ERR_NPES: return "npes out of range";
    case RINGATTN_ERR_DIM: return "dim must be 64 or 128";
    case RINGATTN_ERR_DTYPE: return "dtype must be fp16 (0) or bf16 (1)";
    case RINGATTN_ERR_SEQLEN: return "per-rank sequence lengths must be positive (even with the zigzag layout), and max_seq at least the longest";
    case RINGATTN_ERR_SHAPE: return "batch/heads/kv_heads/layout/scale invalid or sizes overflow";
    case RINGATTN_ERR_WORKSPACE: return "workspace too small";
    case RINGATTN_ERR_RANK: return "rank or step outside [0, npes)";
    case RINGATTN_ERR_PLAN: return "invalid or destroyed plan";
    case RINGATTN_ERR_HIP: return "HIP runtime error";
    case RINGATTN_ERR_ALLOC: return "allocation failed";
    case RINGATTN_ERR_ALIGN: return "pointer not sufficiently aligned";
    default: return "unknown ringattn error";
  }
}

int ringattn_last_hip_error(void) { return g_last_hip_error; }

}  // extern "C"
