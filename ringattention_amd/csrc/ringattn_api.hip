// Host side of the C ABI declared in include/ringattn.h: parameter validation, plan and
// workspace lifetime, the ring step loop over P virtual ranks, optional hipGraph replay.
// It replaces the host functions of the reference -- set_params_fprop
// (csrc/ring_attention.cu:361-395), run_ring_fwd (:669-704) and ring_attention (:706-722).
#include "ringattn.h"
#include "ringattn_kernels.h"

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

constexpr int kMaxGroups = 8;  // block launches per forward
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

// partial O of every slot (fp32, or fp16 with RINGATTN_FLAG_HALF_PARTIALS), then the fp32 partial LSEs
size_t workspace_bytes_of(const ringattn_params* p, const Derived& d) {
  const size_t o_elem = half_partials(*p) ? 2 : 4;
  return (size_t)p->npes * (size_t)d.rows * ((size_t)p->dim * o_elem + sizeof(float));
}

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

}  // namespace

// One block launch of the forward: all ring steps of a few virtual ranks.
struct LaunchGroup {
  int item_begin, item_count;      // slice of the item table
  int region_begin, region_count;  // slice of `regions`: what is merged after this launch
};

// Rows [start, start + len) of every head share one set of active partial slots.
struct MergeRegion {
  int start, len;
  uint64_t active;
};

struct ringattn_plan {
  ringattn_params p{};
  int seqlen[RINGATTN_MAX_NPES]{};
  Derived d{};
  void* ws = nullptr;
  size_t ws_bytes = 0;
  bool own_ws = false;
  void* o_parts = nullptr;     // [npes, rows, dim] fp32 (fp16 with RINGATTN_FLAG_HALF_PARTIALS)
  float* lse_parts = nullptr;  // [npes, rows]
  // Item table (host copy + device copy made at the first forward): first the launch
  // schedule of ringattn_fwd, then one list per ring step for ringattn_block_fwd.
  // The ring steps of different ranks are independent (each item writes its own rows of its
  // step's partial slot), so the forward is issued as a few launches that each hold ALL
  // steps of a few ranks; the merge of those ranks then runs on a second stream underneath
  // the next launch.
  std::vector<ringattn::WorkItem> h_items;
  std::vector<LaunchGroup> groups;
  std::vector<MergeRegion> regions;  // group by group, then (from all_regions on) rank by rank
  int all_regions = 0;
  std::vector<int> step_begin;       // [npes + 1] slices of h_items, one per ring step
  std::vector<int> local_begin;      // [npes * npes + 1] slices of h_items: the items of (rank, step) in
                                     // rank-local rows (queries from 0, keys from 0 of the visited chunk)
  int q_tiles_max = 0;
  ringattn::WorkItem* d_items = nullptr;
  hipStream_t merge_stream = nullptr;
  hipEvent_t ev_group[kMaxGroups]{};
  hipEvent_t ev_done = nullptr;
  hipEvent_t ev_t0[kMaxGroups]{}, ev_t1[kMaxGroups]{};  // RINGATTN_FLAG_TIMING: around each block launch
  bool timed_forward = false;                            // a forward has recorded them
  bool streams_ready = false;
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
void fill_geometry(ringattn::BlockStepArgs& a, const ringattn_params& p, const Derived& d) {
  a.bh_stride = d.S * p.dim;
  a.kv_bh_stride = d.S * p.dim;
  a.part_stride_rows = d.rows;
  a.S = (int)d.S;
  a.slot_bias = 0;
  a.BH = (int)d.BH;
  a.heads = p.heads;
  a.kv_group = p.kv_heads > 0 ? p.heads / p.kv_heads : 1;
  a.scale_log2 = d.scale * kLog2e;
  a.half_partials = half_partials(p) ? 1 : 0;
}

// The rows of rank r that share a set of active slots, with that set: slot s is active for
// a row iff the item list of (r, s) covers the row.
void append_regions(std::vector<MergeRegion>& out, const Derived& d, int P, bool causal, int r) {
  const int q0 = d.start[r], ql = d.start[r + 1] - q0;
  const int parts = d.zigzag ? 2 : 1;
  for (int i = 0; i < parts; ++i) {
    MergeRegion m;
    m.start = q0 + i * (ql / parts);
    m.len = ql / parts;
    m.active = 0;
    std::vector<ringattn::WorkItem> items;
    for (int s = 0; s < P; ++s) {
      items.clear();
      append_items(items, d, P, causal, r, s);
      for (const auto& w : items)
        if (w.q_start <= m.start && m.start + m.len <= w.q_start + w.q_len) m.active |= (uint64_t)1 << s;
    }
    out.push_back(m);
  }
}

// Launch schedule.  Contiguous causal: rank r has r + 1 visible chunks, so ranks are paired
// (P-1-g, g) to give every launch the same work; otherwise (no mask, or zigzag, where all
// ranks have equal work) consecutive ranks.  At most kMaxGroups launches.  Within a launch
// the items of one rank are listed in ring order.
void build_schedule(ringattn_plan* pl) {
  const int P = pl->p.npes;
  const Derived& d = pl->d;
  const bool causal = pl->p.causal != 0;
  const bool paired = causal && !d.zigzag;
  std::vector<int> order;  // ranks in launch order
  if (paired) {
    for (int g = 0; g < (P + 1) / 2; ++g) {
      order.push_back(P - 1 - g);
      if (g != P - 1 - g) order.push_back(g);
    }
  } else if (d.zigzag) {
    // rank 0 merges the fewest partials: last, where the merge is not hidden under a launch
    for (int r = P - 1; r >= 0; --r) order.push_back(r);
  } else {
    for (int r = 0; r < P; ++r) order.push_back(r);
  }
  int n_groups;
  if (P < 4) n_groups = 1;
  else if (paired) n_groups = (P + 1) / 2 < kMaxGroups ? (P + 1) / 2 : kMaxGroups;
  else n_groups = P < 8 ? P / 2 : 4;
  {
    // Splitting only pays when every launch still fills the chip many times over: count the
    // workgroups of the whole forward (128 query rows each) and keep at least 4096 per launch
    // (8 rounds of 2 workgroups on each of 256 CUs).
    std::vector<ringattn::WorkItem> all;
    for (int r = 0; r < P; ++r)
      for (int s = 0; s < P; ++s) append_items(all, d, P, causal, r, s);
    int64_t wgs = 0;
    for (const auto& w : all) wgs += (w.q_len + ringattn::kBlockM - 1) / ringattn::kBlockM;
    wgs *= d.BH;
    const int64_t fit = wgs / 4096;
    if (fit < n_groups) n_groups = fit < 1 ? 1 : (int)fit;
  }
  size_t pos = 0;
  for (int g = 0; g < n_groups; ++g) {
    // even split of the rank list; paired lists come in balanced pairs, keep pairs together
    size_t end = order.size() * (size_t)(g + 1) / (size_t)n_groups;
    if (paired && (end & 1) && end < order.size()) ++end;
    if (g == n_groups - 1) end = order.size();
    if (end <= pos) continue;
    LaunchGroup lg;
    lg.item_begin = (int)pl->h_items.size();
    lg.region_begin = (int)pl->regions.size();
    for (size_t i = pos; i < end; ++i) {
      const int r = order[i];
      append_regions(pl->regions, d, P, causal, r);
      for (int s = 0; s < P; ++s) append_items(pl->h_items, d, P, causal, r, s);
    }
    lg.item_count = (int)pl->h_items.size() - lg.item_begin;
    lg.region_count = (int)pl->regions.size() - lg.region_begin;
    pl->groups.push_back(lg);
    pos = end;
  }
  pl->all_regions = (int)pl->regions.size();
  for (int r = 0; r < P; ++r) append_regions(pl->regions, d, P, causal, r);
  // per-step lists: one ring step of every rank
  for (int s = 0; s < P; ++s) {
    pl->step_begin.push_back((int)pl->h_items.size());
    for (int r = 0; r < P; ++r) append_items(pl->h_items, d, P, causal, r, s);
  }
  pl->step_begin.push_back((int)pl->h_items.size());
  // rank-local lists for ringattn_rank_step_fwd: one (rank, step) at a time, rows counted from the
  // start of the rank's own chunk and of the visited chunk, one partial slot
  for (int r = 0; r < P; ++r)
    for (int s = 0; s < P; ++s) {
      pl->local_begin.push_back((int)pl->h_items.size());
      const size_t first = pl->h_items.size();
      append_items(pl->h_items, d, P, causal, r, s);
      for (size_t i = first; i < pl->h_items.size(); ++i) {
        pl->h_items[i].q_start -= d.start[r];
        pl->h_items[i].kv_start -= d.start[(r + s) % P];
        pl->h_items[i].slot = 0;
      }
    }
  pl->local_begin.push_back((int)pl->h_items.size());
  int longest = 0;
  for (const auto& w : pl->h_items) longest = w.q_len > longest ? w.q_len : longest;
  pl->q_tiles_max = (longest + ringattn::kBlockM - 1) / ringattn::kBlockM;
}

int ensure_streams(ringattn_plan* pl) {
  if (pl->streams_ready) return RINGATTN_OK;
  // a call that failed half way is resumed: nothing is created twice
  const size_t bytes = pl->h_items.size() * sizeof(ringattn::WorkItem);
  if (!pl->d_items) RA_HIP(hipMalloc((void**)&pl->d_items, bytes));
  RA_HIP(hipMemcpy(pl->d_items, pl->h_items.data(), bytes, hipMemcpyHostToDevice));
  if (!pl->merge_stream) RA_HIP(hipStreamCreateWithFlags(&pl->merge_stream, hipStreamNonBlocking));
  for (int i = 0; i < kMaxGroups; ++i)
    if (!pl->ev_group[i]) RA_HIP(hipEventCreateWithFlags(&pl->ev_group[i], hipEventDisableTiming));
  if (!pl->ev_done) RA_HIP(hipEventCreateWithFlags(&pl->ev_done, hipEventDisableTiming));
  if (pl->p.flags & RINGATTN_FLAG_TIMING)
    for (int i = 0; i < kMaxGroups; ++i) {
      if (!pl->ev_t0[i]) RA_HIP(hipEventCreate(&pl->ev_t0[i]));
      if (!pl->ev_t1[i]) RA_HIP(hipEventCreate(&pl->ev_t1[i]));
    }
  pl->streams_ready = true;
  return RINGATTN_OK;
}

// A block launch over a slice of the item table; o_part / lse_part: partial slot `slot_bias`.
int launch_items(const ringattn_plan* pl, int item_begin, int item_count, const void* q, const void* k,
                 const void* v, void* o_part, float* lse_part, int slot_bias, hipStream_t stream) {
  ringattn::BlockStepArgs a;
  fill_geometry(a, pl->p, pl->d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.o_part = o_part;
  a.lse_part = lse_part;
  a.items = pl->d_items + item_begin;
  a.n_items = item_count;
  a.q_tiles_max = pl->q_tiles_max;
  a.slot_bias = slot_bias;
  RA_HIP(ringattn::launch_block_step(a, pl->p.dtype, pl->p.dim, stream));
  return RINGATTN_OK;
}

int launch_region_merge(const ringattn_plan* pl, const void* o_parts, const float* lse_parts, void* out,
                        float* lse, hipStream_t stream, const MergeRegion& reg) {
  ringattn::MergeArgs m;
  m.o_parts = o_parts;
  m.lse_parts = lse_parts;
  m.out = out;
  m.lse = lse;
  m.sel_start = reg.start;
  m.sel_len = reg.len;
  m.rows = pl->d.BH * reg.len;
  m.part_stride_rows = pl->d.rows;
  m.active = reg.active;
  m.half_partials = half_partials(pl->p) ? 1 : 0;
  m.S = (int)pl->d.S;
  RA_HIP(ringattn::launch_merge(m, pl->p.dtype, pl->p.dim, stream));
  return RINGATTN_OK;
}

// The ring step loop (csrc/ring_attention.cu:456-620 moved to the host) plus the merge:
// for every launch group, all ring steps of its ranks, then the merge of those ranks'
// rows on the merge stream while the next group computes.  The last group's merge runs
// on the caller's stream, which finally waits for the merge stream.
int run_forward(ringattn_plan* pl, const void* q, const void* k, const void* v, void* out,
                float* lse, hipStream_t stream) {
  int rc = RINGATTN_OK;
  const size_t G = pl->groups.size();
  const bool timing = (pl->p.flags & RINGATTN_FLAG_TIMING) && !(pl->p.flags & RINGATTN_FLAG_GRAPH);
  for (size_t g = 0; g < G; ++g) {
    const LaunchGroup& lg = pl->groups[g];
    if (timing) RA_HIP(hipEventRecord(pl->ev_t0[g], stream));
    rc = launch_items(pl, lg.item_begin, lg.item_count, q, k, v, pl->o_parts, pl->lse_parts, 0, stream);
    if (rc != RINGATTN_OK) return rc;
    if (timing) RA_HIP(hipEventRecord(pl->ev_t1[g], stream));
    hipStream_t ms = stream;
    if (g + 1 < G) {
      RA_HIP(hipEventRecord(pl->ev_group[g], stream));
      RA_HIP(hipStreamWaitEvent(pl->merge_stream, pl->ev_group[g], 0));
      ms = pl->merge_stream;
    }
    for (int i = 0; i < lg.region_count; ++i) {
      rc = launch_region_merge(pl, pl->o_parts, pl->lse_parts, out, lse, ms, pl->regions[lg.region_begin + i]);
      if (rc != RINGATTN_OK) return rc;
    }
  }
  if (G > 1) {
    RA_HIP(hipEventRecord(pl->ev_done, pl->merge_stream));
    RA_HIP(hipStreamWaitEvent(stream, pl->ev_done, 0));
  }
  if (timing) pl->timed_forward = true;
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
// Device scratch of one call: the rank's per-step partial O [n_parts, c, dim] fp32, partial LSE
// [n_parts, c], a spare LSE row [c] for callers that pass no lse, and the item table.
struct RankCall {
  ringattn_params p;
  Derived d;
  ringattn::ItemPack pack;  // the visible ring steps of the rank in ring order, one compact slot each
  int n_parts = 0;
  int c = 0;                // rows of this rank
  size_t lse_floats = 0;    // floats of the two LSE areas, padded so the item table stays 32-byte aligned
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
  rc->c = d.start[mype + 1] - d.start[mype];
  rc->n_parts = 0;
  for (int s = 0; s < npes; ++s) {
    const int j = (mype + s) % npes;
    if (causal && j > mype) continue;
    rc->pack.items[rc->n_parts] =
        make_item(0, rc->c, d.start[j], d.start[j + 1] - d.start[j], (causal && j == mype) ? 0 : -1, rc->n_parts);
    ++rc->n_parts;
  }
  rc->lse_floats = ((size_t)(rc->n_parts + 1) * rc->c + 7) & ~(size_t)7;
  rc->scratch_bytes = ((size_t)rc->n_parts * rc->c * dim + rc->lse_floats) * sizeof(float) +
                      (size_t)rc->n_parts * sizeof(ringattn::WorkItem);
  return RINGATTN_OK;
}

// Item table (written by a kernel from its arguments), block kernel, merge: three launches on
// `stream`, nothing is allocated or copied from the host.  `scratch`: rc.scratch_bytes of device memory.
int run_rank_call(const RankCall& rc, void* scratch, const void* q, const void* k, const void* v, void* out,
                  float* lse, hipStream_t stream) {
  const int dim = rc.p.dim, c = rc.c, n_parts = rc.n_parts;
  float* o_parts = (float*)scratch;
  float* lse_parts = o_parts + (size_t)n_parts * c * dim;
  float* lse_tmp = lse_parts + (size_t)n_parts * c;
  ringattn::WorkItem* d_items = (ringattn::WorkItem*)(lse_parts + rc.lse_floats);
  RA_HIP(ringattn::launch_write_items(rc.pack, n_parts, d_items, stream));
  ringattn::BlockStepArgs a;
  fill_geometry(a, rc.p, rc.d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.o_part = o_parts;
  a.lse_part = lse_parts;
  a.items = d_items;
  a.n_items = n_parts;
  a.q_tiles_max = (c + ringattn::kBlockM - 1) / ringattn::kBlockM;
  a.bh_stride = (int64_t)c * dim;
  a.part_stride_rows = c;
  a.S = c;
  RA_HIP(ringattn::launch_block_step(a, rc.p.dtype, dim, stream));
  return ringattn_merge(o_parts, lse_parts, n_parts, (int64_t)c, dim, rc.p.dtype, out, lse ? lse : lse_tmp, stream);
}

// Static device scratch of ringattn_ring_attention_noalloc.  In host code the array's name is
// only a handle for hipGetSymbolAddress; the device address is looked up once per device
// (each GPU holds its own copy of the array) and kept.
constexpr size_t kScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

int device_scratch(void** base) {
  int dev = -1;
  RA_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return RINGATTN_ERR_SHAPE;
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    RA_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return RINGATTN_ERR_HIP;
    g_scratch_ptr[dev] = ptr;
  }
  *base = g_scratch_ptr[dev];
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
  } else {
    hipError_t e = hipMalloc(&pl->ws, need);
    if (e != hipSuccess) {
      delete pl;
      g_last_hip_error = (int)e;
      return e == hipErrorOutOfMemory ? RINGATTN_ERR_ALLOC : RINGATTN_ERR_HIP;
    }
    pl->own_ws = true;
  }
  pl->o_parts = pl->ws;
  pl->lse_parts = (float*)((char*)pl->ws + (size_t)params->npes * d.rows * params->dim * (half_partials(*params) ? 2 : 4));
  build_schedule(pl);
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
  // whatever ensure_streams() got to create, also after a failure half way
  if (plan->merge_stream) (void)hipStreamDestroy(plan->merge_stream);
  for (int i = 0; i < kMaxGroups; ++i)
    if (plan->ev_group[i]) (void)hipEventDestroy(plan->ev_group[i]);
  if (plan->ev_done) (void)hipEventDestroy(plan->ev_done);
  for (int i = 0; i < kMaxGroups; ++i) {
    if (plan->ev_t0[i]) (void)hipEventDestroy(plan->ev_t0[i]);
    if (plan->ev_t1[i]) (void)hipEventDestroy(plan->ev_t1[i]);
  }
  if (plan->d_items) (void)hipFree(plan->d_items);
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
  // pair table, merge stream and events: created at the first forward, outside any capture
  int rc0 = ensure_streams(plan);
  if (rc0 != RINGATTN_OK) return rc0;
  if (!(plan->p.flags & RINGATTN_FLAG_GRAPH)) return run_forward(plan, q, k, v, out, lse, stream);

  // hipGraph replay: the launches of a forward are captured once per pointer set on a private
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
  int rc = ensure_streams(plan);
  if (rc != RINGATTN_OK) return rc;
  return launch_items(plan, plan->step_begin[step], plan->step_begin[step + 1] - plan->step_begin[step], q, k, v,
                      o_part, lse_part, step, (hipStream_t)stream);
}

int ringattn_merge_ring(ringattn_plan* plan, const void* o_parts, const float* lse_parts, void* out,
                        float* lse, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (!aligned16(o_parts) || !aligned16(out) || ((uintptr_t)lse_parts & 3u) || ((uintptr_t)lse & 3u)) return RINGATTN_ERR_ALIGN;
  for (size_t i = (size_t)plan->all_regions; i < plan->regions.size(); ++i) {
    int rc = launch_region_merge(plan, o_parts, lse_parts, out, lse, (hipStream_t)stream, plan->regions[i]);
    if (rc != RINGATTN_OK) return rc;
  }
  return RINGATTN_OK;
}

int ringattn_rank_step_fwd(ringattn_plan* plan, int rank, int step, const void* q, const void* k_chunk,
                           const void* v_chunk, void* o_part, float* lse_part, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!q || !k_chunk || !v_chunk || !o_part || !lse_part) return RINGATTN_ERR_NULL;
  const int P = plan->p.npes;
  if (rank < 0 || rank >= P || step < 0 || step >= P) return RINGATTN_ERR_RANK;
  if (!aligned16(q) || !aligned16(k_chunk) || !aligned16(v_chunk) || !aligned16(o_part) || ((uintptr_t)lse_part & 3u)) return RINGATTN_ERR_ALIGN;
  int rc = ensure_streams(plan);
  if (rc != RINGATTN_OK) return rc;
  const int begin = plan->local_begin[rank * P + step], count = plan->local_begin[rank * P + step + 1] - begin;
  if (count == 0) return RINGATTN_OK;  // nothing of the visited chunk is visible to this rank
  const Derived& d = plan->d;
  const int j = (rank + step) % P;
  const int64_t q_rows = d.start[rank + 1] - d.start[rank], kv_rows = d.start[j + 1] - d.start[j];
  ringattn::BlockStepArgs a;
  fill_geometry(a, plan->p, d);
  a.q = q;
  a.k = k_chunk;
  a.v = v_chunk;
  a.o_part = o_part;
  a.lse_part = lse_part;
  a.items = plan->d_items + begin;
  a.n_items = count;
  a.bh_stride = q_rows * plan->p.dim;      // every tensor holds one rank's rows only
  a.kv_bh_stride = kv_rows * plan->p.dim;
  a.S = (int)q_rows;
  a.part_stride_rows = d.BH * q_rows;
  a.q_tiles_max = (int)((q_rows + ringattn::kBlockM - 1) / ringattn::kBlockM);
  RA_HIP(ringattn::launch_block_step(a, plan->p.dtype, plan->p.dim, (hipStream_t)stream));
  return RINGATTN_OK;
}

int ringattn_rank_merge(ringattn_plan* plan, int rank, const void* o_parts, const float* lse_parts, void* out,
                        float* lse, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (rank < 0 || rank >= plan->p.npes) return RINGATTN_ERR_RANK;
  if (!aligned16(o_parts) || !aligned16(out) || ((uintptr_t)lse_parts & 3u) || ((uintptr_t)lse & 3u)) return RINGATTN_ERR_ALIGN;
  const Derived& d = plan->d;
  const int r0 = d.start[rank], r1 = d.start[rank + 1];
  for (size_t i = (size_t)plan->all_regions; i < plan->regions.size(); ++i) {
    const MergeRegion& reg = plan->regions[i];
    if (reg.start < r0 || reg.start >= r1) continue;
    ringattn::MergeArgs m;
    m.o_parts = o_parts;
    m.lse_parts = lse_parts;
    m.out = out;
    m.lse = lse;
    m.sel_start = reg.start - r0;
    m.sel_len = reg.len;
    m.rows = d.BH * reg.len;
    m.S = r1 - r0;
    m.part_stride_rows = d.BH * (int64_t)(r1 - r0);
    m.active = reg.active;
    m.half_partials = half_partials(plan->p) ? 1 : 0;
    RA_HIP(ringattn::launch_merge(m, plan->p.dtype, plan->p.dim, (hipStream_t)stream));
  }
  return RINGATTN_OK;
}

int ringattn_plan_work_items(const ringattn_plan* plan, int step, ringattn_work_item* out, int capacity, int* n_out) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!n_out || (capacity > 0 && !out)) return RINGATTN_ERR_NULL;
  if (step < -1 || step >= plan->p.npes) return RINGATTN_ERR_RANK;
  const int begin = step < 0 ? 0 : plan->step_begin[step];
  const int end = step < 0 ? plan->step_begin[0] : plan->step_begin[step + 1];
  *n_out = end - begin;
  for (int i = begin; i < end && i - begin < capacity; ++i) {
    const ringattn::WorkItem& w = plan->h_items[i];
    out[i - begin] = ringattn_work_item{w.q_start, w.q_len, w.kv_start, w.kv_len, w.diag_off, w.slot};
  }
  return RINGATTN_OK;
}

int ringattn_plan_launch_times(ringattn_plan* plan, float* ms, int capacity, int* n_out) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!n_out || (capacity > 0 && !ms)) return RINGATTN_ERR_NULL;
  if (!plan->timed_forward) return RINGATTN_ERR_PLAN;
  const int n = (int)plan->groups.size();
  *n_out = n;
  for (int g = 0; g < n && g < capacity; ++g) {
    RA_HIP(hipEventSynchronize(plan->ev_t1[g]));
    RA_HIP(hipEventElapsedTime(&ms[g], plan->ev_t0[g], plan->ev_t1[g]));
  }
  return RINGATTN_OK;
}

int ringattn_plan_merge_regions(const ringattn_plan* plan, int* start, int* len, uint64_t* active, int capacity, int* n_out) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!n_out || (capacity > 0 && (!start || !len || !active))) return RINGATTN_ERR_NULL;
  const int n = (int)plan->regions.size() - plan->all_regions;
  *n_out = n;
  for (int i = 0; i < n && i < capacity; ++i) {
    const MergeRegion& m = plan->regions[plan->all_regions + i];
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
  ringattn::MergeArgs m;
  m.o_parts = o_parts;
  m.lse_parts = lse_parts;
  m.out = out;
  m.lse = lse;
  m.rows = rows;
  m.part_stride_rows = rows;
  m.active = n_parts >= 64 ? ~(uint64_t)0 : (((uint64_t)1 << n_parts) - 1);
  m.half_partials = 0;
  m.S = (int)(rows > 0 ? (rows < INT32_MAX ? rows : INT32_MAX) : 1);
  m.sel_start = 0;
  m.sel_len = m.S;
  RA_HIP(ringattn::launch_merge(m, dtype, dim, (hipStream_t)stream));
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
  if (rc_.scratch_bytes > kScratchBytes) return RINGATTN_ERR_WORKSPACE;
  void* base = nullptr;
  rc = device_scratch(&base);
  if (rc != RINGATTN_OK) return rc;
  return run_rank_call(rc_, base, q, k, v, out, lse, (hipStream_t)stream);
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
