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

struct Derived {
  int start[RINGATTN_MAX_NPES + 1] = {};  // rank r owns rows [start[r], start[r+1]) of every head
  int max_len = 0;
  int64_t S = 0;
  int64_t BH = 0;
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
  int64_t S = 0;
  int max_len = 0;
  for (int r = 0; r < p->npes; ++r) {
    const int c = p->h_seqlen[r];
    if (c <= 0 || c % RINGATTN_TILE != 0) return RINGATTN_ERR_SEQLEN;
    S += c;
    if (c > max_len) max_len = c;
  }
  const int64_t BH = (int64_t)p->batch * p->heads;
  if (S > INT32_MAX / 2 || BH > INT32_MAX / 2) return RINGATTN_ERR_SHAPE;
  if (BH * p->npes > (int64_t)INT32_MAX / 64) return RINGATTN_ERR_SHAPE;  // grid size
  if (BH * S > (int64_t)1 << 40) return RINGATTN_ERR_SHAPE;
  if (!std::isfinite(p->softmax_scale)) return RINGATTN_ERR_SHAPE;
  if (d) {
    d->start[0] = 0;
    for (int r = 0; r < p->npes; ++r) d->start[r + 1] = d->start[r] + p->h_seqlen[r];
    d->max_len = max_len;
    d->S = S;
    d->BH = BH;
    d->rows = BH * S;
    d->scale = p->softmax_scale > 0.f ? p->softmax_scale : 1.0f / std::sqrt((float)p->dim);
  }
  return RINGATTN_OK;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

constexpr int kMaxGroups = 8;  // launches per forward

size_t workspace_bytes_of(const ringattn_params* p, const Derived& d) {
  return (size_t)p->npes * (size_t)d.rows * (size_t)(p->dim + 1) * sizeof(float);
}

}  // namespace

// One launch of the forward: the (rank, step) pairs of a few virtual ranks, all their steps.
struct LaunchGroup {
  int pair_begin, pair_count;  // slice of the pair table
  int rank_begin, rank_count;  // slice of group_ranks
};

struct ringattn_plan {
  ringattn_params p{};
  int seqlen[RINGATTN_MAX_NPES]{};
  Derived d{};
  void* ws = nullptr;
  size_t ws_bytes = 0;
  bool own_ws = false;
  float* o_parts = nullptr;    // [npes, rows, dim]
  float* lse_parts = nullptr;  // [npes, rows]
  // Launch schedule of ringattn_fwd.  The ring steps of different ranks are independent
  // (each (rank, step) pair writes its own rows of its step's partial slot), so the forward
  // is issued as a few launches that each hold ALL steps of a few ranks; the merge of those
  // ranks then runs on a second stream underneath the next launch.
  std::vector<int> h_pairs;       // packed (rank << 16 | step), launch by launch
  std::vector<int> group_ranks;
  std::vector<LaunchGroup> groups;
  int* d_pairs = nullptr;         // device copy of h_pairs (allocated at the first forward)
  hipStream_t merge_stream = nullptr;
  hipEvent_t ev_group[kMaxGroups]{};
  hipEvent_t ev_done = nullptr;
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

// Active ranks of ring step s.  Non-causal: all.  Causal: KV chunk j = (r + s) mod P is
// visible iff j <= r, i.e. s == 0 (diagonal) or r + s >= P (wrapped, j < r).
inline void active_ranks(int P, int causal, int s, int* rank_base, int* n_active) {
  if (!causal || s == 0) {
    *rank_base = 0;
    *n_active = P;
  } else {
    *rank_base = P - s;
    *n_active = s;
  }
}

// fields of the launch arguments that depend only on the geometry
void fill_geometry(ringattn::BlockStepArgs& a, const ringattn_params& p, const Derived& d) {
  a.bh_stride = d.S * p.dim;
  a.S = (int)d.S;
  a.q_tiles_max = d.max_len / ringattn::kBlockM;
  a.P = p.npes;
  a.BH = (int)d.BH;
  a.heads = p.heads;
  a.kv_group = p.kv_heads > 0 ? p.heads / p.kv_heads : 1;
  a.causal = p.causal ? 1 : 0;
  a.scale_log2 = d.scale * 1.4426950408889634f;
  for (int r = 0; r <= p.npes; ++r) a.rank_start[r] = d.start[r];
}

int launch_step(const ringattn_plan* pl, int s, const void* q, const void* k, const void* v,
                float* o_part, float* lse_part, hipStream_t stream) {
  ringattn::BlockStepArgs a;
  fill_geometry(a, pl->p, pl->d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.o_part = o_part;
  a.lse_part = lse_part;
  a.pairs = nullptr;
  a.part_stride_rows = 0;
  a.step = s;
  active_ranks(pl->p.npes, pl->p.causal, s, &a.rank_base, &a.n_active);
  RA_HIP(ringattn::launch_block_step(a, pl->p.dtype, pl->p.dim, stream));
  return RINGATTN_OK;
}

// merge of the rows of one virtual rank; with a causal ring, part s of rank r is active iff
// s == 0 or r + s >= P, and inactive parts are never read
int launch_rank_merge(const ringattn_plan* pl, const float* o_parts, const float* lse_parts, void* out,
                      float* lse, hipStream_t stream, int rank) {
  ringattn::MergeArgs m;
  m.o_parts = o_parts;
  m.lse_parts = lse_parts;
  m.out = out;
  m.lse = lse;
  m.sel_start = pl->d.start[rank];
  m.sel_len = pl->d.start[rank + 1] - pl->d.start[rank];
  m.rows = pl->d.BH * m.sel_len;
  m.part_stride_rows = pl->d.rows;
  m.n_parts = pl->p.npes;
  m.first_wrapped = pl->p.causal ? pl->p.npes - rank : 1;
  m.S = (int)pl->d.S;
  RA_HIP(ringattn::launch_merge(m, pl->p.dtype, pl->p.dim, stream));
  return RINGATTN_OK;
}

// Launch schedule.  Causal: rank r has r + 1 visible chunks, so ranks are paired (P-1-g, g)
// to give every launch the same work; non-causal: consecutive ranks.  At most kMaxGroups
// launches.  Within a launch the pairs of one rank are listed in ring order
// (csrc/ring_attention.cu:456-470: step s visits chunk (r + s) mod P).
void build_schedule(ringattn_plan* pl) {
  const int P = pl->p.npes;
  const bool causal = pl->p.causal != 0;
  std::vector<int> order;  // ranks in launch order
  if (causal) {
    for (int g = 0; g < (P + 1) / 2; ++g) {
      order.push_back(P - 1 - g);
      if (g != P - 1 - g) order.push_back(g);
    }
  } else {
    for (int r = 0; r < P; ++r) order.push_back(r);
  }
  const int n_groups = P < 4 ? 1 : (P / 2 < kMaxGroups ? (causal ? (P + 1) / 2 : (P < 8 ? P / 2 : 4)) : (causal ? kMaxGroups : 4));
  size_t pos = 0;
  for (int g = 0; g < n_groups; ++g) {
    // even split of the rank list; causal lists come in balanced pairs, keep pairs together
    size_t end = (size_t)order.size() * (g + 1) / n_groups;
    if (causal && (end & 1) && end < order.size()) ++end;
    if (g == n_groups - 1) end = order.size();
    if (end <= pos) continue;
    LaunchGroup lg;
    lg.pair_begin = (int)pl->h_pairs.size();
    lg.rank_begin = (int)pl->group_ranks.size();
    for (size_t i = pos; i < end; ++i) {
      const int r = order[i];
      pl->group_ranks.push_back(r);
      for (int s = 0; s < P; ++s) {
        const int j = (r + s) % P;
        if (!causal || j <= r) pl->h_pairs.push_back((r << 16) | s);
      }
    }
    lg.pair_count = (int)pl->h_pairs.size() - lg.pair_begin;
    lg.rank_count = (int)pl->group_ranks.size() - lg.rank_begin;
    pl->groups.push_back(lg);
    pos = end;
  }
}

int ensure_streams(ringattn_plan* pl) {
  if (pl->streams_ready) return RINGATTN_OK;
  RA_HIP(hipMalloc((void**)&pl->d_pairs, pl->h_pairs.size() * sizeof(int)));
  RA_HIP(hipMemcpy(pl->d_pairs, pl->h_pairs.data(), pl->h_pairs.size() * sizeof(int), hipMemcpyHostToDevice));
  RA_HIP(hipStreamCreateWithFlags(&pl->merge_stream, hipStreamNonBlocking));
  for (int i = 0; i < kMaxGroups; ++i) RA_HIP(hipEventCreateWithFlags(&pl->ev_group[i], hipEventDisableTiming));
  RA_HIP(hipEventCreateWithFlags(&pl->ev_done, hipEventDisableTiming));
  pl->streams_ready = true;
  return RINGATTN_OK;
}

int launch_group(const ringattn_plan* pl, const LaunchGroup& lg, const void* q, const void* k, const void* v,
                 hipStream_t stream) {
  ringattn::BlockStepArgs a;
  fill_geometry(a, pl->p, pl->d);
  a.q = q;
  a.k = k;
  a.v = v;
  a.o_part = pl->o_parts;
  a.lse_part = pl->lse_parts;
  a.pairs = pl->d_pairs + lg.pair_begin;
  a.part_stride_rows = pl->d.rows;
  a.step = 0;
  a.rank_base = 0;
  a.n_active = lg.pair_count;
  RA_HIP(ringattn::launch_block_step(a, pl->p.dtype, pl->p.dim, stream));
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
  for (size_t g = 0; g < G; ++g) {
    const LaunchGroup& lg = pl->groups[g];
    rc = launch_group(pl, lg, q, k, v, stream);
    if (rc != RINGATTN_OK) return rc;
    hipStream_t ms = stream;
    if (g + 1 < G) {
      RA_HIP(hipEventRecord(pl->ev_group[g], stream));
      RA_HIP(hipStreamWaitEvent(pl->merge_stream, pl->ev_group[g], 0));
      ms = pl->merge_stream;
    }
    for (int i = 0; i < lg.rank_count; ++i) {
      rc = launch_rank_merge(pl, pl->o_parts, pl->lse_parts, out, lse, ms, pl->group_ranks[lg.rank_begin + i]);
      if (rc != RINGATTN_OK) return rc;
    }
  }
  if (G > 1) {
    RA_HIP(hipEventRecord(pl->ev_done, pl->merge_stream));
    RA_HIP(hipStreamWaitEvent(stream, pl->ev_done, 0));
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
  pl->o_parts = (float*)pl->ws;
  pl->lse_parts = pl->o_parts + (size_t)params->npes * d.rows * params->dim;
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
  if (plan->streams_ready) {
    (void)hipStreamDestroy(plan->merge_stream);
    for (int i = 0; i < kMaxGroups; ++i) (void)hipEventDestroy(plan->ev_group[i]);
    (void)hipEventDestroy(plan->ev_done);
    (void)hipFree(plan->d_pairs);
  }
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

  // hipGraph replay: the P + 1 launches are captured once per pointer set on a private
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
                       float* o_part, float* lse_part, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!q || !k || !v || !o_part || !lse_part) return RINGATTN_ERR_NULL;
  if (step < 0 || step >= plan->p.npes) return RINGATTN_ERR_RANK;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o_part) || ((uintptr_t)lse_part & 3u)) return RINGATTN_ERR_ALIGN;
  return launch_step(plan, step, q, k, v, o_part, lse_part, (hipStream_t)stream);
}

int ringattn_merge_ring(ringattn_plan* plan, const float* o_parts, const float* lse_parts, void* out,
                        float* lse, void* stream) {
  if (!plan_ok(plan)) return RINGATTN_ERR_PLAN;
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (!aligned16(o_parts) || !aligned16(out) || ((uintptr_t)lse_parts & 3u) || ((uintptr_t)lse & 3u)) return RINGATTN_ERR_ALIGN;
  for (int r = 0; r < plan->p.npes; ++r) {
    int rc = launch_rank_merge(plan, o_parts, lse_parts, out, lse, (hipStream_t)stream, r);
    if (rc != RINGATTN_OK) return rc;
  }
  return RINGATTN_OK;
}

int ringattn_merge(const float* o_parts, const float* lse_parts, int n_parts, int64_t rows, int dim,
                   int dtype, void* out, float* lse, void* stream) {
  if (!o_parts || !lse_parts || !out || !lse) return RINGATTN_ERR_NULL;
  if (n_parts < 1 || n_parts > RINGATTN_MAX_NPES) return RINGATTN_ERR_NPES;
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
  m.n_parts = n_parts;
  m.first_wrapped = 1;
  m.S = (int)(rows > 0 ? (rows < INT32_MAX ? rows : INT32_MAX) : 1);
  m.sel_start = 0;
  m.sel_len = m.S;
  RA_HIP(ringattn::launch_merge(m, dtype, dim, (hipStream_t)stream));
  return RINGATTN_OK;
}

int ringattn_ring_attention(const void* q, const void* k, const void* v, void* out, float* lse,
                            int npes, int mype, const int* seqlen, int dim, int max_seq,
                            int dtype, int causal, float softmax_scale) {
  ringattn_params p;
  std::memset(&p, 0, sizeof(p));
  p.npes = npes;
  p.h_seqlen = seqlen;
  p.dim = dim;
  p.softmax_scale = softmax_scale;
  p.batch = 1;
  p.heads = 1;
  p.dtype = dtype;
  p.causal = causal;
  Derived d;
  int rc = validate(&p, &d);
  if (rc != RINGATTN_OK) return rc;
  if (mype < 0 || mype >= npes) return RINGATTN_ERR_RANK;
  if (max_seq < d.max_len) return RINGATTN_ERR_SEQLEN;
  if (!q || !k || !v || !out) return RINGATTN_ERR_NULL;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return RINGATTN_ERR_ALIGN;

  // steps in which rank mype has a visible chunk, in ring order
  std::vector<int> steps;
  for (int s = 0; s < npes; ++s) {
    const int j = (mype + s) % npes;
    if (!causal || j <= mype) steps.push_back(s);
  }
  const int n_parts = (int)steps.size();
  const size_t c = (size_t)(d.start[mype + 1] - d.start[mype]);  // rows of this rank
  const size_t first = (size_t)d.start[mype];
  // per-call scratch, like the reference's per-call allocations (:383-394) but freed
  float* ws = nullptr;
  RA_HIP(hipMalloc((void**)&ws, (size_t)n_parts * c * (size_t)(dim + 1) * sizeof(float) + c * sizeof(float)));
  float* o_parts = ws;
  float* lse_parts = ws + (size_t)n_parts * c * dim;
  float* lse_tmp = lse_parts + (size_t)n_parts * c;
  const size_t esz = 2;
  // The kernel addresses the rows of rank r at rank_start[r]: shift the rank-local buffers
  // so that rank mype's rows land on them.  The shifted pointers are never dereferenced
  // outside [start[mype], start[mype + 1]).
  const char* q_shift = (const char*)q - first * dim * esz;
  for (int i = 0; i < n_parts && rc == RINGATTN_OK; ++i) {
    ringattn::BlockStepArgs a;
    fill_geometry(a, p, d);
    a.q = q_shift;
    a.k = k;
    a.v = v;
    a.o_part = o_parts + (size_t)i * c * dim - first * dim;
    a.lse_part = lse_parts + (size_t)i * c - first;
    a.pairs = nullptr;
    a.part_stride_rows = 0;
    a.step = steps[i];
    a.rank_base = mype;
    a.n_active = 1;
    hipError_t e = ringattn::launch_block_step(a, dtype, dim, nullptr);
    if (e != hipSuccess) rc = hip_fail(e);
  }
  if (rc == RINGATTN_OK) rc = ringattn_merge(o_parts, lse_parts, n_parts, (int64_t)c, dim, dtype, out, lse ? lse : lse_tmp, nullptr);
  hipError_t e = hipDeviceSynchronize();  // blocking, as csrc/ring_attention.cu:721
  if (rc == RINGATTN_OK && e != hipSuccess) rc = hip_fail(e);
  (void)hipFree(ws);
  return rc;
}

const char* ringattn_strerror(int code) {
  switch (code) {
    case RINGATTN_OK: return "ok";
    case RINGATTN_ERR_NULL: return "a required pointer is NULL";
    case RINGATTN_ERR_NPES: return "npes out of range";
    case RINGATTN_ERR_DIM: return "dim must be 64 or 128";
    case RINGATTN_ERR_DTYPE: return "dtype must be fp16 (0) or bf16 (1)";
    case RINGATTN_ERR_SEQLEN: return "per-rank sequence lengths must be positive multiples of 128 (and max_seq at least the longest)";
    case RINGATTN_ERR_SHAPE: return "batch/heads/scale invalid or sizes overflow";
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
