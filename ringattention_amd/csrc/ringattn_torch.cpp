// torch.Tensor front end of the C ABI: the extension the reference's
// include/attention_api.cuh was written for (it includes torch/extension.h and defines
// CHECK_CUDA / CHECK_CONTIGUOUS / CHECK_INPUT, :8-18, but the reference never builds one).
// Registers   ringattn::fwd(q, k, v, seqlen, causal, softmax_scale, zigzag) -> (out, lse)
// with the dispatcher.  Only plumbing lives here: tensor checks, output allocation, the
// current stream, a bounded cache of plans (one per parameter set and stream); all computation is
// ringattn_fwd of libringattn.so.
#include <ATen/ATen.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "ringattn.h"

namespace {

// the conventions of include/attention_api.cuh:12-18
#define RA_CHECK_DEVICE(x) TORCH_CHECK((x).device().is_cuda(), #x " must be a CUDA tensor")
#define RA_CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define RA_CHECK_INPUT(x) \
  RA_CHECK_DEVICE(x);     \
  RA_CHECK_CONTIGUOUS(x)

// A plan is meant for one forward at a time (its tables, its timing events, and with
// RINGATTN_FLAG_STEP_PARTIALS its workspace, are single), so the cache holds a plan per
// (parameter set, device, STREAM): forwards on different streams never share one, and
// forwards on one stream are ordered by the stream.  A per-plan mutex keeps two host threads
// from enqueueing on the same plan at once.  The cache is bounded: beyond kMaxPlans the least
// recently used plan that nobody is enqueueing on is destroyed (its device memory goes back to the
// device); hipFree inside ringattn_plan_destroy waits for the work that still uses it.
using PlanKey = std::tuple<int, void*, std::vector<int>, int, int, int, int, int, int, int, float>;
struct Entry {
  ringattn_plan* plan = nullptr;
  std::mutex mu;  // held while a forward is being enqueued on the plan
  uint64_t last_use = 0;
};
constexpr size_t kMaxPlans = 16;
std::mutex g_mu;
std::map<PlanKey, std::shared_ptr<Entry>> g_plans;
uint64_t g_clock = 0;

std::shared_ptr<Entry> plan_for(const PlanKey& key, const ringattn_params& p) {
  std::vector<std::shared_ptr<Entry>> evicted;
  std::shared_ptr<Entry> e;
  int create_rc = RINGATTN_OK;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) {
      it->second->last_use = ++g_clock;
      return it->second;
    }
    while (g_plans.size() >= kMaxPlans) {
      auto victim = g_plans.end();
      for (auto j = g_plans.begin(); j != g_plans.end(); ++j)
        if (j->second.use_count() == 1 && (victim == g_plans.end() || j->second->last_use < victim->second->last_use)) victim = j;
      if (victim == g_plans.end()) break;  // every plan is in use right now: grow
      evicted.push_back(victim->second);
      g_plans.erase(victim);
    }
    e = std::make_shared<Entry>();
    const int rc = ringattn_plan_create(&p, nullptr, 0, &e->plan);
    if (rc == RINGATTN_OK) {
      e->last_use = ++g_clock;
      g_plans.emplace(key, e);
    } else {
      e.reset();
    }
    create_rc = rc;
  }
  // outside the lock, and whether or not the new plan came to be: the evicted plans go back to the device
  for (auto& v : evicted) (void)ringattn_plan_destroy(v->plan);
  TORCH_CHECK(create_rc == RINGATTN_OK, "ringattn_plan_create: ", ringattn_strerror(create_rc));
  return e;
}

std::tuple<at::Tensor, at::Tensor> fwd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                       at::IntArrayRef seqlen, bool causal, double softmax_scale, bool zigzag) {
  RA_CHECK_INPUT(q);
  RA_CHECK_INPUT(k);
  RA_CHECK_INPUT(v);
  TORCH_CHECK(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q, k, v must share a dtype");
  TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, "q, k, v must be [batch, heads, S, dim]");
  TORCH_CHECK(k.sizes() == v.sizes(), "k and v must have the same shape");
  TORCH_CHECK(k.size(0) == q.size(0) && k.size(2) == q.size(2) && k.size(3) == q.size(3),
              "k, v must be [batch, kv_heads, S, dim] for q [batch, heads, S, dim]");
  TORCH_CHECK(k.device() == q.device() && v.device() == q.device(), "q, k, v must be on one device");
  TORCH_CHECK(!seqlen.empty() && seqlen.size() <= RINGATTN_MAX_NPES, "seqlen must name 1..", RINGATTN_MAX_NPES, " ranks");
  int64_t total = 0;
  std::vector<int> lens;
  for (int64_t c : seqlen) {
    TORCH_CHECK(c > 0 && c <= INT32_MAX, "per-rank lengths must be positive");
    lens.push_back((int)c);
    total += c;
  }
  TORCH_CHECK(total == q.size(2), "seqlen must sum to S = ", q.size(2));

  ringattn_params p{};
  p.npes = (int)lens.size();
  p.h_seqlen = lens.data();
  p.dim = (int)q.size(3);
  p.softmax_scale = (float)softmax_scale;
  p.batch = (int)q.size(0);
  p.heads = (int)q.size(1);
  p.dtype = q.scalar_type() == at::kHalf ? RINGATTN_DTYPE_FP16 : RINGATTN_DTYPE_BF16;
  p.causal = causal ? 1 : 0;
  p.flags = 0;
  p.kv_heads = (int)k.size(1) == p.heads ? 0 : (int)k.size(1);
  p.layout = zigzag ? RINGATTN_LAYOUT_ZIGZAG : RINGATTN_LAYOUT_CONTIGUOUS;
  const int device = q.device().index();
  c10::hip::HIPGuard guard(device);  // plan creation allocates on the current device
  hipStream_t stream = c10::hip::getCurrentHIPStream(device).stream();
  const PlanKey key{device, (void*)stream, lens, p.dim, p.batch, p.heads, p.dtype, p.causal, p.kv_heads, p.layout,
                    p.softmax_scale};
  std::shared_ptr<Entry> entry = plan_for(key, p);
  at::Tensor out = at::empty_like(q);
  at::Tensor lse = at::empty({q.size(0), q.size(1), q.size(2)}, q.options().dtype(at::kFloat));
  int rc;
  {
    std::lock_guard<std::mutex> lk(entry->mu);
    rc = ringattn_fwd(entry->plan, q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr<float>(), stream);
  }
  TORCH_CHECK(rc == RINGATTN_OK, "ringattn_fwd: ", ringattn_strerror(rc));
  return {out, lse};
}

}  // namespace

TORCH_LIBRARY(ringattn, m) {
  // catch-all registration: the checks above answer for tensors on any backend
  m.def("fwd(Tensor q, Tensor k, Tensor v, int[] seqlen, bool causal=False, float softmax_scale=0.0, bool zigzag=False)"
        " -> (Tensor, Tensor)", &fwd);
}
