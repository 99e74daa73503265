// Counterpart of the reference's main() (csrc/ring_attention.cu:750-790) on top of the C ABI:
// dim 64, two ranks of 8192 tokens, fp16, every rank's Q/K/V filled with the reference's
// pattern (:731-748), 50 warm-up and 50 timed forwards between an event pair (:767-783), the
// top-left 8 x 8 block of rank 0's output printed (:723-729) and the time per forward as
// "elapsedtime=<ms>" (:789).  One process drives all virtual ranks, so the per-PE
// "mype: N success" lines (:785-787) are printed by it in rank order.
// Plain C++ and the HIP runtime only; links libringattn.so.
//
//   reference_harness [npes] [tokens_per_rank] [loops]
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "ringattn.h"

#define HIP_CHECK(expr)                                                                       \
  do {                                                                                        \
    hipError_t e_ = (expr);                                                                   \
    if (e_ != hipSuccess) {                                                                   \
      fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_));              \
      return 1;                                                                               \
    }                                                                                         \
  } while (0)

static float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31, man = h & 1023;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {  // subnormal
      int e = -1;
      uint32_t m = man;
      while (!(m & 1024)) {
        m <<= 1;
        ++e;
      }
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 1023) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

int main(int argc, char** argv) {
  const int dim = 64;
  const int npes = argc > 1 ? atoi(argv[1]) : 2;
  const int chunk = argc > 2 ? atoi(argv[2]) : 8192;
  const int loops = argc > 3 ? atoi(argv[3]) : 50;
  if (npes < 1 || npes > RINGATTN_MAX_NPES || chunk < 8 || loops < 1) {
    fprintf(stderr, "usage: reference_harness [npes] [tokens_per_rank >= 8] [loops]\n");
    return 2;
  }
  std::vector<int> seqlen((size_t)npes, chunk);
  const size_t S = (size_t)npes * chunk, elems = S * dim, bytes = elems * sizeof(uint16_t);

  // initQKV: every rank holds the same pattern in its block of Q, K and V
  std::vector<uint16_t> host(elems);
  for (int pe = 0; pe < npes; ++pe) {
    const int rc = ringattn_fill_reference_pattern(host.data() + (size_t)pe * chunk * dim, RINGATTN_DTYPE_FP16, chunk, dim);
    if (rc != RINGATTN_OK) {
      fprintf(stderr, "fill: %s\n", ringattn_strerror(rc));
      return 1;
    }
  }
  void *q = nullptr, *k = nullptr, *v = nullptr, *out = nullptr;
  float* lse = nullptr;
  HIP_CHECK(hipMalloc(&q, bytes));
  HIP_CHECK(hipMalloc(&k, bytes));
  HIP_CHECK(hipMalloc(&v, bytes));
  HIP_CHECK(hipMalloc(&out, bytes));
  HIP_CHECK(hipMalloc((void**)&lse, S * sizeof(float)));
  HIP_CHECK(hipMemcpy(q, host.data(), bytes, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(k, host.data(), bytes, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(v, host.data(), bytes, hipMemcpyHostToDevice));

  ringattn_params p;
  memset(&p, 0, sizeof(p));
  p.npes = npes;
  p.h_seqlen = seqlen.data();
  p.dim = dim;
  p.batch = 1;
  p.heads = 1;
  p.dtype = RINGATTN_DTYPE_FP16;
  p.layout = RINGATTN_LAYOUT_CONTIGUOUS;
  ringattn_plan* plan = nullptr;
  int rc = ringattn_plan_create(&p, nullptr, 0, &plan);
  if (rc != RINGATTN_OK) {
    fprintf(stderr, "plan: %s (hip error %d)\n", ringattn_strerror(rc), ringattn_last_hip_error());
    return 1;
  }
  for (int i = 0; i < loops; ++i) {  // warm-up
    rc = ringattn_fwd(plan, q, k, v, out, lse, nullptr);
    if (rc != RINGATTN_OK) {
      fprintf(stderr, "fwd: %s (hip error %d)\n", ringattn_strerror(rc), ringattn_last_hip_error());
      return 1;
    }
  }
  hipEvent_t start, stop;
  HIP_CHECK(hipEventCreate(&start));
  HIP_CHECK(hipEventCreate(&stop));
  HIP_CHECK(hipEventRecord(start, nullptr));
  for (int i = 0; i < loops; ++i) rc |= ringattn_fwd(plan, q, k, v, out, lse, nullptr);
  HIP_CHECK(hipEventRecord(stop, nullptr));
  HIP_CHECK(hipEventSynchronize(stop));
  float elapsed = 0.f;
  HIP_CHECK(hipEventElapsedTime(&elapsed, start, stop));
  if (rc != RINGATTN_OK) {
    fprintf(stderr, "fwd: %s\n", ringattn_strerror(rc));
    return 1;
  }
  for (int pe = 0; pe < npes; ++pe) printf("mype: %d success\n", pe);

  // printDeviceFloat: the 8 x 8 corner of rank 0's output
  std::vector<uint16_t> o((size_t)8 * dim);
  HIP_CHECK(hipMemcpy(o.data(), out, o.size() * sizeof(uint16_t), hipMemcpyDeviceToHost));
  for (int i = 0; i < 8; ++i) {
    for (int j = 0; j < 8; ++j) printf("%10.4f", half_to_float(o[(size_t)i * dim + j]));
    printf("\n");
  }
  printf("elapsedtime=%f\n", elapsed / loops);
  rc = ringattn_plan_destroy(plan);
  (void)hipFree(q);
  (void)hipFree(k);
  (void)hipFree(v);
  (void)hipFree(out);
  (void)hipFree(lse);
  return rc == RINGATTN_OK ? 0 : 1;
}
