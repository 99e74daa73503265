// Seeded host-side input generation: the counterpart of the reference's fillWithNum /
// initQKV (csrc/ring_attention.cu:731-748), which fill a host buffer that is then
// copied to the device.  Pure host code, no HIP.
#include "ringattn.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

inline uint64_t mix64(uint64_t z) {
  z ^= z >> 30;
  z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27;
  z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}
constexpr uint64_t kGamma = 0x9E3779B97F4A7C15ull;

// n-th output (n >= 1) of the splitmix64 stream whose state starts at mix64(seed + gamma)
inline uint64_t stream_at(uint64_t key, uint64_t n) { return mix64(key + n * kGamma); }

inline double to_unit(uint64_t x) { return ((double)(x >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

inline uint16_t float_to_bf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

inline uint16_t float_to_half(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const uint32_t au = u & 0x7fffffffu;
  if (au >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (au > 0x7f800000u ? 0x200u : 0u));
  if (au >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // >= 65520 rounds to inf
  if (au < 0x33000001u) return (uint16_t)sign;               // <= 2^-25 rounds to zero
  int e = (int)(au >> 23) - 127;
  uint32_t man = (au & 0x7fffffu) | 0x800000u;
  int shift;  // bits dropped from the 24-bit significand
  uint32_t base;
  if (e < -14) {  // subnormal half
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  return (uint16_t)(sign | (base + q));  // a carry out of the mantissa bumps the exponent
}

template <typename F>
void parallel_for(int64_t n, F f) {
  unsigned hw = std::thread::hardware_concurrency();
  int64_t nt = std::max<int64_t>(1, std::min<int64_t>(std::min<unsigned>(hw ? hw : 1, 16u), n / 65536));
  if (nt <= 1) {
    f(0, n);
    return;
  }
  std::vector<std::thread> th;
  const int64_t per = (n + nt - 1) / nt;
  for (int64_t t = 0; t < nt; ++t) {
    const int64_t a = t * per, b = std::min(n, a + per);
    if (a >= b) break;
    th.emplace_back([=] { f(a, b); });
  }
  for (auto& x : th) x.join();
}

}  // namespace

extern "C" {

int ringattn_fill_normal(void* dst_host, int dtype, int64_t n, uint64_t seed, int64_t offset, double sigma) {
  if (!dst_host) return RINGATTN_ERR_NULL;
  if (dtype != RINGATTN_DTYPE_FP16 && dtype != RINGATTN_DTYPE_BF16) return RINGATTN_ERR_DTYPE;
  if (n < 0 || offset < 0) return RINGATTN_ERR_SHAPE;
  uint16_t* dst = (uint16_t*)dst_host;
  const uint64_t key = mix64(seed + kGamma);
  parallel_for(n, [=](int64_t a, int64_t b) {
    for (int64_t i = a; i < b; ++i) {
      const uint64_t e = (uint64_t)(offset + i);
      const double u1 = to_unit(stream_at(key, 2 * e + 1));
      const double u2 = to_unit(stream_at(key, 2 * e + 2));
      const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925286766559 * u2);
      const float f = (float)(sigma * z);
      dst[i] = dtype == RINGATTN_DTYPE_BF16 ? float_to_bf16(f) : float_to_half(f);
    }
  });
  return RINGATTN_OK;
}

int ringattn_fill_reference_pattern(void* dst_host, int dtype, int m, int n) {
  if (!dst_host) return RINGATTN_ERR_NULL;
  if (dtype != RINGATTN_DTYPE_FP16 && dtype != RINGATTN_DTYPE_BF16) return RINGATTN_ERR_DTYPE;
  if (m < 0 || n < 0) return RINGATTN_ERR_SHAPE;
  uint16_t* dst = (uint16_t*)dst_host;
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      const float f = (float)(i / 130.0 + j / 110.0 + (double)i * j / 600.0);
      dst[(int64_t)i * n + j] = dtype == RINGATTN_DTYPE_BF16 ? float_to_bf16(f) : float_to_half(f);
    }
  return RINGATTN_OK;
}

}  // extern "C"
