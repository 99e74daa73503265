// Issue-rate probe for gfx950: how much of the MFMA pipe is left when a wave also issues the
// VALU and LDS instructions that block_attention_kernel needs per MFMA.  Stand-alone program:
//
//   hipcc --offload-arch=gfx950 -O2 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         ringattention_amd/csrc/issue_rate_probe.hip -o issue_rate_probe && ./issue_rate_probe
//
// Every mix is a loop of independent instructions (no data dependence between the MFMAs, the
// VALU ops and the LDS reads of an iteration), run by 512-thread workgroups, one per CU: two
// waves per SIMD, the occupancy of block_attention_kernel at d = 128.  Time is read per wave
// with s_memtime around the loop; the table reports it relative to the MFMA-only loop.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define MFMA(acc) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define FMA(x) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(x))
#define EXP(x) asm volatile("v_exp_f32 %0, %0" : "+v"(x))

constexpr int kRepeat = 8;  // groups of 4 MFMAs per loop iteration: the loop overhead must not count

enum Mix { kMfma, kMfmaValu, kMfmaValuLds, kMfmaValuHalfLds, kExp, kFma, kCvt, kMax3, kReadB128, kReadTr };

template <int MIX>
__global__ __launch_bounds__(512) void probe(long long* ticks, float* sink, int iters, float seed) {
  __shared__ float lds[16384];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) lds[i] = seed * i;
  __syncthreads();
  float x[16];
  for (int i = 0; i < 16; ++i) x[i] = seed + i * 0.001f + threadIdx.x * 1e-6f;
  f32x16 acc0 = {0}, acc1 = {0};
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(seed + i);
    b[i] = (__bf16)(seed - i);
  }
  f32x4 q0 = {0}, q1 = {0}, q2, q3;
  f32x2 h0 = {0}, h1 = {0}, h2 = {0}, h3 = {0};
  const unsigned wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const unsigned base = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) void*)lds + (wave & 3) * 8192;
  const unsigned addr16 = base + lane * 16, addr8 = base + lane * 8;  // conflict-free

  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
    if (MIX == kMfma) {
#pragma unroll
      for (int r = 0; r < kRepeat; ++r) {
        MFMA(acc0); MFMA(acc1); MFMA(acc0); MFMA(acc1);
      }
    } else if (MIX == kMfmaValu || MIX == kMfmaValuLds || MIX == kMfmaValuHalfLds) {
      // The kernel's totals per 16 MFMAs: 48 plain VALU ops, 8 conversions, 8 max3, 16 exponentials
      // (on rotating registers: no instruction waits for its neighbour), and 16 KB (or 8 KB) of
      // fragments, each group of reads waited for four MFMAs after its issue.
#pragma unroll
      for (int g = 0; g < 4 * kRepeat; ++g) {
        if ((g & 3) == 0 && MIX != kMfmaValu) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::"v"(q0), "v"(q1), "v"(h0), "v"(h1), "v"(h2), "v"(h3) : "memory");
          if (MIX == kMfmaValuLds) {
            asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:1024" : "=v"(q0), "=v"(q1) : "v"(addr16));
            asm volatile("ds_read_b64_tr_b16 %0, %4\n\tds_read_b64_tr_b16 %1, %4 offset:512\n\t"
                         "ds_read_b64_tr_b16 %2, %4 offset:1024\n\tds_read_b64_tr_b16 %3, %4 offset:1536"
                         : "=v"(h0), "=v"(h1), "=v"(h2), "=v"(h3) : "v"(addr8));
          } else {
            asm volatile("ds_read_b128 %0, %1" : "=v"(q0) : "v"(addr16));
            asm volatile("ds_read_b64_tr_b16 %0, %2\n\tds_read_b64_tr_b16 %1, %2 offset:512" : "=v"(h0), "=v"(h1) : "v"(addr8));
          }
        }
        if (g & 1) MFMA(acc1);
        else MFMA(acc0);
        FMA(x[g & 15]);
        FMA(x[(g + 1) & 15]);
        FMA(x[(g + 2) & 15]);
        if (g & 1) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(x[(g + 4) & 15]));
        else asm volatile("v_max3_f32 %0, %0, %0, %0" : "+v"(x[(g + 4) & 15]));
        EXP(x[(g + 3) & 15]);
      }
    } else if (MIX == kExp) {
#pragma unroll
      for (int i = 0; i < 16; ++i) EXP(x[i]);
    } else if (MIX == kFma) {
#pragma unroll
      for (int i = 0; i < 16; ++i) FMA(x[i]);
    } else if (MIX == kCvt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(x[i]));
    } else if (MIX == kMax3) {
#pragma unroll
      for (int i = 0; i < 16; ++i) asm volatile("v_max3_f32 %0, %0, %0, %0" : "+v"(x[i]));
    } else if (MIX == kReadB128) {
      asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\tds_read_b128 %2, %4 offset:2048\n\t"
                   "ds_read_b128 %3, %4 offset:3072\n\ts_waitcnt lgkmcnt(0)"
                   : "=v"(q0), "=v"(q1), "=v"(q2), "=v"(q3) : "v"(addr16));
      asm volatile("" ::"v"(q0), "v"(q1), "v"(q2), "v"(q3));
    } else if (MIX == kReadTr) {
      asm volatile("ds_read_b64_tr_b16 %0, %4\n\tds_read_b64_tr_b16 %1, %4 offset:512\n\tds_read_b64_tr_b16 %2, %4 offset:1024\n\t"
                   "ds_read_b64_tr_b16 %3, %4 offset:1536\n\ts_waitcnt lgkmcnt(0)"
                   : "=v"(h0), "=v"(h1), "=v"(h2), "=v"(h3) : "v"(addr8));
      asm volatile("" ::"v"(h0), "v"(h1), "v"(h2), "v"(h3));
    }
  }
  const long long t1 = clock64();
  float s = 0;
  for (int i = 0; i < 16; ++i) s += x[i] + acc0[i] + acc1[i];
  if (s == 123.456f) sink[0] = s;  // keeps the loop alive
  if (lane == 0) ticks[blockIdx.x * (blockDim.x / 64) + wave] = t1 - t0;
}

template <int MIX>
double run(int iters) {
  const int blocks = 256, threads = 512, waves = blocks * threads / 64;
  long long* d = nullptr;
  float* sink = nullptr;
  if (hipMalloc(&d, waves * sizeof(long long)) != hipSuccess || hipMalloc(&sink, 4) != hipSuccess) exit(1);
  probe<MIX><<<blocks, threads>>>(d, sink, iters, 0.5f);  // warm-up
  probe<MIX><<<blocks, threads>>>(d, sink, iters, 0.5f);
  if (hipDeviceSynchronize() != hipSuccess) exit(1);
  std::vector<long long> h(waves);
  if (hipMemcpy(h.data(), d, waves * sizeof(long long), hipMemcpyDeviceToHost) != hipSuccess) exit(1);
  double avg = 0;
  for (long long v : h) avg += (double)v;
  (void)hipFree(d);
  (void)hipFree(sink);
  return avg / waves / iters;
}

int main(int argc, char** argv) {
  const int iters = argc > 1 ? atoi(argv[1]) : 5000;
  const double mfma = run<kMfma>(iters) / kRepeat;  // 4 MFMAs per wave, 8 per SIMD
  printf("two waves per SIMD, %d iterations; ticks = s_memtime counts per group of 4 MFMAs and wave\n", iters);
  printf("%-58s %8.1f ticks  MFMA utilisation 100.0 %%\n", "4 mfma_f32_32x32x16_bf16", mfma);
  const double v = run<kMfmaValu>(iters) / kRepeat;
  printf("%-58s %8.1f ticks  MFMA utilisation %5.1f %%\n", "4 mfma + 12 v_fma + 2 v_cvt_pk + 2 v_max3 + 4 v_exp", v, 100 * mfma / v);
  const double l = run<kMfmaValuLds>(iters) / kRepeat;
  printf("%-58s %8.1f ticks  MFMA utilisation %5.1f %%\n", "  + 2 ds_read_b128 + 4 ds_read_b64_tr_b16 (4 KB)", l, 100 * mfma / l);
  const double hl = run<kMfmaValuHalfLds>(iters) / kRepeat;
  printf("%-58s %8.1f ticks  MFMA utilisation %5.1f %%\n", "  + 1 ds_read_b128 + 2 ds_read_b64_tr_b16 (2 KB)", hl, 100 * mfma / hl);
  const double per_mfma = mfma / 8.0;  // ticks of one MFMA (32 cycles) when the pipe is saturated
  printf("single instruction classes, cycles per instruction and wave (one MFMA = 32 cycles):\n");
  printf("  v_exp_f32 %.1f   v_fma_f32 %.1f   v_cvt_pk_bf16_f32 %.1f   v_max3_f32 %.1f\n",
         run<kExp>(iters) / 32 / per_mfma * 32, run<kFma>(iters) / 32 / per_mfma * 32,
         run<kCvt>(iters) / 32 / per_mfma * 32, run<kMax3>(iters) / 32 / per_mfma * 32);
  // 8 waves per CU each read 4 KB (b128) or 2 KB (tr_b64) per iteration
  printf("  LDS bytes per cycle and CU, with a wait after every four reads: ds_read_b128 %.0f   ds_read_b64_tr_b16 %.0f\n",
         8 * 4096.0 / (run<kReadB128>(iters) / per_mfma * 32), 8 * 2048.0 / (run<kReadTr>(iters) / per_mfma * 32));
  return 0;
}
