// Device-side helpers shared by the gfx950 kernels of this library (vector types, direct-to-LDS
// loads, MFMA wrappers, cross-half exchanges, LDS swizzles, the workgroup -> job mapping).
#pragma once
#include "ringattn_kernels.h"

namespace ringattn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// 16 bytes per lane HBM -> LDS without passing through registers: lane i's data lands
// at lds_addr + 16 i (lds_addr is wave-uniform and travels in M0).  Written as inline
// asm so the compiler does not serialise later LDS reads behind the transfer; the
// kernel waits for it explicitly (s_waitcnt vmcnt(0)) before the tile barrier.
// No "memory" clobber: a transfer only ever targets a ring slot that no LDS read between
// the surrounding barriers touches, so the compiler may move LDS reads across it.
// M0 is declared clobbered, and the s_nop is the wait state the hardware needs between a
// scalar write of M0 and the LDS-DMA instruction that reads it (the assembler inserts none
// inside inline asm).
static __device__ __forceinline__ void load_lds_16(const void* base, int voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "m0");
}
// The same transfer for call sites whose base address may have just come out of a v_readfirstlane: a vector
// instruction that wrote a scalar register must be five wait states ahead of the memory instruction that reads it,
// and the compiler does not see into inline asm to provide them.
static __device__ __forceinline__ void load_lds_16_settled(const void* base, int voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "m0");
}
static __device__ __forceinline__ unsigned lds_offset(const void* p) {
  return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

template <int DT> struct Elem;
template <> struct Elem<0> {
  using type = _Float16;
  using vec8 = f16x8;
  using vec4 = f16x4;
  static __device__ __forceinline__ f32x16 mma(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(vec8, a), __builtin_bit_cast(vec8, b), c, 0, 0, 0);
  }
};
template <> struct Elem<1> {
  using type = __bf16;
  using vec8 = bf16x8;
  using vec4 = bf16x4;
  static __device__ __forceinline__ f32x16 mma(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(vec8, a), __builtin_bit_cast(vec8, b), c, 0, 0, 0);
  }
};

// max / sum across the two 32-lane halves of a wave.  v_permlane32_swap exchanges the
// upper half of its first operand with the lower half of its second, so with both
// operands holding x every lane ends up with its own x and the x of the lane 32 away.
// Inline asm on purpose: the compiler builtin, given the same value for both operands,
// merges the two results into one register and drops the exchanged half.  The s_nop
// covers the VALU-write -> permlane-read hazard the assembler does not see inside asm.
static __device__ __forceinline__ void swap_halves(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
static __device__ __forceinline__ float cross_half_max(float x) {
  float a = x, b = x, r;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %1, %2\n\ts_nop 1\n\tv_max_f32 %0, %1, %2" : "=v"(r), "+v"(a), "+v"(b));
  return r;
}
static __device__ __forceinline__ float cross_half_sum(float x) {
  float a = x, b = x;
  swap_halves(a, b);
  return a + b;
}

// XOR swizzles on 16-byte chunk indices within a tile row (row = key, 2*D bytes).
// K is read with ds_read_b128 by 32 lanes on 32 consecutive rows; V is read with
// ds_read_b64_tr_b16 by groups of 16 lanes covering 4 rows x 32 bytes.
template <int D> static __device__ __forceinline__ int k_swizzle(int row) {
  return D == 128 ? (row & 15) : ((row >> 1) & 7);
}
template <int D> static __device__ __forceinline__ int v_swizzle(int row) {
  return D == 128 ? (((row & 3) << 2) | (((row >> 2) & 1) << 1))
                  : ((((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1));
}

// workgroup -> job (segment, head, q tile); false for the holes of the grid.  blockIdx mod 8 is
// the XCD: the q tiles of a (segment, head) group are consecutive workgroups of one XCD and share
// its K and V in that L2.  With a group table the host has dealt the heads to the XCDs and
// listed, per XCD, the segments of one head after the other (busiest first): ranks of a head
// follow each other through the same K and V, which then stay in that XCD's L2 / the
// memory-side cache.  Without one, groups are dealt to the XCDs in segment-major order.
template <int TILE_ROWS>
static __device__ __forceinline__ bool decode_job(const BlockArgs& a, Segment& seg, int& bh, int& qt) {
  const int q_tiles = a.q_tiles_max;
  const int xcd = blockIdx.x & 7, wslot = blockIdx.x >> 3;
  int sg;
  if (a.groups) {
    const int2 g = a.groups[xcd * a.groups_per_xcd + wslot / q_tiles];
    sg = g.x;
    bh = g.y;
    if (sg < 0) return false;
  } else {
    const int group = (wslot / q_tiles) * 8 + xcd;
    if (group >= a.n_segs * a.BH) return false;
    sg = group / a.BH;
    bh = group % a.BH;
  }
  seg = a.segs[sg];
  qt = wslot % q_tiles;
  if (qt * TILE_ROWS >= seg.q_len) return false;  // segments shorter than the longest one
  if (seg.reverse_tiles) qt = (seg.q_len + TILE_ROWS - 1) / TILE_ROWS - 1 - qt;  // most keys first
  return true;
}

// ---- conversions of 8 columns of a row, shared by the merge kernel and the merge at the end of a workgroup
template <int DT> struct Store8;
template <> struct Store8<0> {
  static __device__ __forceinline__ void st(void* p, const float* x) {
    f16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (_Float16)x[e];
    *(f16x8*)p = v;
  }
};
template <> struct Store8<1> {
  static __device__ __forceinline__ void st(void* p, const float* x) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)x[e];
    *(bf16x8*)p = v;
  }
};

// 8 consecutive columns of one partial row as floats
template <bool HP> struct PartRow;
template <> struct PartRow<false> {
  using ptr = const float*;
  static __device__ __forceinline__ void ld(ptr p, f32x4& x0, f32x4& x1) {
    x0 = *(const f32x4*)p;
    x1 = *(const f32x4*)(p + 4);
  }
};
template <> struct PartRow<true> {
  using ptr = const _Float16*;
  static __device__ __forceinline__ void ld(ptr p, f32x4& x0, f32x4& x1) {
    const f16x8 v = *(const f16x8*)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x0[e] = (float)v[e];
      x1[e] = (float)v[4 + e];
    }
  }
};

// ---- merge of one job's rows (BM rows of a segment, one head) over the partials of the
// segment's items.  The same arithmetic, in the same order, as merge_row; only the loads are
// arranged differently: the attention kernel, which runs this at the end of a workgroup, has just two
// waves per SIMD to hide memory latency with, and every round trip it waits for is time its
// compute unit runs half empty.  So all partial LSEs are fetched in one sweep and parked in LDS
// (lse_s: [items][128] floats), and the partial O rows move in batches of 256 bytes per thread
// (two output rows x four or eight parts), three batches in flight at any time.
typedef __attribute__((address_space(3))) float lds_float;
template <int DT, int D, bool HP, int BM, int THREADS>
static __device__ __forceinline__ void merge_job_rows(const void* o_part, const float* lse_part, void* out, float* lse,
                                                      const SegItem* items, const Segment& seg, int bh, int qt, int S,
                                                      lds_float* lse_s) {
  constexpr int WAVES = THREADS / 64;
  constexpr int TPR = D / 8;  // threads per row, 8 columns each
  constexpr int ROWS = THREADS / TPR;
  constexpr int R = 2, G = HP ? 8 : 4;  // rows per thread and parts per batch: 64 registers a batch
  constexpr int RSTEP = R * ROWS;
  constexpr int KMAX = kMaxParts / WAVES;  // parts per wave in the LSE sweep
  constexpr int LR = BM / 64;              // rows per lane in the LSE sweep
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_parts = seg.item_count;
  const SegItem* its = items + seg.item_begin;
  const int row0 = qt * BM;  // first row of the job within the segment
  __syncthreads();  // the partial stores of all waves have completed and are visible to them; the LDS is idle
  {
    float v[KMAX][LR];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int i = wave + WAVES * k;
      if (i < n_parts) {
        const int64_t prow = its[i].part_base + (int64_t)bh * its[i].part_bh_stride + row0;
#pragma unroll
        for (int r = 0; r < LR; ++r) v[k][r] = (row0 + lane + 64 * r < seg.q_len) ? lse_part[prow + lane + 64 * r] : -INFINITY;
      }
    }
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int i = wave + WAVES * k;
      if (i < n_parts) {
#pragma unroll
        for (int r = 0; r < LR; ++r) lse_s[i * BM + lane + 64 * r] = v[k][r];
      }
    }
  }
  __syncthreads();
  const int c8 = tid % TPR, rsub = tid / TPR;
  // this thread's 8 columns of a partial row: 16 bytes as fp16, 32 as fp32
  constexpr int PB = HP ? 16 : 32;
  constexpr int NV = PB / 16;
  const char* o_base = (const char*)o_part + c8 * PB;
  const int n_groups = (n_parts + G - 1) / G;
  const int n_batches = (BM / RSTEP) * n_groups;  // batch b: rows of b / n_groups, parts of b % n_groups
  struct Batch {
    f32x4 raw[R][G][NV];  // as loaded; fp16 partials are widened when they are used
  };
  auto row_of = [&](int b, int j) { return (b / n_groups) * RSTEP + j * ROWS + rsub; };  // within the job
  auto fetch = [&](int b, Batch& t) {
    const int i0 = (b % n_groups) * G;
#pragma unroll
    for (int u = 0; u < G; ++u)
      if (i0 + u < n_parts) {
        const int64_t prow = its[i0 + u].part_base + (int64_t)bh * its[i0 + u].part_bh_stride + row0;
#pragma unroll
        for (int j = 0; j < R; ++j)
          if (row0 + row_of(b, j) < seg.q_len) {
            const char* src = o_base + (prow + row_of(b, j)) * (D * (PB / 8));
#pragma unroll
            for (int v = 0; v < NV; ++v) t.raw[j][u][v] = *(const f32x4*)(src + 16 * v);
          }
      }
  };
  float mx[R], wsum[R], acc[R][8];
  auto accumulate = [&](int b, const Batch& t) {
    const int g = b % n_groups, i0 = g * G;
    if (g == 0) {  // new rows: L = max over the parts first
#pragma unroll
      for (int j = 0; j < R; ++j) {
        mx[j] = -INFINITY;
        wsum[j] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
      }
      for (int i = 0; i < n_parts; ++i)
#pragma unroll
        for (int j = 0; j < R; ++j) mx[j] = fmaxf(mx[j], lse_s[i * BM + row_of(b, j)]);
    }
#pragma unroll
    for (int u = 0; u < G; ++u)
      if (i0 + u < n_parts) {
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const float L = lse_s[(i0 + u) * BM + row_of(b, j)];
          if (row0 + row_of(b, j) >= seg.q_len || L == -INFINITY) continue;  // identity element: its O may hold anything
          const float w = __expf(L - mx[j]);
          wsum[j] += w;
          float x[8];
          if (HP) {
            const f16x8 hv = __builtin_bit_cast(f16x8, t.raw[j][u][0]);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (float)hv[e];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              x[e] = t.raw[j][u][0][e];
              x[4 + e] = t.raw[j][u][NV - 1][e];
            }
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[j][e] = __builtin_fmaf(w, x[e], acc[j][e]);
        }
      }
    if (g == n_groups - 1) {  // all parts in: normalise and store
#pragma unroll
      for (int j = 0; j < R; ++j) {
        if (row0 + row_of(b, j) >= seg.q_len) continue;
        if (mx[j] != -INFINITY) {
          const float inv = 1.f / wsum[j];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[j][e] *= inv;
        }
        const int64_t out_row = (int64_t)bh * S + seg.q_start + row0 + row_of(b, j);
        Store8<DT>::st((char*)out + (out_row * D + c8 * 8) * 2, acc[j]);
        if (c8 == 0) lse[out_row] = (mx[j] == -INFINITY) ? -INFINITY : mx[j] + __logf(wsum[j]);
      }
    }
  };
  // three batches in flight
  Batch t0, t1, t2;
  fetch(0, t0);
  if (1 < n_batches) fetch(1, t1);
#pragma unroll 1
  for (int b = 0; b < n_batches; b += 3) {
    if (b + 2 < n_batches) fetch(b + 2, t2);
    accumulate(b, t0);
    if (b + 3 < n_batches) fetch(b + 3, t0);
    if (b + 1 < n_batches) accumulate(b + 1, t1);
    if (b + 4 < n_batches) fetch(b + 4, t1);
    if (b + 2 < n_batches) accumulate(b + 2, t2);
  }
}

}  // namespace ringattn
