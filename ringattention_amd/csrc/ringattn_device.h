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

}  // namespace ringattn
