// gfx950 (CDNA4) kernels for the ring-attention forward path.
//
//   block_attention_kernel : one ring step for every active virtual rank --
//       S^T = K Q^T, online softmax with running max / sum, O^T += V^T P^T,
//       emitting a normalised fp32 partial O and a natural-log fp32 LSE.
//       It restates the inner KV-tile loop of the reference kernel
//       (csrc/ring_attention.cu:536-610: gemm_smem :278-301, softmax_rescale_o
//       :194-245 completed with the missing `sum += sum_cur` tail,
//       scale_apply_exp2 :173-192, gemm_A_in_regs :304-324) and its epilogue
//       (:621-664), with the tiling of csrc/kernel_traits.h:11-177 replaced by a
//       wave64 / MFMA 32x32x16 design:
//         * each of the 4 waves owns 32 query rows; Q lives in registers as the
//           B operand for the whole launch (the reference re-reads it from smem
//           for every tile, :565);
//         * the score tile is computed TRANSPOSED (keys x queries), so one lane
//           holds 16 keys of ONE query: row max / row sum are in-register
//           reductions plus one cross-half exchange, and the probabilities are
//           already in B-operand layout for O^T += V^T P^T -- the MFMA analogue
//           of convert_layout_rowcol_Aregs (:260-276);
//         * K and V tiles go HBM -> LDS directly (global_load_lds_dwordx4),
//           double-buffered, one barrier per tile; bank conflicts are removed
//           by an XOR swizzle applied on the global-address side;
//         * V^T operands come from ds_read_b64_tr_b16 (the LDS transpose read),
//           replacing ldmatrix.trans of csrc/kernel_traits.h:39.
//   merge_kernel : P-way merge of the per-step (O, LSE) partials.  The reference
//       has no such function: it carries (max, sum, acc-O) in registers across
//       ring steps (:439-443,597).  The merge is the algebraic equivalent on
//       (O, LSE) pairs.
#include "ringattn_kernels.h"
#include <cstdlib>
#include <type_traits>

namespace ringattn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// 16 bytes per lane HBM -> LDS without passing through registers: lane i's data lands
// at lds_addr + 16 i (lds_addr is wave-uniform and travels in M0).  Written as inline
// asm so the compiler does not serialise later LDS reads behind the transfer; the
// kernel waits for it explicitly (s_waitcnt vmcnt(0)) before the tile barrier.
// Nothing else in these kernels uses M0.
static __device__ __forceinline__ void load_lds_16(const void* base, int voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
static __device__ __forceinline__ unsigned lds_offset(const void* p) {
  return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

template <int DT> struct Elem;
template <> struct Elem<0> {
  using type = _Float16;
  using vec8 = f16x8;
  static __device__ __forceinline__ f32x16 mma(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(vec8, a), __builtin_bit_cast(vec8, b), c, 0, 0, 0);
  }
};
template <> struct Elem<1> {
  using type = __bf16;
  using vec8 = bf16x8;
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
  float a = x, b = x;
  swap_halves(a, b);
  return fmaxf(a, b);
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

template <int DT, int D, int BN>
__global__ __launch_bounds__(256, 2) void block_attention_kernel(const BlockStepArgs a) {
  using E = Elem<DT>;
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = D * 2;      // bytes per row
  constexpr int TILE = BN * ROWB;  // bytes per K or V tile
  constexpr int KB = BN / 32;      // 32-key blocks per tile
  constexpr int KS = D / 16;       // contraction slices of QK^T
  constexpr int DB = D / 32;       // 32-wide blocks of the head dim in PV
  constexpr int LD_PER_WAVE = (BN * CPR) / 256;  // LDS-DMA instructions per wave per tile
  static_assert(LD_PER_WAVE >= 1 && (BN * CPR) % 256 == 0, "tile must split over 4 waves");
  __shared__ __attribute__((aligned(1024))) unsigned char smem[4 * TILE];  // K0 K1 V0 V1

  const unsigned smem_base = lds_offset(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;

  // workgroup -> (head, rank, q tile).  Consecutive workgroup ids go round-robin over
  // the 8 XCDs, so all q tiles of one (head, rank) -- which stream the same KV chunk --
  // are placed on one XCD and share its L2.
  const int q_tiles = a.chunk / kBlockM;
  const int groups = a.n_active * a.BH;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int group = (slot / q_tiles) * 8 + xcd;
  if (group >= groups) return;
  const int ridx = group % a.n_active, bh = group / a.n_active;
  const int r = a.rank_base + ridx;
  int j = r + a.step;
  if (j >= a.P) j -= a.P;
  if (a.causal && j > r) return;  // fully masked pair: never launched by the host loop
  const bool diag = a.causal && (j == r);
  int qt = slot % q_tiles;
  if (diag) qt = q_tiles - 1 - qt;  // heaviest q tiles first
  const int n_tiles = diag ? ((qt + 1) * kBlockM) / BN : a.chunk / BN;

  const int64_t head_off = (int64_t)bh * a.bh_stride;
  const char* qbase = (const char*)a.q + (head_off + (int64_t)(r * a.chunk + qt * kBlockM) * D) * 2;
  const char* kbase = (const char*)a.k + (head_off + (int64_t)j * a.chunk * D) * 2;
  const char* vbase = (const char*)a.v + (head_off + (int64_t)j * a.chunk * D) * 2;

  // Q fragment: B operand of S^T = K Q^T.  Lane (n, h) holds Q[row n][16 ks + 8 h .. +8).
  s16x8 qf[KS];
  {
    const char* qrow = qbase + (int64_t)(32 * wave + n) * ROWB + h * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const s16x8*)(qrow + ks * 32);
  }

  // per-lane source offsets of the direct-to-LDS tile loads (swizzle on the global side)
  int goff_k[LD_PER_WAVE], goff_v[LD_PER_WAVE];
#pragma unroll
  for (int i = 0; i < LD_PER_WAVE; ++i) {
    const int p = (wave * LD_PER_WAVE + i) * 64 + lane;
    const int row = p / CPR, pc = p % CPR;
    goff_k[i] = row * ROWB + ((pc ^ k_swizzle<D>(row)) << 4);
    goff_v[i] = row * ROWB + ((pc ^ v_swizzle<D>(row)) << 4);
  }
  // K operand read offsets: lane (n, h) reads row 32 kb + n, logical chunk 2 ks + h
  int koff[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = n * ROWB + (((2 * ks + h) ^ k_swizzle<D>(n)) << 4);
  // V^T operand read offsets (ds_read_b64_tr_b16): within a group of 16 lanes, lane s
  // points at V[k0 + s/4][dbase + 4 (s%4) .. +4) and receives V[k0 .. k0+4)[dbase + s].
  int voff[DB];
  {
    const int s = lane & 15, g1 = (lane >> 4) & 1;
    const int row8 = 4 * h + (s >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int c = 2 * (2 * db + g1) + ((s & 3) >> 1);
      voff[db] = row8 * ROWB + ((c ^ v_swizzle<D>(row8)) << 4) + ((s & 1) << 3);
    }
  }

  float m = -INFINITY, lsum = 0.f;
  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;

  // direct-to-LDS loads of one K or V tile (this wave's share)
  auto issue_k = [&](int t, int buf) {
    const char* kt = kbase + (int64_t)t * TILE;
    const unsigned kd = __builtin_amdgcn_readfirstlane(smem_base + buf * TILE + wave * (LD_PER_WAVE * 1024));
#pragma unroll
    for (int i = 0; i < LD_PER_WAVE; ++i) load_lds_16(kt, goff_k[i], kd + i * 1024);
  };
  auto issue_v = [&](int t, int buf) {
    const char* vt = vbase + (int64_t)t * TILE;
    const unsigned vd = __builtin_amdgcn_readfirstlane(smem_base + (2 + buf) * TILE + wave * (LD_PER_WAVE * 1024));
#pragma unroll
    for (int i = 0; i < LD_PER_WAVE; ++i) load_lds_16(vt, goff_v[i], vd + i * 1024);
  };
  // K fragments (A operand of S^T = K Q^T) of a whole tile, LDS -> registers
  s16x8 kf[KS][KB];
  auto load_k_frags = [&](int buf) {
    const unsigned char* ks_lds = smem + buf * TILE;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) kf[ks][kb] = *(const s16x8*)(ks_lds + kb * 32 * ROWB + koff[ks]);
  };
  // S^T = K Q^T : keys x queries, fp32 accumulate (csrc/ring_attention.cu:565), then the
  // online softmax (:194-245).  Leaves P^T, rounded to the storage type, in pf as B operands.
  s16x8 pf[KB][2];
  auto scores_and_softmax = [&](int t) {
    f32x16 sacc[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) sacc[kb][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) sacc[kb] = E::mma(kf[ks][kb], qf[ks], sacc[kb]);

    // diagonal chunk pair: key visible iff key_local <= query_local
    if (diag && (t + 1) * BN - 1 > qt * kBlockM) {
      const int lim = qt * kBlockM + 32 * wave + n - t * BN - 4 * h;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = 32 * kb + 8 * (e >> 2) + (e & 3);
          if (key > lim) sacc[kb][e] = -INFINITY;
        }
    }

    // this lane's query is n: in-register max, one exchange with the other half
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[kb][e]);
    mx = cross_half_max(mx);
    const float m_new = fmaxf(m, mx);
    // all-masked guard of scale_apply_exp2 (csrc/ring_attention.cu:183)
    const float ms = (m_new == -INFINITY) ? 0.f : m_new * a.scale_log2;
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {  // some row's running max moved
      const float alpha = __builtin_amdgcn_exp2f(m * a.scale_log2 - ms);
      lsum *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
    }
    m = m_new;

    // P^T = exp2(S^T k2 - m k2); row sum from the unrounded values (:242), operands
    // rounded to the storage type (:604)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        typename E::vec8 pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][8 * t2 + e], a.scale_log2, -ms));
          lsum += p;
          pv[e] = (typename E::type)p;
        }
        pf[kb][t2] = __builtin_bit_cast(s16x8, pv);
      }
  };
  // O^T += V^T P^T (csrc/ring_attention.cu:609).  MFMA slice (kb, t2) contracts over keys
  // 32 kb + 16 t2 + {4 h + 0..3, 8 + 4 h + 0..3}, the keys this lane's P values belong to.
  auto pv_product = [&](int buf) {
    const unsigned char* vs_lds = smem + (2 + buf) * TILE;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        const unsigned char* vrow = vs_lds + (32 * kb + 16 * t2) * ROWB;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + voff[db]));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + 8 * ROWB + voff[db]));
          const s16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[db] = E::mma(vf, pf[kb][t2], oacc[db]);
        }
      }
  };

  // Retire the Q loads here, with a wait the compiler can see: otherwise it places
  // counted vmcnt waits at their first use inside the loop, and those would also
  // drain the direct-to-LDS prefetch it does not know about.
  __builtin_amdgcn_s_waitcnt(0);

  // one barrier per tile at the top; K and V of tile t+1 are in flight while tile t is computed
  issue_k(0, 0);
  issue_v(0, 0);
  for (int t = 0; t < n_tiles; ++t) {
    const int buf = t & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // tile t is in LDS; every wave is done with tile t-1
    if (t + 1 < n_tiles) {
      issue_k(t + 1, buf ^ 1);
      issue_v(t + 1, buf ^ 1);
    }
    load_k_frags(buf);
    scores_and_softmax(t);
    pv_product(buf);
  }

  // epilogue (csrc/ring_attention.cu:621-633): normalise, emit partial O and LSE
  const float l = cross_half_sum(lsum);
  const float inv = (l > 0.f) ? 1.f / l : 0.f;
  const int row_g = r * a.chunk + qt * kBlockM + 32 * wave + n;
  float* orow = a.o_part + ((int64_t)bh * a.S + row_g) * D;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f32x4 val;
#pragma unroll
      for (int e = 0; e < 4; ++e) val[e] = oacc[db][4 * q4 + e] * inv;
      *(f32x4*)(orow + 32 * db + 8 * q4 + 4 * h) = val;
    }
  if (h == 0) {
    const float lse = (l > 0.f) ? (m * a.scale_log2 + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
    a.lse_part[(int64_t)bh * a.S + row_g] = lse;
  }
}

// ---- software-pipelined block kernel ---------------------------------------------------
// Same math and data layout as block_attention_kernel, different schedule.  The KV chunk is
// consumed in 32-key tiles held in two 4-deep LDS rings (K and V).  Block u of the loop
// runs, in ONE instruction stream,
//     MFMAs of S^T(u+1) = K(u+1) Q^T      next to   the exponentials of tile u,
//     MFMAs of O^T += V(u)^T P(u)^T       next to   the row-max reduction of tile u+1,
// so every wave feeds the matrix pipe and the VALU at the same time instead of alternating
// between them.  The exponent offset m is a REFERENCE max: it is moved (with the rescale of
// l and acc-O of csrc/ring_attention.cu:226-232) only when some row's tile max exceeds it by
// more than 2^kLazyLog2, decided at the end of a block, which keeps the blocks free of
// branches.  Until then p = exp2((s - m) k2) may exceed 1; O = acc / l and
// LSE = (m k2 + log2 l) ln 2 do not depend on the choice of m.
template <int DT, int D, int SCHED>
__global__ __launch_bounds__(256, 2) void block_attention_pipe_kernel(const BlockStepArgs a) {
  using E = Elem<DT>;
  constexpr int BM = 128;          // query rows per workgroup (4 waves x 32)
  constexpr int BN = 32;           // keys per tile
  constexpr int NBUF = 4;          // ring depth of the K and of the V tiles
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = D * 2;      // bytes per row
  constexpr int TILE = BN * ROWB;  // bytes per tile
  constexpr int KS = D / 16;       // contraction slices of QK^T
  constexpr int DB = D / 32;       // 32-wide blocks of the head dim in PV
  constexpr int LD = (BN * CPR) / 256;  // LDS-DMA instructions per wave per tile
  constexpr float kLazyLog2 = 8.f;
  static_assert(LD >= 1, "tile must split over 4 waves");
  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * NBUF * TILE];  // K ring, V ring

  const unsigned smem_base = lds_offset(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;

  // workgroup -> (head, rank, q tile), XCD-aware as in block_attention_kernel
  const int q_tiles = a.chunk / BM;
  const int groups = a.n_active * a.BH;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int group = (slot / q_tiles) * 8 + xcd;
  if (group >= groups) return;
  const int ridx = group % a.n_active, bh = group / a.n_active;
  const int r = a.rank_base + ridx;
  int j = r + a.step;
  if (j >= a.P) j -= a.P;
  if (a.causal && j > r) return;
  const bool diag = a.causal && (j == r);
  int qt = slot % q_tiles;
  if (diag) qt = q_tiles - 1 - qt;
  const int n_tiles = diag ? ((qt + 1) * BM) / BN : a.chunk / BN;
  const int first_masked = diag ? (qt * BM) / BN : n_tiles;  // tiles >= this need the causal mask

  const int64_t head_off = (int64_t)bh * a.bh_stride;
  const char* qbase = (const char*)a.q + (head_off + (int64_t)(r * a.chunk + qt * BM) * D) * 2;
  const char* kbase = (const char*)a.k + (head_off + (int64_t)j * a.chunk * D) * 2;
  const char* vbase = (const char*)a.v + (head_off + (int64_t)j * a.chunk * D) * 2;

  s16x8 qf[KS];
  {
    const char* qrow = qbase + (int64_t)(32 * wave + n) * ROWB + h * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const s16x8*)(qrow + ks * 32);
  }
  int goff_k[LD], goff_v[LD];
#pragma unroll
  for (int i = 0; i < LD; ++i) {
    const int p = (wave * LD + i) * 64 + lane;
    const int row = p / CPR, pc = p % CPR;
    goff_k[i] = row * ROWB + ((pc ^ k_swizzle<D>(row)) << 4);
    goff_v[i] = row * ROWB + ((pc ^ v_swizzle<D>(row)) << 4);
  }
  int koff[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = n * ROWB + (((2 * ks + h) ^ k_swizzle<D>(n)) << 4);
  int voff[DB];
  {
    const int s = lane & 15, g1 = (lane >> 4) & 1;
    const int row8 = 4 * h + (s >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int c = 2 * (2 * db + g1) + ((s & 3) >> 1);
      voff[db] = row8 * ROWB + ((c ^ v_swizzle<D>(row8)) << 4) + ((s & 1) << 3);
    }
  }

  float m = -INFINITY;  // reference max (raw score units)
  float ms = 0.f;       // m * k2, 0 while m is -inf (guard of csrc/ring_attention.cu:183)
  float ls[4] = {0.f, 0.f, 0.f, 0.f};
  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  f32x16 s_even, s_odd;
  s16x8 pf[2];

  auto issue_k = [&](int t) {
    const char* kt = kbase + (int64_t)t * TILE;
    const unsigned kd = __builtin_amdgcn_readfirstlane(smem_base + (t & (NBUF - 1)) * TILE + wave * (LD * 1024));
#pragma unroll
    for (int i = 0; i < LD; ++i) load_lds_16(kt, goff_k[i], kd + i * 1024);
  };
  auto issue_v = [&](int t) {
    const char* vt = vbase + (int64_t)t * TILE;
    const unsigned vd = __builtin_amdgcn_readfirstlane(smem_base + (NBUF + (t & (NBUF - 1))) * TILE + wave * (LD * 1024));
#pragma unroll
    for (int i = 0; i < LD; ++i) load_lds_16(vt, goff_v[i], vd + i * 1024);
  };
  // S^T = K Q^T of one 32-key tile (csrc/ring_attention.cu:565)
  auto qk = [&](f32x16& sacc, int kslot) {
    const unsigned char* ks_lds = smem + kslot * TILE;
#pragma unroll
    for (int e = 0; e < 16; ++e) sacc[e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const s16x8 kfr = *(const s16x8*)(ks_lds + koff[ks]);
      sacc = E::mma(kfr, qf[ks], sacc);
    }
  };
  auto mask_tile = [&](f32x16& sacc, int t) {
    if (t >= first_masked) {  // diagonal chunk pair: key visible iff key_local <= query_local
      const int lim = qt * BM + 32 * wave + n - t * BN - 4 * h;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int key = 8 * (e >> 2) + (e & 3);
        if (key > lim) sacc[e] = -INFINITY;
      }
    }
  };
  auto tile_max = [&](const f32x16& sacc) {
    // two chains of max(max(m, a), b): the compiler folds each into one v_max3_f32
    float m0 = sacc[0], m1 = sacc[1];
#pragma unroll
    for (int e = 2; e < 16; e += 4) {
      m0 = fmaxf(fmaxf(m0, sacc[e]), sacc[e + 1]);
      if (e + 3 < 16) m1 = fmaxf(fmaxf(m1, sacc[e + 2]), sacc[e + 3]);
    }
    return cross_half_max(fmaxf(m0, m1));
  };
  auto move_reference = [&](float tm) {
    if (__builtin_amdgcn_ballot_w64((tm - m) * a.scale_log2 > kLazyLog2) != 0) {
      const float cand = fmaxf(m, tm);
      const float cs = (cand == -INFINITY) ? 0.f : cand * a.scale_log2;
      const float alpha = __builtin_amdgcn_exp2f(m * a.scale_log2 - cs);
#pragma unroll
      for (int i = 0; i < 4; ++i) ls[i] *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
      m = cand;
      ms = cs;
    }
  };
  // P^T = exp2(S^T k2 - m k2): row sum from the unrounded values (csrc/ring_attention.cu:242),
  // MFMA operands rounded to the storage type (:604)
  auto exponentials = [&](const f32x16& sacc) {
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      typename E::vec8 pv;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[8 * t2 + e], a.scale_log2, -ms));
        ls[e & 3] += p;
        pv[e] = (typename E::type)p;
      }
      pf[t2] = __builtin_bit_cast(s16x8, pv);
    }
  };
  // O^T += V^T P^T of one 32-key tile (csrc/ring_attention.cu:609)
  auto pv_product = [&](int vslot) {
    const unsigned char* vs_lds = smem + (NBUF + vslot) * TILE;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const unsigned char* vrow = vs_lds + 16 * t2 * ROWB;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + voff[db]));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + 8 * ROWB + voff[db]));
        const s16x8 vfr = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        oacc[db] = E::mma(vfr, pf[t2], oacc[db]);
      }
    }
  };

  // Block u.  Even blocks start with the barrier of the pair (u, u+1): K(u+1), K(u+2), V(u)
  // and V(u+1), issued two blocks earlier, have landed, and every wave is past block u-1, so
  // the ring slots of K(u-1), K(u), V(u-2), V(u-1) are free for K(u+3), K(u+4), V(u+2), V(u+3).
  // STEADY blocks (all those tiles exist, tiles u+1 and u+2 unmasked) have compile-time ring
  // slots and no conditions.
  auto block = [&](auto slot_c, auto steady, int u) {
    constexpr int SLOT = decltype(slot_c)::value;  // u mod 4 (STEADY) or u mod 2 (general)
    constexpr bool STEADY = decltype(steady)::value;
    f32x16& cur = (SLOT & 1) ? s_odd : s_even;
    f32x16& nxt = (SLOT & 1) ? s_even : s_odd;
    if (STEADY) {
      if ((SLOT & 1) == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        issue_k(u + 3);
        issue_k(u + 4);
        issue_v(u + 2);
        issue_v(u + 3);
      }
      qk(nxt, (SLOT + 1) & 3);
      exponentials(cur);
      pv_product(SLOT);
      const float tm = tile_max(nxt);
      if constexpr (SCHED == 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
      }
      move_reference(tm);
    } else {
      if ((u & 1) == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (u + 3 < n_tiles) issue_k(u + 3);
        if (u + 4 < n_tiles) issue_k(u + 4);
        if (u + 2 < n_tiles) issue_v(u + 2);
        if (u + 3 < n_tiles) issue_v(u + 3);
      }
      if (u + 1 < n_tiles) {
        qk(nxt, (u + 1) & 3);
        mask_tile(nxt, u + 1);
      }
      exponentials(cur);
      pv_product(u & 3);
      if (u + 1 < n_tiles) move_reference(tile_max(nxt));
    }
  };

  __builtin_amdgcn_s_waitcnt(0);  // retire the Q loads with a wait the compiler can see
  issue_k(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (n_tiles > 1) issue_k(1);
  if (n_tiles > 2) issue_k(2);
  issue_v(0);
  if (n_tiles > 1) issue_v(1);
  qk(s_even, 0);
  mask_tile(s_even, 0);
  move_reference(tile_max(s_even));

  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  using C2 = std::integral_constant<int, 2>;
  using C3 = std::integral_constant<int, 3>;
  // a steady pair (u, u+1), u even, needs u + 4 < n_tiles and u + 2 < first_masked
  const int n_steady = min(n_tiles - 4, first_masked - 2);  // pairs starting at u < n_steady
  int u = 0;
  for (; u + 2 < n_steady; u += 4) {
    block(C0{}, std::true_type{}, u);
    block(C1{}, std::true_type{}, u + 1);
    block(C2{}, std::true_type{}, u + 2);
    block(C3{}, std::true_type{}, u + 3);
  }
  for (; u < n_tiles; ++u) {
    if (u & 1) block(C1{}, std::false_type{}, u);
    else block(C0{}, std::false_type{}, u);
  }

  // epilogue (csrc/ring_attention.cu:621-633): normalise, emit partial O and LSE
  const float l = cross_half_sum((ls[0] + ls[1]) + (ls[2] + ls[3]));
  const float inv = (l > 0.f) ? 1.f / l : 0.f;
  const int row_g = r * a.chunk + qt * BM + 32 * wave + n;
  float* orow = a.o_part + ((int64_t)bh * a.S + row_g) * D;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f32x4 val;
#pragma unroll
      for (int e = 0; e < 4; ++e) val[e] = oacc[db][4 * q4 + e] * inv;
      *(f32x4*)(orow + 32 * db + 8 * q4 + 4 * h) = val;
    }
  if (h == 0) {
    const float lse = (l > 0.f) ? (ms + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
    a.lse_part[(int64_t)bh * a.S + row_g] = lse;
  }
}

// ---- merge ------------------------------------------------------------------------
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

template <int DT, int D>
__global__ __launch_bounds__(256) void merge_kernel(const MergeArgs a) {
  constexpr int TPR = D / 8;  // threads per row, 8 columns each
  constexpr int ROWS = 256 / TPR;
  const int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;
  if (row >= a.rows) return;
  const int c8 = threadIdx.x % TPR;
  int first_wrapped = 1;  // parts s >= first_wrapped are active (besides s == 0)
  if (a.causal_ring) {
    const int r = (int)((row % a.S) / a.chunk);
    first_wrapped = a.P - r;
  }
  float mx = -INFINITY;
  for (int s = 0; s < a.n_parts; ++s) {
    if (s != 0 && s < first_wrapped) continue;
    mx = fmaxf(mx, a.lse_parts[s * a.part_stride_rows + row]);
  }
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  if (mx != -INFINITY) {
    for (int s = 0; s < a.n_parts; ++s) {
      if (s != 0 && s < first_wrapped) continue;
      const float L = a.lse_parts[s * a.part_stride_rows + row];
      if (L == -INFINITY) continue;  // identity element
      const float w = __expf(L - mx);
      wsum += w;
      const float* src = a.o_parts + (s * a.part_stride_rows + row) * D + c8 * 8;
      const f32x4 x0 = *(const f32x4*)src, x1 = *(const f32x4*)(src + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[e] = __builtin_fmaf(w, x0[e], acc[e]);
        acc[4 + e] = __builtin_fmaf(w, x1[e], acc[4 + e]);
      }
    }
    const float inv = 1.f / wsum;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= inv;
  }
  Store8<DT>::st((char*)a.out + (row * D + c8 * 8) * 2, acc);
  if (c8 == 0) a.lse[row] = (mx == -INFINITY) ? -INFINITY : mx + __logf(wsum);
}

// ---- host launchers -----------------------------------------------------------------
hipError_t launch_block_step(const BlockStepArgs& a, int dtype, int dim, hipStream_t stream) {
  if (a.n_active <= 0) return hipSuccess;
  const int q_tiles = a.chunk / kBlockM;
  const int groups = a.n_active * a.BH;
  const unsigned grid = (unsigned)(((groups + 7) / 8) * 8 * q_tiles);
  static const int var = getenv("RINGATTN_VARIANT") ? atoi(getenv("RINGATTN_VARIANT")) : 0;
#define RA_PIPE(SCHED)                                                                                  \
  {                                                                                                     \
    if (dtype == 0 && dim == 64) block_attention_pipe_kernel<0, 64, SCHED><<<grid, 256, 0, stream>>>(a);        \
    else if (dtype == 0 && dim == 128) block_attention_pipe_kernel<0, 128, SCHED><<<grid, 256, 0, stream>>>(a); \
    else if (dtype == 1 && dim == 64) block_attention_pipe_kernel<1, 64, SCHED><<<grid, 256, 0, stream>>>(a);   \
    else if (dtype == 1 && dim == 128) block_attention_pipe_kernel<1, 128, SCHED><<<grid, 256, 0, stream>>>(a); \
    else return hipErrorInvalidValue;                                                                   \
    return hipGetLastError();                                                                           \
  }
  if (var == 1) RA_PIPE(0)
  if (var == 2) RA_PIPE(1)
  if (dtype == 0 && dim == 64) block_attention_kernel<0, 64, 64><<<grid, 256, 0, stream>>>(a);
  else if (dtype == 0 && dim == 128) block_attention_kernel<0, 128, 64><<<grid, 256, 0, stream>>>(a);
  else if (dtype == 1 && dim == 64) block_attention_kernel<1, 64, 64><<<grid, 256, 0, stream>>>(a);
  else if (dtype == 1 && dim == 128) block_attention_kernel<1, 128, 64><<<grid, 256, 0, stream>>>(a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_merge(const MergeArgs& a, int dtype, int dim, hipStream_t stream) {
  if (a.rows <= 0) return hipSuccess;
  const int rows_per_block = 256 / (dim / 8);
  const unsigned grid = (unsigned)((a.rows + rows_per_block - 1) / rows_per_block);
  if (dtype == 0 && dim == 64) merge_kernel<0, 64><<<grid, 256, 0, stream>>>(a);
  else if (dtype == 0 && dim == 128) merge_kernel<0, 128><<<grid, 256, 0, stream>>>(a);
  else if (dtype == 1 && dim == 64) merge_kernel<1, 64><<<grid, 256, 0, stream>>>(a);
  else if (dtype == 1 && dim == 128) merge_kernel<1, 128><<<grid, 256, 0, stream>>>(a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ringattn
