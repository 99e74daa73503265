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
