// gfx950 (CDNA4) kernels for the ring-attention forward path: the ring steps kept apart.
// (The forward that carries the softmax state through the steps is ring_walk_kernel,
// ringattn_walk.hip.)
//
//   block_attention_kernel : the ring steps of every virtual rank.  A workgroup owns 128
//       query rows, keeps their Q in registers and walks the KV chunks those rows meet (the
//       reference's CTA loops over the ring steps in the same way, csrc/ring_attention.cu:
//       439-443,456), per chunk
//       S^T = K Q^T, online softmax with running max / sum, O^T += V^T P^T,
//       emitting a normalised fp32 partial O and a natural-log fp32 LSE per chunk, and, when
//       asked, merging the partials of its rows at the end.
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
//         * K and V go HBM -> LDS directly (global_load_lds_dwordx4) in 32-key
//           tiles, through two 4-deep rings, one barrier per two tiles; bank
//           conflicts are removed by an XOR swizzle applied on the
//           global-address side;
//         * V^T operands come from ds_read_b64_tr_b16 (the LDS transpose read),
//           replacing ldmatrix.trans of csrc/kernel_traits.h:39;
//         * the loop is software-pipelined: the MFMAs of tile u+1's scores run
//           next to the exponentials of tile u (see the kernel's comment).
//   merge_kernel : P-way merge of the per-step (O, LSE) partials.  The reference
//       has no such function: it carries (max, sum, acc-O) in registers across
//       ring steps (:439-443,597).  The merge is the algebraic equivalent on
//       (O, LSE) pairs.
#include "ringattn_device.h"

#include <type_traits>


namespace ringattn {

// ---- merge of one row: shared by the merge kernel and the block kernel's fused merge -------
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

// The parts of one row, in ascending slot order: the set bits of a mask over equally spaced slots.
struct SlotParts {
  uint64_t rest;
  int64_t row, stride;  // the row in slot 0, rows between slots
  __device__ __forceinline__ int left() const { return __builtin_popcountll(rest); }
  __device__ __forceinline__ int64_t take() {
    const int64_t r = row + (int64_t)__builtin_ctzll(rest) * stride;
    rest &= rest - 1;
    return r;
  }
};
// L = logsumexp_s L_s, O = sum_s exp(L_s - L) O_s over the parts of one row; this thread owns
// columns [8 c8, 8 c8 + 8).  A part with L_s = -inf is the identity and its O is not used.
template <int DT, int D, bool HP, class Parts>
static __device__ __forceinline__ void merge_row(Parts parts, const void* o_parts, const float* lse_parts,
                                                 void* out, float* lse, int64_t out_row, int c8) {
  const typename PartRow<HP>::ptr o_base = (typename PartRow<HP>::ptr)o_parts + c8 * 8;
  float mx = -INFINITY;
  {
    Parts p = parts;
    while (p.left()) mx = fmaxf(mx, lse_parts[p.take()]);
  }
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  if (mx != -INFINITY) {
    // four parts per iteration: all their loads are issued before the first is consumed
    Parts p = parts;
    while (p.left() >= 4) {
      float L[4];
      f32x4 x0[4], x1[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t r = p.take();
        L[u] = lse_parts[r];
        PartRow<HP>::ld(o_base + r * D, x0[u], x1[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float w = __expf(L[u] - mx);
        if (L[u] == -INFINITY) continue;  // identity element: its O may hold anything
        wsum += w;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc[e] = __builtin_fmaf(w, x0[u][e], acc[e]);
          acc[4 + e] = __builtin_fmaf(w, x1[u][e], acc[4 + e]);
        }
      }
    }
    while (p.left()) {
      const int64_t r = p.take();
      const float Ls = lse_parts[r];
      const float w = __expf(Ls - mx);
      f32x4 x0, x1;
      PartRow<HP>::ld(o_base + r * D, x0, x1);
      if (Ls == -INFINITY) continue;
      wsum += w;
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
  Store8<DT>::st((char*)out + (out_row * D + c8 * 8) * 2, acc);
  if (c8 == 0) lse[out_row] = (mx == -INFINITY) ? -INFINITY : mx + __logf(wsum);
}

// ---- merge of one job's rows (128 rows of a segment, one head) over the partials of the
// segment's items.  The same arithmetic, in the same order, as merge_row; only the loads are
// arranged differently: the block kernel, which runs this at the end of a workgroup, has just two
// waves per SIMD to hide memory latency with, and every round trip it waits for is time its
// compute unit runs half empty.  So all partial LSEs are fetched in one sweep and parked in LDS
// (lse_s: [items][128] floats), and the partial O rows move in batches of 256 bytes per thread
// (two output rows x four or eight parts), three batches in flight at any time.
typedef __attribute__((address_space(3))) float lds_float;
template <int DT, int D, bool HP>
static __device__ __forceinline__ void merge_job_rows(const void* o_part, const float* lse_part, void* out, float* lse,
                                                      const SegItem* items, const Segment& seg, int bh, int qt, int S,
                                                      lds_float* lse_s) {
  constexpr int BM = kBlockM;
  constexpr int TPR = D / 8;  // threads per row, 8 columns each
  constexpr int ROWS = 256 / TPR;
  constexpr int R = 2, G = HP ? 8 : 4;  // rows per thread and parts per batch: 64 registers a batch
  constexpr int RSTEP = R * ROWS;
  constexpr int KMAX = kMaxParts / 4;  // parts per wave in the LSE sweep
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_parts = seg.item_count;
  const SegItem* its = items + seg.item_begin;
  const int row0 = qt * BM;  // first row of the job within the segment
  __syncthreads();  // the partial stores of all four waves have completed and are visible to them; the LDS is idle
  {
    float v[KMAX][2];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int i = wave + 4 * k;
      if (i < n_parts) {
        const int64_t prow = its[i].part_base + (int64_t)bh * its[i].part_bh_stride + row0;
        v[k][0] = (row0 + lane < seg.q_len) ? lse_part[prow + lane] : -INFINITY;
        v[k][1] = (row0 + lane + 64 < seg.q_len) ? lse_part[prow + lane + 64] : -INFINITY;
      }
    }
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int i = wave + 4 * k;
      if (i < n_parts) {
        lse_s[i * BM + lane] = v[k][0];
        lse_s[i * BM + lane + 64] = v[k][1];
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

// ---- block attention: the ring steps of 128 query rows ----------------------------------
// A KV chunk is consumed in 32-key tiles held in two 4-deep LDS rings (K and V), filled by
// direct-to-LDS loads that run two blocks ahead.  Block u of the loop runs, in ONE
// instruction stream,
//     MFMAs of S^T(u+1) = K(u+1) Q^T      next to   the exponentials of tile u,
//     MFMAs of O^T += V(u)^T P(u)^T       next to   the row-max reduction of tile u+1,
// so every wave feeds the matrix pipe and the VALU at the same time instead of alternating
// between them.  The exponent offset m is a REFERENCE max: it is moved (with the rescale of
// l and acc-O of csrc/ring_attention.cu:226-232) only when some row's tile max exceeds it by
// more than 2^kLazyLog2, decided at the end of a block, which keeps the blocks free of
// branches.  Until then p = exp2((s - m) k2) may exceed 1 (by at most 2^kLazyLog2, well
// inside fp16 and bf16 range); O = acc / l and LSE = (m k2 + log2 l) ln 2 do not depend on
// the choice of m.
// From one KV chunk to the next the tile pipeline keeps running where the shapes allow it
// (the loads that run ahead of the last tiles fetch the first tiles of the next chunk); the
// softmax state is emitted as that chunk's partial and reset.
template <int DT, int D, bool HP>
__global__ __launch_bounds__(256, 2) void block_attention_kernel(const BlockArgs a) {
  using E = Elem<DT>;
  constexpr int QB = 1;            // 32-query blocks per wave
  constexpr int BM = kBlockM;      // query rows per workgroup: 4 waves x 32
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

  Segment seg;
  int bh, qt;
  if (!decode_job<kBlockM>(a, seg, bh, qt)) return;
  const int q_start = seg.q_start, q_len = seg.q_len;
  const int n_items = seg.item_count;
  // items in run order: table order, except that item `last_item` is moved to the end
  auto item_at = [&](int i) -> const SegItem* {
    int idx = i;
    if (seg.last_item >= 0) idx = (i == n_items - 1) ? seg.last_item : (i >= seg.last_item ? i + 1 : i);
    return a.items + seg.item_begin + idx;
  };

  const int64_t head_off = (int64_t)bh * a.bh_stride;
  // grouped-query attention: query head h of a batch entry reads KV head h / kv_group
  const int kv_bh = (bh / a.heads) * (a.heads / a.kv_group) + (bh % a.heads) / a.kv_group;
  const int64_t kv_head_off = (int64_t)kv_bh * a.kv_bh_stride;
  const char* qbase = (const char*)a.q + (head_off + (int64_t)(q_start + qt * BM) * D) * 2;

  // this lane's query rows (local to the q tile): 32 QB wave + 32 qb + n
  s16x8 qf[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int ql = min(qt * BM + 32 * QB * wave + 32 * qb + n, q_len - 1) - qt * BM;
    const char* qrow = qbase + (int64_t)ql * ROWB + h * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[qb][ks] = *(const s16x8*)(qrow + ks * 32);
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

  float m[QB];   // reference max per query block (raw score units)
  float ms[QB];  // m * k2, 0 while m is -inf (guard of csrc/ring_attention.cu:183)
  float ls[QB][4];
  f32x16 oacc[QB][DB];
  auto reset_state = [&]() {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      m[qb] = -INFINITY;
      ms[qb] = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) ls[qb][i] = 0.f;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[qb][db][e] = 0.f;
    }
  };
  reset_state();
  f32x16 s_even[QB], s_odd[QB];
  s16x8 pf[QB][2];

  // ---- the KV chunk being walked (wave-uniform)
  const char *kbase = nullptr, *vbase = nullptr;
  // where the loads that run past the last tile go: the first tiles of the next chunk when
  // the pipeline carries over (stride TILE), else a re-read of the last tile (stride 0)
  int64_t kpast_delta = 0, vpast_delta = 0;  // from the end of this chunk's K (V) to that place
  int past_stride = 0;
  int kv_len = 0, n_tiles = 0, first_masked = 0, kv_tail = -1, diag_rows = 0;
  bool diag = false;
  // Lengths need not be multiples of the tile sizes (the predication the reference leaves as
  // a TODO, csrc/ring_attention.cu:143-145).  The last key tile may reach beyond the KV range:
  // its loads are clamped to the last valid row and its surplus keys masked.  Query rows
  // beyond the range are computed on a copy of the last valid row and not stored.
  auto set_chunk = [&](const SegItem* w) {
    diag = w->diag_off >= 0;
    kv_len = w->kv_len;
    diag_rows = w->diag_off + qt * BM;  // keys below this local index are visible to the whole q tile
    const int kv_tiles = (kv_len + BN - 1) / BN;
    kv_tail = (kv_len % BN) ? kv_len / BN : -1;  // the tile with surplus keys, if any
    n_tiles = diag ? min(kv_tiles, (diag_rows + BM + BN - 1) / BN) : kv_tiles;
    // tiles >= first_masked need a mask (causal diagonal or surplus keys)
    first_masked = min(diag ? diag_rows / BN : n_tiles, kv_tail >= 0 ? kv_tail : n_tiles);
    kbase = (const char*)a.k + (kv_head_off + (int64_t)w->kv_start * D) * 2;
    vbase = (const char*)a.v + (kv_head_off + (int64_t)w->kv_start * D) * 2;
  };

  // bytes to step back so that a row of tile kv_tail beyond the KV range reads the last valid row
  auto surplus = [&](int i) {
    const int row = ((wave * LD + i) * 64 + lane) / CPR;
    return max(0, kv_tail * BN + row - (kv_len - 1)) * ROWB;
  };
  // Byte offset of tile t from the chunk's first tile, in branch-free scalar arithmetic (a
  // branch would split the steady blocks): t < n_tiles gives t TILE; beyond that
  // n_tiles TILE + delta + (t - n_tiles) past_stride, delta being the distance from the end of
  // this chunk to where such loads go.
  auto tile_offset = [&](int t, int64_t delta) -> int64_t {
    const int64_t beyond = (int64_t)((n_tiles - 1 - t) >> 31);  // all ones iff t >= n_tiles
    return (int64_t)min(t, n_tiles) * TILE + (int64_t)max(t - n_tiles, 0) * past_stride + (delta & beyond);
  };
  // `checked`: the tile may be kv_tail (steady blocks never issue that one); checked calls
  // name existing tiles only.  A tile index at or beyond n_tiles comes from a steady block
  // that keeps loading two blocks ahead at the end of the chunk.
  auto issue_k = [&](int t, auto checked) {
    const char* kt = kbase + tile_offset(t, kpast_delta);
    const unsigned kd = __builtin_amdgcn_readfirstlane(smem_base + (t & (NBUF - 1)) * TILE + wave * (LD * 1024));
    if (decltype(checked)::value && t == kv_tail) {
#pragma unroll
      for (int i = 0; i < LD; ++i) load_lds_16(kt, goff_k[i] - surplus(i), kd + i * 1024);
    } else {
#pragma unroll
      for (int i = 0; i < LD; ++i) load_lds_16(kt, goff_k[i], kd + i * 1024);
    }
  };
  auto issue_v = [&](int t, auto checked) {
    const char* vt = vbase + tile_offset(t, vpast_delta);
    const unsigned vd = __builtin_amdgcn_readfirstlane(smem_base + (NBUF + (t & (NBUF - 1))) * TILE + wave * (LD * 1024));
    if (decltype(checked)::value && t == kv_tail) {
#pragma unroll
      for (int i = 0; i < LD; ++i) load_lds_16(vt, goff_v[i] - surplus(i), vd + i * 1024);
    } else {
#pragma unroll
      for (int i = 0; i < LD; ++i) load_lds_16(vt, goff_v[i], vd + i * 1024);
    }
  };
  constexpr std::true_type kChecked{};
  constexpr std::false_type kUnchecked{};
  // S^T = K Q^T of one 32-key tile (csrc/ring_attention.cu:565); each K fragment feeds all
  // QB query blocks of the wave
  auto qk = [&](f32x16(&sacc)[QB], int kslot) {
    const unsigned char* ks_lds = smem + kslot * TILE;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int e = 0; e < 16; ++e) sacc[qb][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const s16x8 kfr = *(const s16x8*)(ks_lds + koff[ks]);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) sacc[qb] = E::mma(kfr, qf[qb][ks], sacc[qb]);
    }
  };
  auto mask_tile = [&](f32x16(&sacc)[QB], int t, auto always) {
    // key visible iff inside the KV range and key_local <= query_local + diag_off
    if (decltype(always)::value || t >= first_masked) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        int lim = kv_len - 1 - t * BN - 4 * h;
        if (diag) lim = min(lim, diag_rows + 32 * QB * wave + 32 * qb + n - t * BN - 4 * h);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = 8 * (e >> 2) + (e & 3);
          if (key > lim) sacc[qb][e] = -INFINITY;
        }
      }
    }
  };
  // max(m, row max of the tile): two chains of max(max(x, a), b) seeded with the reference
  // max, each link one v_max3_f32; one exchange between the halves of the wave
  auto tile_max = [&](const f32x16& sacc, float mref) {
    float m0 = mref, m1 = mref;
#pragma unroll
    for (int e = 0; e < 16; e += 4) {
      m0 = fmaxf(fmaxf(m0, sacc[e]), sacc[e + 1]);
      m1 = fmaxf(fmaxf(m1, sacc[e + 2]), sacc[e + 3]);
    }
    return cross_half_max(fmaxf(m0, m1));
  };
  // cand = max(m, tile max).  The reference moves when some row's cand is far above it (or it
  // is still unset): rescale of l and acc-O as in csrc/ring_attention.cu:226-232.  `live` is
  // false for the scores a steady block computes beyond the last tile of a chunk: they belong
  // to the next chunk (or to nothing) and must not touch this chunk's state.
  auto move_reference = [&](const float (&cand)[QB], bool live) {
    bool far = false;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) far = far || ((cand[qb] - m[qb]) * a.scale_log2 > kLazyLog2);
    if (live && __builtin_amdgcn_ballot_w64(far) != 0) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const float cs = (cand[qb] == -INFINITY) ? 0.f : cand[qb] * a.scale_log2;
        const float alpha = __builtin_amdgcn_exp2f(m[qb] * a.scale_log2 - cs);
#pragma unroll
        for (int i = 0; i < 4; ++i) ls[qb][i] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[qb][db] *= alpha;
        m[qb] = cand[qb];
        ms[qb] = cs;
      }
    }
  };
  // the first tile of a chunk sets the reference: l and acc-O are zero, nothing to rescale
  auto set_reference = [&](const float (&cand)[QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      m[qb] = cand[qb];
      ms[qb] = (cand[qb] == -INFINITY) ? 0.f : cand[qb] * a.scale_log2;
    }
  };
  // P^T = exp2(S^T k2 - m k2): row sum from the unrounded values (csrc/ring_attention.cu:242),
  // MFMA operands rounded to the storage type (:604)
  auto exponentials = [&](const f32x16(&sacc)[QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        typename E::vec8 pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[qb][8 * t2 + e], a.scale_log2, -ms[qb]));
          ls[qb][e & 3] += p;
          pv[e] = (typename E::type)p;
        }
        pf[qb][t2] = __builtin_bit_cast(s16x8, pv);
      }
  };
  // O^T += V^T P^T of one 32-key tile (csrc/ring_attention.cu:609); each V^T fragment feeds
  // all QB query blocks of the wave
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
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) oacc[qb][db] = E::mma(vfr, pf[qb][t2], oacc[qb][db]);
      }
    }
  };
  auto tile_maxes = [&](const f32x16(&sacc)[QB], float (&cand)[QB]) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) cand[qb] = tile_max(sacc[qb], m[qb]);
  };

  // Set between a carried-over chunk boundary and the first pair of the next chunk: the tiles
  // that pair needs were waited for (and the barrier passed) BEFORE the partial was stored, so
  // that the pair does not wait for those stores (stores count in vmcnt too).
  bool synced = false;
  // Block u.  Even blocks start with the barrier of the pair (u, u+1): K(u+1), K(u+2), V(u)
  // and V(u+1), issued during the previous pair, have landed, and every wave is past block
  // u-1, so the ring slots of K(u-1), K(u), V(u-2), V(u-1) are free for K(u+3), K(u+4),
  // V(u+2), V(u+3), which are issued during this pair.
  // STEADY blocks (tiles u+1 and u+2 unmasked or covered by MASKED) have compile-time ring
  // slots and no conditions.
  auto block = [&](auto slot_c, auto steady, auto masked, int u) {
    constexpr int SLOT = decltype(slot_c)::value;  // u mod 4 (STEADY) or u mod 2 (general)
    constexpr bool STEADY = decltype(steady)::value;
    constexpr bool MASKED = decltype(masked)::value;  // STEADY only: tile u+1 gets the mask
    f32x16(&cur)[QB] = (SLOT & 1) ? s_odd : s_even;
    f32x16(&nxt)[QB] = (SLOT & 1) ? s_even : s_odd;
    float cand[QB];
    if (STEADY) {
      // the four tile loads of a pair are spread over its two blocks instead of being
      // issued in one burst behind the barrier
      if ((SLOT & 1) == 0) {
        if (SLOT == 0 && synced) {
          synced = false;  // a carried chunk's first pair: its wait and barrier came before the partial was stored
        } else {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
        }
        issue_k(u + 3, kUnchecked);
      } else {
        issue_v(u + 1, kUnchecked);
      }
      qk(nxt, (SLOT + 1) & 3);
      if (MASKED) mask_tile(nxt, u + 1, kChecked);
      exponentials(cur);
      if ((SLOT & 1) == 0) issue_k(u + 4, kUnchecked);
      else issue_v(u + 2, kUnchecked);
      pv_product(SLOT);
      tile_maxes(nxt, cand);
      // scheduling hint: in the first half of the block every MFMA is preceded by one and
      // followed by two LDS reads, so the reads run ahead of the MFMAs that consume them
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      move_reference(cand, u + 1 < n_tiles);
    } else {
      if ((u & 1) == 0) {
        if (synced) {
          synced = false;
        } else {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
        }
        if (u + 3 < n_tiles) issue_k(u + 3, kChecked);
        if (u + 4 < n_tiles) issue_k(u + 4, kChecked);
        if (u + 2 < n_tiles) issue_v(u + 2, kChecked);
        if (u + 3 < n_tiles) issue_v(u + 3, kChecked);
      }
      if (u + 1 < n_tiles) {
        qk(nxt, (u + 1) & 3);
        mask_tile(nxt, u + 1, kUnchecked);
      }
      exponentials(cur);
      pv_product(u & 3);
      if (u + 1 < n_tiles) {
        tile_maxes(nxt, cand);
        move_reference(cand, true);
      }
    }
  };

  // this chunk's partial (csrc/ring_attention.cu:621-633): normalise, emit O and LSE
  auto emit_partial = [&](const SegItem* w) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float l = cross_half_sum((ls[qb][0] + ls[qb][1]) + (ls[qb][2] + ls[qb][3]));
      const float inv = (l > 0.f) ? 1.f / l : 0.f;
      const int row_l = qt * BM + 32 * QB * wave + 32 * qb + n;
      if (row_l >= q_len) continue;  // a row beyond the query range
      const int64_t prow = w->part_base + (int64_t)bh * w->part_bh_stride + row_l;
      const int64_t opos = prow * D;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          f32x4 val;
#pragma unroll
          for (int e = 0; e < 4; ++e) val[e] = oacc[qb][db][4 * q4 + e] * inv;
          if (HP) {  // fp16 partials: |O_part| <= max |V|, the caller vouches that this fits
            f16x4 hv;
#pragma unroll
            for (int e = 0; e < 4; ++e) hv[e] = (_Float16)val[e];
            *(f16x4*)((_Float16*)a.o_part + opos + 32 * db + 8 * q4 + 4 * h) = hv;
          } else {
            *(f32x4*)((float*)a.o_part + opos + 32 * db + 8 * q4 + 4 * h) = val;
          }
        }
      if (h == 0) {
        const float lse = (l > 0.f) ? (ms[qb] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
        a.lse_part[prow] = lse;
      }
    }
  };

  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  using C2 = std::integral_constant<int, 2>;
  using C3 = std::integral_constant<int, 3>;

  bool carried = false;  // the previous chunk's pipeline ran on into this one
  for (int it = 0; it < n_items; ++it) {
    const SegItem* w = item_at(it);
    set_chunk(w);
    // The pipeline carries over into the next chunk when this one ends in plain steady groups
    // on a multiple of four tiles (ring slots then line up with a fresh start) and the next
    // chunk has its first three tiles in full.
    bool carry = false;
    if (it + 1 < n_items) {
      const SegItem* wn = item_at(it + 1);
      carry = !diag && kv_tail < 0 && (n_tiles & 3) == 0 && wn->kv_len >= 4 * BN;
      if (carry) {
        const int64_t next_first = ((int64_t)wn->kv_start - w->kv_start) * ROWB;  // from this chunk's first tile
        kpast_delta = vpast_delta = next_first - (int64_t)n_tiles * TILE;
        past_stride = TILE;
      }
    }
    if (!carry) {
      kpast_delta = vpast_delta = -(int64_t)TILE;
      past_stride = 0;
    }

    if (!carried) {
      if (it > 0) __syncthreads();  // every wave is done with the ring slots of the previous chunk
      // the first tiles go out next to the Q loads: one memory latency for all of them
      issue_k(0, kChecked);
      if (n_tiles > 1) issue_k(1, kChecked);
      if (n_tiles > 2) issue_k(2, kChecked);
      issue_v(0, kChecked);
      if (n_tiles > 1) issue_v(1, kChecked);
      __builtin_amdgcn_s_waitcnt(0);  // retire the Q loads with a wait the compiler can see (and the tiles)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      qk(s_even, 0);
    }
    // (carried: K(0) was consumed by the last block of the previous chunk, which left the
    // scores of tile 0 in s_even; K(1), K(2), V(0), V(1) are in flight)
    {
      float cand[QB];
      mask_tile(s_even, 0, kUnchecked);
      tile_maxes(s_even, cand);
      set_reference(cand);
    }

    // Steady blocks come in groups of four (ring slots are compile-time constants).  A group
    // starting at u computes the scores of tiles u+1 .. u+4 and loads up to tile u+6:
    //   plain groups   while those four tiles need no mask; without any mask in the chunk the last
    //                  group runs up to tile n_tiles-1 and its last block computes the scores of
    //                  the tile after the last one (the next chunk's first, or nothing of use);
    //   masked groups  (diagonal chunks) for the rest: every block masks its tile u+1;
    //   a chunk with surplus keys in its last tile keeps clear of that tile (its loads need the
    //   clamped form) and leaves the rest to the general blocks.
    const bool ragged = kv_tail >= 0;
    const int plain_end = ragged ? min(first_masked, kv_tail - 2) : (diag ? first_masked : n_tiles + 1);
    const int masked_end = (diag && !ragged) ? n_tiles + 1 : 0;
    int u = 0;
    for (; u + 4 < plain_end; u += 4) {
      block(C0{}, std::true_type{}, std::false_type{}, u);
      block(C1{}, std::true_type{}, std::false_type{}, u + 1);
      block(C2{}, std::true_type{}, std::false_type{}, u + 2);
      block(C3{}, std::true_type{}, std::false_type{}, u + 3);
    }
    for (; u + 4 < masked_end; u += 4) {
      block(C0{}, std::true_type{}, std::true_type{}, u);
      block(C1{}, std::true_type{}, std::true_type{}, u + 1);
      block(C2{}, std::true_type{}, std::true_type{}, u + 2);
      block(C3{}, std::true_type{}, std::true_type{}, u + 3);
    }
    for (; u < n_tiles; ++u) {
      if (u & 1) block(C1{}, std::false_type{}, std::false_type{}, u);
      else block(C0{}, std::false_type{}, std::false_type{}, u);
    }
    carried = carry;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next chunk's first tiles, or re-reads of the last tile
    if (carry) {
      __syncthreads();
      synced = true;
    }
    emit_partial(w);
    reset_state();
  }
  // ---- fused merge: this workgroup's rows over the partials it has just written
  if (a.mode == kBlockPartialsMerged) {
    static_assert(sizeof(smem) >= kMaxParts * BM * sizeof(float), "partial LSEs of a q tile fit the rings");
    merge_job_rows<DT, D, HP>(a.o_part, a.lse_part, a.out, a.lse, a.items, seg, bh, qt, a.S,
                              (lds_float*)(__attribute__((address_space(3))) void*)smem);
  }
}

// ---- merge ------------------------------------------------------------------------
template <int DT, int D, bool HP>
__global__ __launch_bounds__(256) void merge_kernel(const MergeArgs a) {
  constexpr int TPR = D / 8;  // threads per row, 8 columns each
  constexpr int ROWS = 256 / TPR;
  const MergeRegion reg = a.regions ? a.regions[blockIdx.y] : a.single;
  const int64_t idx = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;  // over heads x reg.len
  if (idx >= (int64_t)a.heads * reg.len) return;
  const int64_t row = (idx / reg.len) * a.S + reg.start + idx % reg.len;
  SlotParts parts{reg.active, row, a.part_stride_rows};
  merge_row<DT, D, HP>(parts, a.o_parts, a.lse_parts, a.out, a.lse, row, threadIdx.x % TPR);
}

// ---- segment + item table from kernel arguments -------------------------------------
__global__ __launch_bounds__(64) void write_table_kernel(const TablePack pack, int n, Segment* seg_dst, SegItem* item_dst) {
  const int i = threadIdx.x;
  if (i < n) item_dst[i] = pack.items[i];
  if (i == 0) *seg_dst = pack.seg;
}

// ---- host launchers -----------------------------------------------------------------
hipError_t launch_block(const BlockArgs& a, int dtype, int dim, hipStream_t stream) {
  if (a.n_segs <= 0) return hipSuccess;
  if (a.mode != kBlockPartials && a.mode != kBlockPartialsMerged) return hipErrorInvalidValue;  // carry mode: launch_walk
  const int q_tiles = a.q_tiles_max;
  const int64_t groups = (int64_t)a.n_segs * a.BH;
  const int64_t blocks = (a.groups ? (int64_t)a.groups_per_xcd : (groups + 7) / 8) * 8 * q_tiles;
  if (q_tiles <= 0 || blocks > INT32_MAX) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)blocks;
#define RA_LAUNCH_BLOCK(DT_, D_)                                                            \
  do {                                                                                   \
    if (a.half_partials) block_attention_kernel<DT_, D_, true><<<grid, 256, 0, stream>>>(a);  \
    else block_attention_kernel<DT_, D_, false><<<grid, 256, 0, stream>>>(a);                \
  } while (0)
  if (dtype == 0 && dim == 64) RA_LAUNCH_BLOCK(0, 64);
  else if (dtype == 0 && dim == 128) RA_LAUNCH_BLOCK(0, 128);
  else if (dtype == 1 && dim == 64) RA_LAUNCH_BLOCK(1, 64);
  else if (dtype == 1 && dim == 128) RA_LAUNCH_BLOCK(1, 128);
#undef RA_LAUNCH_BLOCK
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_write_table(const TablePack& pack, int n, Segment* seg_dst, SegItem* item_dst, hipStream_t stream) {
  if (n <= 0 || n > kMaxParts) return hipErrorInvalidValue;
  write_table_kernel<<<1, 64, 0, stream>>>(pack, n, seg_dst, item_dst);
  return hipGetLastError();
}

hipError_t launch_merge(const MergeArgs& a, int dtype, int dim, hipStream_t stream) {
  if (a.n_regions <= 0 || a.max_len <= 0 || a.heads <= 0) return hipSuccess;
  const int rows_per_block = 256 / (dim / 8);
  const int64_t cols = ((int64_t)a.heads * a.max_len + rows_per_block - 1) / rows_per_block;
  if (cols > INT32_MAX || a.n_regions > 65535) return hipErrorInvalidValue;
  const dim3 grid((unsigned)cols, (unsigned)a.n_regions);
#define RA_LAUNCH_MERGE(DT_, D_)                                                 \
  do {                                                                        \
    if (a.half_partials) merge_kernel<DT_, D_, true><<<grid, 256, 0, stream>>>(a);  \
    else merge_kernel<DT_, D_, false><<<grid, 256, 0, stream>>>(a);                \
  } while (0)
  if (dtype == 0 && dim == 64) RA_LAUNCH_MERGE(0, 64);
  else if (dtype == 0 && dim == 128) RA_LAUNCH_MERGE(0, 128);
  else if (dtype == 1 && dim == 64) RA_LAUNCH_MERGE(1, 64);
  else if (dtype == 1 && dim == 128) RA_LAUNCH_MERGE(1, 128);
#undef RA_LAUNCH_MERGE
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ringattn
