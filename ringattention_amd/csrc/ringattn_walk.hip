// gfx950 (CDNA4) kernel: block attention over the ring steps of 256 query rows.
//
//   ring_walk_kernel : a workgroup of EIGHT waves owns 256 query rows of a segment (one head),
//       keeps their Q in registers and walks the KV chunks those rows meet, as the reference's
//       CTA walks its ring steps (csrc/ring_attention.cu:439-443,456), per chunk
//       S^T = K Q^T, online softmax with running max / sum, O^T += V^T P^T.
//       Between two chunks it either carries max, sum and acc-O on (the reference's own way,
//       :597, with O = acc / l (:621-664) and the LSE written once at the end), or emits the
//       chunk's normalised partial (O, LSE) and starts afresh (the ring steps kept apart; the
//       partials of its rows can then be merged at the end of the workgroup).
//       It restates the inner KV-tile loop of the reference kernel
//       (csrc/ring_attention.cu:536-610: gemm_smem :278-301, softmax_rescale_o
//       :194-245 completed with the missing `sum += sum_cur` tail,
//       scale_apply_exp2 :173-192, gemm_A_in_regs :304-324) and its epilogue
//       (:621-664), with the tiling of csrc/kernel_traits.h:11-177 replaced by a
//       wave64 / MFMA 32x32x16 design:
//         * each of the 8 waves owns 32 query rows; Q lives in registers as the
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
//         * the exponent offset m is a REFERENCE max: it is moved (with the rescale of l and
//           acc-O of :226-232) only when some row's tile max exceeds it by more than
//           2^kLazyLog2, decided by a wave-uniform branch.  Until then p = exp2((s - m) k2)
//           may exceed 1 (by at most 2^kLazyLog2, well inside fp16 and bf16 range); O = acc / l
//           and LSE = (m k2 + log2 l) ln 2 do not depend on the choice of m.  At d = 64, where this
//           work bounds the kernel, a tile's row maximum is not even computed as long as its
//           exponentials against the standing reference stay small (softmax_phase).
//
//       A tile's work is laid out in time in two phases.  The eight waves sit two per SIMD
//       (wave w and wave w + 4).  Per tile every wave has an MFMA phase (O^T += V(u)^T P(u)^T, then
//       S^T(u+1) = K(u+1) Q^T: 16 MFMAs and their 24 fragment reads from LDS at d = 128) and a
//       softmax phase (row max, reference move, exponentials, row sum, conversion of P: VALU
//       only).  Waves 0-3 run MFMA phase then softmax phase, waves 4-7 softmax phase then MFMA
//       phase, between the same barriers: while one wave of a SIMD keeps the matrix pipe busy the
//       other keeps the VALU busy, instead of both mixing the two kinds of work and colliding.
//       Measured on synthetic tiles (same instruction mix, barrier and loads): 63.6 % of the
//       MFMA-only rate against 53.4 % for a stream that mixes both kinds of work in every wave.
//
//       From one KV chunk to the next the tile pipeline keeps running where the shapes allow it
//       (the loads that run ahead of the last tiles fetch the first tiles of the next chunk).
#include "ringattn_device.h"

#include <type_traits>

namespace ringattn {

// KEEP: the softmax state is carried through the chunks (kBlockCarryState); otherwise a partial is emitted per
// chunk (kBlockPartials, kBlockPartialsMerged; HP: partial O as fp16).
template <int DT, int D, bool HP, bool KEEP>
__global__ __launch_bounds__(512, 1) void ring_walk_kernel(const BlockArgs a) {
  using E = Elem<DT>;
  constexpr int WAVES = 8;
  constexpr int BM = kWalkM;       // query rows per workgroup: 8 waves x 32
  constexpr int BN = 32;           // keys per tile
  constexpr int NBUF = 4;          // ring depth of the K and of the V tiles
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = D * 2;      // bytes per row
  constexpr int TILE = BN * ROWB;  // bytes per tile
  constexpr int KS = D / 16;       // contraction slices of QK^T
  constexpr int DB = D / 32;       // 32-wide blocks of the head dim in PV
  constexpr int PIECES = TILE / 1024;  // 1 KB wave-loads per tile: 8 at d = 128, 4 at d = 64
  constexpr float kLazyLog2 = 8.f;
  static_assert(BM == 32 * WAVES, "one 32-row block per wave");
  static_assert(PIECES == WAVES || 2 * PIECES == WAVES, "a tile is loaded by all waves, or K and V by half of them each");
  // K ring, V ring; at the end of a workgroup that merges its partials, their LSEs ([parts][256] floats)
  constexpr int kRingBytes = 2 * NBUF * TILE, kLseBytes = KEEP ? 0 : kMaxParts * BM * (int)sizeof(float);
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kRingBytes > kLseBytes ? kRingBytes : kLseBytes];

  const unsigned smem_base = lds_offset(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  Segment seg;
  int bh, qt;
  if (!decode_job<BM>(a, seg, bh, qt)) return;
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

  // this lane's query row (local to the q tile): 32 wave + n; rows beyond the range read the last valid row
  s16x8 qf[KS];
  {
    const int ql = min(qt * BM + 32 * wave + n, q_len - 1) - qt * BM;
    const char* qrow = qbase + (int64_t)ql * ROWB + h * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const s16x8*)(qrow + ks * 32);
  }
  // the 1 KB piece of a tile this wave loads: all waves a piece of K and of V each (d = 128), or waves 0-3 the
  // K tile and waves 4-7 the V tile (d = 64)
  const bool loads_k = PIECES == WAVES || wave < PIECES;
  const bool loads_v = PIECES == WAVES || wave >= WAVES - PIECES;
  const int piece_k = wave, piece_v = PIECES == WAVES ? wave : wave - (WAVES - PIECES);
  int goff_k, goff_v;
  {
    const int pk = piece_k * 64 + lane, pv = piece_v * 64 + lane;
    goff_k = (pk / CPR) * ROWB + (((pk % CPR) ^ k_swizzle<D>(pk / CPR)) << 4);
    goff_v = (pv / CPR) * ROWB + (((pv % CPR) ^ v_swizzle<D>(pv / CPR)) << 4);
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
  auto reset_state = [&]() {
    m = -INFINITY;
    ms = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) ls[i] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  };
  f32x16 sacc;   // scores of the tile in flight: written by an MFMA phase, consumed by the next softmax phase
  s16x8 pf[2];   // its probabilities in B-operand layout: written by a softmax phase, consumed by the next MFMA phase

  // ---- the KV chunk being walked (wave-uniform)
  const char *kbase = nullptr, *vbase = nullptr;
  // where the loads that run past the last tile go: the first tiles of the next chunk when
  // the pipeline carries over (stride TILE), else a re-read of the last tile (stride 0)
  int64_t past_delta = 0;  // from the end of this chunk's K (V) to that place
  int past_stride = 0;
  int kv_len = 0, n_tiles = 0, first_masked = 0, kv_tail = -1, diag_rows = 0;
  bool diag = false;
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
  auto surplus = [&](int piece) {
    const int row = (piece * 64 + lane) / CPR;
    return max(0, kv_tail * BN + row - (kv_len - 1)) * ROWB;
  };
  // byte offset of tile t from the chunk's first tile, branch-free: t < n_tiles gives t TILE; beyond that
  // n_tiles TILE + past_delta + (t - n_tiles) past_stride
  auto tile_offset = [&](int t) -> int64_t {
    const int64_t beyond = (int64_t)((n_tiles - 1 - t) >> 31);  // all ones iff t >= n_tiles
    return (int64_t)min(t, n_tiles) * TILE + (int64_t)max(t - n_tiles, 0) * past_stride + (past_delta & beyond);
  };
  // `checked`: the tile may be kv_tail (steady blocks never issue that one)
  auto issue_k = [&](int t, auto checked) {
    if (!loads_k) return;
    const char* kt = kbase + tile_offset(t);
    const unsigned kd = __builtin_amdgcn_readfirstlane(smem_base + (t & (NBUF - 1)) * TILE + piece_k * 1024);
    if (decltype(checked)::value && t == kv_tail) load_lds_16(kt, goff_k - surplus(piece_k), kd);
    else load_lds_16(kt, goff_k, kd);
  };
  auto issue_v = [&](int t, auto checked) {
    if (!loads_v) return;
    const char* vt = vbase + tile_offset(t);
    const unsigned vd = __builtin_amdgcn_readfirstlane(smem_base + (NBUF + (t & (NBUF - 1))) * TILE + piece_v * 1024);
    if (decltype(checked)::value && t == kv_tail) load_lds_16(vt, goff_v - surplus(piece_v), vd);
    else load_lds_16(vt, goff_v, vd);
  };
  // the same for a tile given by address (interior groups keep running pointers instead of recomputing
  // tile_offset: two scalar instructions per load instead of eighteen)
  auto issue_k_at = [&](const char* kt, int slot) {
    const unsigned kd = __builtin_amdgcn_readfirstlane(smem_base + slot * TILE + piece_k * 1024);
    load_lds_16(kt, goff_k, kd);
  };
  auto issue_v_at = [&](const char* vt, int slot) {
    const unsigned vd = __builtin_amdgcn_readfirstlane(smem_base + (NBUF + slot) * TILE + piece_v * 1024);
    load_lds_16(vt, goff_v, vd);
  };
  constexpr std::true_type kChecked{};
  constexpr std::false_type kUnchecked{};

  // S^T = K Q^T of one 32-key tile (csrc/ring_attention.cu:565)
  auto qk = [&](int kslot) {
    const unsigned char* ks_lds = smem + kslot * TILE;
#pragma unroll
    for (int e = 0; e < 16; ++e) sacc[e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const s16x8 kfr = *(const s16x8*)(ks_lds + koff[ks]);
      sacc = E::mma(kfr, qf[ks], sacc);
    }
  };
  // key visible iff inside the KV range and key_local <= query_local + diag_off
  auto mask_tile = [&](int t, auto always) {
    if (decltype(always)::value || t >= first_masked) {
      int lim = kv_len - 1 - t * BN - 4 * h;
      if (diag) lim = min(lim, diag_rows + 32 * wave + n - t * BN - 4 * h);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int key = 8 * (e >> 2) + (e & 3);
        if (key > lim) sacc[e] = -INFINITY;
      }
    }
  };
  // max(m, row max of the tile): two chains of max(max(x, a), b), each link one v_max3_f32; one
  // exchange between the halves of the wave
  auto tile_max = [&]() {
    float m0 = m, m1 = m;
#pragma unroll
    for (int e = 0; e < 16; e += 4) {
      m0 = fmaxf(fmaxf(m0, sacc[e]), sacc[e + 1]);
      m1 = fmaxf(fmaxf(m1, sacc[e + 2]), sacc[e + 3]);
    }
    return cross_half_max(fmaxf(m0, m1));
  };
  // The reference max moves when some row's cand = max(m, tile max) is far above it (or it is still
  // unset): rescale of l and acc-O as in csrc/ring_attention.cu:226-232.
  auto move_reference = [&](float cand) {
    const bool far = (cand - m) * a.scale_log2 > kLazyLog2;
    if (__builtin_amdgcn_ballot_w64(far) != 0) {
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
  auto exponentials = [&](float (&sums)[4]) {
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      typename E::vec8 pv;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[8 * t2 + e], a.scale_log2, -ms));
        sums[e & 3] += p;
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
  // the softmax phase of the tile whose scores are in sacc
  // At d = 64 the kernel is bound by this phase (the same VALU work per score as at d = 128 for half the
  // MFMA work), and the phase runs speculatively: exponentials against the reference as it stands, and the
  // tile's row maximum is only looked at when some probability came out large (a sum of four of them above
  // kSpecLimit, which fp16 still holds; an infinity or a NaN also lands here) or a row has no reference yet.
  // At d = 128 the same change measured 6-9 % slower: the decision then sits at the end of the phase, between
  // the wave's last VALU result and the first fragment reads of its next MFMA phase.
  constexpr bool kSpeculate = D == 64;
  constexpr float kSpecLimit = 16384.f;
  auto softmax_phase = [&]() {
    if (!kSpeculate) {
      move_reference(tile_max());
      exponentials(ls);
      return;
    }
    float sums[4] = {0.f, 0.f, 0.f, 0.f};
    exponentials(sums);
    const float largest = fmaxf(fmaxf(sums[0], sums[1]), fmaxf(sums[2], sums[3]));
    const bool again = !(largest <= kSpecLimit) || m == -INFINITY;
    if (__builtin_amdgcn_ballot_w64(again) != 0) {
      move_reference(tile_max());
#pragma unroll
      for (int i = 0; i < 4; ++i) sums[i] = 0.f;
      exponentials(sums);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) ls[i] += sums[i];
  };
  auto phase_fence = [&]() { __builtin_amdgcn_sched_barrier(0); };  // keeps the compiler from mixing the phases
  // The MFMA phase of a steady block: O += P(u) V(u), then S(u+1) = K(u+1) Q^T.  Scheduling hint: the
  // fragment reads run ahead of the MFMAs that consume them (8 reads up front, two more behind each of
  // the PV MFMAs: the K fragments are all on their way when the QK MFMAs start), so the matrix pipe does
  // not wait for LDS latency inside the phase.
  auto mfma_phase = [&](int vslot, int kslot) {
    pv_product(vslot);
    qk(kslot);
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
    for (int i = 0; i < 2 * DB; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int i = 0; i < KS; ++i) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  };
  // Set between a carried-over chunk boundary and the first pair of the next chunk when a partial is stored
  // in between: the tiles that pair needs were waited for (and the barrier passed) BEFORE the stores, so that
  // the pair does not wait for them (stores count in vmcnt too).
  bool synced = false;
  auto ring_barrier = [&]() {
    if (synced) {
      synced = false;
      return;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  // a chunk's partial (csrc/ring_attention.cu:621-633): normalise, emit O and LSE
  auto emit_partial = [&](const SegItem* w) {
    const float l = cross_half_sum((ls[0] + ls[1]) + (ls[2] + ls[3]));
    const float inv = (l > 0.f) ? 1.f / l : 0.f;
    const int row_l = qt * BM + 32 * wave + n;
    if (row_l >= q_len) return;  // a row beyond the query range
    int64_t prow = w->part_base + (int64_t)bh * w->part_bh_stride + row_l;
    if (w->part_row_mul > 0) prow = prow * w->part_row_mul + w->slot;  // a row's steps next to each other
    const int64_t opos = prow * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 val;
#pragma unroll
        for (int e = 0; e < 4; ++e) val[e] = oacc[db][4 * q4 + e] * inv;
        if (HP) {  // fp16 partials: |O_part| <= max |V|, the caller vouches that this fits
          f16x4 hv;
#pragma unroll
          for (int e = 0; e < 4; ++e) hv[e] = (_Float16)val[e];
          *(f16x4*)((_Float16*)a.o_part + opos + 32 * db + 8 * q4 + 4 * h) = hv;
        } else {
          *(f32x4*)((float*)a.o_part + opos + 32 * db + 8 * q4 + 4 * h) = val;
        }
      }
    if (h == 0) a.lse_part[prow] = (l > 0.f) ? (ms + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
  };
  // (KEEP fixes it at compile time; the other instantiations decide at run time, which also gives the
  // emission path the better code: as a compile-time constant it measured 8 % slower at cfg4)
  const bool keep_state = KEEP || a.mode == kBlockCarryState;

  // The walk of all items, for one half of the workgroup.  At the start of block u the waves of the
  // first half hold P(u) (their softmax phase of tile u is done), those of the second half the raw
  // scores S(u).  Block u: the even ones start with the barrier of the pair (u, u+1) -- K(u+1),
  // K(u+2), V(u), V(u+1), issued during the previous pair, have landed, and every wave is past
  // block u-1, so the ring slots of K(u-1), K(u), V(u-2), V(u-1) are free for K(u+3), K(u+4),
  // V(u+2), V(u+3), which are issued during this pair -- then
  //     first half :  O += P(u) V(u), S(u+1) = K(u+1) Q^T  |  softmax of S(u+1)
  //     second half:  softmax of S(u)                      |  O += P(u) V(u), S(u+1) = K(u+1) Q^T
  auto walk = [&](auto second_c) {
    constexpr bool SECOND = decltype(second_c)::value;
    // STEADY blocks (tiles u+1 and u+2 unmasked or covered by MASKED) have compile-time ring slots
    // which tiles this half of the workgroup loads: all waves a piece of each (d = 128), or the first half K and
    // the second half V (d = 64)
    constexpr bool LOADS_K = PIECES == WAVES || !SECOND, LOADS_V = PIECES == WAVES || SECOND;
    const char *k_next = nullptr, *v_next = nullptr;  // interior groups: the next K and the next V tile to load
    auto block = [&](auto slot_c, auto steady, auto masked, auto interior, int u) {
      constexpr int SLOT = decltype(slot_c)::value;  // u mod 4 (STEADY only)
      constexpr bool STEADY = decltype(steady)::value;
      constexpr bool MASKED = decltype(masked)::value;  // STEADY only: tile u+1 gets the mask
      constexpr bool INTERIOR = decltype(interior)::value;  // STEADY only: every tile loaded lies inside the chunk
      if (STEADY) {
        // the two tile loads of a block go out next to the softmax phase of the wave (the VALU side has issue
        // slots to spare): K(u+3), K(u+4) in even blocks, V(u+1), V(u+2) in odd ones
        auto issue_loads = [&]() {
          if (INTERIOR) {
            if ((SLOT & 1) == 0) {
              if (LOADS_K) {
                issue_k_at(k_next, (SLOT + 3) & 3);
                issue_k_at(k_next + TILE, SLOT);
                k_next += 2 * TILE;
              }
            } else if (LOADS_V) {
              issue_v_at(v_next, (SLOT + 1) & 3);
              issue_v_at(v_next + TILE, (SLOT + 2) & 3);
              v_next += 2 * TILE;
            }
          } else if ((SLOT & 1) == 0) {
            issue_k(u + 3, kUnchecked);
            issue_k(u + 4, kUnchecked);
          } else {
            issue_v(u + 1, kUnchecked);
            issue_v(u + 2, kUnchecked);
          }
        };
        if ((SLOT & 1) == 0) ring_barrier();
        if (SECOND) issue_loads();
        phase_fence();
        if (!SECOND) {
          mfma_phase(SLOT, (SLOT + 1) & 3);
          if (MASKED) mask_tile(u + 1, kChecked);
        } else {
          softmax_phase();
        }
        phase_fence();
        if (!SECOND) issue_loads();
        phase_fence();
        if (!SECOND) {
          // the scores past the end of a chunk belong to the next chunk (or to nothing): its start handles them
          if (u + 1 < n_tiles) softmax_phase();
        } else {
          mfma_phase(SLOT, (SLOT + 1) & 3);
          if (MASKED) mask_tile(u + 1, kChecked);
        }
        phase_fence();
      } else {
        if ((u & 1) == 0) {
          ring_barrier();
          if (u + 3 < n_tiles) issue_k(u + 3, kChecked);
          if (u + 4 < n_tiles) issue_k(u + 4, kChecked);
          if (u + 2 < n_tiles) issue_v(u + 2, kChecked);
          if (u + 3 < n_tiles) issue_v(u + 3, kChecked);
        }
        if (SECOND) softmax_phase();
        pv_product(u & 3);
        if (u + 1 < n_tiles) {
          qk((u + 1) & 3);
          mask_tile(u + 1, kUnchecked);
          if (!SECOND) softmax_phase();
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
          past_delta = ((int64_t)wn->kv_start - w->kv_start) * ROWB - (int64_t)n_tiles * TILE;
          past_stride = TILE;
        }
      }
      if (!carry) {
        past_delta = -(int64_t)TILE;
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
        ring_barrier();
        qk(0);
      }
      // (carried: the last block of the previous chunk left the scores of tile 0 in sacc; K(1), K(2),
      // V(0), V(1) are in flight)
      mask_tile(0, kUnchecked);
      if (!SECOND) softmax_phase();

      // Steady blocks come in groups of four.  A group starting at u computes the scores of tiles
      // u+1 .. u+4 and loads up to tile u+6:
      //   plain groups   while those four tiles need no mask; without any mask in the chunk the last
      //                  group runs up to tile n_tiles-1 and its last block computes the scores of
      //                  the tile after the last one (the next chunk's first, or nothing of use);
      //   masked groups  (diagonal chunks) for the rest: every block masks its tile u+1;
      //   a chunk with surplus keys in its last tile keeps clear of that tile (its loads need the
      //   clamped form) and leaves the rest to the general blocks.
      const bool ragged = kv_tail >= 0;
      const int plain_end = ragged ? min(first_masked, kv_tail - 2) : (diag ? first_masked : n_tiles + 1);
      const int masked_end = (diag && !ragged) ? n_tiles + 1 : 0;
      constexpr std::true_type kYes{};
      constexpr std::false_type kNo{};
      int u = 0;
      // interior plain groups: the group at u loads K up to tile u+6 and V up to tile u+5, all inside the chunk
      k_next = kbase + 3 * TILE;
      v_next = vbase + 2 * TILE;
      // (d = 64 only: +9 % on cfg2, whose softmax phase is what a wave spends its issue slots on; at d = 128 the
      // same change measured 2-6 % slower, as did everything else that shortened the softmax phase there)
      constexpr bool kInteriorGroups = D == 64;
      for (; kInteriorGroups && u + 4 < plain_end && u + 6 < n_tiles; u += 4) {
        block(C0{}, kYes, kNo, kYes, u);
        block(C1{}, kYes, kNo, kYes, u + 1);
        block(C2{}, kYes, kNo, kYes, u + 2);
        block(C3{}, kYes, kNo, kYes, u + 3);
      }
      for (; u + 4 < plain_end; u += 4) {
        block(C0{}, kYes, kNo, kNo, u);
        block(C1{}, kYes, kNo, kNo, u + 1);
        block(C2{}, kYes, kNo, kNo, u + 2);
        block(C3{}, kYes, kNo, kNo, u + 3);
      }
      for (; u + 4 < masked_end; u += 4) {
        block(C0{}, kYes, kYes, kNo, u);
        block(C1{}, kYes, kYes, kNo, u + 1);
        block(C2{}, kYes, kYes, kNo, u + 2);
        block(C3{}, kYes, kYes, kNo, u + 3);
      }
      for (; u < n_tiles; ++u) block(C0{}, kNo, kNo, kNo, u);
      carried = carry;
      if (keep_state) {
        // the softmax state runs on into the next chunk; with the pipeline carried over as well, the chunk
        // boundary is just another tile boundary
        if (!carry) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // re-reads of the last tile
        continue;
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next chunk's first tiles, or re-reads of the last tile
      if (carry) {
        __syncthreads();
        synced = true;
      }
      emit_partial(w);
      reset_state();
    }
  };
  if (wave < WAVES / 2) walk(std::false_type{});
  else walk(std::true_type{});

  if (!KEEP && a.mode == kBlockPartialsMerged)  // this workgroup's rows over the partials it has just written
    merge_job_rows<DT, D, HP, BM, 64 * WAVES>(a.o_part, a.lse_part, a.out, a.lse, a.items, seg, bh, qt, a.S,
                                              (lds_float*)(__attribute__((address_space(3))) void*)smem);
  // the rows' result from a carried state: the reference's epilogue (csrc/ring_attention.cu:621-664), O = acc / l
  // in the storage type, plus the LSE
  if (keep_state) {
    const float l = cross_half_sum((ls[0] + ls[1]) + (ls[2] + ls[3]));
    const float inv = (l > 0.f) ? 1.f / l : 0.f;
    const int row_l = qt * BM + 32 * wave + n;
    if (row_l < q_len) {  // not a row beyond the query range
      const int64_t row = (int64_t)bh * a.S + q_start + row_l;
      typename E::type* orow = (typename E::type*)a.out + row * D;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          typename E::vec4 val;
#pragma unroll
          for (int e = 0; e < 4; ++e) val[e] = (typename E::type)(oacc[db][4 * q4 + e] * inv);
          *(typename E::vec4*)(orow + 32 * db + 8 * q4 + 4 * h) = val;
        }
      if (h == 0 && a.lse) a.lse[row] = (l > 0.f) ? (ms + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
    }
  }
}

hipError_t launch_walk(const BlockArgs& a, int dtype, int dim, hipStream_t stream) {
  if (a.n_segs <= 0) return hipSuccess;
  const int q_tiles = a.q_tiles_max;  // kWalkM-row tiles of the longest segment
  const int64_t groups = (int64_t)a.n_segs * a.BH;
  const int64_t blocks = (a.groups ? (int64_t)a.groups_per_xcd : (groups + 7) / 8) * 8 * q_tiles;
  if (q_tiles <= 0 || blocks > INT32_MAX) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)blocks;
  if (a.mode != kBlockCarryState && a.mode != kBlockPartials && a.mode != kBlockPartialsMerged) return hipErrorInvalidValue;
#define RA_LAUNCH_WALK(DT_, D_)                                                                          \
  do {                                                                                                \
    if (a.mode == kBlockCarryState) ring_walk_kernel<DT_, D_, false, true><<<grid, 512, 0, stream>>>(a);   \
    else if (a.half_partials) ring_walk_kernel<DT_, D_, true, false><<<grid, 512, 0, stream>>>(a);         \
    else ring_walk_kernel<DT_, D_, false, false><<<grid, 512, 0, stream>>>(a);                             \
  } while (0)
  if (dtype == 0 && dim == 64) RA_LAUNCH_WALK(0, 64);
  else if (dtype == 0 && dim == 128) RA_LAUNCH_WALK(0, 128);
  else if (dtype == 1 && dim == 64) RA_LAUNCH_WALK(1, 64);
  else if (dtype == 1 && dim == 128) RA_LAUNCH_WALK(1, 128);
#undef RA_LAUNCH_WALK
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ringattn
