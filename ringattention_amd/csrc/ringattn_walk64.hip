// gfx950 (CDNA4) kernel: block attention over the ring steps of 256 query rows, 64 rows per wave.
//
//   ring_walk64_kernel : the forward of ring_walk_kernel (ringattn_walk.hip; the reference's CTA
//       that walks its ring steps with max / sum / acc-O in registers,
//       csrc/ring_attention.cu:439-443,456-620, epilogue :621-664; or, chunk by chunk, with a partial
//       (O, LSE) per ring step and their merge at the end), laid out for ONE wave
//       per SIMD: a workgroup of FOUR waves owns the same 256 query rows, each wave two 32-query
//       blocks.  Every K fragment and every V^T fragment read from LDS then feeds two MFMAs (one per
//       block) instead of one: half the LDS fragment traffic per MFMA.  With 512 registers per wave
//       the tile pipeline is skewed by a tile on either side so that, within one iteration, the
//       matrix work and the vector work have no dependence on each other and interleave freely in
//       the single instruction stream:
//           iteration u :  S(u+1) = K(u+1) Q^T   |   P(u) = exp2(S(u) k2 - m k2), row sums   |   O += P(u-1) V(u-1)
//       The reference max for tile u+1 is decided at the end of iteration u (wave-uniform branch,
//       as in ring_walk_kernel); its rescale of acc-O (:226-232) is applied one iteration later,
//       once P(u) -- computed against the old reference -- has been accumulated.
//       The KV chunks of a segment are walked as ONE sequence of 32-key tiles (the diagonal chunk
//       last): a chunk boundary is only a jump of the load address.
//       One wave per SIMD has nobody to wait behind, so nothing may be waited for: the K and V rings are eight
//       tiles deep (128 KB of LDS) and a tile is loaded four or more iterations before the barrier that hands it
//       over (s_waitcnt vmcnt(12): the loads of the last three iterations stay in flight).
//       Described for d = 128; at d = 64 (state carried only) a tile is 4 KB, an iteration has 16 MFMAs and the
//       rings take 64 KB.  Shapes it takes: every KV range a multiple of 32 keys and at least 128 (the host checks);
//       anything else runs ring_walk_kernel.
#include "ringattn_device.h"

#include <type_traits>

namespace ringattn {

// Merge of the workgroup's 256 rows over the partials the workgroup has written (what merge_job_rows does for
// ring_walk_kernel; the arithmetic and its order are merge_row's, so the bits are the merge kernel's).  With one wave
// per SIMD nobody covers for a wave that waits for memory, so the partial rows are not fetched into registers a
// batch at a time but streamed through LDS, which the rings have left free: every wave merges eight rows of each
// group of 32 and keeps six blocks (eight rows of one part: 4 KB, 2 KB as fp16) in flight in a ring of its own,
// with no barrier between the waves.  LDS: the partial LSEs [parts][256], the parts' first rows, the four rings.
constexpr int kStagedMergeMaxParts = 24;  // LSEs of at most this many parts fit below the rings
template <int DT, bool HP>
static __device__ __forceinline__ void merge_rows_staged(const BlockArgs& a, const Segment& seg, int bh, int qt,
                                                         unsigned char* smem, unsigned smem_base) {
  constexpr int D = 128, BM = kWalkM;
  constexpr int RB = HP ? D * 2 : D * 4;  // bytes per partial row
  constexpr int SLOT = 8 * RB;            // a block: eight rows of one part
  constexpr int LPB = SLOT / 1024;        // load instructions per block (1 KB per wave and instruction)
  constexpr int NS = 6;                   // blocks in flight per wave
  constexpr int PPR = RB / 16;            // 16-byte pieces per row
  constexpr int NK = PPR / 8;             // pieces per lane and row
  constexpr int CPP = HP ? 8 : 4;         // columns per piece
  constexpr int kBaseAt = kStagedMergeMaxParts * BM * 4;  // behind the LSEs: the parts' first rows (int64 each)
  constexpr int kRingAt = kBaseAt + 1024;  // (every 1 KB transfer stays inside a 1 KB block of LDS)
  static_assert(kStagedMergeMaxParts * 8 <= 1024, "the parts' first rows fit");
  static_assert(kRingAt + 4 * NS * SLOT <= 2 * 8 * 8192 + 8 * (kMaxParts + 4), "inside the kernel's LDS (rings and chunk list)");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_parts = seg.item_count;
  const SegItem* its = a.items + seg.item_begin;
  const int row0 = qt * BM;
  const int rows_here = min(BM, seg.q_len - row0);
  const int n_groups = (rows_here + 31) / 32;
  float* lse_s = (float*)smem;
  int64_t* base_s = (int64_t*)(smem + kBaseAt);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();  // the partial stores of all waves have completed and are visible to them; the LDS is idle
  for (int i0 = 0; i0 < n_parts; i0 += 8) {  // thread tid: the LSEs of row tid
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (i0 + u < n_parts) {
        const int64_t prow = its[i0 + u].part_base + (int64_t)bh * its[i0 + u].part_bh_stride + row0;
        v[u] = tid < rows_here ? a.lse_part[prow + tid] : -INFINITY;
        if (tid == 0) base_s[i0 + u] = prow;
      }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (i0 + u < n_parts) lse_s[(i0 + u) * BM + tid] = v[u];
  }
  __syncthreads();

  // block t = (group, part) in that order; this wave's rows of a group: 32 group + 8 wave + [0, 8)
  const int total = n_groups * n_parts;
  const unsigned ring = smem_base + kRingAt + wave * (NS * SLOT);
  int ig = 0, ii = 0;  // group and part of the next block to issue
  auto issue_block = [&](int slot) {
    const int64_t prow = base_s[ii];
    const uint64_t addr = (uint64_t)(uintptr_t)a.o_part + (uint64_t)prow * RB;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)addr), hi = __builtin_amdgcn_readfirstlane((unsigned)(addr >> 32));
    const char* src = (const char*)(uintptr_t)(((uint64_t)hi << 32) | lo);  // row 0 of the job in part ii
    const int r_first = 32 * ig + 8 * wave;
#pragma unroll
    for (int k = 0; k < LPB; ++k) {
      const int pos = k * 64 + lane;  // 16-byte position within the block
      const int r = pos / PPR, piece = (pos % PPR) ^ (8 * (r & 1));
      const int rr = min(r_first + r, rows_here - 1);  // rows past the end of the segment: its last row again
      load_lds_16_settled(src, rr * RB + piece * 16, ring + slot * SLOT + k * 1024);
    }
    if (++ii == n_parts) {
      ii = 0;
      ++ig;
    }
  };
  for (int t = 0; t < NS && t < total; ++t) issue_block(t);

  const int r8 = lane >> 3, c = lane & 7;
  float mx = -INFINITY, wsum = 0.f, acc[NK * CPP];
  int cg = 0, ci = 0;  // group and part of the block to consume
  int slot = 0;
  for (int t = 0; t < total; ++t) {
    if (t + NS <= total) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 1) * LPB) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const int row = 32 * cg + 8 * wave + r8;  // within the job
    f32x4 x[NK];
    const unsigned char* blk = smem + kRingAt + wave * (NS * SLOT) + slot * SLOT + r8 * RB;
#pragma unroll
    for (int k = 0; k < NK; ++k) x[k] = *(const f32x4*)(blk + (((c + 8 * k) ^ (8 * (r8 & 1))) << 4));
    if (ci == 0) {  // new rows: L = max over the parts first
      mx = -INFINITY;
      wsum = 0.f;
#pragma unroll
      for (int e = 0; e < NK * CPP; ++e) acc[e] = 0.f;
      for (int i = 0; i < n_parts; ++i) mx = fmaxf(mx, lse_s[i * BM + row]);
    }
    const float L = lse_s[ci * BM + row];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the block is in registers: its slot takes the block NS further on
    if (t + NS < total) issue_block(slot);
    if (row < rows_here && L != -INFINITY) {  // (-inf: the identity element, its O may hold anything)
      const float w = __expf(L - mx);
      wsum += w;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        if (HP) {
          const f16x8 hv = __builtin_bit_cast(f16x8, x[k]);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[8 * k + e] = __builtin_fmaf(w, (float)hv[e], acc[8 * k + e]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[4 * k + e] = __builtin_fmaf(w, x[k][e], acc[4 * k + e]);
        }
      }
    }
    if (ci == n_parts - 1 && row < rows_here) {  // all parts in: normalise and store
      if (mx != -INFINITY) {
        const float inv = 1.f / wsum;
#pragma unroll
        for (int e = 0; e < NK * CPP; ++e) acc[e] *= inv;
      }
      const int64_t out_row = (int64_t)bh * a.S + seg.q_start + row0 + row;
      typename Elem<DT>::type* orow = (typename Elem<DT>::type*)a.out + out_row * D;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        if (HP) {
          Store8<DT>::st(orow + (c + 8 * k) * 8, &acc[8 * k]);
        } else {
          typename Elem<DT>::vec4 o4;
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = (typename Elem<DT>::type)acc[4 * k + e];
          *(typename Elem<DT>::vec4*)(orow + (c + 8 * k) * 4) = o4;
        }
      }
      if (c == 0) a.lse[out_row] = (mx == -INFINITY) ? -INFINITY : mx + __logf(wsum);
    }
    if (++ci == n_parts) {
      ci = 0;
      ++cg;
    }
    slot = slot + 1 == NS ? 0 : slot + 1;
  }
}

// KEEP: max / sum / acc-O run through all chunks of the q tile and the rows' result is written once (kBlockCarryState).
// Otherwise the chunks are walked one by one, each as a sequence of its own -- prologue, loop, drain --, and each
// ends in its normalised partial (O, LSE) (kBlockPartials, kBlockPartialsMerged; HP: partial O as fp16).
// D = 64 (state carried only): half the MFMAs per tile for the same vector work, 4 KB tiles (one 1 KB piece per wave),
// 64 KB of rings.
template <int DT, int D, bool KEEP, bool HP>
__global__ __launch_bounds__(256, 1) void ring_walk64_kernel(const BlockArgs a) {
  using E = Elem<DT>;
  static_assert(D == 128 || (D == 64 && KEEP && !HP), "d = 64 is built with the state carried only");
  constexpr int WAVES = 4;
  constexpr int BM = kWalkM;       // query rows per workgroup: 4 waves x 64
  constexpr int BN = 32;           // keys per tile
  constexpr int NBUF = 8;          // ring depth of the K and of the V tiles: loads run seven to eight tiles ahead of the products
  constexpr int CPR = D / 8;       // 16-byte chunks per row
  constexpr int ROWB = D * 2;      // bytes per row
  constexpr int TILE = BN * ROWB;  // bytes per tile
  constexpr int PIECES = TILE / 4096;  // 1 KB pieces of a tile per wave
  constexpr int KS = D / 16;       // contraction slices of QK^T
  constexpr int DB = D / 32;       // 32-wide blocks of the head dim in PV
  constexpr float kLazyLog2 = 8.f;
  static_assert(BM == 64 * WAVES, "two 32-row blocks per wave");
  constexpr int kListAt = 2 * NBUF * TILE;  // behind the rings: the chunks of this q tile in walking order, (byte offset, tiles) each
  __shared__ __attribute__((aligned(1024))) unsigned char smem[kListAt + 8 * (kMaxParts + 4)];

  const unsigned smem_base = lds_offset(smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  Segment seg;
  int bh, qt;
  if (!decode_job<BM>(a, seg, bh, qt)) return;
  const int q_start = seg.q_start, q_len = seg.q_len;
  const int all_items = seg.item_count;
  // items in run order: table order, except that item `last_item` (the diagonal one) is moved to the end
  auto item_in_order = [&](int i) -> const SegItem* {
    int idx = i;
    if (seg.last_item >= 0) idx = (i == all_items - 1) ? seg.last_item : (i >= seg.last_item ? i + 1 : i);
    return a.items + seg.item_begin + idx;
  };
  const int64_t head_off = (int64_t)bh * a.bh_stride;
  const int kv_bh = (bh / a.heads) * (a.heads / a.kv_group) + (bh % a.heads) / a.kv_group;
  const int64_t kv_head_off = (int64_t)kv_bh * a.kv_bh_stride;
  const char* qbase = (const char*)a.q + (head_off + (int64_t)(q_start + qt * BM) * D) * 2;
  const char* k_head = (const char*)a.k + kv_head_off * 2;
  const char* v_head = (const char*)a.v + kv_head_off * 2;

  // Q of this lane's two rows (B operands for the whole launch); rows beyond the range read the last valid row
  s16x8 qf[2][KS];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int ql = min(qt * BM + 64 * wave + 32 * b + n, q_len - 1) - qt * BM;
    const char* qrow = qbase + (int64_t)ql * ROWB + h * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[b][ks] = *(const s16x8*)(qrow + ks * 32);
  }
  // the 1 KB pieces of a tile this wave loads (d = 128: pieces 2 wave and 2 wave + 1 of eight; d = 64: piece wave of four)
  int goff_k[PIECES], goff_v[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int pk = (PIECES * wave + j) * 64 + lane;
    goff_k[j] = (pk / CPR) * ROWB + (((pk % CPR) ^ k_swizzle<D>(pk / CPR)) << 4);
    goff_v[j] = (pk / CPR) * ROWB + (((pk % CPR) ^ v_swizzle<D>(pk / CPR)) << 4);
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

  // ---- a pass walks n_items chunks from item `first` on as one sequence: all of them (KEEP), or one
  const int n_items = KEEP ? all_items : 1;
  for (int first = 0; first < all_items; first += n_items) {
  auto item_at = [&](int i) -> const SegItem* { return item_in_order(first + i); };
  // ---- the flattened tile sequence of the pass: item i contributes tiles_of(i) tiles
  const int diag_item = (n_items > 0 && item_at(n_items - 1)->diag_off >= 0) ? n_items - 1 : -1;
  auto tiles_of = [&](const SegItem* w) {
    const int kv_tiles = w->kv_len / BN;
    return w->diag_off >= 0 ? min(kv_tiles, (w->diag_off + qt * BM + BM - 1) / BN + 1) : kv_tiles;
  };
  int N = 0;
  for (int i = 0; i < n_items; ++i) N += tiles_of(item_at(i));
  // this wave's share of the diagonal chunk: tiles below Mw are visible to all its rows, tiles from Ew on to none
  int Mw = N, Ew = N, diag_base = 0, diag_rows = 0;
  if (diag_item >= 0) {
    const SegItem* w = item_at(diag_item);
    const int n_last = tiles_of(w);
    diag_base = N - n_last;
    diag_rows = w->diag_off + qt * BM;  // keys below this local index are visible to the whole q tile
    Mw = diag_base + min(n_last, (diag_rows + 64 * wave + 1) / BN);
    Ew = diag_base + min(n_last, (diag_rows + 64 * wave + 63) / BN + 1);
  }

  // ---- load streams: K is loaded seven to eight tiles ahead of its product, V four to five.  A stream is a byte
  // offset from the head's first row; past the last chunk it goes round the first four tiles of the head (valid
  // memory: some KV range of 128 keys lies in every head; nobody reads these tiles from LDS), so that every
  // iteration issues the same number of loads.  At most nine tiles are loaded past the end: three such rounds.
  struct Stream {
    unsigned off;  // the next tile to load
    int left;      // tiles left in its chunk, that one included
    int idx;       // the chunk
  };
  auto chunk_of = [&](int i, unsigned& off, int& cnt) {
    if (i < n_items) {
      const SegItem* w = item_at(i);
      off = (unsigned)w->kv_start * ROWB;
      cnt = tiles_of(w);
    } else {
      off = 0;
      cnt = 4;
    }
  };
  auto step = [&](Stream& s) {
    s.off += TILE;
    if (--s.left == 0) {
      s.idx += 1;
      chunk_of(s.idx, s.off, s.left);
    }
  };
  Stream kst, vst;
  kst.idx = vst.idx = 0;
  chunk_of(0, kst.off, kst.left);
  chunk_of(0, vst.off, vst.left);
  auto issue_k = [&](int slot) {
    const unsigned dst = __builtin_amdgcn_readfirstlane(smem_base + slot * TILE + PIECES * wave * 1024);
    const char* p = k_head + __builtin_amdgcn_readfirstlane(kst.off);
#pragma unroll
    for (int j = 0; j < PIECES; ++j) load_lds_16_settled(p, goff_k[j], dst + 1024 * j);
    step(kst);
  };
  auto issue_v = [&](int slot) {
    const unsigned dst = __builtin_amdgcn_readfirstlane(smem_base + (NBUF + slot) * TILE + PIECES * wave * 1024);
    const char* p = v_head + __builtin_amdgcn_readfirstlane(vst.off);
#pragma unroll
    for (int j = 0; j < PIECES; ++j) load_lds_16_settled(p, goff_v[j], dst + 1024 * j);
    step(vst);
  };

  // ---- softmax state of the two blocks
  float m[2] = {-INFINITY, -INFINITY};  // reference max (raw score units)
  float ms[2] = {0.f, 0.f};             // m * k2, 0 while m is -inf (guard of csrc/ring_attention.cu:183)
  float ls[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  float cand[2] = {-INFINITY, -INFINITY};
  float apend[2] = {1.f, 1.f};  // rescale of acc-O that is still to be applied
  bool pend = false;
  f32x16 oacc[2][DB];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[b][db][e] = 0.f;
  f32x16 sacc[2];     // scores of tile u, consumed by the exponentials of iteration u
  s16x8 pprev[2][2];  // probabilities of tile u-1 (B operands), consumed by the PV product of iteration u
#pragma unroll
  for (int b = 0; b < 2; ++b) {
#pragma unroll
    for (int e = 0; e < 16; ++e) sacc[b][e] = 0.f;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int e = 0; e < 8; ++e) pprev[b][t2][e] = 0;
  }

  // S^T = K Q^T of one 32-key tile for both blocks (csrc/ring_attention.cu:565): each K fragment feeds two MFMAs
  auto qk = [&](int kbytes, f32x16 (&s)[2]) {
    const unsigned char* ks_lds = smem + kbytes;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[b][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const s16x8 kfr = *(const s16x8*)(ks_lds + koff[ks]);
      s[0] = E::mma(kfr, qf[0][ks], s[0]);
      s[1] = E::mma(kfr, qf[1][ks], s[1]);
    }
  };
  // O^T += V^T P^T of one 32-key tile for both blocks (csrc/ring_attention.cu:609): each V^T fragment feeds two MFMAs
  auto pv = [&](int vbytes, const s16x8 (&p)[2][2]) {
    const unsigned char* vs_lds = smem + vbytes;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const unsigned char* vrow = vs_lds + 16 * t2 * ROWB;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + voff[db]));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vrow + 8 * ROWB + voff[db]));
        const s16x8 vfr = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        oacc[0][db] = E::mma(vfr, p[0][t2], oacc[0][db]);
        oacc[1][db] = E::mma(vfr, p[1][t2], oacc[1][db]);
      }
    }
  };
  // P^T = exp2(S^T k2 - m k2): row sum from the unrounded values (csrc/ring_attention.cu:242), MFMA operands
  // rounded to the storage type (:604)
  auto exps = [&](const f32x16 (&s)[2], s16x8 (&p)[2][2]) {
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        typename E::vec8 pv8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(s[b][8 * t2 + e], a.scale_log2, -ms[b]));
          ls[b][e & 3] += pe;
          pv8[e] = (typename E::type)pe;
        }
        p[b][t2] = __builtin_bit_cast(s16x8, pv8);
      }
  };
  // max(m, row max of the tile): two chains of v_max3_f32, one exchange between the halves of the wave
  auto tile_max = [&](const f32x16& s, float mb) {
    float m0 = mb, m1 = mb;
#pragma unroll
    for (int e = 0; e < 16; e += 4) {
      m0 = fmaxf(fmaxf(m0, s[e]), s[e + 1]);
      m1 = fmaxf(fmaxf(m1, s[e + 2]), s[e + 3]);
    }
    return cross_half_max(fmaxf(m0, m1));
  };
  // causal mask of flattened tile t (a tile of the diagonal chunk): key visible iff key_local <= query_local + diag_off
  auto mask_tile = [&](f32x16 (&s)[2], int t) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int lim = diag_rows + 64 * wave + 32 * b + n - (t - diag_base) * BN - 4 * h;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int key = 8 * (e >> 2) + (e & 3);
        if (key > lim) s[b][e] = -INFINITY;
      }
    }
  };
  // End of an iteration, seldom taken.  First the rescale of acc-O that was decided an iteration ago (the
  // probabilities computed against the old reference are all in by now); then, if some row's cand = max(m, tile max)
  // is far above its reference (or the reference is unset), the move of csrc/ring_attention.cu:226-232: l at once,
  // acc-O after the next iteration.
  auto settle = [&](bool far_any) {
    if (pend) {
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[b][db] *= apend[b];
      pend = false;
    }
    if (far_any) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const float cs = (cand[b] == -INFINITY) ? 0.f : cand[b] * a.scale_log2;
        const float alpha = __builtin_amdgcn_exp2f(m[b] * a.scale_log2 - cs);
#pragma unroll
        for (int i = 0; i < 4; ++i) ls[b][i] *= alpha;
        apend[b] = alpha;
        m[b] = cand[b];
        ms[b] = cs;
      }
      pend = true;
    }
  };
  auto far_now = [&]() {
    const bool far = (cand[0] - m[0]) * a.scale_log2 > kLazyLog2 || (cand[1] - m[1]) * a.scale_log2 > kLazyLog2;
    return __builtin_amdgcn_ballot_w64(far) != 0;
  };
  // the barrier of a pair of iterations: every wave's loads of four and more iterations ago have landed (each
  // iteration issues two tiles: 2 PIECES loads); the loads of the last three stay in flight
  auto ring_barrier = [&]() {
    if (PIECES == 2) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    __syncthreads();
  };

  // ---- any iteration: u from 0 to N; products and loads that fall outside the sequence (or outside this wave's
  // share of the diagonal chunk) are left out, tiles of the diagonal chunk are masked
  auto general = [&](int u) {
    if ((u & 1) == 0) {
      ring_barrier();
      issue_k((u + 7) & 7);
      issue_k(u & 7);
    } else {
      issue_v((u + 4) & 7);
      issue_v((u + 5) & 7);
    }
    const bool do_qk = u + 1 < Ew, do_sm = u < Ew, do_pv = u >= 1 && u - 1 < Ew;
    f32x16 snext[2];
    s16x8 pf[2][2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      snext[b] = sacc[b];
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) pf[b][t2] = pprev[b][t2];
    }
    if (do_pv) pv((NBUF + ((u - 1) & 7)) * TILE, pprev);
    if (do_sm) exps(sacc, pf);
    if (do_qk) {
      qk(((u + 1) & 7) * TILE, snext);
      if (u + 1 >= Mw) mask_tile(snext, u + 1);
      cand[0] = tile_max(snext[0], m[0]);
      cand[1] = tile_max(snext[1], m[1]);
    }
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      sacc[b] = snext[b];
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) pprev[b][t2] = pf[b][t2];
    }
    const bool far_any = do_qk && far_now();
    if (far_any || pend) settle(far_any);
  };

  // ---- prologue: K(0) .. K(6) and V(0) .. V(4) next to the Q loads; the scores of tile 0.  V ring slot 7 -- "tile
  // -1", which the first iteration multiplies with all-zero probabilities -- is cleared.
  if (first > 0) __syncthreads();  // every wave is done with the rings and the chunk list of the pass before
  for (int t = 0; t < 7; ++t) issue_k(t);
  for (int t = 0; t < 5; ++t) issue_v(t);
  if (tid < n_items + 4) {  // the chunk list the hand-scheduled loop steps its load streams through
    unsigned o;
    int c;
    chunk_of(tid, o, c);
    *(int2*)(smem + kListAt + 8 * tid) = int2{(int)o, c};
  }
  {
    f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < TILE / 4096; ++j) *(f32x4*)(smem + (NBUF + 7) * TILE + tid * (TILE / 256) + 16 * j) = zero;
  }
  __builtin_amdgcn_s_waitcnt(0);  // retire the Q loads with a wait the compiler can see (and the tiles)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (Ew > 0) {
    qk(0, sacc);
    if (0 >= Mw) mask_tile(sacc, 0);
    cand[0] = tile_max(sacc[0], m[0]);
    cand[1] = tile_max(sacc[1], m[1]);
    settle(far_now());
    // acc-O is still zero: the rescale that the first reference leaves pending is void
    pend = false;
  }

  // LDS addresses for the hand-scheduled loop: fragment offsets from the start of LDS, and where this wave's two
  // tile pieces go in ring slot 0 of K and of V
  int koff_a[KS], voff_a[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff_a[ks] = koff[ks] + (int)smem_base;
#pragma unroll
  for (int db = 0; db < DB; ++db) voff_a[db] = voff[db] + (int)smem_base + NBUF * TILE;  // from the start of the V ring
  const unsigned lds_dst_k = __builtin_amdgcn_readfirstlane(smem_base + PIECES * wave * 1024);
  const unsigned lds_dst_v = lds_dst_k + NBUF * TILE;
  auto uni = [](unsigned x) { return (unsigned)__builtin_amdgcn_readfirstlane((int)x); };
  const unsigned kh_lo = uni((unsigned)(uintptr_t)k_head), kh_hi = uni((unsigned)((uintptr_t)k_head >> 32));
  const unsigned vh_lo = uni((unsigned)(uintptr_t)v_head), vh_hi = uni((unsigned)((uintptr_t)v_head >> 32));
  const unsigned k2_bits = uni(__builtin_bit_cast(unsigned, a.scale_log2));

  // The hand-scheduled loop (ringattn_walk64_loop.inc) runs all iterations of the workgroup, 0 to N: every iteration
  // whose score tile u+1 this wave computes -- masking the tiles of the diagonal chunk that need it --, the wave's last
  // two iterations, and then only the wave's share of the loads and the barriers.  A wave with no second score tile
  // walks the iterations in plain code.
  if (1 < Ew) {
    const int u = 0;  // where the loop starts
    unsigned asm_u = 0, asm_far = 0;
    const unsigned asm_stop = uni((unsigned)(Ew - 1)), asm_mw1 = uni((unsigned)(Mw - 1));
    int vlim[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) vlim[b] = diag_rows + 64 * wave + 32 * b + n - 4 * h - (u + 1 - diag_base) * BN;
    const uint64_t kp = (uint64_t)(uintptr_t)k_head + kst.off, vp = (uint64_t)(uintptr_t)v_head + vst.off;
    unsigned k_lo = uni((unsigned)kp), k_hi = uni((unsigned)(kp >> 32)), v_lo = uni((unsigned)vp), v_hi = uni((unsigned)(vp >> 32));
    unsigned k_left = uni((unsigned)kst.left), v_left = uni((unsigned)vst.left);
    unsigned k_next = uni(smem_base + kListAt + 8 * (kst.idx + 1)), v_next = uni(smem_base + kListAt + 8 * (vst.idx + 1));
    const unsigned asm_n = uni((unsigned)N);
    if constexpr (D == 128) {
#include "ringattn_walk64_loop.inc"
    } else {
#include "ringattn_walk64_loop_d64.inc"
    }
  } else {
    for (int u = 0; u <= N; ++u) general(u);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (pend) settle(false);

  if (KEEP) {
    // ---- the rows' result: the reference's epilogue (csrc/ring_attention.cu:621-664), O = acc / l in the storage
    // type, plus the LSE
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float l = cross_half_sum((ls[b][0] + ls[b][1]) + (ls[b][2] + ls[b][3]));
      const float inv = (l > 0.f) ? 1.f / l : 0.f;
      const int row_l = qt * BM + 64 * wave + 32 * b + n;
      if (row_l < q_len) {  // not a row beyond the query range
        const int64_t row = (int64_t)bh * a.S + q_start + row_l;
        typename E::type* orow = (typename E::type*)a.out + row * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            typename E::vec4 val;
#pragma unroll
            for (int e = 0; e < 4; ++e) val[e] = (typename E::type)(oacc[b][db][4 * q4 + e] * inv);
            *(typename E::vec4*)(orow + 32 * db + 8 * q4 + 4 * h) = val;
          }
        if (h == 0 && a.lse) a.lse[row] = (l > 0.f) ? (ms[b] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
      }
    }
  } else {
    // ---- the chunk's partial (csrc/ring_attention.cu:621-633): normalised O and LSE at the rows of the queries
    const SegItem* w = item_at(0);
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float l = cross_half_sum((ls[b][0] + ls[b][1]) + (ls[b][2] + ls[b][3]));
      const float inv = (l > 0.f) ? 1.f / l : 0.f;
      const int row_l = qt * BM + 64 * wave + 32 * b + n;
      if (row_l < q_len) {
        int64_t prow = w->part_base + (int64_t)bh * w->part_bh_stride + row_l;
        if (w->part_row_mul > 0) prow = prow * w->part_row_mul + w->slot;  // a row's steps next to each other
        const int64_t opos = prow * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            f32x4 val;
#pragma unroll
            for (int e = 0; e < 4; ++e) val[e] = oacc[b][db][4 * q4 + e] * inv;
            if (HP) {  // fp16 partials: |O_part| <= max |V|, the caller vouches that this fits
              f16x4 hv;
#pragma unroll
              for (int e = 0; e < 4; ++e) hv[e] = (_Float16)val[e];
              *(f16x4*)((_Float16*)a.o_part + opos + 32 * db + 8 * q4 + 4 * h) = hv;
            } else {
              *(f32x4*)((float*)a.o_part + opos + 32 * db + 8 * q4 + 4 * h) = val;
            }
          }
        if (h == 0) a.lse_part[prow] = (l > 0.f) ? (ms[b] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f : -INFINITY;
      }
    }
  }
  }  // passes
  if constexpr (!KEEP) {
    if (a.mode == kBlockPartialsMerged) {  // this workgroup's rows over the partials it has just written
      if (all_items <= kStagedMergeMaxParts)
        merge_rows_staged<DT, HP>(a, seg, bh, qt, smem, smem_base);
      else
        merge_job_rows<DT, D, HP, BM, 64 * WAVES>(a.o_part, a.lse_part, a.out, a.lse, a.items, seg, bh, qt, a.S,
                                                  (lds_float*)(__attribute__((address_space(3))) void*)smem);
    }
  }
}

hipError_t launch_walk64(const BlockArgs& a, int dtype, int dim, hipStream_t stream) {
  if (a.n_segs <= 0) return hipSuccess;
  const int q_tiles = a.q_tiles_max;
  const int64_t groups = (int64_t)a.n_segs * a.BH;
  const int64_t blocks = (a.groups ? (int64_t)a.groups_per_xcd : (groups + 7) / 8) * 8 * q_tiles;
  if (q_tiles <= 0 || blocks > INT32_MAX) return hipErrorInvalidValue;
  if (a.mode != kBlockCarryState && a.mode != kBlockPartials && a.mode != kBlockPartialsMerged) return hipErrorInvalidValue;
  if (dtype != 0 && dtype != 1) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)blocks;
  if (dim == 64) {  // state carried only
    if (a.mode != kBlockCarryState) return hipErrorInvalidValue;
    if (dtype == 0) ring_walk64_kernel<0, 64, true, false><<<grid, 256, 0, stream>>>(a);
    else ring_walk64_kernel<1, 64, true, false><<<grid, 256, 0, stream>>>(a);
    return hipGetLastError();
  }
  if (dim != 128) return hipErrorInvalidValue;
#define RA_LAUNCH_WALK64(DT_)                                                                            \
  do {                                                                                                  \
    if (a.mode == kBlockCarryState) ring_walk64_kernel<DT_, 128, true, false><<<grid, 256, 0, stream>>>(a);  \
    else if (a.half_partials) ring_walk64_kernel<DT_, 128, false, true><<<grid, 256, 0, stream>>>(a);        \
    else ring_walk64_kernel<DT_, 128, false, false><<<grid, 256, 0, stream>>>(a);                            \
  } while (0)
  if (dtype == 0) RA_LAUNCH_WALK64(0);
  else RA_LAUNCH_WALK64(1);
#undef RA_LAUNCH_WALK64
  return hipGetLastError();
}

}  // namespace ringattn
