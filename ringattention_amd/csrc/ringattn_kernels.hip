// gfx950 (CDNA4) kernels around the attention kernel (ring_walk_kernel, ringattn_walk.hip).
//
//   merge_kernel : P-way merge of per-step (O, LSE) partials over row ranges.  The reference
//       has no such function: it carries (max, sum, acc-O) in registers across ring steps
//       (csrc/ring_attention.cu:439-443,597).  The merge is the algebraic equivalent on
//       (O, LSE) pairs (:207-245,621-633).
//   write_table_kernel : a segment + item table from kernel arguments to device memory, for
//       callers that may not copy from the host.
#include "ringattn_device.h"

#include <type_traits>


namespace ringattn {

// ---- merge of one row: the merge kernel's arithmetic (the attention kernel's merge at the end of a workgroup follows it) -------
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

// ---- merge ------------------------------------------------------------------------
template <int DT, int D, bool HP>
__global__ __launch_bounds__(256) void merge_kernel(const MergeArgs a) {
  constexpr int TPR = D / 8;  // threads per row, 8 columns each
  constexpr int ROWS = 256 / TPR;
  const MergeRegion reg = a.regions ? a.regions[blockIdx.y] : a.single;
  const int64_t idx = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;  // over heads x reg.len
  if (idx >= (int64_t)a.heads * reg.len) return;
  const int64_t row = (idx / reg.len) * a.S + reg.start + idx % reg.len;
  // slot-major partials: slot s of a row lies part_stride_rows rows further on; row-major: at entry row_mul row + s
  SlotParts parts{reg.active, a.row_mul > 0 ? row * a.row_mul : row, a.row_mul > 0 ? (int64_t)1 : a.part_stride_rows};
  merge_row<DT, D, HP>(parts, a.o_parts, a.lse_parts, a.out, a.lse, row, threadIdx.x % TPR);
}

// ---- segment + item table from kernel arguments -------------------------------------
__global__ __launch_bounds__(64) void write_table_kernel(const TablePack pack, int n, Segment* seg_dst, SegItem* item_dst) {
  const int i = threadIdx.x;
  if (i < n) item_dst[i] = pack.items[i];
  if (i == 0) *seg_dst = pack.seg;
}

// ---- host launchers -----------------------------------------------------------------
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
