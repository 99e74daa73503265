/*
 * CPU oracle for ring-attention forward.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg may load it.  The product path
 * (ringattention_amd/) must never link, import or call anything in here.
 *
 * What it restates (all citations are into the reference tree):
 *   - the attention math of csrc/self_attention.py:22-26 (scores = Q K^T,
 *     softmax over keys, output = weights V), evaluated per query row in
 *     fp64 on the widened fp16/bf16 inputs, with the conventions the build
 *     adds on top: logits scaled by softmax_scale, base-e softmax, optional
 *     causal mask on GLOBAL token indices, and the natural-log LSE per row;
 *   - the online-softmax recurrence of csrc/ring_attention.cu:194-245
 *     (running max, rescale of the running sum and of acc-O, sum taken from
 *     the unrounded probabilities) together with its guards at :183 and :626
 *     and the final 1/sum normalisation at :621-633 -- completed with the
 *     `sum += sum_cur` tail that is missing from the truncated reference;
 *   - the ring visiting order of csrc/ring_attention.cu:456-470,531,611-619:
 *     at step s rank r works on KV chunk (r + s) mod P;
 *   - the cross-step merge, which has no function in the reference: it is the
 *     algebraic equivalent of carrying (max, sum, acc-O) across steps
 *     (csrc/ring_attention.cu:439-443,597) expressed on (O, LSE) partials.
 *
 * Parity status: the reference ships no test vector, fixture or assertion for
 * this path, and its kernel source is truncated and cannot be built
 * (csrc/ring_attention.cu:244-248), so no function here is pinned by the
 * reference's own tests.  Every function is pinned instead by
 * tests/test_oracle.py against independent routines (torch CPU fp64
 * matmul/softmax, scipy logsumexp), closed forms (Q = 0, constant V, causal
 * row 0, a dominant key), brute force on tiny shapes and algebraic invariants
 * (order independence of the ring, merge identity/commutativity); the causal
 * ring partials step by step, a block partial with a shifted diagonal and the
 * rounded-probability form against scipy softmax / logsumexp on explicitly
 * masked scores.
 *
 * Build: gcc -O3 -fopenmp -shared -fPIC (see oracle/build.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_FP16 0
#define ORACLE_BF16 1

/* ---- 16-bit storage types -------------------------------------------------- */

static float half_bits_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static float bf16_bits_to_float(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

float oracle_to_float(uint16_t bits, int dtype) {
  return dtype == ORACLE_BF16 ? bf16_bits_to_float(bits) : half_bits_to_float(bits);
}

/* Round-to-nearest-even of a double into the 16-bit storage type
 * (csrc/ring_attention.cu:249-258 uses round-to-nearest for the fp16 store).
 * Goes through float first only when that is exact for the purpose: a double
 * rounded to float and then to 16 bits can double-round, so do it directly. */
static uint16_t double_to_bf16_bits(double x) {
  if (isnan(x)) return 0x7fc0u;
  float f = (float)x; /* candidate; fix double rounding below */
  uint32_t u;
  memcpy(&u, &f, 4);
  /* neighbours on the bf16 grid around x */
  uint32_t lo = u & 0xffff0000u;
  float flo;
  memcpy(&flo, &lo, 4);
  if ((double)flo == x) return (uint16_t)(lo >> 16);
  if (isinf(f)) return (uint16_t)(u >> 16);
  /* flo is toward zero from f; make [a, b] bracket x in magnitude */
  uint32_t hi = lo + 0x10000u;
  float fhi;
  memcpy(&fhi, &hi, 4);
  double ax = fabs(x), a = fabs((double)flo), b = fabs((double)fhi);
  if (ax < a) { /* float rounding moved f up across a bf16 grid point */
    hi = lo; lo = lo - 0x10000u;
    memcpy(&flo, &lo, 4); memcpy(&fhi, &hi, 4);
    a = fabs((double)flo); b = fabs((double)fhi);
  }
  double da = ax - a, db = b - ax;
  if (da < db) return (uint16_t)(lo >> 16);
  if (db < da) return (uint16_t)(hi >> 16);
  return (uint16_t)(((lo >> 16) & 1u) ? (hi >> 16) : (lo >> 16));
}

static uint16_t double_to_half_bits(double x) {
  if (isnan(x)) return 0x7e00u;
  uint16_t sign = signbit(x) ? 0x8000u : 0;
  double ax = fabs(x);
  if (ax >= 65520.0) return sign | 0x7c00u; /* rounds to inf */
  if (ax < 5.9604644775390625e-08 * 0.5) return sign; /* below half the least subnormal */
  int e;
  (void)frexp(ax, &e); /* ax = m * 2^e, m in [0.5,1) -> exponent of leading bit is e-1 */
  int lead = e - 1;
  if (lead < -14) lead = -14; /* subnormal grid spacing 2^-24 */
  double ulp = ldexp(1.0, lead - 10);
  double q = ax / ulp; /* exact: power-of-two scaling */
  double fl = floor(q);
  double r = q - fl;
  if (r > 0.5 || (r == 0.5 && fmod(fl, 2.0) == 1.0)) fl += 1.0;
  double y = fl * ulp;
  /* encode y (exactly representable) */
  if (y >= 65536.0) return sign | 0x7c00u;
  if (y < 6.103515625e-05) { /* subnormal */
    return sign | (uint16_t)(y / 5.9604644775390625e-08);
  }
  (void)frexp(y, &e);
  int ex = e - 1;
  uint32_t man = (uint32_t)(y / ldexp(1.0, ex - 10)) - 1024u;
  return sign | (uint16_t)((ex + 15) << 10) | (uint16_t)man;
}

uint16_t oracle_from_double(double x, int dtype) {
  return dtype == ORACLE_BF16 ? double_to_bf16_bits(x) : double_to_half_bits(x);
}

void oracle_round_array(const double* src, uint16_t* dst, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; ++i) dst[i] = oracle_from_double(src[i], dtype);
}

void oracle_widen_array(const uint16_t* src, double* dst, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; ++i) dst[i] = (double)oracle_to_float(src[i], dtype);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- direct form --------------------------------------------------------------
 * One query row against keys [0, nkeys): csrc/self_attention.py:22-26 with the
 * scale and LSE added.  kf/vf are float-widened [S, d] slabs of one head.
 * Two passes (max, then sums) so nothing depends on a running rescale. */
static void direct_row(const float* q, const float* kf, const float* vf, int d, int64_t nkeys,
                       double scale, double* sbuf, double* o, double* lse) {
  double m = -INFINITY;
  for (int64_t t = 0; t < nkeys; ++t) {
    const float* kr = kf + t * d;
    double acc = 0.0;
    for (int c = 0; c < d; ++c) acc += (double)q[c] * (double)kr[c];
    acc *= scale;
    sbuf[t] = acc;
    if (acc > m) m = acc;
  }
  for (int c = 0; c < d; ++c) o[c] = 0.0;
  if (nkeys == 0) { *lse = -INFINITY; return; }
  double l = 0.0;
  for (int64_t t = 0; t < nkeys; ++t) {
    double p = exp(sbuf[t] - m);
    l += p;
    const float* vr = vf + t * d;
    for (int c = 0; c < d; ++c) o[c] += p * (double)vr[c];
  }
  for (int c = 0; c < d; ++c) o[c] /= l;
  *lse = m + log(l);
}

/*
 * Direct attention for selected rows.
 *   q, k, v : [B, H, S, d] storage-dtype bits (fp16 or bf16), contiguous
 *   rows    : nrows flat indices into [B*H*S] (row = (b*H + h)*S + i), or NULL
 *             for all rows in order (then nrows must be B*H*S)
 *   o_out   : [nrows, d] fp64,  lse_out : [nrows] fp64
 * causal: query i sees keys t <= i (global indices).
 * Returns 0, or -1 on bad arguments / allocation failure.
 */
int oracle_attention_rows(const uint16_t* q, const uint16_t* k, const uint16_t* v, int dtype,
                          int B, int H, int64_t S, int d, double scale, int causal,
                          const int64_t* rows, int64_t nrows, double* o_out, double* lse_out) {
  if (!q || !k || !v || !o_out || !lse_out || B <= 0 || H <= 0 || S <= 0 || d <= 0) return -1;
  const int64_t BH = (int64_t)B * H;
  if (!rows && nrows != BH * S) return -1;
  /* group rows by head so K/V are widened once per head: sort an index array by head */
  int64_t* order = (int64_t*)malloc(sizeof(int64_t) * (size_t)(nrows > 0 ? nrows : 1));
  int64_t* head_start = (int64_t*)calloc((size_t)BH + 1, sizeof(int64_t));
  if (!order || !head_start) { free(order); free(head_start); return -1; }
  for (int64_t r = 0; r < nrows; ++r) {
    int64_t fr = rows ? rows[r] : r;
    if (fr < 0 || fr >= BH * S) { free(order); free(head_start); return -1; }
    head_start[fr / S + 1]++;
  }
  for (int64_t g = 0; g < BH; ++g) head_start[g + 1] += head_start[g];
  {
    int64_t* fill = (int64_t*)malloc(sizeof(int64_t) * (size_t)BH);
    if (!fill) { free(order); free(head_start); return -1; }
    memcpy(fill, head_start, sizeof(int64_t) * (size_t)BH);
    for (int64_t r = 0; r < nrows; ++r) {
      int64_t fr = rows ? rows[r] : r;
      order[fill[fr / S]++] = r;
    }
    free(fill);
  }
  float* kf = (float*)malloc(sizeof(float) * (size_t)(S * d));
  float* vf = (float*)malloc(sizeof(float) * (size_t)(S * d));
  if (!kf || !vf) { free(order); free(head_start); free(kf); free(vf); return -1; }
  int rc = 0;
  for (int64_t g = 0; g < BH; ++g) {
    int64_t n0 = head_start[g], n1 = head_start[g + 1];
    if (n0 == n1) continue;
    const uint16_t* kh = k + g * S * d;
    const uint16_t* vh = v + g * S * d;
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < S * d; ++e) {
      kf[e] = oracle_to_float(kh[e], dtype);
      vf[e] = oracle_to_float(vh[e], dtype);
    }
#pragma omp parallel
    {
      double* sbuf = (double*)malloc(sizeof(double) * (size_t)S);
      float* qf = (float*)malloc(sizeof(float) * (size_t)d);
      if (!sbuf || !qf) {
#pragma omp atomic write
        rc = -1;
      } else {
#pragma omp for schedule(dynamic, 4)
        for (int64_t x = n0; x < n1; ++x) {
          int64_t r = order[x];
          int64_t fr = rows ? rows[r] : r;
          int64_t i = fr % S;
          const uint16_t* qr = q + fr * d;
          for (int c = 0; c < d; ++c) qf[c] = oracle_to_float(qr[c], dtype);
          int64_t nkeys = causal ? i + 1 : S;
          direct_row(qf, kf, vf, d, nkeys, scale, sbuf, o_out + r * d, lse_out + r);
        }
      }
      free(sbuf);
      free(qf);
    }
  }
  free(order); free(head_start); free(kf); free(vf);
  return rc;
}

/* ---- blockwise / ring form ------------------------------------------------------
 * Online softmax over key tiles for one query row against one KV chunk:
 * csrc/ring_attention.cu:194-245 (+ the missing `sum += sum_cur`), guards
 * :183 (max == -inf -> p = 0) and :626 (sum == 0 -> no divide).
 *   nvis      : number of visible keys of this chunk for this row (prefix)
 *   tile      : keys per tile (the reference uses 64, csrc/ring_attention.cu:708)
 *   round_p   : if non-zero, probabilities are rounded to the storage dtype
 *               before the PV product (csrc/ring_attention.cu:604) while the
 *               row sum keeps the unrounded values (:242)
 * Outputs the normalised partial O (fp64) and LSE = m + ln(l), -inf if nvis == 0.
 */
static void online_row(const float* q, const float* kf, const float* vf, int d, int64_t nvis,
                       int tile, double scale, int round_p, int dtype, double* pbuf,
                       double* o, double* lse) {
  double m = -INFINITY, l = 0.0;
  for (int c = 0; c < d; ++c) o[c] = 0.0;
  for (int64_t t0 = 0; t0 < nvis; t0 += tile) {
    int64_t t1 = t0 + tile < nvis ? t0 + tile : nvis;
    double mt = -INFINITY;
    for (int64_t t = t0; t < t1; ++t) {
      const float* kr = kf + t * d;
      double acc = 0.0;
      for (int c = 0; c < d; ++c) acc += (double)q[c] * (double)kr[c];
      acc *= scale;
      pbuf[t - t0] = acc;
      if (acc > mt) mt = acc;
    }
    double mn = mt > m ? mt : m;
    double alpha = (m == -INFINITY) ? 0.0 : exp(m - mn);
    l *= alpha;
    for (int c = 0; c < d; ++c) o[c] *= alpha;
    for (int64_t t = t0; t < t1; ++t) {
      double p = (mn == -INFINITY) ? 0.0 : exp(pbuf[t - t0] - mn);
      l += p;
      if (round_p) p = (double)oracle_to_float(oracle_from_double(p, dtype), dtype);
      const float* vr = vf + t * d;
      for (int c = 0; c < d; ++c) o[c] += p * (double)vr[c];
    }
    m = mn;
  }
  if (l == 0.0 || l != l) {
    *lse = -INFINITY;
  } else {
    for (int c = 0; c < d; ++c) o[c] /= l;
    *lse = m + log(l);
  }
}

/* Merge of n (O, LSE) partials of one row.  L = logsumexp(L_s); O = sum exp(L_s - L) O_s.
 * A partial with LSE = -inf is the identity element.  All fp64. */
void oracle_merge_row(const double* o_parts, const double* lse_parts, int n, int d, double* o, double* lse) {
  double mx = -INFINITY;
  for (int s = 0; s < n; ++s) if (lse_parts[s] > mx) mx = lse_parts[s];
  for (int c = 0; c < d; ++c) o[c] = 0.0;
  if (mx == -INFINITY) { *lse = -INFINITY; return; }
  double sum = 0.0;
  for (int s = 0; s < n; ++s) sum += exp(lse_parts[s] - mx);
  double L = mx + log(sum);
  for (int s = 0; s < n; ++s) {
    if (lse_parts[s] == -INFINITY) continue;
    double w = exp(lse_parts[s] - L);
    for (int c = 0; c < d; ++c) o[c] += w * o_parts[(int64_t)s * d + c];
  }
  *lse = L;
}

/* n-way merge over arrays: o_parts [n, rows, d], lse_parts [n, rows] -> o [rows, d], lse [rows]. */
int oracle_merge(const double* o_parts, const double* lse_parts, int n, int64_t rows, int d,
                 double* o, double* lse) {
  if (!o_parts || !lse_parts || !o || !lse || n <= 0 || rows < 0 || d <= 0) return -1;
  int rc = 0;
#pragma omp parallel
  {
    double* op = (double*)malloc(sizeof(double) * (size_t)n * d);
    double* lp = (double*)malloc(sizeof(double) * (size_t)n);
    if (!op || !lp) {
#pragma omp atomic write
      rc = -1;
    } else {
#pragma omp for schedule(static)
      for (int64_t r = 0; r < rows; ++r) {
        for (int s = 0; s < n; ++s) {
          memcpy(op + (int64_t)s * d, o_parts + ((int64_t)s * rows + r) * d, sizeof(double) * (size_t)d);
          lp[s] = lse_parts[(int64_t)s * rows + r];
        }
        oracle_merge_row(op, lp, n, d, o + r * d, lse + r);
      }
    }
    free(op);
    free(lp);
  }
  return rc;
}

/*
 * One (Q chunk, KV chunk) block: partial O and LSE of every row of the Q chunk
 * against the KV chunk.  q [cq, d], k, v [ck, d] storage bits for ONE head.
 *   mask_mode 0: every key visible; 1: local causal, key t visible to row i
 *   iff t <= i + diag_offset (diag_offset = 0 for equal chunks on the diagonal).
 * o_part [cq, d] fp64, lse_part [cq] fp64.
 */
int oracle_block_partial(const uint16_t* q, const uint16_t* k, const uint16_t* v, int dtype,
                         int64_t cq, int64_t ck, int d, double scale, int mask_mode,
                         int64_t diag_offset, int tile, int round_p,
                         double* o_part, double* lse_part) {
  if (!q || !k || !v || !o_part || !lse_part || cq <= 0 || ck <= 0 || d <= 0 || tile <= 0) return -1;
  float* kf = (float*)malloc(sizeof(float) * (size_t)(ck * d));
  float* vf = (float*)malloc(sizeof(float) * (size_t)(ck * d));
  if (!kf || !vf) { free(kf); free(vf); return -1; }
  for (int64_t e = 0; e < ck * d; ++e) { kf[e] = oracle_to_float(k[e], dtype); vf[e] = oracle_to_float(v[e], dtype); }
  int rc = 0;
#pragma omp parallel
  {
    double* pbuf = (double*)malloc(sizeof(double) * (size_t)tile);
    float* qf = (float*)malloc(sizeof(float) * (size_t)d);
    if (!pbuf || !qf) {
#pragma omp atomic write
      rc = -1;
    } else {
#pragma omp for schedule(dynamic, 8)
      for (int64_t i = 0; i < cq; ++i) {
        for (int c = 0; c < d; ++c) qf[c] = oracle_to_float(q[i * d + c], dtype);
        int64_t nvis = ck;
        if (mask_mode == 1) {
          nvis = i + diag_offset + 1;
          if (nvis < 0) nvis = 0;
          if (nvis > ck) nvis = ck;
        }
        online_row(qf, kf, vf, d, nvis, tile, scale, round_p, dtype, pbuf, o_part + i * d, lse_part + i);
      }
    }
    free(pbuf);
    free(qf);
  }
  free(kf); free(vf);
  return rc;
}

/*
 * Ring form for selected rows: P virtual ranks, chunk lengths seqlen[0..P) (sum = S),
 * chunks in sequence order.  For the row's rank r, steps s = 0..P-1 visit KV chunk
 * j = (r + s) mod P (csrc/ring_attention.cu:463,531,615); causal: j < r full,
 * j == r lower-triangular on local indices, j > r skipped.  Each visited chunk yields
 * a partial (O, LSE) by the online recurrence; partials are merged in visiting order.
 * `order` (may be NULL) overrides the visiting order: order[s] is the step executed
 * s-th -- used to test that the result does not depend on the ring order.
 * parts_o / parts_lse (may be NULL): per-step partials [nrows, P, d] / [nrows, P]
 * (skipped steps hold O = 0, LSE = -inf).
 */
int oracle_ring_rows(const uint16_t* q, const uint16_t* k, const uint16_t* v, int dtype,
                     int B, int H, int P, const int* seqlen, int d, double scale, int causal,
                     int tile, int round_p, const int* order,
                     const int64_t* rows, int64_t nrows,
                     double* o_out, double* lse_out, double* parts_o, double* parts_lse) {
  if (!q || !k || !v || !seqlen || !rows || !o_out || !lse_out || P <= 0 || d <= 0 || tile <= 0) return -1;
  int64_t S = 0;
  int64_t* start = (int64_t*)malloc(sizeof(int64_t) * (size_t)(P + 1));
  if (!start) return -1;
  for (int r = 0; r < P; ++r) { if (seqlen[r] <= 0) { free(start); return -1; } start[r] = S; S += seqlen[r]; }
  start[P] = S;
  const int64_t BH = (int64_t)B * H;
  int rc = 0;
#pragma omp parallel
  {
    int64_t maxc = 0;
    for (int r = 0; r < P; ++r) if (seqlen[r] > maxc) maxc = seqlen[r];
    float* kf = (float*)malloc(sizeof(float) * (size_t)(maxc * d));
    float* vf = (float*)malloc(sizeof(float) * (size_t)(maxc * d));
    float* qf = (float*)malloc(sizeof(float) * (size_t)d);
    double* pbuf = (double*)malloc(sizeof(double) * (size_t)tile);
    double* po = (double*)malloc(sizeof(double) * (size_t)P * d);
    double* pl = (double*)malloc(sizeof(double) * (size_t)P);
    if (!kf || !vf || !qf || !pbuf || !po || !pl) {
#pragma omp atomic write
      rc = -1;
    } else {
#pragma omp for schedule(dynamic, 1)
      for (int64_t x = 0; x < nrows; ++x) {
        int64_t fr = rows[x];
        if (fr < 0 || fr >= BH * S) {
#pragma omp atomic write
          rc = -1;
          continue;
        }
        int64_t g = fr / S, i = fr % S;
        int r = 0;
        while (i >= start[r + 1]) ++r;
        int64_t il = i - start[r];
        for (int c = 0; c < d; ++c) qf[c] = oracle_to_float(q[fr * d + c], dtype);
        for (int s = 0; s < P; ++s) {
          int step = order ? order[s] : s;
          int j = (r + step) % P;
          int64_t ck = seqlen[j];
          int64_t nvis = ck;
          if (causal) {
            if (j > r) nvis = 0;
            else if (j == r) nvis = il + 1;
          }
          double* os = po + (int64_t)s * d;
          if (nvis == 0) {
            for (int c = 0; c < d; ++c) os[c] = 0.0;
            pl[s] = -INFINITY;
          } else {
            const uint16_t* kc = k + (g * S + start[j]) * d;
            const uint16_t* vc = v + (g * S + start[j]) * d;
            for (int64_t e = 0; e < nvis * d; ++e) { kf[e] = oracle_to_float(kc[e], dtype); vf[e] = oracle_to_float(vc[e], dtype); }
            online_row(qf, kf, vf, d, nvis, tile, scale, round_p, dtype, pbuf, os, &pl[s]);
          }
          if (parts_o) memcpy(parts_o + (x * P + step) * d, os, sizeof(double) * (size_t)d);
          if (parts_lse) parts_lse[x * P + step] = pl[s];
        }
        oracle_merge_row(po, pl, P, d, o_out + x * d, lse_out + x);
      }
    }
    free(kf); free(vf); free(qf); free(pbuf); free(po); free(pl);
  }
  free(start);
  return rc;
}
