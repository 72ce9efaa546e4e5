/*
 * tbe_oracle.c -- TEST INFRASTRUCTURE, NOT A PRODUCT PATH.
 *
 * Scalar CPU restatement of the reference's table-batched embedding-bag
 * arithmetic, used only as the checker in tests/, in __graft_entry__.smoke()
 * and as the cpu_baseline leg of bench.py.  Nothing in the shipped package may
 * import, link or call it.
 *
 * Every function follows the reference lines cited at its head
 * (tbe.cu = table_batched_embeddings_cuda.cu).  Arithmetic is done in the
 * reference's accumulator type: float for fp16/fp32 weights, double for fp64
 * (acc_type<scalar_t, true>), fp16 stored with round-to-nearest-even
 * (tbe.cu:62-84).  Compile with -ffp-contract=off so float expressions are
 * evaluated as written.
 *
 * Pinning (which independent check covers which function) is listed in
 * tests/test_oracle.py; in short: forward / SGD / Adagrad against
 * torch.nn.EmbeddingBag + the Python optimizer of
 * test_table_batched_embeddings.py:184-193, 296-318 (golden fixture and live),
 * approximate Adagrad against the same EmbeddingBag + Python optimizer with
 * indices drawn without replacement (test_table_batched_embeddings.py:244),
 * hand-computed repeated-row cases and a closed form for one row looked up
 * n times, sort against numpy's stable argsort, segments against numpy.unique,
 * construct_offsets against its closed form, fp16 conversion against numpy's
 * float16 over all 65536 bit patterns.  The cache model restates this
 * repository's own specification (the reference has no cache): its parity is
 * pinned only by invariants and a brute-force model, not by reference vectors.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { F32 = 0, F16 = 1, F64 = 2 };

/* ------------------------------------------------------------ fp16 <-> fp32 */
float oracle_half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: renormalise */
      int shift = 0;
      while (!(man & 0x400u)) { man <<= 1; ++shift; }
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
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

/* round-to-nearest-even, as __float22half2_rn (tbe.cu:81-82) */
uint16_t oracle_float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u | ((ax >> 13) & 0x3ffu) : 0u));
  }
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to >= 65520 -> inf */
  if (ax < 0x33000001u) return sign;                        /* < 2^-25 (or == 2^-25: tie to even 0) */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u;
  uint32_t shift, half_exp;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(e + 15);
  }
  uint32_t q = m >> shift;
  const uint32_t rem = m & ((1u << shift) - 1u);
  const uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
  /* q carries the implicit bit for normals; adding the exponent field handles mantissa overflow */
  uint32_t out;
  if (half_exp == 0) out = q; /* subnormal (q may reach 0x400 = smallest normal) */
  else out = ((half_exp - 1) << 10) + q;
  return (uint16_t)(sign | out);
}

static inline double load_elem(const void *p, int dtype, int64_t i) {
  if (dtype == F32) return ((const float *)p)[i];
  if (dtype == F16) return oracle_half_to_float(((const uint16_t *)p)[i]);
  return ((const double *)p)[i];
}
static inline float load_f(const void *p, int dtype, int64_t i) {
  return dtype == F32 ? ((const float *)p)[i] : oracle_half_to_float(((const uint16_t *)p)[i]);
}
static inline void store_f(void *p, int dtype, int64_t i, float v) {
  if (dtype == F32) ((float *)p)[i] = v;
  else ((uint16_t *)p)[i] = oracle_float_to_half(v);
}

/* -------------------------------------------------------- stochastic rounding
 * Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
 * SC'11) -- the generator behind curandStatePhilox4_32_10_t, which the reference draws its
 * rounding bits from (tbe.cu:595-599, 627-631).  cuRAND is not part of the reference tree and
 * its per-thread stream layout cannot be reproduced, so the BITS of a stochastically rounded
 * result are PARITY UNPINNED against the reference; the rounding rule itself
 * (stochastic_rounding_vector, tbe.cu:564-578: add 13 random bits to the fp32 pattern, truncate
 * toward zero) is restated exactly.  Pinned by the Random123 known-answer vectors and by
 * statistical tests (unbiased, within one fp16 ulp, exact values unchanged).
 */
void oracle_philox4x32_10(const uint32_t ctr_in[4], const uint32_t key_in[2], uint32_t out[4]) {
  uint32_t c0 = ctr_in[0], c1 = ctr_in[1], c2 = ctr_in[2], c3 = ctr_in[3];
  uint32_t k0 = key_in[0], k1 = key_in[1];
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* __float2half_rz */
static uint16_t float_to_half_rz(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
  if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7bffu); /* >= 65536: truncates to the largest finite half */
  const int32_t e = (int32_t)(ax >> 23) - 127;
  if (e < -24) return sign;
  const uint32_t m = (ax & 0x7fffffu) | 0x800000u;
  if (e < -14) return (uint16_t)(sign | (m >> (13 + (-14 - e))));
  return (uint16_t)(sign | (((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3ffu)));
}

/* one element: stochastic_rounding_vector (tbe.cu:569-576) */
uint16_t oracle_stochastic_round(float value, uint32_t random_bits) {
  uint32_t x;
  memcpy(&x, &value, 4);
  x += random_bits >> 19;
  float f;
  memcpy(&f, &x, 4);
  return float_to_half_rz(f);
}

void oracle_stochastic_round_many(const float *values, const uint32_t *random_bits, uint16_t *out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = oracle_stochastic_round(values[i], random_bits[i]);
}

/* Stores `count` (a multiple of 4) fp16 values starting at table element `element` (a multiple
 * of 4): element e takes word e % 4 of Philox(counter = {e / 4, offset}, key = seed). */
static void store_row_stochastic(uint16_t *dst, const float *values, int32_t count, int64_t element,
                                 uint64_t seed, uint64_t offset) {
  for (int32_t q = 0; q < count; q += 4) {
    const uint64_t group = (uint64_t)(element + q) / 4;
    const uint32_t ctr[4] = {(uint32_t)group, (uint32_t)(group >> 32), (uint32_t)offset, (uint32_t)(offset >> 32)};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t r[4];
    oracle_philox4x32_10(ctr, key, r);
    for (int k = 0; k < 4; ++k) dst[q + k] = oracle_stochastic_round(values[q + k], r[k]);
  }
}

/* ------------------------------------------------------------------ forward
 * batched_embedding_forward_kernel_1 (tbe.cu:193-251) with UnweightedForward /
 * WeightedForward (tbe.cu:166-191): b_t = t*B + b; serial sum over the bag in
 * index order; output[b][t][d].
 */
int oracle_forward(const void *weights, int dtype, int32_t D, const int32_t *table_offsets,
                   int32_t T, const int32_t *indices, const int32_t *offsets, int32_t B,
                   const void *psw, void *output) {
  for (int32_t b_t = 0; b_t < T * B; ++b_t) {
    const int32_t t = b_t / B, b = b_t % B;
    const int64_t table_offset = table_offsets[t];
    const int32_t start = offsets[t * B + b], end = offsets[t * B + b + 1];
    const int64_t out0 = ((int64_t)b * T + t) * D;
    for (int32_t d = 0; d < D; ++d) {
      if (dtype == F64) {
        double sum = 0;
        for (int32_t l = start; l < end; ++l) {
          const double w = ((const double *)weights)[(table_offset + indices[l]) * D + d];
          if (psw) sum += w * ((const double *)psw)[l];
          else sum += w;
        }
        ((double *)output)[out0 + d] = sum;
      } else {
        float sum = 0;
        for (int32_t l = start; l < end; ++l) {
          const float w = load_f(weights, dtype, (table_offset + indices[l]) * D + d);
          if (psw) sum += w * load_f(psw, dtype, l);
          else sum += w;
        }
        store_f(output, dtype, out0 + d, sum);
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------- linearize
 * linear_index_weight_offsets_kernel (tbe.cu:1471-1497): key = table_offset + idx,
 * info = {b_t, indices_idx} (IndexInfo, tbe.cu:1215-1218).
 */
void oracle_linearize(const int32_t *table_offsets, int32_t T, const int32_t *indices,
                      const int32_t *offsets, int32_t B, int32_t *keys, int32_t *info_b_t,
                      int32_t *info_indices_idx) {
  for (int32_t b_t = 0; b_t < T * B; ++b_t) {
    const int32_t t = b_t / B, b = b_t % B;
    const int32_t table_offset = table_offsets[t];
    const int32_t start = offsets[t * B + b], end = offsets[t * B + b + 1];
    for (int32_t i = start; i < end; ++i) {
      keys[i] = table_offset + indices[i];
      info_b_t[i] = b_t;
      info_indices_idx[i] = i;
    }
  }
}

/* --------------------------------------------------------------------- sort
 * Contract of cub::DeviceRadixSort::SortPairs(keys, values, n, begin_bit=0, end_bit)
 * as called at tbe.cu:1639-1655: ascending on key bits [0, end_bit), stable.
 * CUB is not part of the reference tree (include path in setup.py:7, no version
 * pinned); this restates its published contract as a least-significant-digit
 * counting sort.  `values` are positions (IndexInfo.indices_idx).
 */
void oracle_sort_pairs(const int32_t *keys_in, const int32_t *values_in, int32_t *keys_out,
                       int32_t *values_out, int64_t n, int32_t end_bit) {
  uint32_t *ka = (uint32_t *)malloc((size_t)(n > 0 ? n : 1) * 4);
  uint32_t *va = (uint32_t *)malloc((size_t)(n > 0 ? n : 1) * 4);
  uint32_t *kb = (uint32_t *)malloc((size_t)(n > 0 ? n : 1) * 4);
  uint32_t *vb = (uint32_t *)malloc((size_t)(n > 0 ? n : 1) * 4);
  for (int64_t i = 0; i < n; ++i) {
    ka[i] = (uint32_t)keys_in[i];
    va[i] = values_in ? (uint32_t)values_in[i] : (uint32_t)i;
  }
  for (int shift = 0; shift < end_bit; shift += 8) {
    const int bits = end_bit - shift < 8 ? end_bit - shift : 8;
    const uint32_t mask = (1u << bits) - 1u;
    int64_t count[257];
    memset(count, 0, sizeof(count));
    for (int64_t i = 0; i < n; ++i) ++count[((ka[i] >> shift) & mask) + 1];
    for (int d = 0; d < 256; ++d) count[d + 1] += count[d];
    for (int64_t i = 0; i < n; ++i) {
      const int64_t dst = count[(ka[i] >> shift) & mask]++;
      kb[dst] = ka[i];
      vb[dst] = va[i];
    }
    uint32_t *t = ka; ka = kb; kb = t;
    t = va; va = vb; vb = t;
  }
  for (int64_t i = 0; i < n; ++i) {
    keys_out[i] = (int32_t)ka[i];
    values_out[i] = (int32_t)va[i];
  }
  free(ka); free(va); free(kb); free(vb);
}

/* ----------------------------------------------------------------- segments
 * Segment-head rule and run length of batched_embedding_backward_adagrad_exact_kernel_1
 * (tbe.cu:1523-1539).  Writes segment_starts[0..U] (last = n); returns U.
 */
int64_t oracle_segments(const int32_t *keys_sorted, int64_t n, int32_t *segment_starts) {
  int64_t U = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int head = (i == 0 || keys_sorted[i - 1] != keys_sorted[i]);
    if (!head) continue;
    int64_t SL = 1;
    while (i + SL < n && keys_sorted[i + SL] == keys_sorted[i]) ++SL;
    segment_starts[U++] = (int32_t)i;
    (void)SL;
  }
  segment_starts[U] = (int32_t)n;
  return U;
}

/* ----------------------------------------------------------------- backward
 * Shared skeleton of the exact backward: linearize -> sort -> one pass per
 * segment (tbe.cu:1589-1706, kernel :1499-1587).  For each unique row:
 *   G[d] = sum over the run, in sorted (= ascending position) order, of
 *          (psw[p] *) grad_output[b][t][d]                    (tbe.cu:1548-1558)
 * optimizer 0 = exact SGD: w -= G * lr (SGDFunctor arithmetic, tbe.cu:322-330,
 *   applied once per distinct row, i.e. the semantics of the reference's own
 *   test oracle w - lr * grad, test_table_batched_embeddings.py:190-193);
 * optimizer 1 = row-wise Adagrad (AdaGradFunctor, tbe.cu:437-471):
 *   gss = sum_d G[d]^2; state = old + gss;
 *   mult = lr * (1.0 / (sqrt(old + gss) + eps)); w -= G * mult.
 * Weighted runs multiply each gradient row by psw[indices_idx] and emit
 *   grad_psw[p] = <w_before_update, grad_output[b][t]>  (WeightedAdaGradFunctor
 *   sample_weight_state, tbe.cu:529-553), which the reference's exact kernel
 *   leaves as a TODO (tbe.cu:1552, 1678-1679).
 * `total_rows` sets the sorted bit range int(log2(total_rows) + 1) (tbe.cu:1643).
 * keys_sorted / positions_sorted / segment_starts may be NULL or receive the
 * intermediate results; *num_unique receives U.  With stochastic_rounding (fp16 only) the
 * updated row is rounded by store_row_stochastic (StochasticRoundingAdaGradFunctor, tbe.cu:618-646).
 */
int oracle_backward(int optimizer, const void *grad_output, void *weights, int dtype,
                    int64_t total_rows, int32_t D, const int32_t *table_offsets, int32_t T,
                    const int32_t *indices, int64_t n, const int32_t *offsets, int32_t B,
                    const void *psw, void *optimizer_state, float lr, float eps, void *grad_psw,
                    int32_t *keys_sorted_out, int32_t *positions_sorted_out,
                    int32_t *segment_starts_out, int64_t *num_unique, int32_t stochastic_rounding,
                    uint64_t sr_seed, uint64_t sr_offset) {
  const size_t nn = (size_t)(n > 0 ? n : 1);
  int32_t *keys = (int32_t *)malloc(nn * 4), *b_ts = (int32_t *)malloc(nn * 4);
  int32_t *pos = (int32_t *)malloc(nn * 4), *keys_s = (int32_t *)malloc(nn * 4);
  int32_t *pos_s = (int32_t *)malloc(nn * 4), *seg = (int32_t *)malloc((nn + 1) * 4);
  oracle_linearize(table_offsets, T, indices, offsets, B, keys, b_ts, pos);
  const int end_bit = (int)(log2((double)total_rows) + 1);
  oracle_sort_pairs(keys, pos, keys_s, pos_s, n, end_bit);
  const int64_t U = oracle_segments(keys_s, n, seg);
  if (num_unique) *num_unique = U;
  if (keys_sorted_out) memcpy(keys_sorted_out, keys_s, (size_t)n * 4);
  if (positions_sorted_out) memcpy(positions_sorted_out, pos_s, (size_t)n * 4);
  if (segment_starts_out) memcpy(segment_starts_out, seg, (size_t)(U + 1) * 4);

  double *Gd = (double *)malloc((size_t)D * 8);
  float *Gf = (float *)malloc((size_t)D * 4);
  for (int64_t u = 0; u < U; ++u) {
    const int32_t s0 = seg[u], s1 = seg[u + 1];
    const int64_t row = keys_s[s0]; /* == table_offset + idx (tbe.cu:1544-1545, 1583) */
    if (dtype == F64) {
      for (int32_t d = 0; d < D; ++d) Gd[d] = 0;
      for (int32_t i = s0; i < s1; ++i) {
        const int32_t p = pos_s[i], b_t = b_ts[p];
        const int32_t t = b_t / B, b = b_t % B;
        const double *g = (const double *)grad_output + ((int64_t)b * T + t) * D;
        const double *w = (const double *)weights + row * D;
        if (psw) {
          double dot = 0;
          for (int32_t d = 0; d < D; ++d) dot += w[d] * g[d];
          ((double *)grad_psw)[p] = dot;
          const double pw = ((const double *)psw)[p];
          for (int32_t d = 0; d < D; ++d) Gd[d] += g[d] * pw;
        } else {
          for (int32_t d = 0; d < D; ++d) Gd[d] += g[d];
        }
      }
      double mult = lr;
      if (optimizer == 1) {
        double gss = 0;
        for (int32_t d = 0; d < D; ++d) gss += Gd[d] * Gd[d];
        double *st = (double *)optimizer_state + row;
        const double old = *st;
        *st = old + gss;
        mult = lr * (1.0 / (sqrt(old + gss) + eps));
      }
      double *w = (double *)weights + row * D;
      for (int32_t d = 0; d < D; ++d) w[d] -= Gd[d] * mult;
    } else {
      for (int32_t d = 0; d < D; ++d) Gf[d] = 0;
      for (int32_t i = s0; i < s1; ++i) {
        const int32_t p = pos_s[i], b_t = b_ts[p];
        const int32_t t = b_t / B, b = b_t % B;
        const int64_t g0 = ((int64_t)b * T + t) * D;
        if (psw) {
          float dot = 0;
          for (int32_t d = 0; d < D; ++d)
            dot += load_f(weights, dtype, row * D + d) * load_f(grad_output, dtype, g0 + d);
          store_f(grad_psw, dtype, p, dot);
          const float pw = load_f(psw, dtype, p);
          for (int32_t d = 0; d < D; ++d) Gf[d] += load_f(grad_output, dtype, g0 + d) * pw;
        } else {
          for (int32_t d = 0; d < D; ++d) Gf[d] += load_f(grad_output, dtype, g0 + d);
        }
      }
      float mult = lr;
      if (optimizer == 1) {
        float gss = 0;
        for (int32_t d = 0; d < D; ++d) gss += Gf[d] * Gf[d];
        float *st = (float *)optimizer_state + row;
        const float old = *st;
        *st = old + gss;
        mult = (float)(lr * (1.0 / (sqrtf(old + gss) + eps)));
      }
      if (stochastic_rounding && dtype == F16) {
        for (int32_t d = 0; d < D; ++d) Gf[d] = load_f(weights, dtype, row * D + d) - Gf[d] * mult;
        store_row_stochastic((uint16_t *)weights + row * D, Gf, D, row * D, sr_seed, sr_offset);
      } else {
        for (int32_t d = 0; d < D; ++d) {
          float w = load_f(weights, dtype, row * D + d);
          w -= Gf[d] * mult;
          store_f(weights, dtype, row * D + d, w);
        }
      }
    }
  }
  free(Gd); free(Gf);
  free(keys); free(b_ts); free(pos); free(keys_s); free(pos_s); free(seg);
  return 0;
}

/* ---------------------------------------------- approximate row-wise Adagrad
 * batched_embedding_backward_adagrad_approx_kernel_1 (tbe.cu:648-704) and its mixed-D twin
 * (tbe.cu:1006-1074) with AdaGradFunctor / WeightedAdaGradFunctor (tbe.cu:437-471, 483-553).
 * Per bag (t, b): gss = sum_d grad_output[b][t][d]^2; then per lookup p of the bag
 *   wss    = gss (* psw[p] * psw[p])
 *   old    = state[row]; state[row] = old + wss                       (update_momentum)
 *   mult   = (psw[p] *) lr * (1.0 / (sqrt(old + wss) + eps))
 *   grad_psw[p] = <weights[row], grad_output[b][t]>                   (weighted: the row as it is now)
 *   weights[row] -= grad_output[b][t] * mult, stored in the weights' type  (update_weight)
 * The reference runs the bags concurrently with plain loads and stores, so its result is only
 * defined when no row occurs twice in a batch (the only case its test draws,
 * test_table_batched_embeddings.py:244).  This restatement is the same kernel run ONE LOOKUP AT A
 * TIME in position order (table-major bags, then the bag's lookups): the outcome every
 * interleaving of the reference agrees with when rows do not repeat, and the serial one when
 * they do.  fp16 weights are rounded after every lookup, as update_weight's store does; with
 * stochastic rounding the k-th update of a row in a call draws its bits with the Philox key
 * seed ^ (k * 0x9E3779B97F4A7C15) (k = 0 is the exact update's stream).
 * Uniform tables: D > 0, table_offsets = first ROW of each table [T], mixed_* NULL.
 * Mixed-D tables: D = 0, mixed_table_offsets = first ELEMENT [T+1], table_dim_offsets = first row id
 * [T+1], dim_offsets = first output column [T+1], grad_output [B][total_D].
 */
int oracle_backward_approx(const void *grad_output, void *weights, int dtype, int64_t total_rows,
                           int32_t D, const int32_t *table_offsets,
                           const int64_t *mixed_table_offsets, const int32_t *table_dim_offsets,
                           const int32_t *dim_offsets, int32_t total_D, int32_t T,
                           const int32_t *indices, const int32_t *offsets, int32_t B, const void *psw,
                           void *optimizer_state, float lr, float eps, void *grad_psw,
                           int32_t stochastic_rounding, uint64_t sr_seed, uint64_t sr_offset) {
  const int mixed = D == 0;
  int32_t *times = (int32_t *)calloc((size_t)(total_rows > 0 ? total_rows : 1), 4);
  int32_t max_D = D;
  if (mixed)
    for (int32_t t = 0; t < T; ++t)
      if (dim_offsets[t + 1] - dim_offsets[t] > max_D) max_D = dim_offsets[t + 1] - dim_offsets[t];
  float *tmp = (float *)malloc((size_t)(max_D > 0 ? max_D : 1) * 4);
  for (int32_t t = 0; t < T; ++t) {
    const int32_t Dt = mixed ? dim_offsets[t + 1] - dim_offsets[t] : D;
    for (int32_t b = 0; b < B; ++b) {
      const int64_t g0 = mixed ? (int64_t)b * total_D + dim_offsets[t] : ((int64_t)b * T + t) * D;
      double gss_d = 0;
      float gss_f = 0;
      for (int32_t d = 0; d < Dt; ++d) {
        if (dtype == F64) { const double g = ((const double *)grad_output)[g0 + d]; gss_d += g * g; }
        else { const float g = load_f(grad_output, dtype, g0 + d); gss_f += g * g; }
      }
      for (int32_t p = offsets[t * B + b]; p < offsets[t * B + b + 1]; ++p) {
        const int64_t row = mixed ? (int64_t)table_dim_offsets[t] + indices[p] : (int64_t)table_offsets[t] + indices[p];
        const int64_t w0 = mixed ? mixed_table_offsets[t] + (int64_t)indices[p] * Dt : row * D;
        const int32_t k = times[row]++;
        if (dtype == F64) {
          const double pw = psw ? ((const double *)psw)[p] : 1.0;
          const double wss = psw ? gss_d * pw * pw : gss_d;
          double *st = (double *)optimizer_state + row;
          const double old = *st;
          *st = old + wss;
          const double mult = psw ? pw * lr * (1.0 / (sqrt(old + wss) + eps)) : lr * (1.0 / (sqrt(old + wss) + eps));
          double *w = (double *)weights + w0;
          const double *g = (const double *)grad_output + g0;
          if (psw) {
            double dot = 0;
            for (int32_t d = 0; d < Dt; ++d) dot += w[d] * g[d];
            ((double *)grad_psw)[p] = dot;
          }
          for (int32_t d = 0; d < Dt; ++d) w[d] -= g[d] * mult;
        } else {
          const float pw = psw ? load_f(psw, dtype, p) : 1.0f;
          const float wss = psw ? gss_f * pw * pw : gss_f;
          float *st = (float *)optimizer_state + row;
          const float old = *st;
          *st = old + wss;
          const float mult = psw ? (float)(pw * lr * (1.0 / (sqrtf(old + wss) + eps)))
                                 : (float)(lr * (1.0 / (sqrtf(old + wss) + eps)));
          if (psw) {
            float dot = 0;
            for (int32_t d = 0; d < Dt; ++d) dot += load_f(weights, dtype, w0 + d) * load_f(grad_output, dtype, g0 + d);
            store_f(grad_psw, dtype, p, dot);
          }
          if (stochastic_rounding && dtype == F16) {
            for (int32_t d = 0; d < Dt; ++d)
              tmp[d] = load_f(weights, dtype, w0 + d) - load_f(grad_output, dtype, g0 + d) * mult;
            store_row_stochastic((uint16_t *)weights + w0, tmp, Dt, w0,
                                 sr_seed ^ ((uint64_t)k * 0x9E3779B97F4A7C15ull), sr_offset);
          } else {
            for (int32_t d = 0; d < Dt; ++d) {
              float w = load_f(weights, dtype, w0 + d);
              w -= load_f(grad_output, dtype, g0 + d) * mult;
              store_f(weights, dtype, w0 + d, w);
            }
          }
        }
      }
    }
  }
  free(times);
  free(tmp);
  return 0;
}

/* --------------------------------------------------------- construct_offsets
 * construct_offsets_kernel (tbe.cu:1165-1188): out[0] = 0 (at::zeros, :1201),
 * out[1 + t*B + b] = next start (or table total for the last bag) - start.
 */
void oracle_construct_offsets(const int32_t *batch_offsets_per_table,
                              const int32_t *total_indices_per_table, int32_t T, int32_t B,
                              int32_t *output) {
  output[0] = 0;
  for (int32_t b_t = 0; b_t < T * B; ++b_t) {
    const int32_t b = b_t % B, t = b_t / B;
    int32_t upper;
    if (b != B - 1) upper = batch_offsets_per_table[t * B + b + 1];
    else upper = total_indices_per_table[t];
    output[1 + t * B + b] = upper - batch_offsets_per_table[t * B + b];
  }
}

/* ======================================================= per-table dimension
 * Mixed-D layout of table_batched_embeddings_ops.py:324-379: weights 1-D with int64
 * element offsets table_offsets[T+1], global row ids from table_dim_offsets[T+1]
 * (cumulative row counts), output columns from dim_offsets[T+1], output [B][total_D].
 */

/* batched_embedding_forward_kernel_mixed_D_1 (tbe.cu:882-943) */
void oracle_forward_mixed(const void *weights, int dtype, const int64_t *table_offsets,
                          const int32_t *dim_offsets, int32_t total_D, int32_t T,
                          const int32_t *indices, const int32_t *offsets, int32_t B,
                          const void *psw, void *output) {
  for (int32_t b_t = 0; b_t < T * B; ++b_t) {
    const int32_t t = b_t / B, b = b_t % B;
    const int32_t dim_start = dim_offsets[t], D = dim_offsets[t + 1] - dim_start;
    const int64_t table_offset = table_offsets[t];
    const int32_t start = offsets[t * B + b], end = offsets[t * B + b + 1];
    const int64_t out0 = (int64_t)b * total_D + dim_start;
    for (int32_t d = 0; d < D; ++d) {
      if (dtype == F64) {
        double sum = 0;
        for (int32_t l = start; l < end; ++l) {
          const double w = ((const double *)weights)[table_offset + (int64_t)indices[l] * D + d];
          if (psw) sum += w * ((const double *)psw)[l];
          else sum += w;
        }
        ((double *)output)[out0 + d] = sum;
      } else {
        float sum = 0;
        for (int32_t l = start; l < end; ++l) {
          const float w = load_f(weights, dtype, table_offset + (int64_t)indices[l] * D + d);
          if (psw) sum += w * load_f(psw, dtype, l);
          else sum += w;
        }
        store_f(output, dtype, out0 + d, sum);
      }
    }
  }
}

/* linear_index_weight_offsets_mixed_D_kernel (tbe.cu:1220-1247), the sort (tbe.cu:1400-1416)
 * and batched_embedding_backward_adagrad_exact_kernel_mixed_D_1 (tbe.cu:1249-1348); optimizer
 * and weighting as in oracle_backward. */
int oracle_backward_mixed(int optimizer, const void *grad_output, void *weights, int dtype,
                          int64_t total_rows, const int64_t *table_offsets,
                          const int32_t *table_dim_offsets, const int32_t *dim_offsets,
                          int32_t total_D, int32_t T, const int32_t *indices, int64_t n,
                          const int32_t *offsets, int32_t B, const void *psw,
                          void *optimizer_state, float lr, float eps, void *grad_psw) {
  const size_t nn = (size_t)(n > 0 ? n : 1);
  int32_t *keys = (int32_t *)malloc(nn * 4), *b_ts = (int32_t *)malloc(nn * 4);
  int32_t *pos = (int32_t *)malloc(nn * 4), *keys_s = (int32_t *)malloc(nn * 4);
  int32_t *pos_s = (int32_t *)malloc(nn * 4), *seg = (int32_t *)malloc((nn + 1) * 4);
  oracle_linearize(table_dim_offsets, T, indices, offsets, B, keys, b_ts, pos);
  oracle_sort_pairs(keys, pos, keys_s, pos_s, n, (int)(log2((double)total_rows) + 1));
  const int64_t U = oracle_segments(keys_s, n, seg);
  double *G = (double *)malloc((size_t)total_D * 8);
  for (int64_t u = 0; u < U; ++u) {
    const int32_t s0 = seg[u], s1 = seg[u + 1];
    const int32_t t = b_ts[pos_s[s0]] / B;
    const int32_t dim_start = dim_offsets[t], D = dim_offsets[t + 1] - dim_start;
    const int64_t row = keys_s[s0];
    const int64_t w0 = table_offsets[t] + (row - table_dim_offsets[t]) * D;
    for (int32_t d = 0; d < D; ++d) G[d] = 0;
    for (int32_t i = s0; i < s1; ++i) {
      const int32_t p = pos_s[i], b = b_ts[p] % B;
      const int64_t g0 = (int64_t)b * total_D + dim_start;
      if (dtype == F64) {
        const double *g = (const double *)grad_output + g0;
        const double *w = (const double *)weights + w0;
        double pw = 1;
        if (psw) {
          double dot = 0;
          for (int32_t d = 0; d < D; ++d) dot += w[d] * g[d];
          ((double *)grad_psw)[p] = dot;
          pw = ((const double *)psw)[p];
        }
        for (int32_t d = 0; d < D; ++d) G[d] += psw ? g[d] * pw : g[d];
      } else {
        float pw = 1;
        if (psw) {
          float dot = 0;
          for (int32_t d = 0; d < D; ++d) dot += load_f(weights, dtype, w0 + d) * load_f(grad_output, dtype, g0 + d);
          store_f(grad_psw, dtype, p, dot);
          pw = load_f(psw, dtype, p);
        }
        for (int32_t d = 0; d < D; ++d) {
          const float g = load_f(grad_output, dtype, g0 + d);
          G[d] = (double)((float)G[d] + (psw ? g * pw : g));
        }
      }
    }
    if (dtype == F64) {
      double mult = lr;
      if (optimizer == 1) {
        double gss = 0;
        for (int32_t d = 0; d < D; ++d) gss += G[d] * G[d];
        double *st = (double *)optimizer_state + row;
        const double old = *st;
        *st = old + gss;
        mult = lr * (1.0 / (sqrt(old + gss) + eps));
      }
      double *w = (double *)weights + w0;
      for (int32_t d = 0; d < D; ++d) w[d] -= G[d] * mult;
    } else {
      float mult = lr;
      if (optimizer == 1) {
        float gss = 0;
        for (int32_t d = 0; d < D; ++d) gss += (float)G[d] * (float)G[d];
        float *st = (float *)optimizer_state + row;
        const float old = *st;
        *st = old + gss;
        mult = (float)(lr * (1.0 / (sqrtf(old + gss) + eps)));
      }
      for (int32_t d = 0; d < D; ++d) {
        float w = load_f(weights, dtype, w0 + d);
        w -= (float)G[d] * mult;
        store_f(weights, dtype, w0 + d, w);
      }
    }
  }
  free(G);
  free(keys); free(b_ts); free(pos); free(keys_s); free(pos_s); free(seg);
  return 0;
}

/* ================================================== interleaved [E][T][D] tables
 * The older kernels: sparse_embedding_cuda_forward_offsets_kernel_impl
 * (sparse_embedding_cuda_kernel.cu:221-284; the dense variant :349-379 is the special case of
 * equal bag lengths) and the fused update (:464-499), the latter made exact: each distinct
 * (row, table) gets -lr * (sum of its bags' gradients) once.  fp32 only (what the tests use).
 * offsets is the flattened [B*T+1] array, bag (b,t) = offsets[b*T+t] .. offsets[b*T+t+1].
 */
void oracle_forward_etd(const float *weights, int32_t E, int32_t T, int32_t D, const int32_t *indices,
                        const int32_t *offsets, int32_t B, float *output) {
  (void)E;
  for (int32_t b = 0; b < B; ++b)
    for (int32_t t = 0; t < T; ++t)
      for (int32_t d = 0; d < D; ++d) {
        float sum = 0.0f;
        for (int32_t l = offsets[b * T + t]; l < offsets[b * T + t + 1]; ++l)
          sum += weights[((int64_t)indices[l] * T + t) * D + d];
        output[((int64_t)b * T + t) * D + d] = sum;
      }
}

void oracle_backward_etd(const float *grad_output, float *weights, int32_t E, int32_t T, int32_t D,
                         const int32_t *indices, const int32_t *offsets, int32_t B, float lr) {
  float *G = (float *)calloc((size_t)E * T * D, sizeof(float));
  uint8_t *hit = (uint8_t *)calloc((size_t)E * T, 1);
  for (int32_t b = 0; b < B; ++b)
    for (int32_t t = 0; t < T; ++t)
      for (int32_t l = offsets[b * T + t]; l < offsets[b * T + t + 1]; ++l) {
        const int64_t row = (int64_t)indices[l] * T + t;
        hit[row] = 1;
        for (int32_t d = 0; d < D; ++d) G[row * D + d] += grad_output[((int64_t)b * T + t) * D + d];
      }
  for (int64_t row = 0; row < (int64_t)E * T; ++row)
    if (hit[row])
      for (int32_t d = 0; d < D; ++d) weights[row * D + d] -= G[row * D + d] * lr;
  free(G);
  free(hit);
}
