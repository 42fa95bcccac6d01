/* orc_sumcheck.c -- the sumcheck prover (folding path with split eq weights) and verifier,
 * restated from src/sumcheck.lisp (test oracle; see orc.h).
 *
 * The statement arrives as its canonical sum of monomials (src/forms.lisp:57-78) instead of the
 * nested form the reference compiles; both are the same polynomial over an exact field, so every
 * round sum is the same field element (the reference's own tests rely on the same fact,
 * tests/tests.lisp:329-395).  The small-value first rounds (src/sumcheck.lisp:319-510) are not
 * restated: they send the same messages as folding (tests/tests.lisp:374-395).
 */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

int orc_stmt_degree(const orc_stmt *st) { /* src/sumcheck.lisp:33-35, src/forms.lisp:101-106 */
  int degree = 0;
  for (int t = 0; t < st->nterms; t++) {
    int d = 0;
    for (int k = st->start[t]; k < st->start[t + 1]; k++) d += st->vars[k] < st->T;
    if (d > degree) degree = d;
  }
  return degree;
}

void orc_stmt_eval(const orc_stmt *st, int D, const uint32_t *tv, const uint32_t *consts, uint32_t *out) {
  uint32_t acc[ORC_MAXD] = {0};
  for (int t = 0; t < st->nterms; t++) {
    uint32_t term[ORC_MAXD] = {1};
    for (int k = st->start[t]; k < st->start[t + 1]; k++) {
      int v = st->vars[k];
      const uint32_t *x = v < st->T ? tv + (size_t)v * D : consts + (size_t)(v - st->T) * D;
      orc_ext_mul(D, term, x, term);
    }
    orc_ext_scale(D, term, st->coeff[t], term);
    orc_ext_add(D, acc, term, acc);
  }
  memcpy(out, acc, D * sizeof(uint32_t));
}

/* TABLE-ENTRY, src/sumcheck.lisp:75-82: a base value v lifts to (v, 0, ..., 0) */
static void table_entry(int D, const uint32_t *entries, int stride, uint64_t x, uint32_t *out) {
  for (int c = 0; c < D; c++) out[c] = c < stride ? entries[stride * x + c] : 0;
}

/* WEIGHTS, src/sumcheck.lisp:37-41 */
static uint32_t *weights(int D, const uint32_t *eq, int from, int to) {
  int k = to - from;
  uint64_t len = (uint64_t)1 << k;
  uint32_t *w = (uint32_t *)calloc(len * D, sizeof(uint32_t));
  if (eq)
    orc_eq_table(D, k, eq + (size_t)from * D, w);
  else
    for (uint64_t i = 0; i < len; i++) w[i * D] = 1;
  return w;
}

/* HYPERCUBE-SUM, src/sumcheck.lisp:112-127 */
void orc_hypercube_sum(const orc_stmt *st, int n, int D, const uint32_t *const *tables,
                       const int32_t *strides, const uint32_t *eq, const uint32_t *consts, uint32_t *out) {
  uint32_t *w = weights(D, eq, 0, n);
  uint32_t sum[ORC_MAXD] = {0}, tv[16 * ORC_MAXD], f[ORC_MAXD];
  for (uint64_t x = 0; x < ((uint64_t)1 << n); x++) {
    for (int t = 0; t < st->T; t++) table_entry(D, tables[t], strides[t], x, tv + t * D);
    orc_stmt_eval(st, D, tv, consts, f);
    orc_ext_mul(D, w + x * D, f, f);
    orc_ext_add(D, sum, f, sum);
  }
  free(w);
  memcpy(out, sum, D * sizeof(uint32_t));
}

/* one prover round, ROUND-KERNEL-CODE / GENERIC-ROUND-SUMS, src/sumcheck.lisp:190-311 */
void orc_round_sums(const orc_stmt *st, int D, int points, uint64_t n_low, uint64_t n_high,
                    const uint32_t *const *tables, const int32_t *strides, const uint32_t *low,
                    const uint32_t *high, const uint32_t *consts, uint32_t *out) {
  int T = st->T;
  uint32_t lines[16][17][ORC_MAXD]; /* [table][X] */
  uint32_t inner[16][ORC_MAXD], slope[ORC_MAXD], tv[16 * ORC_MAXD], f[ORC_MAXD];
  memset(out, 0, (size_t)points * D * sizeof(uint32_t));
  for (uint64_t h = 0; h < n_high; h++) {
    memset(inner, 0, sizeof(inner));
    for (uint64_t l = 0; l < n_low; l++) {
      uint64_t i = h * n_low + l;
      for (int t = 0; t < T; t++) {
        table_entry(D, tables[t], strides[t], 2 * i, lines[t][0]);
        table_entry(D, tables[t], strides[t], 2 * i + 1, lines[t][1]);
        orc_ext_sub(D, lines[t][1], lines[t][0], slope);
        for (int x = 2; x <= points; x++) orc_ext_add(D, lines[t][x - 1], slope, lines[t][x]);
      }
      for (int k = 0; k < points; k++) { /* X = 0, 2, 3, ..., points */
        int x = k == 0 ? 0 : k + 1;
        for (int t = 0; t < T; t++) memcpy(tv + t * D, lines[t][x], D * sizeof(uint32_t));
        orc_stmt_eval(st, D, tv, consts, f);
        orc_ext_mul(D, low + l * D, f, f);
        orc_ext_add(D, inner[k], f, inner[k]);
      }
    }
    for (int k = 0; k < points; k++) {
      orc_ext_mul(D, high + h * D, inner[k], f);
      orc_ext_add(D, out + (size_t)k * D, f, out + (size_t)k * D);
    }
  }
}

/* FOLD-FLAT-TABLE, src/sumcheck.lisp:84-104 */
void orc_fold_flat(int D, uint64_t len, const uint32_t *entries, int stride, const uint32_t *r, uint32_t *out) {
  for (uint64_t i = 0; i < len / 2; i++) {
    uint32_t term[ORC_MAXD];
    if (stride == 1) {
      uint32_t lo = entries[2 * i];
      orc_ext_scale(D, r, orc_fsub(entries[2 * i + 1], lo), term);
      term[0] = orc_fadd(term[0], lo);
    } else {
      uint32_t lo[ORC_MAXD], hi[ORC_MAXD];
      table_entry(D, entries, stride, 2 * i, lo);
      table_entry(D, entries, stride, 2 * i + 1, hi);
      orc_ext_sub(D, hi, lo, term);
      orc_ext_mul(D, r, term, term);
      orc_ext_add(D, lo, term, term);
    }
    memcpy(out + i * D, term, D * sizeof(uint32_t));
  }
}

/* HEADER, src/sumcheck.lisp:24-27: label | n u16 | degree u16 | blocks u32 */
static void absorb_header(orc_tr *tr, const uint8_t *label, uint64_t label_len, int n, int degree, int blocks) {
  uint8_t *h = (uint8_t *)malloc(label_len + 9);
  memcpy(h, label, label_len);
  h[label_len] = '|';
  uint8_t *p = h + label_len + 1;
  p[0] = (uint8_t)n;
  p[1] = (uint8_t)(n >> 8);
  p[2] = (uint8_t)degree;
  p[3] = (uint8_t)(degree >> 8);
  for (int i = 0; i < 4; i++) p[4 + i] = (uint8_t)((uint32_t)blocks >> (8 * i));
  orc_tr_absorb(tr, h, label_len + 9);
  free(h);
}

/* PROVE, src/sumcheck.lisp:512-571 (folding rounds) */
int orc_sumcheck_prove(orc_tr *tr, int n, const orc_stmt *st, const uint32_t *const *tables,
                       const int32_t *strides, const uint32_t *eq, const uint32_t *consts,
                       const uint8_t *label, uint64_t label_len, const uint32_t *bw, int K, int degree,
                       uint32_t *out_chal, uint32_t *out_finals, uint32_t *const *out_folded) {
  int D = orc_tr_degree(tr), T = st->T;
  if (T > 16 || K < 1) return ORC_E_PARAM;
  if (degree < 0) degree = orc_stmt_degree(st);
  int points = degree > 1 ? degree : 1;
  if (points > 16) return ORC_E_PARAM;
  uint64_t size = (uint64_t)K << n; /* entries per table */
  uint32_t *flat[16];
  int32_t stride[16];
  const uint32_t *cur[16];
  for (int t = 0; t < T; t++) {
    flat[t] = NULL;
    cur[t] = tables[t];
    stride[t] = strides[t];
  }
  absorb_header(tr, label, label_len, n, degree, bw ? K : 1);
  for (int j = 0; j < n; j++) {
    uint32_t *low, *high;
    uint64_t n_low, n_high;
    if (bw) { /* :549-550 */
      low = weights(D, eq, j + 1, n);
      n_low = (uint64_t)1 << (n - j - 1);
      high = (uint32_t *)malloc((size_t)K * D * sizeof(uint32_t));
      memcpy(high, bw, (size_t)K * D * sizeof(uint32_t));
      n_high = (uint64_t)K;
    } else { /* SPLIT-WEIGHTS, :43-49 */
      int from = j + 1, middle = from + (n - from) / 2;
      low = weights(D, eq, from, middle);
      high = weights(D, eq, middle, n);
      n_low = (uint64_t)1 << (middle - from);
      n_high = (uint64_t)1 << (n - middle);
    }
    uint32_t sums[16 * ORC_MAXD];
    const int fast = orc_fast_threads();
    if (fast > 0)
      orc_round_sums_fast(st, D, points, n_low, n_high, cur, stride, low, high, consts, fast, sums);
    else
      orc_round_sums(st, D, points, n_low, n_high, cur, stride, low, high, consts, sums);
    free(low);
    free(high);
    uint64_t dims[2] = {(uint64_t)points, (uint64_t)D};
    int status = orc_tr_send(tr, sums, 2, dims, NULL);
    if (status) return status;
    uint32_t *r = out_chal + (size_t)j * D;
    orc_tr_challenge(tr, D, r);
    for (int t = 0; t < T; t++) {
      uint32_t *next = (uint32_t *)malloc((size / 2) * D * sizeof(uint32_t) + 4);
      if (fast > 0)
        orc_fold_flat_fast(D, size, cur[t], stride[t], r, fast, next);
      else
        orc_fold_flat(D, size, cur[t], stride[t], r, next);
      free(flat[t]);
      flat[t] = next;
      cur[t] = next;
      stride[t] = D;
    }
    size /= 2;
  }
  for (int t = 0; t < T; t++) {
    table_entry(D, cur[t], stride[t], 0, out_finals + (size_t)t * D);
    if (out_folded && out_folded[t])
      for (uint64_t x = 0; x < size; x++) table_entry(D, cur[t], stride[t], x, out_folded[t] + x * D);
    free(flat[t]);
  }
  return ORC_OK;
}

/* NEXT-CLAIM, src/sumcheck.lisp:137-145 */
static int next_claim(int D, int points, const uint32_t *claim, const uint32_t *message,
                      const uint32_t *eq_rj, const uint32_t *x, uint32_t *out) {
  uint32_t vals[18 * ORC_MAXD];
  const uint32_t *g0 = message;
  uint32_t *g1 = vals + D;
  memcpy(vals, g0, D * sizeof(uint32_t));
  if (eq_rj) { /* claim = (1 - r) g(0) + r g(1) */
    uint32_t one[ORC_MAXD] = {1}, t[ORC_MAXD], inv[ORC_MAXD];
    orc_ext_sub(D, one, eq_rj, t);
    orc_ext_mul(D, t, g0, t);
    orc_ext_sub(D, claim, t, t);
    int status = orc_ext_inv(D, eq_rj, inv);
    if (status) return status;
    orc_ext_mul(D, t, inv, g1);
  } else {
    orc_ext_sub(D, claim, g0, g1);
  }
  memcpy(vals + 2 * D, message + D, (size_t)(points - 1) * D * sizeof(uint32_t));
  orc_lagrange(D, points + 1, vals, x, out);
  return ORC_OK;
}

/* VERIFY, src/sumcheck.lisp:147-163 */
int orc_sumcheck_verify(orc_tr *tr, int n, const orc_stmt *st, const uint32_t *claim_in,
                        const uint32_t *eq, const uint32_t *consts, int blocks, const uint8_t *label,
                        uint64_t label_len, int degree, uint32_t *out_chal, uint32_t *out_reduced) {
  (void)consts;
  int D = orc_tr_degree(tr);
  if (degree < 0) degree = orc_stmt_degree(st);
  int points = degree > 1 ? degree : 1;
  if (points > 16) return ORC_E_PARAM;
  uint32_t claim[ORC_MAXD];
  for (int c = 0; c < D; c++) claim[c] = claim_in[c] % ORC_P;
  absorb_header(tr, label, label_len, n, degree, blocks);
  for (int j = 0; j < n; j++) {
    uint32_t message[16 * ORC_MAXD];
    uint64_t dims[2] = {(uint64_t)points, (uint64_t)D};
    int status = orc_tr_send(tr, NULL, 2, dims, message);
    if (status) return status;
    uint32_t *r = out_chal + (size_t)j * D;
    orc_tr_challenge(tr, D, r);
    status = next_claim(D, points, claim, message, eq ? eq + (size_t)j * D : NULL, r, claim);
    if (status) return status;
  }
  memcpy(out_reduced, claim, D * sizeof(uint32_t));
  return ORC_OK;
}

/* CHECK-FINAL, src/sumcheck.lisp:165-172 */
int orc_check_final(const orc_stmt *st, int D, const uint32_t *reduced, const uint32_t *finals,
                    const uint32_t *consts) {
  uint32_t expected[ORC_MAXD];
  orc_stmt_eval(st, D, finals, consts, expected);
  return memcmp(expected, reduced, D * sizeof(uint32_t)) == 0 ? ORC_OK : ORC_E_REJECT;
}
