/* orc_pcs.c -- the commitment's data-parallel part: leaf digests, Merkle trees with caps, column
 * commitment, combine-columns and the BaseFold loop, restated from src/pcs.lisp:37-101, 271-304, 434-441, 473-483,
 * 569-657
 * (test oracle; see orc.h).  BaseFold runs here on one class; the opening over several size classes, query
 * verification and trees with injections are in orc_open.c.  The multi-unit bookkeeping around them (units,
 * merge sets, segments, point reductions) is not restated. */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

#define CHUNK 64 /* columns per BLAKE3 call in a leaf digest, src/pcs.lisp:35 */
#define CAPLOG 7
#define FLOG 5

/* LEAF-DIGEST, src/pcs.lisp:44-52: rows hashed 64 at a time, chained h = BLAKE3(h || d_i) */
void orc_leaf_digest(const uint32_t *rows, uint64_t nrows, const uint8_t *previous, uint8_t out[32]) {
  uint8_t h[32], d[32], buf[CHUNK * 16], hd[64];
  int have = 0;
  if (previous) {
    memcpy(h, previous, 32);
    have = 1;
  }
  for (uint64_t start = 0; start < nrows; start += CHUNK) {
    uint64_t cnt = nrows - start < CHUNK ? nrows - start : CHUNK;
    for (uint64_t k = 0; k < 4 * cnt; k++) {
      uint32_t v = rows[4 * start + k];
      buf[4 * k] = (uint8_t)v, buf[4 * k + 1] = (uint8_t)(v >> 8), buf[4 * k + 2] = (uint8_t)(v >> 16),
              buf[4 * k + 3] = (uint8_t)(v >> 24);
    }
    orc_blake3_hash(buf, 16 * cnt, d, 32);
    if (have) {
      memcpy(hd, h, 32);
      memcpy(hd + 32, d, 32);
      orc_blake3_hash(hd, 64, h, 32);
    } else {
      memcpy(h, d, 32);
      have = 1;
    }
  }
  if (have)
    memcpy(out, h, 32);
  else
    memset(out, 0, 32); /* no rows and no previous digest: the reference returns NIL */
}

void orc_node(const uint8_t left[32], const uint8_t right[32], uint8_t out[32]) { /* :54-55 */
  uint8_t lr[64];
  memcpy(lr, left, 32);
  memcpy(lr + 32, right, 32);
  orc_blake3_hash(lr, 64, out, 32);
}

int orc_cap_level(uint64_t leaves) { /* :57-59 */
  int il = 0;
  for (uint64_t v = leaves; v; v >>= 1) il++;
  int l = il - 1 - CAPLOG;
  return l > 0 ? l : 0;
}

/* MERKLE-LEVELS without injections, src/pcs.lisp:64-77 */
void orc_merkle_levels(const uint8_t *leaves, uint64_t n, uint8_t *out) {
  memcpy(out, leaves, 32 * n);
  uint8_t *level = out;
  while (n > 1) {
    uint8_t *next = level + 32 * n;
    for (uint64_t i = 0; i < n; i += 2) orc_node(level + 32 * i, level + 32 * (i + 1), next + 32 * (i / 2));
    level = next;
    n /= 2;
  }
}

/* CHECK-PATH, src/pcs.lisp:86-95 */
int orc_check_path(const uint8_t h_in[32], const uint8_t *path, int depth, uint64_t i, const uint8_t *cap) {
  uint8_t h[32];
  memcpy(h, h_in, 32);
  for (int l = 0; l < depth; l++) {
    const uint8_t *sib = path + 32 * l;
    if (i & 1)
      orc_node(sib, h, h);
    else
      orc_node(h, sib, h);
    i >>= 1;
  }
  return memcmp(h, cap + 32 * i, 32) == 0;
}

static const uint8_t *level_ptr(const uint8_t *levels, uint64_t nleaves, int level) {
  const uint8_t *p = levels;
  for (int l = 0; l < level; l++, nleaves /= 2) p += 32 * nleaves;
  return p;
}

/* PCS-COMMIT for one class of one unit, src/pcs.lisp:271-304 */
uint64_t orc_commit_columns(const uint32_t *const *columns, int ncols, int c, uint32_t *codewords,
                            uint8_t *levels, uint8_t *cap) {
  uint64_t cwlen = (uint64_t)1 << (c + 1), nleaves = (uint64_t)1 << (c - 1);
  for (int k = 0; k < ncols; k++) orc_rs_encode(columns[k], c + 1, codewords + (uint64_t)k * cwlen);
  uint8_t *digests = (uint8_t *)malloc(32 * nleaves);
  uint32_t *rows = (uint32_t *)malloc((size_t)ncols * 4 * sizeof(uint32_t));
  for (uint64_t l = 0; l < nleaves; l++) { /* LEAF-ROWS, :275-277 */
    for (int k = 0; k < ncols; k++)
      for (int s = 0; s < 4; s++) rows[4 * k + s] = codewords[(uint64_t)k * cwlen + 4 * l + s];
    orc_leaf_digest(rows, ncols, NULL, digests + 32 * l);
  }
  orc_merkle_levels(digests, nleaves, levels);
  int lc = orc_cap_level(nleaves);
  uint64_t cap_rows = nleaves >> lc;
  memcpy(cap, level_ptr(levels, nleaves, lc), 32 * cap_rows);
  free(digests);
  free(rows);
  return cap_rows;
}

/* ENCODE-EXT, src/pcs.lisp:569-575: coordinate by coordinate */
static void encode_ext(const uint32_t *table, int c, uint32_t *cw) {
  uint64_t len = (uint64_t)1 << c;
  uint32_t *col = (uint32_t *)malloc(len * sizeof(uint32_t)), *ccw = (uint32_t *)malloc(2 * len * sizeof(uint32_t));
  for (int d = 0; d < 8; d++) {
    for (uint64_t i = 0; i < len; i++) col[i] = table[i * 8 + d];
    orc_rs_encode(col, c + 1, ccw);
    for (uint64_t i = 0; i < 2 * len; i++) cw[i * 8 + d] = ccw[i];
  }
  free(col);
  free(ccw);
}

/* DOT-PAIRS, src/pcs.lisp:473-483 */
void orc_dot_pairs(const uint32_t *e, const uint32_t *v, uint64_t len, int parity, uint32_t *out) {
  uint32_t acc[8] = {0}, a[8], b[8], t[8];
  for (uint64_t i = 0; i < len; i += 2) {
    const uint32_t *tabs[2] = {e, v};
    uint32_t *dst[2] = {a, b};
    for (int k = 0; k < 2; k++) {
      const uint32_t *lo = tabs[k] + i * 8, *hi = lo + 8;
      if (parity == 0)
        memcpy(dst[k], lo, 32);
      else if (parity == 1)
        memcpy(dst[k], hi, 32);
      else {
        orc_ext_scale(8, hi, 2, t);
        orc_ext_sub(8, t, lo, dst[k]);
      }
    }
    orc_ext_mul(8, a, b, t);
    orc_ext_add(8, acc, t, acc);
  }
  memcpy(out, acc, 32);
}

/* the oracle tree of a folded codeword: leaf l = 8 rows (one per coordinate) of symbols 4l..4l+3
   (ORACLE-ROWS, :577-579) */
static void oracle_leaf_rows(const uint32_t *cw, uint64_t l, uint32_t rows[32]) {
  for (int d = 0; d < 8; d++)
    for (int s = 0; s < 4; s++) rows[4 * d + s] = cw[(4 * l + s) * 8 + d];
}

typedef struct {
  int level;
  uint32_t *cw;
  uint64_t cwlen;
  uint8_t *levels;
  uint64_t nleaves;
  int lc;
} oracle_t;

/* BASEFOLD, prover side, src/pcs.lisp:581-657, for one class c = nv */
int orc_basefold_prove(orc_tr *tr, int nv, const uint32_t *rr, const uint32_t *v, const uint32_t *h,
                       int grind_bits, int queries, uint64_t *out_qs, uint32_t *out_chal, uint32_t *out_final) {
  int fl = nv - FLOG > 0 ? nv - FLOG : 0, status = ORC_OK;
  uint64_t len = (uint64_t)1 << nv;
  uint32_t prf[8] = {1}, claim[8];
  memcpy(claim, v, 32);
  uint32_t *tt = (uint32_t *)malloc(len * 32), *et = (uint32_t *)malloc(len * 32), *cw = (uint32_t *)malloc(2 * len * 32);
  memcpy(tt, h, len * 32);
  encode_ext(h, nv, cw);
  orc_eq_table(8, nv, rr, et);
  uint32_t *tw = (uint32_t *)malloc(orc_twiddles_size(nv + 1) * sizeof(uint32_t));
  orc_twiddles(nv + 1, tw);
  const uint32_t *tw_level = tw;
  oracle_t oracles[32];
  int noracles = 0;
  for (int i = 0; i < fl; i++) {
    uint64_t cur = len >> i;
    uint32_t ev[24];
    for (int parity = 0; parity < 3; parity++) /* a = prf * ysum = 0: every class has joined */
      orc_dot_pairs(tt, et, cur, parity, ev + 8 * parity);
    uint64_t dims[2] = {3, 8};
    if ((status = orc_tr_send(tr, ev, 2, dims, NULL))) goto done;
    uint32_t s[8];
    orc_ext_add(8, ev, ev + 8, s);
    if (memcmp(s, claim, 32)) {
      status = ORC_E_REJECT;
      goto done;
    }
    uint32_t x[8], e1[8];
    orc_tr_challenge(tr, 8, x);
    if (out_chal) memcpy(out_chal + 8 * i, x, 32);
    orc_lagrange(8, 3, ev, x, claim);
    orc_ext_eq1(8, rr + 8 * i, x, e1);
    orc_ext_mul(8, prf, e1, prf);
    orc_fold_table(8, cur, tt, x, tt);
    orc_fold_table(8, cur, et, x, et);
    {
      uint32_t *ncw = (uint32_t *)malloc(cur * 32);
      orc_rs_fold(8, cur, cw, tw_level, x, ncw);
      free(cw);
      cw = ncw;
    }
    tw_level += cur; /* level i has 2^(nv - i) twiddles */
    int l = i + 1;
    if (l >= 2 && l < fl && l % 2 == 0) { /* oracle levels 2, 4, ... below fl */
      uint64_t cwlen = cur, nleaves = cwlen / 4;
      uint8_t *digests = (uint8_t *)malloc(32 * nleaves);
      uint32_t rows[32];
      for (uint64_t li = 0; li < nleaves; li++) {
        oracle_leaf_rows(cw, li, rows);
        orc_leaf_digest(rows, 8, NULL, digests + 32 * li);
      }
      uint8_t *levels = (uint8_t *)malloc(32 * (2 * nleaves));
      orc_merkle_levels(digests, nleaves, levels);
      free(digests);
      int lc = orc_cap_level(nleaves);
      uint64_t cap_rows = nleaves >> lc;
      if ((status = orc_tr_send_bytes(tr, level_ptr(levels, nleaves, lc), (int64_t)(32 * cap_rows), NULL, 0, NULL))) {
        free(levels);
        goto done;
      }
      oracle_t *o = &oracles[noracles++];
      o->level = l;
      o->cwlen = cwlen;
      o->cw = (uint32_t *)malloc(cwlen * 32);
      memcpy(o->cw, cw, cwlen * 32);
      o->levels = levels;
      o->nleaves = nleaves;
      o->lc = lc;
    }
  }
  {
    uint64_t mlen = len >> fl;
    uint64_t dims[2] = {mlen, 8};
    if ((status = orc_tr_send(tr, tt, 2, dims, NULL))) goto done;
    if (out_final) memcpy(out_final, tt, mlen * 32);
    uint32_t mval[8], t[8];
    if (fl < nv)
      orc_mle_eval(8, nv - fl, tt, 8, rr + 8 * fl, mval);
    else
      memcpy(mval, tt, 32);
    orc_ext_mul(8, prf, mval, t);
    if (memcmp(t, claim, 32)) {
      status = ORC_E_REJECT;
      goto done;
    }
    orc_tr_grind(tr, grind_bits);
    uint64_t *qs = out_qs ? out_qs : (uint64_t *)malloc(8 * (size_t)queries + 8);
    orc_tr_challenge_bits(tr, nv - 1, queries, qs);
    for (int k = 0; k < noracles && !status; k++) { /* the oracle openings, recorded, :651-655 */
      oracle_t *o = &oracles[k];
      uint32_t *lv = (uint32_t *)malloc((size_t)queries * 32 * sizeof(uint32_t) + 4);
      uint8_t *paths = (uint8_t *)malloc((size_t)queries * o->lc * 32 + 1);
      for (int q = 0; q < queries; q++) {
        uint64_t li = qs[q] >> o->level;
        oracle_leaf_rows(o->cw, li, lv + 32 * q);
        const uint8_t *level = o->levels;
        uint64_t n = o->nleaves, idx = li;
        for (int d = 0; d < o->lc; d++) { /* PATH, :79-84 */
          memcpy(paths + 32 * ((size_t)q * o->lc + d), level + 32 * (idx ^ 1), 32);
          level += 32 * n;
          n /= 2;
          idx >>= 1;
        }
      }
      uint64_t d3[3] = {(uint64_t)queries, 8, 4};
      status = orc_tr_record(tr, lv, 3, d3, NULL);
      if (!status) status = orc_tr_record_bytes(tr, paths, (int64_t)queries * o->lc * 32, NULL, 0, NULL);
      free(lv);
      free(paths);
    }
    if (!out_qs) free(qs);
  }
done:
  for (int k = 0; k < noracles; k++) {
    free(oracles[k].cw);
    free(oracles[k].levels);
  }
  free(tt);
  free(et);
  free(cw);
  free(tw);
  return status;
}

/* BASEFOLD, verifier side (the sumcheck rounds, the final claim, grinding and the query positions;
   the query openings are taken and checked against the oracle caps for shape only by the caller) */
int orc_basefold_verify(orc_tr *tr, int nv, const uint32_t *rr, const uint32_t *v, int grind_bits,
                        int queries, uint64_t *out_qs) {
  int fl = nv - FLOG > 0 ? nv - FLOG : 0, status;
  uint32_t prf[8] = {1}, claim[8];
  memcpy(claim, v, 32);
  for (int i = 0; i < fl; i++) {
    uint32_t ev[24], s[8], x[8], e1[8];
    uint64_t dims[2] = {3, 8};
    if ((status = orc_tr_send(tr, NULL, 2, dims, ev))) return status;
    orc_ext_add(8, ev, ev + 8, s);
    if (memcmp(s, claim, 32)) return ORC_E_REJECT;
    orc_tr_challenge(tr, 8, x);
    orc_lagrange(8, 3, ev, x, claim);
    orc_ext_eq1(8, rr + 8 * i, x, e1);
    orc_ext_mul(8, prf, e1, prf);
    int l = i + 1;
    if (l >= 2 && l < fl && l % 2 == 0) {
      uint64_t nleaves = ((uint64_t)1 << (nv + 1 - l)) / 4;
      uint64_t cap_rows = nleaves >> orc_cap_level(nleaves);
      if ((status = orc_tr_send_bytes(tr, NULL, (int64_t)(32 * cap_rows), NULL, 0, NULL))) return status;
    }
  }
  uint64_t mlen = (uint64_t)1 << (nv - fl);
  uint32_t *m = (uint32_t *)malloc(mlen * 32);
  uint64_t dims[2] = {mlen, 8};
  if ((status = orc_tr_send(tr, NULL, 2, dims, m))) {
    free(m);
    return status;
  }
  uint32_t mval[8], t[8];
  if (fl < nv)
    orc_mle_eval(8, nv - fl, m, 8, rr + 8 * fl, mval);
  else
    memcpy(mval, m, 32);
  free(m);
  orc_ext_mul(8, prf, mval, t);
  if (memcmp(t, claim, 32)) return ORC_E_REJECT;
  uint64_t nonce;
  if ((status = orc_tr_verify_grind(tr, grind_bits, &nonce))) return status;
  uint64_t *qs = out_qs ? out_qs : (uint64_t *)malloc(8 * (size_t)queries + 8);
  orc_tr_challenge_bits(tr, nv - 1, queries, qs);
  if (!out_qs) free(qs);
  return ORC_OK;
}

/* COMBINE-COLUMNS, src/pcs.lisp:434-441: g[x] = sum_k coefficient_k * column_k[x] for base columns (column k at
   columns + k * len) and extension coefficients; the sum starts from zero and runs in column order */
void orc_combine_columns(int D, int ncols, uint64_t len, const uint32_t *columns, const uint32_t *coefficients,
                         uint32_t *out) {
  for (uint64_t x = 0; x < len; x++) {
    uint32_t g[ORC_MAXD] = {0}, term[ORC_MAXD];
    for (int k = 0; k < ncols; k++) {
      orc_ext_scale(D, coefficients + (size_t)k * D, columns[(uint64_t)k * len + x], term);
      orc_ext_add(D, g, term, g);
    }
    memcpy(out + x * D, g, D * sizeof(uint32_t));
  }
}

/* the opening's table per class, src/pcs.lisp:709-716: h[x] <- h[x] + scale * column[x] over EXT8s (one call
   per unit or pulled unit of the class, starting from zeros) */
void orc_scale_add(int D, uint64_t len, const uint32_t *scale, const uint32_t *column, uint32_t *h) {
  for (uint64_t x = 0; x < len; x++) {
    uint32_t t[ORC_MAXD];
    orc_ext_mul(D, scale, column + x * D, t);
    orc_ext_add(D, h + x * D, t, h + x * D);
  }
}

/* OPEN-QUERIES' recorded data for one (unit, class), src/pcs.lisp:721-734: the (Q, rows, 4) array of the queried
   leaves (LEAF-ROWS :275-277 through FIELD-ARRAY-OF-LEAVES :659-665) and, with LEVELS (all levels, leaves
   first, as orc_merkle_levels lays them out), each leaf's PATH (:79-84) up to the cap level.  Returns that depth. */
int orc_open_queries(const uint32_t *codewords, int ncols, int c, const uint8_t *levels, const uint64_t *leaves,
                     int count, uint32_t *out_leaves, uint8_t *out_paths) {
  const uint64_t nleaves = (uint64_t)1 << (c - 1), cw_len = (uint64_t)1 << (c + 1);
  const int depth = levels ? orc_cap_level(nleaves) : 0;
  for (int q = 0; q < count; q++) {
    for (int k = 0; k < ncols; k++)
      for (int sym = 0; sym < 4; sym++)
        out_leaves[((size_t)q * ncols + k) * 4 + sym] = codewords[(uint64_t)k * cw_len + 4 * leaves[q] + sym];
    uint64_t i = leaves[q], level_size = nleaves;
    const uint8_t *level = levels;
    for (int l = 0; l < depth; l++) {
      memcpy(out_paths + ((size_t)q * depth + l) * 32, level + (i ^ 1) * 32, 32);
      level += level_size * 32;
      level_size >>= 1;
      i >>= 1;
    }
  }
  return depth;
}
