/* orc_open.c -- the final opening over several size classes, restated from src/pcs.lisp (test oracle; see orc.h):
 * Merkle trees of mixed height (MERKLE-LEVELS with injections :64-77, CHECK-PATH with INJECTED-AT :86-95), BASEFOLD
 * with classes joining at later levels (:581-657), OPEN-QUERIES (:721-734) and VERIFY-QUERIES (:752-843).
 *
 * The unit bookkeeping around them is reduced to what the data-parallel part needs: one key per size class, each a
 * unit of its own with its own tree (a set of one unit, whose "mixed" tree is that class alone), columns combined
 * with the coefficients the caller gives (UC-COEF).  Merge sets, segments and the cross-unit sumcheck are not
 * restated.
 *
 * Pinned by the reference's frozen commitment cases (tests/tests.lisp:728-758, digest at :905): under the reference's
 * scheduler restated in tests/golden/pcs_cases.py, orc_basefold_classes and the Merkle levels with injections
 * produce the three proofs of EXPORT-PCS-CASES byte for byte (tests/test_oracle_frozen_cases.py).  orc_pcs_open's
 * own query openings (one tree per key) and the verifier's side are held to: prover -> verifier
 * acceptance; rejection of every flipped opened symbol, path byte, cap byte and final-table entry; each opened
 * leaf hashing up its path to the committed cap; fold(encode(m)) = encode(fold(m)) through the oracles down to
 * the final table's codeword, which is what VERIFY-QUERIES itself recomputes; the single-class case being
 * orc_basefold_prove byte for byte. */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

#define FLOG 5

/* MERKLE-LEVELS with injections, src/pcs.lisp:64-77: after level l's nodes are formed, node = H(node, injected) */
void orc_merkle_levels_injected(const uint8_t *leaves, uint64_t n, int ninj, const int32_t *inj_level,
                                const uint8_t *const *inj, uint8_t *out) {
  memcpy(out, leaves, 32 * n);
  uint8_t *level = out;
  for (int l = 1; n > 1; l++) {
    uint8_t *next = level + 32 * n;
    for (uint64_t i = 0; i < n; i += 2) orc_node(level + 32 * i, level + 32 * (i + 1), next + 32 * (i / 2));
    n /= 2;
    for (int k = 0; k < ninj; k++)
      if (inj_level[k] == l)
        for (uint64_t i = 0; i < n; i++) orc_node(next + 32 * i, inj[k] + 32 * i, next + 32 * i);
    level = next;
  }
}

/* CHECK-PATH with INJECTED-AT, src/pcs.lisp:86-95 */
int orc_check_path_injected(const uint8_t h_in[32], const uint8_t *path, int depth, uint64_t i, const uint8_t *cap,
                            int ninj, const int32_t *inj_level, const uint8_t *inj_digests) {
  uint8_t h[32];
  memcpy(h, h_in, 32);
  for (int l = 1; l <= depth; l++) {
    const uint8_t *sib = path + 32 * (l - 1);
    if (i & 1)
      orc_node(sib, h, h);
    else
      orc_node(h, sib, h);
    i >>= 1;
    for (int k = 0; k < ninj; k++)
      if (inj_level[k] == l) orc_node(h, inj_digests + 32 * k, h);
  }
  return memcmp(h, cap + 32 * i, 32) == 0;
}

/* ENCODE-EXT, src/pcs.lisp:569-575 */
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

static void oracle_leaf_rows(const uint32_t *cw, uint64_t l, uint32_t rows[32]) { /* ORACLE-ROWS, :577-579 */
  for (int d = 0; d < 8; d++)
    for (int s = 0; s < 4; s++) rows[4 * d + s] = cw[(4 * l + s) * 8 + d];
}

static const uint8_t *level_ptr(const uint8_t *levels, uint64_t nleaves, int level) {
  const uint8_t *p = levels;
  for (int l = 0; l < level; l++, nleaves /= 2) p += 32 * nleaves;
  return p;
}

typedef struct {
  int level;
  uint32_t *cw;
  uint64_t cwlen;
  uint8_t *levels;
  uint64_t nleaves;
  int lc;
} oracle_t;

static void add_table(uint32_t *acc, const uint32_t *h, uint64_t len) {
  for (uint64_t i = 0; i < len; i++) orc_ext_add(8, acc + i * 8, h + i * 8, acc + i * 8);
}

/* BASEFOLD, prover side, src/pcs.lisp:581-657; classes ascending, class c joins at level nv - c; then OPEN-QUERIES
   (:721-734) over the keys, each the last (and only) unit of its set */
static int open_classes(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr, const uint32_t *v,
                        int grind_bits, int queries, uint64_t *out_qs, int open_keys) {
  int fl = nv - FLOG > 0 ? nv - FLOG : 0, status = ORC_OK;
  uint64_t len = (uint64_t)1 << nv;
  for (int k = 0; k < nkeys; k++)
    if (keys[k].c > nv || keys[k].c < 1 || (k && keys[k].c <= keys[k - 1].c)) return ORC_E_PARAM;
  if (nkeys < 1 || keys[nkeys - 1].c != nv || queries < 1) return ORC_E_PARAM;
  uint32_t prf[8] = {1}, claim[8], ysum[8] = {0};
  uint32_t(*yc)[8] = (uint32_t(*)[8])calloc(nkeys, 32);
  memcpy(claim, v, 32);
  for (int k = 0; k < nkeys; k++) { /* y_c = H_c(point-tail rr c nv); ysum over the classes still to join */
    orc_mle_eval(8, keys[k].c, keys[k].h, 8, rr + 8 * (size_t)(nv - keys[k].c), yc[k]);
    if (nv - keys[k].c > 0) orc_ext_add(8, ysum, yc[k], ysum);
  }
  uint32_t *tt = (uint32_t *)calloc(len * 8, 4), *et = (uint32_t *)malloc(len * 32), *cw = (uint32_t *)calloc(2 * len * 8, 4);
  orc_eq_table(8, nv, rr, et);
  for (int k = 0; k < nkeys; k++)
    if (keys[k].c == nv) {
      uint32_t *e = (uint32_t *)malloc(2 * len * 32);
      add_table(tt, keys[k].h, len);
      encode_ext(keys[k].h, nv, e);
      add_table(cw, e, 2 * len);
      free(e);
    }
  uint32_t *tw = (uint32_t *)malloc(orc_twiddles_size(nv + 1) * sizeof(uint32_t));
  orc_twiddles(nv + 1, tw);
  const uint32_t *tw_level = tw;
  oracle_t oracles[32];
  int noracles = 0;
  uint64_t *qs = out_qs ? out_qs : (uint64_t *)malloc(8 * (size_t)queries + 8);
  for (int i = 0; i < fl; i++) {
    uint64_t cur = len >> i;
    const uint32_t *ri = rr + 8 * (size_t)i;
    uint32_t ev[24], a[8], one[8] = {1}, one_r[8], eqx[3][8], t[8];
    orc_ext_mul(8, prf, ysum, a);
    orc_ext_sub(8, one, ri, one_r);
    memcpy(eqx[0], one_r, 32);
    memcpy(eqx[1], ri, 32);
    orc_ext_scale(8, ri, 2, t);
    orc_ext_sub(8, t, one_r, eqx[2]);
    for (int parity = 0; parity < 3; parity++) {
      orc_dot_pairs(tt, et, cur, parity, ev + 8 * parity);
      orc_ext_mul(8, a, eqx[parity], t);
      orc_ext_add(8, ev + 8 * parity, t, ev + 8 * parity);
    }
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
    orc_lagrange(8, 3, ev, x, claim);
    orc_ext_eq1(8, ri, x, e1);
    orc_ext_mul(8, prf, e1, prf);
    orc_fold_table(8, cur, tt, x, tt);
    orc_fold_table(8, cur, et, x, et);
    {
      uint32_t *ncw = (uint32_t *)malloc(cur * 32);
      orc_rs_fold(8, cur, cw, tw_level, x, ncw);
      free(cw);
      cw = ncw;
    }
    tw_level += cur;
    int l = i + 1;
    if (l >= 2 && l < fl && l % 2 == 0) {
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
      if ((status = orc_tr_send_bytes(tr, level_ptr(levels, nleaves, lc), (int64_t)(32 * (nleaves >> lc)), NULL, 0, NULL))) {
        free(levels);
        goto done;
      }
      oracle_t *o = &oracles[noracles++];
      o->level = l, o->cwlen = cwlen, o->levels = levels, o->nleaves = nleaves, o->lc = lc;
      o->cw = (uint32_t *)malloc(cwlen * 32);
      memcpy(o->cw, cw, cwlen * 32);
    }
    for (int k = 0; k < nkeys; k++) /* the classes that join here, :635-639 */
      if (nv - keys[k].c == l) {
        uint64_t clen = (uint64_t)1 << keys[k].c;
        uint32_t *e = (uint32_t *)malloc(2 * clen * 32);
        add_table(tt, keys[k].h, clen);
        encode_ext(keys[k].h, keys[k].c, e);
        add_table(cw, e, 2 * clen);
        free(e);
        orc_ext_sub(8, ysum, yc[k], ysum);
      }
  }
  {
    uint64_t mlen = len >> fl;
    uint64_t dims[2] = {mlen, 8};
    if ((status = orc_tr_send(tr, tt, 2, dims, NULL))) goto done;
    uint32_t mval[8], t[8];
    if (fl < nv)
      orc_mle_eval(8, nv - fl, tt, 8, rr + 8 * (size_t)fl, mval);
    else
      memcpy(mval, tt, 32);
    orc_ext_mul(8, prf, mval, t);
    if (memcmp(t, claim, 32)) {
      status = ORC_E_REJECT;
      goto done;
    }
    orc_tr_grind(tr, grind_bits);
    orc_tr_challenge_bits(tr, nv - 1, queries, qs);
    for (int k = 0; k < noracles && !status; k++) { /* the oracle openings, recorded, :651-655 */
      oracle_t *o = &oracles[k];
      uint32_t *lv = (uint32_t *)malloc((size_t)queries * 32 * sizeof(uint32_t) + 4);
      uint8_t *paths = (uint8_t *)malloc((size_t)queries * o->lc * 32 + 1);
      for (int q = 0; q < queries; q++) {
        uint64_t li = qs[q] >> o->level, n = o->nleaves, idx = li;
        oracle_leaf_rows(o->cw, li, lv + 32 * q);
        const uint8_t *level = o->levels;
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
  }
  /* OPEN-QUERIES, :721-734: each key's queried leaves, then (it is its set's last) its tree's paths */
  for (int k = 0; k < nkeys && !status && open_keys; k++) {
    const orc_open_key *key = &keys[k];
    int c = key->c, depth = orc_cap_level((uint64_t)1 << (c - 1));
    uint64_t *leaves = (uint64_t *)malloc(8 * (size_t)queries);
    for (int q = 0; q < queries; q++) leaves[q] = qs[q] >> (nv - c);
    uint32_t *rows = (uint32_t *)malloc((size_t)queries * key->ncols * 4 * sizeof(uint32_t) + 4);
    uint8_t *paths = (uint8_t *)malloc((size_t)queries * depth * 32 + 1);
    orc_open_queries(key->codewords, key->ncols, c, key->levels, leaves, queries, rows, paths);
    uint64_t d3[3] = {(uint64_t)queries, (uint64_t)key->ncols, 4};
    status = orc_tr_record(tr, rows, 3, d3, NULL);
    if (!status) status = orc_tr_record_bytes(tr, paths, (int64_t)queries * depth * 32, NULL, 0, NULL);
    free(leaves);
    free(rows);
    free(paths);
  }
done:
  for (int k = 0; k < noracles; k++) {
    free(oracles[k].cw);
    free(oracles[k].levels);
  }
  if (!out_qs) free(qs);
  free(yc);
  free(tt);
  free(et);
  free(cw);
  free(tw);
  return status;
}

int orc_pcs_open(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr, const uint32_t *v,
                 int grind_bits, int queries, uint64_t *out_qs) {
  return open_classes(tr, nv, nkeys, keys, rr, v, grind_bits, queries, out_qs, 1);
}

/* BASEFOLD alone (src/pcs.lisp:581-657) over the classes' combined columns (a key's c and h; nothing else of it is
   read): what a caller that opens merged sets and mixed trees itself (tests/golden/pcs_cases.py) builds on */
int orc_basefold_classes(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr, const uint32_t *v,
                         int grind_bits, int queries, uint64_t *out_qs) {
  return open_classes(tr, nv, nkeys, keys, rr, v, grind_bits, queries, out_qs, 0);
}

/* BASEFOLD's verifier side and VERIFY-QUERIES (src/pcs.lisp:581-657, 752-843) over the same keys (class, column
   count, cap and coefficients are read) */
int orc_pcs_verify_opening(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr,
                           const uint32_t *v, int grind_bits, int queries) {
  int fl = nv - FLOG > 0 ? nv - FLOG : 0, status = ORC_OK, nolv = 0, olv[32];
  if (nkeys < 1 || keys[nkeys - 1].c != nv || queries < 1) return ORC_E_PARAM;
  uint32_t prf[8] = {1}, claim[8];
  uint32_t *chal = (uint32_t *)calloc((size_t)(fl + 1) * 8, 4);
  uint8_t *caps[32];
  uint64_t cap_rows[32];
  memcpy(claim, v, 32);
  for (int i = 0; i < fl; i++) {
    uint32_t ev[24], s[8], e1[8], *x = chal + 8 * (size_t)i;
    uint64_t dims[2] = {3, 8};
    if ((status = orc_tr_send(tr, NULL, 2, dims, ev))) goto done0;
    orc_ext_add(8, ev, ev + 8, s);
    if (memcmp(s, claim, 32)) {
      status = ORC_E_REJECT;
      goto done0;
    }
    orc_tr_challenge(tr, 8, x);
    orc_lagrange(8, 3, ev, x, claim);
    orc_ext_eq1(8, rr + 8 * (size_t)i, x, e1);
    orc_ext_mul(8, prf, e1, prf);
    int l = i + 1;
    if (l >= 2 && l < fl && l % 2 == 0) {
      uint64_t got = 0;
      caps[nolv] = (uint8_t *)malloc(32 * 128);
      if ((status = orc_tr_send_bytes(tr, NULL, -1, caps[nolv], 32 * 128, &got))) {
        free(caps[nolv]);
        goto done0;
      }
      cap_rows[nolv] = got / 32;
      olv[nolv++] = l;
    }
  }
  uint64_t mlen = (uint64_t)1 << (nv - fl);
  uint32_t *m = (uint32_t *)malloc(mlen * 32);
  {
    uint64_t dims[2] = {mlen, 8};
    uint32_t mval[8], t[8];
    if ((status = orc_tr_send(tr, NULL, 2, dims, m))) goto done1;
    if (fl < nv)
      orc_mle_eval(8, nv - fl, m, 8, rr + 8 * (size_t)fl, mval);
    else
      memcpy(mval, m, 32);
    orc_ext_mul(8, prf, mval, t);
    if (memcmp(t, claim, 32)) {
      status = ORC_E_REJECT;
      goto done1;
    }
  }
  uint64_t nonce;
  if ((status = orc_tr_verify_grind(tr, grind_bits, &nonce))) goto done1;
  {
    const int Q = queries;
    uint64_t *qs = (uint64_t *)malloc(8 * (size_t)Q + 8);
    orc_tr_challenge_bits(tr, nv - 1, Q, qs);
    /* ---- VERIFY-QUERIES */
    uint32_t *oleaves[32] = {0};                                             /* per oracle: Q leaves of 8 rows of 4 */
    uint32_t *inj = (uint32_t *)calloc((size_t)nkeys * Q * 4 * 8, 4);        /* [key][query][symbol] EXT8 */
    for (int o = 0; o < nolv && !status; o++) { /* the oracles' leaves and paths, :763-774 */
      int l = olv[o];
      uint64_t nleaves = (uint64_t)1 << (nv - 1 - l);
      int depth = orc_cap_level(nleaves);
      uint64_t d3[3] = {(uint64_t)Q, 8, 4}, got = 0;
      oleaves[o] = (uint32_t *)malloc((size_t)Q * 32 * 4 + 4);
      uint8_t *paths = (uint8_t *)malloc((size_t)Q * depth * 32 + 1);
      status = orc_tr_record(tr, NULL, 3, d3, oleaves[o]);
      if (!status) status = orc_tr_record_bytes(tr, NULL, -1, paths, (uint64_t)Q * depth * 32 + 1, &got);
      if (!status && got != (uint64_t)Q * depth * 32) status = ORC_E_REJECT; /* "merkle path length" */
      if (!status && cap_rows[o] != nleaves >> depth) status = ORC_E_REJECT; /* "oracle opening shape" */
      for (int q = 0; q < Q && !status; q++) {
        uint8_t h[32];
        orc_leaf_digest(oleaves[o] + 32 * q, 8, NULL, h);
        if (!orc_check_path(h, paths + 32 * (size_t)q * depth, depth, qs[q] >> l, caps[o])) status = ORC_E_REJECT;
      }
      free(paths);
    }
    for (int k = 0; k < nkeys && !status; k++) { /* every key's leaves, then its tree's paths, :776-808 */
      const orc_open_key *key = &keys[k];
      int c = key->c, nc = key->ncols;
      uint64_t nleaves = (uint64_t)1 << (c - 1);
      int depth = orc_cap_level(nleaves);
      uint64_t d3[3] = {(uint64_t)Q, (uint64_t)nc, 4}, got = 0;
      uint32_t *leaves = (uint32_t *)malloc((size_t)Q * nc * 4 * 4 + 4);
      uint8_t *paths = (uint8_t *)malloc((size_t)Q * depth * 32 + 1);
      status = orc_tr_record(tr, NULL, 3, d3, leaves);
      if (!status) status = orc_tr_record_bytes(tr, NULL, -1, paths, (uint64_t)Q * depth * 32 + 1, &got);
      if (!status && got != (uint64_t)Q * depth * 32) status = ORC_E_REJECT;
      for (int q = 0; q < Q && !status; q++) {
        uint8_t h[32];
        orc_leaf_digest(leaves + (size_t)q * nc * 4, nc, NULL, h);
        if (!orc_check_path(h, paths + 32 * (size_t)q * depth, depth, qs[q] >> (nv - c), key->cap)) status = ORC_E_REJECT;
        for (int s = 0; s < 4; s++) { /* inj_c += sum_k coef_k leaf_k */
          uint32_t *held = inj + (((size_t)k * Q + q) * 4 + s) * 8, t[8];
          for (int col = 0; col < nc; col++) {
            orc_ext_scale(8, key->coef + 8 * (size_t)col, leaves[((size_t)q * nc + col) * 4 + s], t);
            orc_ext_add(8, held, t, held);
          }
        }
      }
      free(leaves);
      free(paths);
    }
    if (!status) { /* fold each query's symbols down to the final table's codeword, :810-843 */
      uint32_t *tw = (uint32_t *)malloc(orc_twiddles_size(nv + 1) * sizeof(uint32_t));
      orc_twiddles(nv + 1, tw);
      uint32_t *menc = (uint32_t *)malloc(2 * mlen * 32);
      encode_ext(m, nv - fl, menc);
      uint32_t inv2;
      orc_finv(2, &inv2);
      for (int q = 0; q < Q && !status; q++) {
        uint64_t base = 4 * qs[q];
        uint32_t held[4][8];
        int nheld = 4;
        memset(held, 0, sizeof(held));
        const uint32_t *tw_level = tw;
        for (int level = 0; level <= fl; level++) {
          if (level > 0) {
            int l = level - 1;
            for (int t2 = 0; t2 < nheld / 2; t2++) { /* RS:FOLD of the pair at twiddle index base / 2 + t2 */
              uint64_t s = base / 2 + (uint64_t)t2;
              uint32_t f0[8], f1[8], t[8], ix;
              orc_finv(orc_fmul(2, tw_level[s]), &ix);
              orc_ext_add(8, held[2 * t2], held[2 * t2 + 1], f0);
              orc_ext_scale(8, f0, inv2, f0);
              orc_ext_sub(8, held[2 * t2], held[2 * t2 + 1], f1);
              orc_ext_scale(8, f1, ix, f1);
              orc_ext_sub(8, f1, f0, t);
              orc_ext_mul(8, chal + 8 * (size_t)l, t, t);
              orc_ext_add(8, f0, t, held[t2]);
            }
            nheld /= 2;
            base /= 2;
            tw_level += (uint64_t)1 << (nv - l);
            for (int o = 0; o < nolv; o++)
              if (olv[o] == level) {
                const uint32_t *leaf = oleaves[o] + 32 * (size_t)q;
                uint64_t ob = 4 * (qs[q] >> level);
                uint32_t sym[4][8];
                for (int s = 0; s < 4; s++)
                  for (int d = 0; d < 8; d++) sym[s][d] = leaf[4 * d + s];
                if (memcmp(sym[base - ob], held[0], 32)) status = ORC_E_REJECT; /* "fold consistency" */
                memcpy(held, sym, sizeof(sym));
                nheld = 4;
                base = ob;
              }
          }
          for (int k = 0; k < nkeys; k++) /* INJECT, :817-823 */
            if (nv - keys[k].c == level) {
              uint64_t cb = 4 * (qs[q] >> level);
              for (int s = 0; s < nheld; s++)
                orc_ext_add(8, held[s], inj + (((size_t)k * Q + q) * 4 + (base - cb) + s) * 8, held[s]);
            }
        }
        for (int s = 0; s < nheld && !status; s++)
          if (memcmp(held[s], menc + (base + s) * 8, 32)) status = ORC_E_REJECT; /* "final codeword consistency" */
      }
      free(tw);
      free(menc);
    }
    for (int o = 0; o < nolv; o++) free(oleaves[o]);
    free(inj);
    free(qs);
  }
done1:
  free(m);
done0:
  for (int o = 0; o < nolv; o++) free(caps[o]);
  free(chal);
  return status;
}
