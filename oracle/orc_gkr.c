/* orc_gkr.c -- batched LogUp-GKR fractional sums, restated from src/gkr.lisp (test oracle; see orc.h). */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

static int block_bits(int k) { /* src/gkr.lisp:23-25: integer-length of k - 1 */
  int b = 0;
  for (int v = k - 1; v > 0; v >>= 1) b++;
  return b;
}

/* LAYER-STATEMENT, src/gkr.lisp:30-41: sum_l a_l p0 q1 + a_l p1 q0 + (a_l lambda) q0 q1, tables
   p0,p1,q0,q1 per lookup, constants a_l, a_l lambda per lookup.  With EXTRA = 1 the statement is
   (* bw statement): table 0 is bw and every other table index moves up by one. */
typedef struct {
  orc_stmt st;
  uint32_t *coeff;
  int32_t *start, *vars;
} layer_stmt;

static void layer_stmt_make(layer_stmt *ls, int lookups, int extra) {
  int T = 4 * lookups + extra, nterms = 3 * lookups, per = 3 + extra;
  ls->coeff = (uint32_t *)malloc(nterms * sizeof(uint32_t));
  ls->start = (int32_t *)malloc((nterms + 1) * sizeof(int32_t));
  ls->vars = (int32_t *)malloc((size_t)nterms * per * sizeof(int32_t));
  int k = 0;
  for (int l = 0; l < lookups; l++) {
    int p0 = extra + 4 * l, p1 = p0 + 1, q0 = p0 + 2, q1 = p0 + 3, a = T + 2 * l, al = a + 1;
    int terms[3][3] = {{a, p0, q1}, {a, p1, q0}, {al, q0, q1}};
    for (int t = 0; t < 3; t++) {
      ls->coeff[3 * l + t] = 1;
      ls->start[3 * l + t] = k;
      if (extra) ls->vars[k++] = 0;
      for (int v = 0; v < 3; v++) ls->vars[k++] = terms[t][v];
    }
  }
  ls->start[nterms] = k;
  memset(&ls->st, 0, sizeof(ls->st));
  ls->st.T = T;
  ls->st.C = 2 * lookups;
  ls->st.nterms = nterms;
  ls->st.coeff = ls->coeff;
  ls->st.start = ls->start;
  ls->st.vars = ls->vars;
}
static void layer_stmt_free(layer_stmt *ls) {
  free(ls->coeff);
  free(ls->start);
  free(ls->vars);
}

/* LAYER-CHALLENGES, src/gkr.lisp:43-51: a_l from one stream, then lambda; constants a_l, a_l lambda */
static void layer_challenges(orc_tr *tr, int D, int lookups, uint32_t *consts, uint32_t *as, uint32_t *lam) {
  orc_tr_challenges(tr, lookups, D, as);
  orc_tr_challenge(tr, D, lam);
  for (int l = 0; l < lookups; l++) {
    memcpy(consts + (size_t)(2 * l) * D, as + (size_t)l * D, D * sizeof(uint32_t));
    orc_ext_mul(D, as + (size_t)l * D, lam, consts + (size_t)(2 * l + 1) * D);
  }
}

/* LAYER-CLAIM, src/gkr.lisp:53-55 */
static void layer_claim(int D, int lookups, const uint32_t *as, const uint32_t *lam, const uint32_t *cp,
                        const uint32_t *cq, uint32_t *out) {
  uint32_t acc[ORC_MAXD] = {0}, t[ORC_MAXD];
  for (int l = 0; l < lookups; l++) {
    orc_ext_mul(D, lam, cq + (size_t)l * D, t);
    orc_ext_add(D, cp + (size_t)l * D, t, t);
    orc_ext_mul(D, as + (size_t)l * D, t, t);
    orc_ext_add(D, acc, t, acc);
  }
  memcpy(out, acc, D * sizeof(uint32_t));
}

static void fold_pair(int D, const uint32_t *lo, const uint32_t *hi, const uint32_t *r, uint32_t *out) {
  uint32_t t[ORC_MAXD];
  orc_ext_sub(D, hi, lo, t);
  orc_ext_mul(D, r, t, t);
  orc_ext_add(D, lo, t, out);
}

/* NEXT-CLAIMS, src/gkr.lisp:57-63; finals in the order p0,p1,q0,q1 per lookup */
static void next_claims(int D, int lookups, const uint32_t *finals, const uint32_t *tt, uint32_t *cp, uint32_t *cq) {
  for (int l = 0; l < lookups; l++) {
    const uint32_t *f = finals + (size_t)(4 * l) * D;
    fold_pair(D, f, f + D, tt, cp + (size_t)l * D);
    fold_pair(D, f + 2 * D, f + 3 * D, tt, cq + (size_t)l * D);
  }
}

/* PADDED-MASS, src/gkr.lisp:68-71 */
static void padded_mass(int D, int lk, int K, const uint32_t *rb, uint32_t *out) {
  uint64_t len = (uint64_t)1 << lk;
  uint32_t *e = (uint32_t *)malloc(len * D * sizeof(uint32_t));
  orc_eq_table(D, lk, rb, e);
  memset(out, 0, D * sizeof(uint32_t));
  for (uint64_t b = K; b < len; b++) orc_ext_add(D, out, e + b * D, out);
  free(e);
}

/* BLOCK-WEIGHTS, src/gkr.lisp:73-77 */
static uint32_t *block_weights(int D, int lk, int K, const uint32_t *rb) {
  uint64_t len = (uint64_t)1 << lk;
  uint32_t *e = (uint32_t *)calloc(len * D, sizeof(uint32_t));
  if (lk == 0)
    e[0] = 1;
  else
    orc_eq_table(D, lk, rb, e);
  (void)K;
  return e; /* the first K entries are the weights */
}

/* one in-block reduction, FRACTION-TREES src/gkr.lisp:157-170: children (b, x) and (b, x + 2^m) */
void orc_gkr_reduce_layer(int D, int K, int m, const uint32_t *p, const uint32_t *q, uint32_t *pp, uint32_t *qq) {
  uint64_t half = (uint64_t)1 << m;
  for (int b = 0; b < K; b++)
    for (uint64_t x = 0; x < half; x++) {
      uint64_t c0 = (uint64_t)b * 2 * half + x, c1 = c0 + half, o = (uint64_t)b * half + x;
      uint32_t t0[ORC_MAXD], t1[ORC_MAXD];
      orc_ext_mul(D, p + c0 * D, q + c1 * D, t0);
      orc_ext_mul(D, p + c1 * D, q + c0 * D, t1);
      orc_ext_add(D, t0, t1, pp + o * D);
      orc_ext_mul(D, q + c0 * D, q + c1 * D, qq + o * D);
    }
}

/* HALVES-PER-BLOCK, src/gkr.lisp:190-197 */
static void halves_per_block(int D, int K, uint64_t size, const uint32_t *v, uint32_t *lower, uint32_t *upper) {
  for (int b = 0; b < K; b++) {
    memcpy(lower + (uint64_t)b * size * D, v + (uint64_t)b * 2 * size * D, size * D * sizeof(uint32_t));
    memcpy(upper + (uint64_t)b * size * D, v + ((uint64_t)b * 2 * size + size) * D, size * D * sizeof(uint32_t));
  }
}

/* SEND-FINALS, src/gkr.lisp:208-213 */
static int send_finals(orc_tr *tr, int D, int ntables, const uint32_t *finals, uint32_t *tt) {
  uint64_t dims[2] = {1, (uint64_t)D};
  for (int t = 0; t < ntables; t++) {
    int status = orc_tr_send(tr, finals + (size_t)t * D, 2, dims, NULL);
    if (status) return status;
  }
  orc_tr_challenge(tr, D, tt);
  return ORC_OK;
}

static uint8_t *label_plus(const uint8_t *label, uint64_t len, const char *suffix, uint64_t *out_len) {
  uint64_t sl = strlen(suffix);
  uint8_t *l = (uint8_t *)malloc(len + sl + 1);
  memcpy(l, label, len);
  memcpy(l + len, suffix, sl);
  *out_len = len + sl;
  return l;
}

/* PROVE-UPPER, src/gkr.lisp:215-272 */
int orc_gkr_prove_upper(orc_tr *tr, int n, int K, int lookups, const uint32_t *const *leaves,
                        const uint8_t *label, uint64_t label_len, uint32_t *out_ri, uint32_t *out_rb,
                        uint32_t *out_cp, uint32_t *out_cq) {
  int D = orc_tr_degree(tr), lk = block_bits(K), L = lookups, status = ORC_OK;
  if (L < 1 || 4 * L + 1 > 16 || n < 0) return ORC_E_PARAM;
  uint64_t Kp = (uint64_t)1 << lk;
  /* FRACTION-TREES: layers[m][2l], layers[m][2l+1] = p, q of lookup l with K 2^m entries */
  uint32_t ***layers = (uint32_t ***)calloc(n + 1, sizeof(uint32_t **));
  for (int m = n; m >= 0; m--) {
    layers[m] = (uint32_t **)calloc(2 * L, sizeof(uint32_t *));
    for (int l = 0; l < L; l++) {
      uint64_t len = (uint64_t)K << m;
      uint32_t *p = (uint32_t *)malloc(len * D * sizeof(uint32_t)), *q = (uint32_t *)malloc(len * D * sizeof(uint32_t));
      if (m == n) {
        memcpy(p, leaves[2 * l], len * D * sizeof(uint32_t));
        memcpy(q, leaves[2 * l + 1], len * D * sizeof(uint32_t));
      } else {
        orc_gkr_reduce_layer(D, K, m, layers[m + 1][2 * l], layers[m + 1][2 * l + 1], p, q);
      }
      layers[m][2 * l] = p;
      layers[m][2 * l + 1] = q;
    }
  }
  /* the top tree over the block index, padded with 0/1 (:171-187) */
  uint32_t ***top = (uint32_t ***)calloc(lk + 1, sizeof(uint32_t **));
  for (int j = lk; j >= 0; j--) {
    top[j] = (uint32_t **)calloc(2 * L, sizeof(uint32_t *));
    uint64_t len = (uint64_t)1 << j;
    for (int l = 0; l < L; l++) {
      uint32_t *p = (uint32_t *)calloc(len * D, sizeof(uint32_t)), *q = (uint32_t *)calloc(len * D, sizeof(uint32_t));
      if (j == lk) {
        memcpy(p, layers[0][2 * l], (size_t)K * D * sizeof(uint32_t));
        memcpy(q, layers[0][2 * l + 1], (size_t)K * D * sizeof(uint32_t));
        for (uint64_t b = K; b < Kp; b++) q[b * D] = 1;
      } else {
        orc_gkr_reduce_layer(D, 1, j, top[j + 1][2 * l], top[j + 1][2 * l + 1], p, q);
      }
      top[j][2 * l] = p;
      top[j][2 * l + 1] = q;
    }
  }

  layer_stmt ls, ls_blk;
  layer_stmt_make(&ls, L, 0);
  layer_stmt_make(&ls_blk, L, 1);
  int NT = 4 * L;
  uint32_t *cp = out_cp, *cq = out_cq;
  uint32_t consts[2 * 4 * ORC_MAXD], as[4 * ORC_MAXD], lam[ORC_MAXD], tt[ORC_MAXD];
  uint32_t finals[17 * ORC_MAXD];
  uint32_t *r = (uint32_t *)calloc((size_t)(lk + n + 2) * D, sizeof(uint32_t));  /* top-tree point */
  uint32_t *ri = (uint32_t *)calloc((size_t)(n + 2) * D, sizeof(uint32_t));      /* in-block point */
  uint32_t *rho = (uint32_t *)calloc((size_t)(lk + n + 2) * D, sizeof(uint32_t));
  int r_len = 0, ri_len = 0;
  uint64_t dims2[2] = {2, (uint64_t)D};

  for (int l = 0; l < L; l++) { /* roots, :225-230 */
    uint32_t root[2 * ORC_MAXD];
    memcpy(root, top[0][2 * l], D * sizeof(uint32_t));
    memcpy(root + D, top[0][2 * l + 1], D * sizeof(uint32_t));
    if ((status = orc_tr_send(tr, root, 2, dims2, NULL))) goto done;
    memcpy(cp + (size_t)l * D, root, D * sizeof(uint32_t));
    memcpy(cq + (size_t)l * D, root + D, D * sizeof(uint32_t));
  }
  uint64_t tl;
  uint8_t *top_label = label_plus(label, label_len, "-top", &tl);
  uint64_t bl;
  uint8_t *blk_label = label_plus(label, label_len, "-blk", &bl);

  for (int j = 0; j < lk; j++) { /* the top tree, :232-241 */
    layer_challenges(tr, D, L, consts, as, lam);
    uint64_t size = (uint64_t)1 << j;
    uint32_t *tabs[16];
    const uint32_t *ctabs[16];
    int32_t strides[16];
    for (int l = 0; l < L; l++)
      for (int w = 0; w < 2; w++) {
        uint32_t *lo = (uint32_t *)malloc(size * D * sizeof(uint32_t)), *hi = (uint32_t *)malloc(size * D * sizeof(uint32_t));
        halves_per_block(D, 1, size, top[j + 1][2 * l + w], lo, hi);
        tabs[4 * l + 2 * w] = lo;
        tabs[4 * l + 2 * w + 1] = hi;
      }
    for (int t = 0; t < NT; t++) ctabs[t] = tabs[t], strides[t] = D;
    status = orc_sumcheck_prove(tr, j, &ls.st, ctabs, strides, j > 0 ? r : NULL, consts, top_label, tl, NULL, 1,
                                j > 0 ? 2 : 0, rho, finals, NULL);
    for (int t = 0; t < NT; t++) free(tabs[t]);
    if (status) goto done2;
    if ((status = send_finals(tr, D, NT, finals, tt))) goto done2;
    next_claims(D, L, finals, tt, cp, cq);
    memcpy(r, rho, (size_t)j * D * sizeof(uint32_t));
    memcpy(r + (size_t)j * D, tt, D * sizeof(uint32_t));
    r_len = j + 1;
  }
  {
    uint32_t *rb = (uint32_t *)calloc((size_t)(lk + 1) * D, sizeof(uint32_t));
    int rb_len = r_len;
    memcpy(rb, r, (size_t)r_len * D * sizeof(uint32_t));
    if (Kp != (uint64_t)K) { /* :244-246 */
      uint32_t mass[ORC_MAXD];
      padded_mass(D, lk, K, rb, mass);
      for (int l = 0; l < L; l++) orc_ext_sub(D, cq + (size_t)l * D, mass, cq + (size_t)l * D);
    }
    for (int layer = 0; layer < n - 1 && !status; layer++) { /* the in-block layers, :248-271 */
      layer_challenges(tr, D, L, consts, as, lam);
      uint32_t *bw = block_weights(D, rb_len, K, rb);
      uint64_t size = (uint64_t)1 << layer;
      uint32_t *tabs[16], *folded[16];
      const uint32_t *ctabs[17];
      int32_t strides[17];
      for (int l = 0; l < L; l++)
        for (int w = 0; w < 2; w++) {
          uint32_t *lo = (uint32_t *)malloc(K * size * D * sizeof(uint32_t)), *hi = (uint32_t *)malloc(K * size * D * sizeof(uint32_t));
          halves_per_block(D, K, size, layers[layer + 1][2 * l + w], lo, hi);
          tabs[4 * l + 2 * w] = lo;
          tabs[4 * l + 2 * w + 1] = hi;
        }
      for (int t = 0; t < NT; t++) {
        ctabs[t] = tabs[t];
        strides[t] = D;
        folded[t] = (uint32_t *)calloc(Kp * D, sizeof(uint32_t)); /* zero padded to 2^lk */
      }
      status = orc_sumcheck_prove(tr, layer, &ls.st, ctabs, strides, layer > 0 ? ri : NULL, consts, label, label_len,
                                  bw, K, layer > 0 ? 2 : 0, rho, finals, folded);
      int rbn_len = 0;
      uint32_t rbn[32 * ORC_MAXD];
      if (!status && lk > 0) { /* bind the block index, :257-267 */
        uint32_t *bwp = (uint32_t *)calloc(Kp * D, sizeof(uint32_t));
        memcpy(bwp, bw, (size_t)K * D * sizeof(uint32_t));
        ctabs[0] = bwp;
        strides[0] = D;
        for (int t = 0; t < NT; t++) ctabs[t + 1] = folded[t], strides[t + 1] = D;
        uint32_t f2[17 * ORC_MAXD];
        status = orc_sumcheck_prove(tr, lk, &ls_blk.st, ctabs, strides, NULL, consts, blk_label, bl, NULL, 1, -1,
                                    rbn, f2, NULL);
        memcpy(finals, f2 + D, (size_t)NT * D * sizeof(uint32_t)); /* finals of the tables (bw's is first) */
        rbn_len = lk;
        free(bwp);
      }
      for (int t = 0; t < NT; t++) {
        free(tabs[t]);
        free(folded[t]);
      }
      free(bw);
      if (status) break;
      if ((status = send_finals(tr, D, NT, finals, tt))) break;
      next_claims(D, L, finals, tt, cp, cq);
      memcpy(ri, rho, (size_t)layer * D * sizeof(uint32_t));
      memcpy(ri + (size_t)layer * D, tt, D * sizeof(uint32_t));
      ri_len = layer + 1;
      memcpy(rb, rbn, (size_t)rbn_len * D * sizeof(uint32_t));
      rb_len = rbn_len;
    }
    if (!status) {
      if (out_ri) memcpy(out_ri, ri, (size_t)ri_len * D * sizeof(uint32_t));
      if (out_rb) memcpy(out_rb, rb, (size_t)rb_len * D * sizeof(uint32_t));
    }
    free(rb);
  }
done2:
  free(top_label);
  free(blk_label);
done:
  layer_stmt_free(&ls);
  layer_stmt_free(&ls_blk);
  for (int m = 0; m <= n; m++) {
    for (int i = 0; i < 2 * L; i++) free(layers[m][i]);
    free(layers[m]);
  }
  free(layers);
  for (int j = 0; j <= lk; j++) {
    for (int i = 0; i < 2 * L; i++) free(top[j][i]);
    free(top[j]);
  }
  free(top);
  free(r);
  free(ri);
  free(rho);
  return status;
}

static int receive_finals(orc_tr *tr, int D, int ntables, uint32_t *finals, uint32_t *tt) { /* :84-89 */
  uint64_t dims[2] = {1, (uint64_t)D};
  for (int t = 0; t < ntables; t++) {
    int status = orc_tr_send(tr, NULL, 2, dims, finals + (size_t)t * D);
    if (status) return status;
  }
  orc_tr_challenge(tr, D, tt);
  return ORC_OK;
}

/* VERIFY-UPPER, src/gkr.lisp:91-145 */
int orc_gkr_verify_upper(orc_tr *tr, int n, int K, int lookups, const uint8_t *label, uint64_t label_len,
                         uint32_t *out_roots, uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp,
                         uint32_t *out_cq) {
  int D = orc_tr_degree(tr), lk = block_bits(K), L = lookups, status = ORC_OK;
  if (L < 1 || 4 * L + 1 > 16) return ORC_E_PARAM;
  uint64_t Kp = (uint64_t)1 << lk;
  int NT = 4 * L;
  uint32_t *cp = out_cp, *cq = out_cq;
  uint64_t dims2[2] = {2, (uint64_t)D};
  for (int l = 0; l < L; l++) {
    uint32_t root[2 * ORC_MAXD];
    if ((status = orc_tr_send(tr, NULL, 2, dims2, root))) return status;
    if (out_roots) memcpy(out_roots + (size_t)l * 2 * D, root, 2 * D * sizeof(uint32_t));
    memcpy(cp + (size_t)l * D, root, D * sizeof(uint32_t));
    memcpy(cq + (size_t)l * D, root + D, D * sizeof(uint32_t));
  }
  layer_stmt ls, ls_blk;
  layer_stmt_make(&ls, L, 0);
  layer_stmt_make(&ls_blk, L, 1);
  uint64_t tl, bl;
  uint8_t *top_label = label_plus(label, label_len, "-top", &tl);
  uint8_t *blk_label = label_plus(label, label_len, "-blk", &bl);
  uint32_t consts[2 * 4 * ORC_MAXD], as[4 * ORC_MAXD], lam[ORC_MAXD], tt[ORC_MAXD], claim[ORC_MAXD];
  uint32_t reduced[ORC_MAXD], expected[ORC_MAXD], finals[17 * ORC_MAXD];
  uint32_t *r = (uint32_t *)calloc((size_t)(lk + n + 2) * D, sizeof(uint32_t));
  uint32_t *ri = (uint32_t *)calloc((size_t)(n + 2) * D, sizeof(uint32_t));
  uint32_t *rho = (uint32_t *)calloc((size_t)(lk + n + 2) * D, sizeof(uint32_t));
  uint32_t *rb = (uint32_t *)calloc((size_t)(lk + 1) * D, sizeof(uint32_t));
  int r_len = 0, ri_len = 0, rb_len = 0;

  for (int j = 0; j < lk; j++) { /* the top tree, :107-116 */
    layer_challenges(tr, D, L, consts, as, lam);
    layer_claim(D, L, as, lam, cp, cq, claim);
    if ((status = orc_sumcheck_verify(tr, j, &ls.st, claim, j > 0 ? r : NULL, consts, 1, top_label, tl,
                                      j > 0 ? 2 : 0, rho, reduced)))
      goto done;
    if ((status = receive_finals(tr, D, NT, finals, tt))) goto done;
    orc_stmt_eval(&ls.st, D, finals, consts, expected);
    if (memcmp(reduced, expected, D * sizeof(uint32_t))) {
      status = ORC_E_REJECT; /* :gkr-top */
      goto done;
    }
    next_claims(D, L, finals, tt, cp, cq);
    memcpy(r, rho, (size_t)j * D * sizeof(uint32_t));
    memcpy(r + (size_t)j * D, tt, D * sizeof(uint32_t));
    r_len = j + 1;
  }
  memcpy(rb, r, (size_t)r_len * D * sizeof(uint32_t));
  rb_len = r_len;
  if (Kp != (uint64_t)K) { /* :120-122 */
    uint32_t mass[ORC_MAXD];
    padded_mass(D, lk, K, rb, mass);
    for (int l = 0; l < L; l++) orc_ext_sub(D, cq + (size_t)l * D, mass, cq + (size_t)l * D);
  }
  for (int layer = 0; layer < n - 1; layer++) { /* the in-block layers, :124-144 */
    layer_challenges(tr, D, L, consts, as, lam);
    uint32_t *bw = block_weights(D, rb_len, K, rb);
    layer_claim(D, L, as, lam, cp, cq, claim);
    status = orc_sumcheck_verify(tr, layer, &ls.st, claim, layer > 0 ? ri : NULL, consts, K, label, label_len,
                                 layer > 0 ? 2 : 0, rho, reduced);
    uint32_t rbn[32 * ORC_MAXD];
    int rbn_len = 0;
    if (!status && lk > 0) {
      uint32_t red2[ORC_MAXD];
      status = orc_sumcheck_verify(tr, lk, &ls_blk.st, reduced, NULL, consts, 1, blk_label, bl, -1, rbn, red2);
      memcpy(reduced, red2, sizeof(red2));
      rbn_len = lk;
    }
    if (!status) status = receive_finals(tr, D, NT, finals, tt);
    if (!status) {
      uint32_t weight[ORC_MAXD] = {0}, t[ORC_MAXD];
      if (K > 1) { /* sum_b bw_b eq(rbn, b), :136-138 */
        uint32_t *e = (uint32_t *)malloc(Kp * D * sizeof(uint32_t));
        orc_eq_table(D, lk, rbn, e);
        for (int b = 0; b < K; b++) {
          orc_ext_mul(D, bw + (size_t)b * D, e + (size_t)b * D, t);
          orc_ext_add(D, weight, t, weight);
        }
        free(e);
      } else {
        memcpy(weight, bw, D * sizeof(uint32_t));
      }
      orc_stmt_eval(&ls.st, D, finals, consts, expected);
      orc_ext_mul(D, weight, expected, expected);
      if (memcmp(reduced, expected, D * sizeof(uint32_t))) status = ORC_E_REJECT; /* :gkr-layer */
    }
    free(bw);
    if (status) goto done;
    next_claims(D, L, finals, tt, cp, cq);
    memcpy(ri, rho, (size_t)layer * D * sizeof(uint32_t));
    memcpy(ri + (size_t)layer * D, tt, D * sizeof(uint32_t));
    ri_len = layer + 1;
    memcpy(rb, rbn, (size_t)rbn_len * D * sizeof(uint32_t));
    rb_len = rbn_len;
  }
  if (out_ri) memcpy(out_ri, ri, (size_t)ri_len * D * sizeof(uint32_t));
  if (out_rb) memcpy(out_rb, rb, (size_t)rb_len * D * sizeof(uint32_t));
done:
  free(top_label);
  free(blk_label);
  layer_stmt_free(&ls);
  layer_stmt_free(&ls_blk);
  free(r);
  free(ri);
  free(rho);
  free(rb);
  return status;
}
