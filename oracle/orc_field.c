/* orc_field.c -- KoalaBear and its tower, restated from src/field.lisp (test oracle; see orc.h). */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

#define P ORC_P

/* src/field.lisp:50-72 */
uint32_t orc_fadd(uint32_t a, uint32_t b) {
  int64_t s = (int64_t)a + b - P;
  return (uint32_t)(s + (P & (s >> 63)));
}
uint32_t orc_fsub(uint32_t a, uint32_t b) {
  int64_t d = (int64_t)a - b;
  return (uint32_t)(d + (P & (d >> 63)));
}
uint32_t orc_fmul(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) % P); }

/* src/field.lisp:74-82 */
uint32_t orc_fpow(uint32_t a, uint64_t e) {
  uint32_t result = 1, base = a % P;
  for (; e; e >>= 1) {
    if (e & 1) result = orc_fmul(result, base);
    base = orc_fmul(base, base);
  }
  return result;
}

/* src/field.lisp:84-96: the inverse of zero is an error; *out = 0 is the RETURN-ZERO restart */
int orc_finv(uint32_t a, uint32_t *out) {
  a %= P;
  if (!a) {
    *out = 0;
    return ORC_E_DIVZERO;
  }
  *out = orc_fpow(a, P - 2);
  return ORC_OK;
}

static uint32_t times3(uint32_t a) { return orc_fadd(orc_fadd(a, a), a); } /* field.lisp:65-68 */

void orc_ext_add(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) {
  for (int i = 0; i < D; i++) out[i] = orc_fadd(a[i], b[i]);
}
void orc_ext_sub(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) {
  for (int i = 0; i < D; i++) out[i] = orc_fsub(a[i], b[i]);
}
void orc_ext_neg(int D, const uint32_t *a, uint32_t *out) {
  for (int i = 0; i < D; i++) out[i] = orc_fsub(0, a[i]);
}
void orc_ext_scale(int D, const uint32_t *a, uint32_t s, uint32_t *out) {
  s %= P;
  for (int i = 0; i < D; i++) out[i] = orc_fmul(a[i], s);
}

static int bit_reverse(int i, int bits) { /* field.lisp:195-197 */
  int r = 0;
  for (int b = 0; b < bits; b++) r |= ((i >> b) & 1) << (bits - 1 - b);
  return r;
}
static int log2i(int d) {
  int b = 0;
  while ((1 << b) < d) b++;
  return b;
}

/* MUL*, src/field.lisp:213-234: the schoolbook product in F_p[w]/(w^d - 3) on the power-ordered
   coordinates, the wrapping b's tripled first, each coefficient reduced once per four products
   (four products below p^2 fit an unsigned 64-bit word).  d: any power of two up to 8. */
static void mul_star(int d, const uint32_t *a_t, const uint32_t *b_t, uint32_t *out_t) {
  int bits = log2i(d);
  uint32_t a[ORC_MAXD], b[ORC_MAXD], b3[ORC_MAXD], c[ORC_MAXD];
  for (int e = 0; e < d; e++) {
    a[e] = a_t[bit_reverse(e, bits)];
    b[e] = b_t[bit_reverse(e, bits)];
  }
  for (int j = 1; j < d; j++) b3[j] = times3(b[j]);
  for (int e = 0; e < d; e++) {
    uint32_t sum = 0;
    int have = 0;
    uint64_t acc = 0;
    int in_acc = 0;
    for (int i = 0; i < d; i++) {
      int j = ((e - i) % d + d) % d;
      acc += (uint64_t)a[i] * (i > e ? b3[j] : b[j]);
      if (++in_acc == 4 || i == d - 1) {
        uint32_t r = (uint32_t)(acc % P);
        sum = have ? orc_fadd(sum, r) : r;
        have = 1;
        acc = 0;
        in_acc = 0;
      }
    }
    c[e] = sum;
  }
  for (int e = 0; e < d; e++) out_t[e] = c[bit_reverse(e, bits)];
}

void orc_ext_mul_plain(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) { mul_star(D, a, b, out); }
void orc_ext_mul(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) {
  if (D == 4)
    orc_ext_mul4(a, b, out);
  else if (D == 8)
    orc_ext_mul8(a, b, out);
  else
    mul_star(D, a, b, out);
}

/* A w for the generator w of A's level, src/field.lisp:206-211 */
static void mul_by_generator(int d, const uint32_t *a, uint32_t *out) {
  if (d == 1) {
    out[0] = times3(a[0]);
    return;
  }
  int h = d / 2;
  uint32_t tmp[ORC_MAXD];
  mul_by_generator(h, a + h, tmp);
  memcpy(tmp + h, a, h * sizeof(uint32_t));
  memcpy(out, tmp, d * sizeof(uint32_t));
}

/* INV*, src/field.lisp:236-243: (A0 + A1 w)^-1 = (A0 - A1 w) / (A0^2 - A1^2 w^2) */
static void inv_star(int d, const uint32_t *a, uint32_t *out) {
  if (d == 1) {
    orc_finv(a[0], out);
    return;
  }
  int h = d / 2;
  const uint32_t *a0 = a, *a1 = a + h;
  uint32_t s0[ORC_MAXD], s1[ORC_MAXD], g[ORC_MAXD], norm[ORC_MAXD], ninv[ORC_MAXD], r[ORC_MAXD];
  mul_star(h, a0, a0, s0);
  mul_star(h, a1, a1, s1);
  mul_by_generator(h, s1, g);
  orc_ext_sub(h, s0, g, norm);
  inv_star(h, norm, ninv);
  mul_star(h, a0, ninv, r);
  mul_star(h, a1, ninv, s1);
  orc_ext_neg(h, s1, r + h);
  memcpy(out, r, d * sizeof(uint32_t));
}

/* src/field.lisp:291-302 */
int orc_ext_inv(int D, const uint32_t *a, uint32_t *out) {
  int nonzero = 0;
  for (int i = 0; i < D; i++) nonzero |= a[i] != 0;
  if (!nonzero) {
    memset(out, 0, D * sizeof(uint32_t));
    return ORC_E_DIVZERO;
  }
  inv_star(D, a, out);
  return ORC_OK;
}

/* eq(a, b) = a b + (1 - a)(1 - b), src/field.lisp:314-317 */
void orc_ext_eq1(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) {
  uint32_t one[ORC_MAXD] = {1}, ab[ORC_MAXD], na[ORC_MAXD], nb[ORC_MAXD], t[ORC_MAXD];
  orc_ext_mul(D, a, b, ab);
  orc_ext_sub(D, one, a, na);
  orc_ext_sub(D, one, b, nb);
  orc_ext_mul(D, na, nb, t);
  orc_ext_add(D, ab, t, out);
}

/* prod_k eq(a_k, b_k), src/field.lisp:319-321 */
void orc_ext_eq(int D, int k, const uint32_t *as, const uint32_t *bs, uint32_t *out) {
  uint32_t acc[ORC_MAXD] = {1}, e[ORC_MAXD];
  for (int i = 0; i < k; i++) {
    orc_ext_eq1(D, as + (size_t)i * D, bs + (size_t)i * D, e);
    orc_ext_mul(D, acc, e, acc);
  }
  memcpy(out, acc, D * sizeof(uint32_t));
}

/* src/field.lisp:327-352: sum_i w_i v_i prod_{j /= i} (x - j), w_i = 1 / prod_{j /= i} (i - j) */
void orc_lagrange(int D, int count, const uint32_t *values, const uint32_t *x, uint32_t *out) {
  int d = count - 1;
  uint32_t xm[16][ORC_MAXD];
  uint32_t acc[ORC_MAXD] = {0};
  for (int j = 0; j <= d; j++) {
    uint32_t jj[ORC_MAXD] = {0};
    jj[0] = (uint32_t)j;
    orc_ext_sub(D, x, jj, xm[j]);
  }
  for (int i = 0; i <= d; i++) {
    uint32_t w = 1, term[ORC_MAXD];
    for (int j = 0; j <= d; j++)
      if (j != i) w = orc_fmul(w, (uint32_t)(((int64_t)(i - j) % P + P) % P));
    orc_finv(w, &w);
    memcpy(term, values + (size_t)i * D, D * sizeof(uint32_t));
    for (int j = 0; j <= d; j++)
      if (j != i) orc_ext_mul(D, term, xm[j], term);
    orc_ext_scale(D, term, w, term);
    orc_ext_add(D, acc, term, acc);
  }
  memcpy(out, acc, D * sizeof(uint32_t));
}

/* src/field.lisp:354-363: each variable maps e -> (e - e r_b, e r_b), upper half appended */
void orc_eq_table(int D, int k, const uint32_t *r, uint32_t *out) {
  memset(out, 0, D * sizeof(uint32_t));
  out[0] = 1;
  uint64_t len = 1;
  for (int b = 0; b < k; b++) {
    const uint32_t *rb = r + (size_t)b * D;
    for (uint64_t i = 0; i < len; i++) {
      uint32_t *e = out + i * D, *u = out + (len + i) * D;
      orc_ext_mul(D, e, rb, u);
      orc_ext_sub(D, e, u, e);
    }
    len *= 2;
  }
}

/* src/field.lisp:365-370 */
void orc_fold_table(int D, uint64_t len, const uint32_t *table, const uint32_t *r, uint32_t *out) {
  for (uint64_t i = 0; i < len / 2; i++) {
    const uint32_t *lo = table + 2 * i * D, *hi = lo + D;
    uint32_t t[ORC_MAXD];
    orc_ext_sub(D, hi, lo, t);
    orc_ext_mul(D, r, t, t);
    orc_ext_add(D, lo, t, out + i * D);
  }
}

/* src/field.lisp:372-377; stride 1: base values, stride D: EXTs */
void orc_mle_eval(int D, int k, const uint32_t *values, int stride, const uint32_t *r, uint32_t *out) {
  uint64_t len = (uint64_t)1 << k;
  uint32_t *t = (uint32_t *)calloc(len * D, sizeof(uint32_t));
  for (uint64_t i = 0; i < len; i++) {
    if (stride == 1)
      t[i * D] = values[i] % P;
    else
      memcpy(t + i * D, values + i * D, D * sizeof(uint32_t));
  }
  for (int b = 0; b < k; b++) {
    orc_fold_table(D, len, t, r + (size_t)b * D, t); /* in place: entry i is written after 2i, 2i+1 are read */
    len /= 2;
  }
  memcpy(out, t, D * sizeof(uint32_t));
  free(t);
}
