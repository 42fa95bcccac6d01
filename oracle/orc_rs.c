/* orc_rs.c -- the rate-1/2 Reed-Solomon code over KoalaBear, restated from src/rs.lisp
 * (test oracle; see orc.h). */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

/* src/rs.lisp:24-28: w_k = 3^((p-1)/2^k), k <= 24 */
int orc_root_of_unity(int k, uint32_t *out) {
  if (k < 0 || k > 24) return ORC_E_PARAM;
  *out = orc_fpow(3, (uint64_t)(ORC_P - 1) >> k);
  return ORC_OK;
}

static uint64_t bitrev(uint64_t i, int bits) { /* src/rs.lisp:30-33 */
  uint64_t r = 0;
  for (int b = 0; b < bits; b++) r |= ((i >> b) & 1) << (bits - 1 - b);
  return r;
}

/* the powers w^0..w^(len-1) in bit-reversed order (src/rs.lisp:35-42) */
static void bitrev_powers(uint32_t w, int bits, uint32_t *out) {
  uint64_t len = (uint64_t)1 << bits;
  uint32_t x = 1;
  for (uint64_t i = 0; i < len; i++) {
    out[bitrev(i, bits)] = x;
    x = orc_fmul(x, w);
  }
}

uint64_t orc_twiddles_size(int n) {
  int levels = n - 1 > 1 ? n - 1 : 1;
  uint64_t total = 0, len = (uint64_t)1 << (n - 1);
  for (int l = 0; l < levels; l++, len /= 2) total += len;
  return total;
}

/* src/rs.lisp:44-55: level 0 = bit-reversed powers of w_n, level l+1[s] = level l[2s]^2 */
void orc_twiddles(int n, uint32_t *out) {
  uint32_t w;
  orc_root_of_unity(n, &w);
  bitrev_powers(w, n - 1, out);
  int levels = n - 1 > 1 ? n - 1 : 1;
  uint32_t *level = out;
  uint64_t len = (uint64_t)1 << (n - 1);
  for (int l = 1; l < levels; l++) {
    uint32_t *next = level + len;
    for (uint64_t i = 0; i < len; i += 2) next[i / 2] = orc_fmul(level[i], level[i]);
    level = next;
    len /= 2;
  }
}

void orc_domain_points(int n, uint32_t *out) { /* src/rs.lisp:57-58 */
  uint32_t w;
  orc_root_of_unity(n, &w);
  bitrev_powers(w, n, out);
}

/* FFT, src/rs.lisp:60-73, on twiddle levels from `level`; tw_levels[l] points at level l */
static void fft(uint32_t *x, uint32_t *const *tw_levels, int level, int size_bits) {
  for (int b = size_bits - 2; b >= 0; b--) {
    uint64_t half = (uint64_t)1 << b;
    const uint32_t *tw = tw_levels[level + b];
    uint64_t nblocks = ((uint64_t)1 << size_bits) / (2 * half);
    for (uint64_t k = 0; k < nblocks; k++) {
      uint32_t tg = tw[k];
      uint64_t base = k * 2 * half;
      for (uint64_t i = base; i < base + half; i++) {
        uint32_t a = x[i], tc = orc_fmul(tg, x[i + half]);
        x[i] = orc_fadd(a, tc);
        x[i + half] = orc_fsub(a, tc);
      }
    }
  }
}

/* ENCODE, src/rs.lisp:75-85: x = m || m, then the butterflies */
int orc_rs_encode(const uint32_t *message, int n, uint32_t *codeword) {
  if (n < 1 || n > 24) return ORC_E_PARAM;
  uint64_t half = (uint64_t)1 << (n - 1);
  for (uint64_t i = 0; i < half; i++) codeword[i] = codeword[half + i] = message[i] % ORC_P;
  uint32_t *tw = (uint32_t *)malloc(orc_twiddles_size(n) * sizeof(uint32_t));
  orc_twiddles(n, tw);
  uint32_t *levels[32];
  uint32_t *p = tw;
  uint64_t len = half;
  int nlevels = n - 1 > 1 ? n - 1 : 1;
  for (int l = 0; l < nlevels; l++, len /= 2) {
    levels[l] = p;
    p += len;
  }
  fft(codeword, levels, 0, n);
  free(tw);
  return ORC_OK;
}

/* BRUTE-EVAL, src/rs.lisp:87-91: Horner on the domain points */
void orc_rs_brute_eval(const uint32_t *message, int n, uint32_t *out) {
  uint64_t len = (uint64_t)1 << n, mlen = len / 2;
  uint32_t *pts = (uint32_t *)malloc(len * sizeof(uint32_t));
  orc_domain_points(n, pts);
  for (uint64_t t = 0; t < len; t++) {
    uint32_t acc = 0;
    for (uint64_t j = mlen; j-- > 0;) acc = orc_fadd(orc_fmul(acc, pts[t]), message[j] % ORC_P);
    out[t] = acc;
  }
  free(pts);
}

/* FOLD, src/rs.lisp:93-101: f0 = (a + b)/2, f1 = (a - b)/(2x), out = f0 + (f1 - f0) r */
void orc_rs_fold(int D, uint64_t m, const uint32_t *codeword, const uint32_t *twiddle_level,
                 const uint32_t *r, uint32_t *out) {
  uint32_t inv2;
  orc_finv(2, &inv2);
  for (uint64_t s = 0; s < m; s++) {
    const uint32_t *a = codeword + 2 * s * D, *b = a + D;
    uint32_t f0[ORC_MAXD], f1[ORC_MAXD], t[ORC_MAXD], ix;
    orc_finv(orc_fmul(2, twiddle_level[s]), &ix);
    orc_ext_add(D, a, b, f0);
    orc_ext_scale(D, f0, inv2, f0);
    orc_ext_sub(D, a, b, f1);
    orc_ext_scale(D, f1, ix, f1);
    orc_ext_sub(D, f1, f0, t);
    if (D == 1)
      t[0] = orc_fmul(t[0], r[0]);
    else
      orc_ext_mul(D, t, r, t);
    orc_ext_add(D, f0, t, out + s * D);
  }
}
