/* orc_fast.c -- the sumcheck prover's round sums and fold once more, organised the way the reference's
 * compiled round kernel is (test oracle; see orc.h): the statement as straight-line code in its written shape
 * (ARITHMETIC-FORM / IN-PLACE-CODE, src/forms.lisp:113-185) instead of its monomial expansion, the tables' lines
 * by addition (src/sumcheck.lisp:236-242, 248-253), base-field lines and statement with one EXT-SCALE per point
 * when every table is a base table and there are no constants (:236-246, :552-553), extension products with one
 * reduction per four products (src/field.lisp:213-218) unrolled for D = 4 and 8, and the HIGH blocks (or, with few
 * of them, ranges of LOW) spread over threads.
 *
 * Every value here is a canonical residue of an exact field computation, so these functions return the very words
 * orc_round_sums / orc_fold_flat return; tests/test_oracle_fast.py checks that on every shape, and the plain
 * functions are the ones the reference's golden proofs pin.  orc_set_fast(threads) makes orc_sumcheck_prove (and
 * through it the GKR and opening provers) use this path: it is what the benchmark times as the CPU baseline and
 * what writes the full-size fixtures.
 */
#include "orc.h"
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define P ORC_P
#define INLINE static inline __attribute__((always_inline))

static int g_fast_threads = 0;
void orc_set_fast(int threads) { g_fast_threads = threads < 0 ? 0 : threads; }
int orc_fast_threads(void) { return g_fast_threads; }
int orc_host_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

INLINE uint32_t fadd(uint32_t a, uint32_t b) {
  uint32_t s = a + b;
  return s >= P ? s - P : s;
}
INLINE uint32_t fsub(uint32_t a, uint32_t b) { return a >= b ? a - b : a + P - b; }
INLINE uint32_t fmul(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) % P); }

/* tower index <-> power index: bit reversal over log2 D bits (src/field.lisp:195-204) */
INLINE int brev(const int D, int i) {
  return D == 4 ? (((i & 1) << 1) | ((i >> 1) & 1)) : D == 8 ? (((i & 1) << 2) | (i & 2) | ((i >> 2) & 1)) : i;
}

/* MUL* unrolled (src/field.lisp:213-234); out may alias a or b */
INLINE void mulD(const int D, const uint32_t *at, const uint32_t *bt, uint32_t *ot) {
  uint32_t a[8], b[8], b3[8], c[8];
#pragma GCC unroll 8
  for (int e = 0; e < D; e++) a[e] = at[brev(D, e)], b[e] = bt[brev(D, e)];
#pragma GCC unroll 8
  for (int j = 1; j < D; j++) b3[j] = fadd(fadd(b[j], b[j]), b[j]);
#pragma GCC unroll 8
  for (int e = 0; e < D; e++) {
    uint64_t acc = 0;
    uint32_t sum = 0;
#pragma GCC unroll 8
    for (int i = 0; i < D; i++) {
      int j = (e - i) & (D - 1);
      acc += (uint64_t)a[i] * (i > e ? b3[j] : b[j]);
      if ((i & 3) == 3) {
        uint32_t r = (uint32_t)(acc % P);
        sum = i == 3 ? r : fadd(sum, r);
        acc = 0;
      }
    }
    c[e] = sum;
  }
#pragma GCC unroll 8
  for (int e = 0; e < D; e++) ot[brev(D, e)] = c[e];
}
INLINE void addD(const int D, const uint32_t *a, const uint32_t *b, uint32_t *o) {
#pragma GCC unroll 8
  for (int i = 0; i < D; i++) o[i] = fadd(a[i], b[i]);
}
INLINE void subD(const int D, const uint32_t *a, const uint32_t *b, uint32_t *o) {
#pragma GCC unroll 8
  for (int i = 0; i < D; i++) o[i] = fsub(a[i], b[i]);
}

/* the unrolled products, for the rest of the oracle */
void orc_ext_mul4(const uint32_t *a, const uint32_t *b, uint32_t *out) { mulD(4, a, b, out); }
void orc_ext_mul8(const uint32_t *a, const uint32_t *b, uint32_t *out) { mulD(8, a, b, out); }

/* ---- the statement as a postfix program.  ops: 0 table, 1 constant, 2 integer (arg = value mod p), 3 +, 4 -,
   5 *, 6 unary -.  An n-ary chain arrives as its left-to-right binary reduction (src/forms.lisp:124-127). */
enum { OP_TABLE = 0, OP_CONST, OP_INT, OP_ADD, OP_SUB, OP_MUL, OP_NEG };
#define STACK 24

INLINE void eval_ext(const int D, const orc_stmt *st, const uint32_t *const *tv, const uint32_t *consts, uint32_t *out) {
  if (st->nops > 0) {
    uint32_t stack[STACK][8];
    int sp = 0;
    for (int k = 0; k < st->nops; k++) {
      const int32_t a = st->args[k];
      switch (st->ops[k]) {
        case OP_TABLE: memcpy(stack[sp++], tv[a], D * 4); break;
        case OP_CONST: memcpy(stack[sp++], consts + (size_t)a * D, D * 4); break;
        case OP_INT:
          memset(stack[sp], 0, D * 4);
          stack[sp++][0] = (uint32_t)a;
          break;
        case OP_ADD: sp--, addD(D, stack[sp - 1], stack[sp], stack[sp - 1]); break;
        case OP_SUB: sp--, subD(D, stack[sp - 1], stack[sp], stack[sp - 1]); break;
        case OP_MUL: sp--, mulD(D, stack[sp - 1], stack[sp], stack[sp - 1]); break;
        default: {
          uint32_t z[8] = {0};
          subD(D, z, stack[sp - 1], stack[sp - 1]);
        }
      }
    }
    memcpy(out, stack[0], D * 4);
    return;
  }
  uint32_t acc[8] = {0};
  for (int t = 0; t < st->nterms; t++) {
    uint32_t term[8] = {1};
    for (int k = st->start[t]; k < st->start[t + 1]; k++) {
      int v = st->vars[k];
      mulD(D, term, v < st->T ? tv[v] : consts + (size_t)(v - st->T) * D, term);
    }
    if (st->coeff[t] != 1) {
#pragma GCC unroll 8
      for (int c = 0; c < D; c++) term[c] = fmul(term[c], st->coeff[t]);
    }
    addD(D, acc, term, acc);
  }
  memcpy(out, acc, D * 4);
}

static uint32_t eval_base(const orc_stmt *st, const uint32_t *tv) {
  if (st->nops > 0) {
    uint32_t stack[STACK];
    int sp = 0;
    for (int k = 0; k < st->nops; k++) {
      const int32_t a = st->args[k];
      switch (st->ops[k]) {
        case OP_TABLE: stack[sp++] = tv[a]; break;
        case OP_INT: stack[sp++] = (uint32_t)a; break;
        case OP_ADD: sp--, stack[sp - 1] = fadd(stack[sp - 1], stack[sp]); break;
        case OP_SUB: sp--, stack[sp - 1] = fsub(stack[sp - 1], stack[sp]); break;
        case OP_MUL: sp--, stack[sp - 1] = fmul(stack[sp - 1], stack[sp]); break;
        case OP_NEG: stack[sp - 1] = fsub(0, stack[sp - 1]); break;
        default: stack[sp++] = 0; /* a constant: base mode has none */
      }
    }
    return stack[0];
  }
  uint32_t acc = 0;
  for (int t = 0; t < st->nterms; t++) {
    uint32_t term = st->coeff[t];
    for (int k = st->start[t]; k < st->start[t + 1]; k++) term = fmul(term, tv[st->vars[k]]);
    acc = fadd(acc, term);
  }
  return acc;
}

/* one block h, LOW entries [l0, l1): inner[k] += LOW[l] * F(lines at X_k)   (src/sumcheck.lisp:230-255) */
INLINE void block_range(const int D, const int BASE, const orc_stmt *st, int points, uint64_t n_low, uint64_t h,
                        uint64_t l0, uint64_t l1, const uint32_t *const *tables, const int32_t *strides,
                        const uint32_t *low, const uint32_t *consts, uint32_t (*inner)[8]) {
  const int T = st->T;
  for (uint64_t l = l0; l < l1; l++) {
    const uint64_t i = h * n_low + l;
    const uint32_t *w = low + l * D;
    if (BASE) {
      uint32_t lines[16][18];
      for (int t = 0; t < T; t++) {
        const uint32_t lo = tables[t][2 * i], hi = tables[t][2 * i + 1], s = fsub(hi, lo);
        lines[t][0] = lo, lines[t][1] = hi;
        for (int x = 2; x <= points; x++) lines[t][x] = fadd(lines[t][x - 1], s);
      }
      for (int k = 0; k < points; k++) {
        const int x = k == 0 ? 0 : k + 1;
        uint32_t tv[16];
        for (int t = 0; t < T; t++) tv[t] = lines[t][x];
        const uint32_t f = eval_base(st, tv);
#pragma GCC unroll 8
        for (int c = 0; c < D; c++) inner[k][c] = fadd(inner[k][c], fmul(w[c], f)); /* EXT-SCALE, :245-246 */
      }
    } else {
      uint32_t lines[16][18][8], slope[8], f[8];
      for (int t = 0; t < T; t++) {
        if (strides[t] == 1) { /* TABLE-ENTRY lifts a base value, :75-82 */
          memset(lines[t][0], 0, D * 4), memset(lines[t][1], 0, D * 4);
          lines[t][0][0] = tables[t][2 * i], lines[t][1][0] = tables[t][2 * i + 1];
        } else {
          memcpy(lines[t][0], tables[t] + 2 * i * D, D * 4), memcpy(lines[t][1], tables[t] + (2 * i + 1) * D, D * 4);
        }
        subD(D, lines[t][1], lines[t][0], slope);
        for (int x = 2; x <= points; x++) addD(D, lines[t][x - 1], slope, lines[t][x]);
      }
      for (int k = 0; k < points; k++) {
        const int x = k == 0 ? 0 : k + 1;
        const uint32_t *tv[16];
        for (int t = 0; t < T; t++) tv[t] = lines[t][x];
        eval_ext(D, st, tv, consts, f);
        mulD(D, w, f, f);
        addD(D, inner[k], f, inner[k]);
      }
    }
  }
}

INLINE void round_sums_D(const int D, const int BASE, const orc_stmt *st, int points, uint64_t n_low, uint64_t n_high,
                         const uint32_t *const *tables, const int32_t *strides, const uint32_t *low,
                         const uint32_t *high, const uint32_t *consts, int threads, uint32_t *out) {
  uint32_t total[16][8];
  memset(total, 0, sizeof(total));
  if (threads < 1) threads = 1;
  if (n_high >= (uint64_t)threads * 2 || threads == 1) {
#pragma omp parallel num_threads(threads)
    {
      uint32_t mine[16][8], inner[16][8], f[8];
      memset(mine, 0, sizeof(mine));
#pragma omp for schedule(static)
      for (uint64_t h = 0; h < n_high; h++) {
        memset(inner, 0, sizeof(inner));
        block_range(D, BASE, st, points, n_low, h, 0, n_low, tables, strides, low, consts, inner);
        for (int k = 0; k < points; k++) { /* sum_X += HIGH[h] * inner_X, :256-257 */
          mulD(D, high + h * D, inner[k], f);
          addD(D, mine[k], f, mine[k]);
        }
      }
#pragma omp critical
      for (int k = 0; k < points; k++) addD(D, total[k], mine[k], total[k]);
    }
  } else {
    for (uint64_t h = 0; h < n_high; h++) {
      uint32_t inner[16][8], f[8];
      memset(inner, 0, sizeof(inner));
#pragma omp parallel num_threads(threads)
      {
        uint32_t mine[16][8];
        memset(mine, 0, sizeof(mine));
#ifdef _OPENMP
        const uint64_t parts = (uint64_t)omp_get_num_threads(), me = (uint64_t)omp_get_thread_num();
#else
        const uint64_t parts = 1, me = 0;
#endif
        block_range(D, BASE, st, points, n_low, h, n_low * me / parts, n_low * (me + 1) / parts, tables, strides, low,
                    consts, mine);
#pragma omp critical
        for (int k = 0; k < points; k++) addD(D, inner[k], mine[k], inner[k]);
      }
      for (int k = 0; k < points; k++) {
        mulD(D, high + h * D, inner[k], f);
        addD(D, total[k], f, total[k]);
      }
    }
  }
  for (int k = 0; k < points; k++) memcpy(out + (size_t)k * D, total[k], D * 4);
}

int orc_round_sums_fast(const orc_stmt *st, int D, int points, uint64_t n_low, uint64_t n_high,
                        const uint32_t *const *tables, const int32_t *strides, const uint32_t *low,
                        const uint32_t *high, const uint32_t *consts, int threads, uint32_t *out) {
  if ((D != 4 && D != 8) || st->T > 16 || points > 16) return ORC_E_PARAM;
  int base = st->C == 0;
  for (int t = 0; t < st->T; t++) base = base && strides[t] == 1;
  for (int k = 0; k < st->nops; k++) base = base && st->ops[k] != OP_CONST;
  if (D == 4 && base)
    round_sums_D(4, 1, st, points, n_low, n_high, tables, strides, low, high, consts, threads, out);
  else if (D == 4)
    round_sums_D(4, 0, st, points, n_low, n_high, tables, strides, low, high, consts, threads, out);
  else if (base)
    round_sums_D(8, 1, st, points, n_low, n_high, tables, strides, low, high, consts, threads, out);
  else
    round_sums_D(8, 0, st, points, n_low, n_high, tables, strides, low, high, consts, threads, out);
  return ORC_OK;
}

/* FOLD-FLAT-TABLE over threads, src/sumcheck.lisp:84-104 */
INLINE void fold_D(const int D, uint64_t len, const uint32_t *entries, int stride, const uint32_t *r, int threads,
                   uint32_t *out) {
#pragma omp parallel for schedule(static) num_threads(threads)
  for (uint64_t i = 0; i < len / 2; i++) {
    uint32_t term[8];
    if (stride == 1) {
      const uint32_t lo = entries[2 * i], s = fsub(entries[2 * i + 1], lo);
#pragma GCC unroll 8
      for (int c = 0; c < D; c++) term[c] = fmul(r[c], s);
      term[0] = fadd(term[0], lo);
    } else {
      const uint32_t *lo = entries + 2 * i * D, *hi = lo + D;
      subD(D, hi, lo, term);
      mulD(D, r, term, term);
      addD(D, lo, term, term);
    }
    memcpy(out + i * D, term, D * 4);
  }
}
int orc_fold_flat_fast(int D, uint64_t len, const uint32_t *entries, int stride, const uint32_t *r, int threads,
                       uint32_t *out) {
  if (threads < 1) threads = 1;
  if (D == 4)
    fold_D(4, len, entries, stride, r, threads, out);
  else if (D == 8)
    fold_D(8, len, entries, stride, r, threads, out);
  else
    return ORC_E_PARAM;
  return ORC_OK;
}

/* Seeded synthetic field elements: SplitMix64(seed), each output's top 31 bits, kept when below p -- the rule
   the transcript's challenges follow (src/transcript.lisp:159-164) and the rule exh_table_random uses. */
void orc_splitmix_field(uint64_t seed, uint64_t count, uint32_t *out) {
  uint64_t x = seed;
  for (uint64_t i = 0; i < count;) {
    x += 0x9E3779B97F4A7C15ull;
    uint64_t z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const uint32_t w = (uint32_t)(z >> 33);
    if (w < P) out[i++] = w;
  }
}
