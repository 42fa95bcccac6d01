// field.hpp -- KoalaBear F_p (p = 2^31 - 2^24 + 1) and its towers F_p^4 / F_p^8 for gfx950.
//
// Values in memory are canonical residues in [0, p), extension elements are D words in the
// reference's tower order (src/field.lisp:8-11): coordinate i is the coefficient of w^bitrev(i) in
// F_p[w]/(w^D - 3).  Products go through 32-bit Montgomery reduction (R = 2^32): mont_mul(a, b) is
// a b / R, so a caller that wants the exact product passes one operand pre-multiplied by R, or
// corrects a whole sum afterwards by a power of R.  Sums of products are accumulated unreduced
// (four products below p^2 fit 64 bits, as in src/field.lisp:213-218; longer sums use a 96-bit
// accumulator) and reduced once.
#pragma once
// (a run-time compilation of these kernels has the runtime's declarations built in and no host headers)
#if !defined(__HIPCC_RTC__)
#include <stdint.h>
#else
typedef unsigned char uint8_t;
typedef unsigned short uint16_t;
typedef unsigned int uint32_t;
typedef int int32_t;
typedef unsigned long long uint64_t;
typedef long long int64_t;
typedef __SIZE_TYPE__ size_t;
#define offsetof(type, member) __builtin_offsetof(type, member)
namespace std {
template <class A, class B> struct is_same { static constexpr bool value = false; };
template <class A> struct is_same<A, A> { static constexpr bool value = true; };
template <bool C, class A, class B> struct conditional { typedef A type; };
template <class A, class B> struct conditional<false, A, B> { typedef B type; };
}  // namespace std
#endif

#if defined(__HIPCC_RTC__)
#define EXH_HD __host__ __device__ inline __attribute__((always_inline))
#elif defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define EXH_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define EXH_HD inline
#endif

namespace exh {

constexpr uint32_t P = 0x7f000001u;      // 2130706433
constexpr uint32_t PINV = 0x81000001u;   // p^-1 mod 2^32
constexpr uint32_t R1 = 33554430u;       // 2^32 mod p
constexpr uint32_t R2 = 402124772u;      // 2^64 mod p
constexpr uint32_t R3 = 414154551u;      // 2^96 mod p
constexpr uint32_t INV2 = 1065353217u;   // 1/2 mod p

EXH_HD uint32_t umin32(uint32_t a, uint32_t b) { return a < b ? a : b; }

// a + b and a - b for a, b in [0, p): the wrapped alternative is the larger unsigned value
EXH_HD uint32_t fadd(uint32_t a, uint32_t b) {
  uint32_t s = a + b;
  return umin32(s, s - P);
}
EXH_HD uint32_t fsub(uint32_t a, uint32_t b) {
  uint32_t d = a - b;
  return umin32(d, d + P);
}
EXH_HD uint32_t fneg(uint32_t a) { return fsub(0u, a); }
EXH_HD uint32_t fdbl(uint32_t a) { return fadd(a, a); }
EXH_HD uint32_t times3(uint32_t a) { return fadd(fadd(a, a), a); }

// t / R mod p for t < 2^32 p (one product, or two products below p^2): result in [0, p)
EXH_HD uint32_t mont_reduce(uint64_t t) {
  uint32_t m = (uint32_t)t * PINV;
  uint32_t u = (uint32_t)(((uint64_t)m * P) >> 32);
  uint32_t r = (uint32_t)(t >> 32) - u;  // low words cancel exactly
  return umin32(r, r + P);
}
// t / R mod p for any t < 4 p^2 < 2^64 (a sum of four products): result in [0, p)
EXH_HD uint32_t mont_reduce4(uint64_t t) {
  uint32_t m = (uint32_t)t * PINV;
  uint32_t u = (uint32_t)(((uint64_t)m * P) >> 32);  // < p
  uint32_t hi = (uint32_t)(t >> 32);                 // < 1.99 p
  hi = umin32(hi, hi - P);                           // < p (the wrapped alternative is the larger unsigned value)
  uint32_t r = hi - u;                               // in (-p, p): no comparison, no select
  return umin32(r, r + P);
}
EXH_HD uint32_t mont_mul(uint32_t a, uint32_t b) { return mont_reduce((uint64_t)a * b); }
// exact a b mod p (two reductions; host-side helpers and rare device paths)
EXH_HD uint32_t fmul(uint32_t a, uint32_t b) { return mont_mul(mont_mul(a, b), R2); }
EXH_HD uint32_t to_mont(uint32_t a) { return mont_mul(a, R2); }

EXH_HD uint32_t fpow(uint32_t a, uint64_t e) {
  uint32_t result = 1, base = a;
  for (; e; e >>= 1) {
    if (e & 1) result = fmul(result, base);
    base = fmul(base, base);
  }
  return result;
}
EXH_HD uint32_t finv(uint32_t a) { return fpow(a, P - 2); }  // 0 -> 0

// ---- unreduced accumulation: a 96-bit sum of 64-bit terms
struct Acc96 {
  uint64_t lo;
  uint32_t hi;
};
EXH_HD void acc_zero(Acc96 &a) {
  a.lo = 0;
  a.hi = 0;
}
// (the carry of the 64-bit addition taken from the addition itself: three additions chained by the carry; written
// as a comparison of the sum with a term it costs a 64-bit comparison and a select on top)
EXH_HD void acc_add(Acc96 &a, uint64_t t) {
  unsigned long long s;
  const bool carry = __builtin_uaddll_overflow(a.lo, t, &s);
  a.hi += carry ? 1u : 0u;
  a.lo = s;
}
EXH_HD void acc_mad(Acc96 &a, uint32_t x, uint32_t y) { acc_add(a, (uint64_t)x * y); }
// the accumulator mod p, exactly
EXH_HD uint32_t acc_reduce(const Acc96 &a) {
  // hi 2^64 + mid 2^32 + lo = (hi R^3 + mid R^2 + lo R) / R: two Montgomery reductions, no division
  uint64_t v = (a.lo >> 32) * (uint64_t)R2 + (uint64_t)(uint32_t)a.lo * R1;  // < 2^32 (p + R1) < 4 p^2
  return fadd(mont_reduce4(v), mont_mul(a.hi, R3));
}

// ---- tower arithmetic on D = 4 or 8 words in tower order
constexpr int brev(int i, int D) {
  int bits = D == 8 ? 3 : D == 4 ? 2 : D == 2 ? 1 : 0, r = 0;
  for (int b = 0; b < bits; b++) r |= ((i >> b) & 1) << (bits - 1 - b);
  return r;
}

template <int D>
struct Ext {
  uint32_t c[D];
};

template <int D>
EXH_HD Ext<D> ext_zero() {
  Ext<D> z;
#pragma unroll
  for (int i = 0; i < D; i++) z.c[i] = 0;
  return z;
}
template <int D>
EXH_HD Ext<D> ext_lift(uint32_t v) {
  Ext<D> z = ext_zero<D>();
  z.c[0] = v;
  return z;
}
template <int D>
EXH_HD Ext<D> ext_add(const Ext<D> &a, const Ext<D> &b) {
  Ext<D> o;
#pragma unroll
  for (int i = 0; i < D; i++) o.c[i] = fadd(a.c[i], b.c[i]);
  return o;
}
template <int D>
EXH_HD Ext<D> ext_sub(const Ext<D> &a, const Ext<D> &b) {
  Ext<D> o;
#pragma unroll
  for (int i = 0; i < D; i++) o.c[i] = fsub(a.c[i], b.c[i]);
  return o;
}
// a * s / R for a base value s
template <int D>
EXH_HD Ext<D> ext_scale_mont(const Ext<D> &a, uint32_t s) {
  Ext<D> o;
#pragma unroll
  for (int i = 0; i < D; i++) o.c[i] = mont_mul(a.c[i], s);
  return o;
}

// The D unreduced coefficient sums of a * b in F_p[w]/(w^D - 3), each a sum of D products with the
// wrapping b's tripled first (src/field.lisp:220-234); emit(e_tower, group, sum) receives them in
// groups of at most four products.
template <int D, class F>
EXH_HD void ext_mul_sums(const Ext<D> &a, const Ext<D> &b, F emit) {
  uint32_t pa[D], pb[D], pb3[D];
#pragma unroll
  for (int e = 0; e < D; e++) {
    pa[e] = a.c[brev(e, D)];
    pb[e] = b.c[brev(e, D)];
  }
  pb3[0] = 0;
#pragma unroll
  for (int j = 1; j < D; j++) pb3[j] = times3(pb[j]);
#pragma unroll
  for (int e = 0; e < D; e++) {
#pragma unroll
    for (int g = 0; g < D; g += 4) {
      uint64_t t = 0;
#pragma unroll
      for (int i = g; i < g + 4; i++) {
        int j = (e - i) & (D - 1);
        t += (uint64_t)pa[i] * (i > e ? pb3[j] : pb[j]);
      }
      emit(brev(e, D), g / 4, t);
    }
  }
}

// a b / R
template <int D>
EXH_HD Ext<D> ext_mul_mont(const Ext<D> &a, const Ext<D> &b) {
  Ext<D> o;
  ext_mul_sums<D>(a, b, [&](int e, int g, uint64_t t) {
    uint32_t r = mont_reduce4(t);
    o.c[e] = g == 0 ? r : fadd(o.c[e], r);
  });
  return o;
}
// exact a b (host-side helpers)
template <int D>
EXH_HD Ext<D> ext_mul(const Ext<D> &a, const Ext<D> &b) {
  Ext<D> o = ext_mul_mont<D>(a, b);
#pragma unroll
  for (int i = 0; i < D; i++) o.c[i] = mont_mul(o.c[i], R2);
  return o;
}

// acc += a b, unreduced (D 96-bit accumulators in tower order)
template <int D>
EXH_HD void ext_mul_acc(Acc96 *acc, const Ext<D> &a, const Ext<D> &b) {
  ext_mul_sums<D>(a, b, [&](int e, int, uint64_t t) { acc_add(acc[e], t); });
}
// acc += a * s for a base value s
#if defined(__HIP_DEVICE_COMPILE__)
// Four accumulators at once: the multiply-add's own carry-out feeds the add to the third word, two
// instructions per accumulator (written in C++ the carry is recomputed by a 64-bit add and a compare: four).
// The carries go through four scalar pairs so that three other instructions separate each write from its read.
__device__ __forceinline__ void acc_mad4(Acc96 *acc, const uint32_t *a, uint32_t s) {
  uint64_t c0, c1, c2, c3;
  asm("v_mad_u64_u32 %0, %8, %12, %16, %0\n\t"
      "v_mad_u64_u32 %1, %9, %13, %16, %1\n\t"
      "v_mad_u64_u32 %2, %10, %14, %16, %2\n\t"
      "v_mad_u64_u32 %3, %11, %15, %16, %3\n\t"
      "v_addc_co_u32_e64 %4, %8, 0, %4, %8\n\t"
      "v_addc_co_u32_e64 %5, %9, 0, %5, %9\n\t"
      "v_addc_co_u32_e64 %6, %10, 0, %6, %10\n\t"
      "v_addc_co_u32_e64 %7, %11, 0, %7, %11"
      : "+v"(acc[0].lo), "+v"(acc[1].lo), "+v"(acc[2].lo), "+v"(acc[3].lo), "+v"(acc[0].hi), "+v"(acc[1].hi),
        "+v"(acc[2].hi), "+v"(acc[3].hi), "=&s"(c0), "=&s"(c1), "=&s"(c2), "=&s"(c3)
      : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(s));
}
template <int D>
__device__ __forceinline__ void ext_scale_acc(Acc96 *acc, const Ext<D> &a, uint32_t s) {
  static_assert(D % 4 == 0, "accumulators go four at a time");
#pragma unroll
  for (int i = 0; i < D; i += 4) acc_mad4(acc + i, a.c + i, s);
}
#else
template <int D>
EXH_HD void ext_scale_acc(Acc96 *acc, const Ext<D> &a, uint32_t s) {
#pragma unroll
  for (int i = 0; i < D; i++) acc_mad(acc[i], a.c[i], s);
}
#endif
template <int D>
EXH_HD Ext<D> acc_reduce_ext(const Acc96 *acc) {
  Ext<D> o;
#pragma unroll
  for (int i = 0; i < D; i++) o.c[i] = acc_reduce(acc[i]);
  return o;
}

#if defined(__HIPCC__)
// ---- KoalaBear in double precision, for the products of base-field values that are sums and differences of
// table entries: integers below 2^53 are exact there, so the lines' values need no reduction between additions
// (three integer operations each otherwise) and a product mod p takes six operations, as a Montgomery product
// with its final correction does.  Every step below is exact integer arithmetic: a product a b is held as the
// pair (h, l) of its rounded value and the rounding error, the quotient estimate q = rint(h / p) is off by far
// less than one, and h - q p + l is then a small integer.
constexpr double F_P = 2130706433.0, F_PINV = 1.0 / 2130706433.0, F_MAGIC = 6755399441055744.0;  // 1.5 * 2^52
// v mod p in about [-p/2, p/2] for an integer |v| < 2^80
__device__ __forceinline__ double f_reduce(double v) {
  double q = __builtin_fma(v, F_PINV, F_MAGIC) - F_MAGIC;  // rint(v / p) for |v / p| < 2^51
  return __builtin_fma(-q, F_P, v);
}
// a b mod p in about [-p/2 - 2^27, p/2 + 2^27] for integers |a b| < 2^80
__device__ __forceinline__ double f_mul(double a, double b) {
  double h = a * b;
  double l = __builtin_fma(a, b, -h);
  double q = __builtin_fma(h, F_PINV, F_MAGIC) - F_MAGIC;
  return __builtin_fma(-q, F_P, h) + l;
}
// c x for a table value x and a statement's integer coefficient c (a residue: large ones stand for negatives)
__device__ __forceinline__ double f_scale(double x, uint32_t c) {
  return c == 1 ? x : c == P - 1 ? -x : f_mul(x, c > P / 2 ? (double)c - F_P : (double)c);
}
// a residue of v below 2^32 as an integer, for |v| < p + 2^28: v + p sits in the low word of v + p + 1.5 * 2^52
__device__ __forceinline__ uint32_t f_residue32(double v) {
  return (uint32_t)__double_as_longlong(v + (F_P + F_MAGIC));
}
// the canonical residue of an integer |v| < 2^80
__device__ __forceinline__ uint32_t f_canonical(double v) {
  const int32_t r = (int32_t)f_reduce(v);
  return r < 0 ? (uint32_t)(r + (int32_t)P) : (uint32_t)r;
}
#endif

}  // namespace exh
