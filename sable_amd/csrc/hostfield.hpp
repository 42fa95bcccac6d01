// hostfield.hpp -- exact tower arithmetic on the host with a run-time degree (4 or 8), for the
// O(rounds) protocol logic around the kernels: message assembly, claims, the verifier.
#pragma once
#include <string.h>

#include <vector>

#include "field.hpp"

namespace exh {
namespace hf {

typedef std::vector<uint32_t> E;  // D canonical words, tower order

inline E zero(int D) { return E(D, 0u); }
inline E lift(uint32_t v, int D) {
  E e(D, 0u);
  e[0] = v % P;
  return e;
}
inline E from(const uint32_t *p, int D) { return E(p, p + D); }
inline E add(const E &a, const E &b) {
  E o(a.size());
  for (size_t i = 0; i < a.size(); i++) o[i] = fadd(a[i], b[i]);
  return o;
}
inline E sub(const E &a, const E &b) {
  E o(a.size());
  for (size_t i = 0; i < a.size(); i++) o[i] = fsub(a[i], b[i]);
  return o;
}
inline E neg(const E &a) { return sub(zero((int)a.size()), a); }
inline E scale(const E &a, uint32_t s) {
  E o(a.size());
  for (size_t i = 0; i < a.size(); i++) o[i] = fmul(a[i], s % P);
  return o;
}
inline void mul_raw(int D, const uint32_t *a, const uint32_t *b, uint32_t *out) {
  if (D == 4) {
    Ext<4> x, y;
    memcpy(x.c, a, 16), memcpy(y.c, b, 16);
    Ext<4> z = ext_mul<4>(x, y);
    memcpy(out, z.c, 16);
  } else if (D == 8) {
    Ext<8> x, y;
    memcpy(x.c, a, 32), memcpy(y.c, b, 32);
    Ext<8> z = ext_mul<8>(x, y);
    memcpy(out, z.c, 32);
  } else if (D == 2) {  // F_p[x]/(x^2 - 3), for the inverse's descent
    uint32_t c0 = fadd(fmul(a[0], b[0]), times3(fmul(a[1], b[1])));
    uint32_t c1 = fadd(fmul(a[0], b[1]), fmul(a[1], b[0]));
    out[0] = c0, out[1] = c1;
  } else {
    out[0] = fmul(a[0], b[0]);
  }
}
inline E mul(const E &a, const E &b) {
  E o(a.size());
  mul_raw((int)a.size(), a.data(), b.data(), o.data());
  return o;
}
// a times the generator of a's level: (A0 + A1 w) w = A1 w^2 + A0 w (src/field.lisp:206-211)
inline E mul_by_generator(const E &a) {
  if (a.size() == 1) return E{times3(a[0])};
  size_t h = a.size() / 2;
  E a0(a.begin(), a.begin() + h), a1(a.begin() + h, a.end());
  E g = mul_by_generator(a1);
  g.insert(g.end(), a0.begin(), a0.end());
  return g;
}
// 1/a by norms down the tower (src/field.lisp:236-243); zero -> zero (the RETURN-ZERO convention),
// callers that must signal check is_zero first
inline E inv(const E &a) {
  if (a.size() == 1) return E{finv(a[0])};
  size_t h = a.size() / 2;
  E a0(a.begin(), a.begin() + h), a1(a.begin() + h, a.end());
  E norm = sub(mul(a0, a0), mul_by_generator(mul(a1, a1)));
  E ninv = inv(norm);
  E r0 = mul(a0, ninv), r1 = neg(mul(a1, ninv));
  r0.insert(r0.end(), r1.begin(), r1.end());
  return r0;
}
inline bool is_zero(const E &a) {
  for (uint32_t v : a)
    if (v) return false;
  return true;
}
inline E eq1(const E &a, const E &b) {  // a b + (1 - a)(1 - b)
  E one = lift(1, (int)a.size());
  return add(mul(a, b), mul(sub(one, a), sub(one, b)));
}
// the polynomial through (xs[i], values[i]) at x, xs small distinct integers
inline E interpolate(const std::vector<int> &xs, const std::vector<E> &values, const E &x) {
  int D = (int)x.size();
  E acc = zero(D);
  for (size_t i = 0; i < xs.size(); i++) {
    uint32_t w = 1;
    E term = values[i];
    for (size_t j = 0; j < xs.size(); j++) {
      if (j == i) continue;
      int64_t diff = xs[i] - xs[j];
      w = fmul(w, (uint32_t)(((diff % (int64_t)P) + P) % P));
      term = mul(term, sub(x, lift((uint32_t)xs[j], D)));
    }
    acc = add(acc, scale(term, finv(w)));
  }
  return acc;
}
// LAGRANGE on the nodes 0..d (src/field.lisp:340-352)
inline E lagrange(const std::vector<E> &values, const E &x) {
  std::vector<int> xs(values.size());
  for (size_t i = 0; i < xs.size(); i++) xs[i] = (int)i;
  return interpolate(xs, values, x);
}
// EQ-TABLE (src/field.lisp:354-363), flat: 2^k entries of D words
inline std::vector<uint32_t> eq_table(const uint32_t *r, int k, int D) {
  std::vector<uint32_t> t((size_t)D << k, 0u);
  t[0] = 1;
  size_t len = 1;
  for (int b = 0; b < k; b++) {
    for (size_t i = 0; i < len; i++) {
      uint32_t up[8];
      mul_raw(D, &t[i * D], r + (size_t)b * D, up);
      for (int c = 0; c < D; c++) {
        t[(len + i) * D + c] = up[c];
        t[i * D + c] = fsub(t[i * D + c], up[c]);
      }
    }
    len *= 2;
  }
  return t;
}
// the multilinear extension of 2^k EXTs at r (LSB first), src/field.lisp:372-377
inline E mle_eval(const uint32_t *values, int k, const uint32_t *r, int D) {
  std::vector<uint32_t> t(values, values + ((size_t)D << k));
  size_t len = (size_t)1 << k;
  for (int b = 0; b < k; b++) {
    for (size_t i = 0; i < len / 2; i++) {
      uint32_t d[8], m[8];
      for (int c = 0; c < D; c++) d[c] = fsub(t[(2 * i + 1) * D + c], t[2 * i * D + c]);
      mul_raw(D, r + (size_t)b * D, d, m);
      for (int c = 0; c < D; c++) t[i * D + c] = fadd(t[2 * i * D + c], m[c]);
    }
    len /= 2;
  }
  return E(t.begin(), t.begin() + D);
}

}  // namespace hf
}  // namespace exh
