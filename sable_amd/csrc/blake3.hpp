// blake3.hpp -- the BLAKE3 compression function and single-chunk hashing, shared by the host
// transcript and the device Merkle kernels.  Every hash on the commitment path is a single chunk
// (at most 1024 bytes: src/pcs.lisp:35, 44-55), so no chunk tree is needed on the device.
#pragma once
#if !defined(__HIPCC_RTC__)
#include <stdint.h>
#endif

#include "field.hpp"

namespace exh {

enum : uint32_t { B3_CHUNK_START = 1, B3_CHUNK_END = 2, B3_PARENT = 4, B3_ROOT = 8 };

#define EXH_B3_IV0 0x6A09E667u
#define EXH_B3_IV1 0xBB67AE85u
#define EXH_B3_IV2 0x3C6EF372u
#define EXH_B3_IV3 0xA54FF53Au
#define EXH_B3_IV4 0x510E527Fu
#define EXH_B3_IV5 0x9B05688Cu
#define EXH_B3_IV6 0x1F83D9ABu
#define EXH_B3_IV7 0x5BE0CD19u

EXH_HD uint32_t b3_rotr(uint32_t w, int n) { return (w >> n) | (w << (32 - n)); }

EXH_HD void b3_iv(uint32_t cv[8]) {
  cv[0] = EXH_B3_IV0, cv[1] = EXH_B3_IV1, cv[2] = EXH_B3_IV2, cv[3] = EXH_B3_IV3;
  cv[4] = EXH_B3_IV4, cv[5] = EXH_B3_IV5, cv[6] = EXH_B3_IV6, cv[7] = EXH_B3_IV7;
}

#define EXH_B3_G(a, b, c, d, x, y) \
  a = a + b + (x);                 \
  d = b3_rotr(d ^ a, 16);          \
  c = c + d;                       \
  b = b3_rotr(b ^ c, 12);          \
  a = a + b + (y);                 \
  d = b3_rotr(d ^ a, 8);           \
  c = c + d;                       \
  b = b3_rotr(b ^ c, 7);

// One round with the message schedule of round R written out, so the message words stay in
// registers under a fixed permutation (src/blake3.lisp:37-40, 74-83).
#define EXH_B3_ROUND(m, i0, i1, i2, i3, i4, i5, i6, i7, i8, i9, i10, i11, i12, i13, i14, i15) \
  EXH_B3_G(v0, v4, v8, v12, m[i0], m[i1])                                                     \
  EXH_B3_G(v1, v5, v9, v13, m[i2], m[i3])                                                     \
  EXH_B3_G(v2, v6, v10, v14, m[i4], m[i5])                                                    \
  EXH_B3_G(v3, v7, v11, v15, m[i6], m[i7])                                                    \
  EXH_B3_G(v0, v5, v10, v15, m[i8], m[i9])                                                    \
  EXH_B3_G(v1, v6, v11, v12, m[i10], m[i11])                                                  \
  EXH_B3_G(v2, v7, v8, v13, m[i12], m[i13])                                                   \
  EXH_B3_G(v3, v4, v9, v14, m[i14], m[i15])

// compress(cv, m, counter, block_len, flags) -> first 8 output words in out (the chaining value);
// with full != 0 all 16 words.
EXH_HD void b3_compress(const uint32_t cv[8], const uint32_t m[16], uint64_t counter, uint32_t block_len,
                        uint32_t flags, uint32_t *out, int full) {
  uint32_t v0 = cv[0], v1 = cv[1], v2 = cv[2], v3 = cv[3], v4 = cv[4], v5 = cv[5], v6 = cv[6], v7 = cv[7];
  uint32_t v8 = EXH_B3_IV0, v9 = EXH_B3_IV1, v10 = EXH_B3_IV2, v11 = EXH_B3_IV3;
  uint32_t v12 = (uint32_t)counter, v13 = (uint32_t)(counter >> 32), v14 = block_len, v15 = flags;
  EXH_B3_ROUND(m, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15)
  EXH_B3_ROUND(m, 2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8)
  EXH_B3_ROUND(m, 3, 4, 10, 12, 13, 2, 7, 14, 6, 5, 9, 0, 11, 15, 8, 1)
  EXH_B3_ROUND(m, 10, 7, 12, 9, 14, 3, 13, 15, 4, 0, 11, 2, 5, 8, 1, 6)
  EXH_B3_ROUND(m, 12, 13, 9, 11, 15, 10, 14, 8, 7, 2, 5, 3, 0, 1, 6, 4)
  EXH_B3_ROUND(m, 9, 14, 11, 5, 8, 12, 15, 1, 13, 3, 0, 10, 2, 6, 4, 7)
  EXH_B3_ROUND(m, 11, 15, 5, 0, 1, 9, 8, 6, 14, 10, 2, 12, 3, 4, 7, 13)
  out[0] = v0 ^ v8, out[1] = v1 ^ v9, out[2] = v2 ^ v10, out[3] = v3 ^ v11;
  out[4] = v4 ^ v12, out[5] = v5 ^ v13, out[6] = v6 ^ v14, out[7] = v7 ^ v15;
  if (full) {
    out[8] = v8 ^ cv[0], out[9] = v9 ^ cv[1], out[10] = v10 ^ cv[2], out[11] = v11 ^ cv[3];
    out[12] = v12 ^ cv[4], out[13] = v13 ^ cv[5], out[14] = v14 ^ cv[6], out[15] = v15 ^ cv[7];
  }
}

// The 32-byte digest (8 words) of a single-chunk message given as NWORDS little-endian words
// (NWORDS * 4 bytes <= 1024, a multiple of 4 bytes): standard BLAKE3, src/blake3.lisp:157-233.
EXH_HD void b3_hash_words(const uint32_t *words, int nwords, uint32_t out[8]) {
  uint32_t cv[8], m[16];
  b3_iv(cv);
  int nblocks = nwords == 0 ? 1 : (nwords + 15) / 16;
  for (int b = 0; b < nblocks; b++) {
    int have = nwords - 16 * b;
    if (have > 16) have = 16;
    for (int i = 0; i < 16; i++) m[i] = i < have ? words[16 * b + i] : 0u;
    uint32_t flags = (b == 0 ? B3_CHUNK_START : 0u) | (b == nblocks - 1 ? (B3_CHUNK_END | B3_ROOT) : 0u);
    b3_compress(cv, m, 0, (uint32_t)(4 * have), flags, cv, 0);
  }
  for (int i = 0; i < 8; i++) out[i] = cv[i];
}

// node = BLAKE3(left || right): one 64-byte block (src/pcs.lisp:54-55)
EXH_HD void b3_node(const uint32_t left[8], const uint32_t right[8], uint32_t out[8]) {
  uint32_t cv[8], m[16];
  b3_iv(cv);
  for (int i = 0; i < 8; i++) m[i] = left[i], m[8 + i] = right[i];
  b3_compress(cv, m, 0, 64, B3_CHUNK_START | B3_CHUNK_END | B3_ROOT, out, 0);
}

}  // namespace exh
