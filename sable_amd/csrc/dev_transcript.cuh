// dev_transcript.cuh -- the Fiat-Shamir transcript on the device, so the rounds of a sumcheck run back
// to back without a host round trip: the sequential BLAKE3 mode (src/blake3.lisp:125-155) and the
// transcript operations a prover round needs (src/transcript.lisp:95-100, 116-128, 152-176).  It absorbs
// and squeezes exactly the bytes the host transcript would; the host replays the logged messages into
// its own transcript afterwards and checks that it draws the same challenges.
//
// One wavefront runs it, every lane executing the same (uniform) steps.  The compression function is
// spread over the four lanes of each quad: lane i holds column i of the 4x4 state, so the four G
// functions of a half-round run side by side and the diagonal step is three DPP quad rotations; the
// chain of dependent operations is about a third of the one-lane version.  Between launches the state
// is a DevB3S in device memory; while running, the pending block is a 128-byte ring in LDS (two 64-byte
// halves used alternately), so words are appended with one (possibly unaligned) store.
#pragma once
#include "blake3.cuh"

namespace exh {

struct DevB3S {
  uint32_t cv[8];
  uint32_t block[16];  // the pending block as little-endian words, zero beyond `used`
  uint32_t used;       // bytes taken in the pending block
  uint32_t counter_lo, counter_hi;
};

// message word used by G number g (0..7: columns 0-3, then diagonals 0-3) of round r, first and second
// operand: the BLAKE3 message permutation applied r times (src/blake3.lisp:37-40)
__device__ const uint8_t B3_SCHEDULE[7][16] = {
    {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8},
    {3, 4, 10, 12, 13, 2, 7, 14, 6, 5, 9, 0, 11, 15, 8, 1}, {10, 7, 12, 9, 14, 3, 13, 15, 4, 0, 11, 2, 5, 8, 1, 6},
    {12, 13, 9, 11, 15, 10, 14, 8, 7, 2, 5, 3, 0, 1, 6, 4}, {9, 14, 11, 5, 8, 12, 15, 1, 13, 3, 0, 10, 2, 6, 4, 7},
    {11, 15, 5, 0, 1, 9, 8, 6, 14, 10, 2, 12, 3, 4, 7, 13}};

#define EXH_QUAD(v, ctrl) ((uint32_t)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xf, 0xf, false))

// compress(cv, m, counter, block_len, flags) with the state's columns spread over the lanes of a quad.
// cv: uniform registers; m: the 16 message words in LDS.  Lane i of each quad returns
// w0 = out[i], w1 = out[4+i], w2 = out[8+i], w3 = out[12+i].
__device__ __forceinline__ void b3_compress_quad(const uint32_t cv[8], const uint32_t *m, uint64_t counter,
                                                 uint32_t block_len, uint32_t flags, uint32_t &w0, uint32_t &w1,
                                                 uint32_t &w2, uint32_t &w3) {
  const uint32_t i = threadIdx.x & 3;
  const uint32_t iv = i == 0 ? EXH_B3_IV0 : i == 1 ? EXH_B3_IV1 : i == 2 ? EXH_B3_IV2 : EXH_B3_IV3;
  const uint32_t cva = i == 0 ? cv[0] : i == 1 ? cv[1] : i == 2 ? cv[2] : cv[3];
  const uint32_t cvb = i == 0 ? cv[4] : i == 1 ? cv[5] : i == 2 ? cv[6] : cv[7];
  uint32_t a = cva, b = cvb, c = iv;
  uint32_t d = i == 0 ? (uint32_t)counter : i == 1 ? (uint32_t)(counter >> 32) : i == 2 ? block_len : flags;
  uint32_t mx[7][2], my[7][2];
#pragma unroll
  for (int r = 0; r < 7; r++) {  // no dependence on the state: issued ahead of the rounds
    mx[r][0] = m[B3_SCHEDULE[r][2 * i]], my[r][0] = m[B3_SCHEDULE[r][2 * i + 1]];
    mx[r][1] = m[B3_SCHEDULE[r][8 + 2 * i]], my[r][1] = m[B3_SCHEDULE[r][9 + 2 * i]];
  }
#pragma unroll
  for (int r = 0; r < 7; r++) {
    EXH_B3_G(a, b, c, d, mx[r][0], my[r][0])  // the four columns
    b = EXH_QUAD(b, 0x39), c = EXH_QUAD(c, 0x4E), d = EXH_QUAD(d, 0x93);  // rotate rows by 1, 2, 3
    EXH_B3_G(a, b, c, d, mx[r][1], my[r][1])  // the four diagonals
    b = EXH_QUAD(b, 0x93), c = EXH_QUAD(c, 0x4E), d = EXH_QUAD(d, 0x39);
  }
  w0 = a ^ c, w1 = b ^ d, w2 = c ^ cva, w3 = d ^ cvb;
}

// the first 8 output words, uniform
__device__ __forceinline__ void b3_quad_cv(uint32_t w0, uint32_t w1, uint32_t out[8]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    out[i] = (uint32_t)__builtin_amdgcn_readlane((int)w0, i);
    out[4 + i] = (uint32_t)__builtin_amdgcn_readlane((int)w1, i);
  }
}

// The running state: chaining value and counters in registers, the pending block as a 128-byte ring in
// LDS (`ring`, 32 words) whose two halves are used alternately.
struct RunB3S {
  uint32_t cv[8];
  uint32_t *ring;
  uint32_t used, half;
  uint64_t counter;
};

__device__ inline void rb3s_load(RunB3S &s, uint32_t *ring, const DevB3S *g) {
#pragma unroll
  for (int i = 0; i < 8; i++) s.cv[i] = g->cv[i];
#pragma unroll
  for (int i = 0; i < 16; i++) ring[i] = g->block[i], ring[16 + i] = 0;
  s.ring = ring;
  s.used = g->used, s.half = 0;
  s.counter = ((uint64_t)g->counter_hi << 32) | g->counter_lo;
}
__device__ inline void rb3s_store(const RunB3S &s, DevB3S *g) {
#pragma unroll
  for (int i = 0; i < 8; i++) g->cv[i] = s.cv[i];
#pragma unroll
  for (int i = 0; i < 16; i++) g->block[i] = s.ring[16 * s.half + i];
  g->used = s.used;
  g->counter_lo = (uint32_t)s.counter, g->counter_hi = (uint32_t)(s.counter >> 32);
}

// the pending block is full and more input arrives: compress it, move to the other half
__device__ inline void rb3s_flush(RunB3S &s) {
  uint32_t w0, w1, w2, w3;
  b3_compress_quad(s.cv, s.ring + 16 * s.half, s.counter, 64, 0, w0, w1, w2, w3);
  b3_quad_cv(w0, w1, s.cv);
  s.counter++;
  s.half ^= 1;
#pragma unroll
  for (int i = 0; i < 16; i++) s.ring[16 * s.half + i] = 0;
  s.used = 0;
}

// append the low NBYTES (1..4) bytes of W
__device__ inline void rb3s_append(RunB3S &s, uint32_t w, uint32_t nbytes) {
  uint8_t *bytes = reinterpret_cast<uint8_t *>(s.ring) + 64 * s.half;
  if (s.used + nbytes <= 64) {  // the common case: one store, aligned or not
    if (nbytes == 4)
      __builtin_memcpy(bytes + s.used, &w, 4);
    else
      for (uint32_t b = 0; b < nbytes; b++) bytes[s.used + b] = (uint8_t)(w >> (8 * b));
    s.used += nbytes;
    return;
  }
  for (uint32_t b = 0; b < nbytes; b++) {  // the word straddles two blocks
    if (s.used == 64) {
      rb3s_flush(s);
      bytes = reinterpret_cast<uint8_t *>(s.ring) + 64 * s.half;
    }
    bytes[s.used++] = (uint8_t)(w >> (8 * b));
  }
}

// 48 bytes of output for everything absorbed so far (state unchanged)
__device__ inline void rb3s_digest48(const RunB3S &s, uint32_t out[12]) {
  uint32_t w0, w1, w2, w3;
  b3_compress_quad(s.cv, s.ring + 16 * s.half, 0, s.used, B3_CHUNK_END | B3_ROOT, w0, w1, w2, w3);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    out[i] = (uint32_t)__builtin_amdgcn_readlane((int)w0, i);
    out[4 + i] = (uint32_t)__builtin_amdgcn_readlane((int)w1, i);
    out[8 + i] = (uint32_t)__builtin_amdgcn_readlane((int)w2, i);
  }
}

// absorb(data) for NWORDS little-endian words: the length as u64 LE, then the bytes
// (src/transcript.lisp:95-100)
__device__ inline void dev_absorb_words(RunB3S &s, const uint32_t *words, uint32_t nwords) {
  rb3s_append(s, 4 * nwords, 4);
  rb3s_append(s, 0, 4);
  for (uint32_t i = 0; i < nwords; i++) rb3s_append(s, words[i], 4);
}

// K <= 8 base-field challenges (CHALLENGE-BASE, src/transcript.lisp:159-172): squeeze 4 (missing + 4)
// bytes, keep the 31-bit words below p, repeat until K are kept; each squeeze then absorbs "squeeze" and
// the first min(32, n) bytes of its output (src/transcript.lisp:152-157).
__device__ inline void dev_challenge(RunB3S &s, int k, uint32_t *out) {
  int have = 0;
  while (have < k) {
    uint32_t n = 4u * (uint32_t)(k - have + 4);  // at most 48 bytes: one output block
    uint32_t o[12];
    rb3s_digest48(s, o);
    rb3s_append(s, 0x65757173u, 4);  // "sque"
    rb3s_append(s, 0x00657a65u, 3);  // "eze"
#pragma unroll
    for (uint32_t i = 0; i < 8; i++)
      if (4 * i < n) rb3s_append(s, o[i], 4);
#pragma unroll
    for (uint32_t i = 0; i < 12; i++) {
      uint32_t w = o[i] & 0x7fffffffu;
      if (4 * i < n && have < k && w < P) out[have++] = w;
    }
  }
}

}  // namespace exh
