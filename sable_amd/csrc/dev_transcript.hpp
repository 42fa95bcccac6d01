// dev_transcript.hpp -- the Fiat-Shamir transcript on the device, so the rounds of a sumcheck run back
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
#include "blake3.hpp"

namespace exh {

struct DevB3S {
  uint32_t cv[8];
  uint32_t block[16];  // the pending block as little-endian words, zero beyond `used`
  uint32_t used;       // bytes taken in the pending block
  uint32_t counter_lo, counter_hi;
};

// S[r][k]: the message word used k-th in round r (G number g = k / 2 of columns 0-3 then diagonals 0-3, first
// and second operand): the BLAKE3 message permutation applied r times (src/blake3.lisp:37-40).  Lane i of a
// quad needs S[r][first + 2 i]: the four numbers, one nibble each, as a compile-time constant.
__host__ __device__ constexpr uint32_t b3_lane_words(int r, int first) {
  constexpr uint8_t S[7][16] = {
      {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8},
      {3, 4, 10, 12, 13, 2, 7, 14, 6, 5, 9, 0, 11, 15, 8, 1}, {10, 7, 12, 9, 14, 3, 13, 15, 4, 0, 11, 2, 5, 8, 1, 6},
      {12, 13, 9, 11, 15, 10, 14, 8, 7, 2, 5, 3, 0, 1, 6, 4}, {9, 14, 11, 5, 8, 12, 15, 1, 13, 3, 0, 10, 2, 6, 4, 7},
      {11, 15, 5, 0, 1, 9, 8, 6, 14, 10, 2, 12, 3, 4, 7, 13}};
  return (uint32_t)S[r][first] | (uint32_t)S[r][first + 2] << 4 | (uint32_t)S[r][first + 4] << 8 |
         (uint32_t)S[r][first + 6] << 12;
}

#define EXH_QUAD(v, ctrl) ((uint32_t)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xf, 0xf, false))

// compress(cv, m, counter, block_len, flags) with the state's columns spread over the lanes of a quad.
// cv: the chaining value's 8 words in LDS (lane i takes words i and 4 + i: from registers the choice by lane
// becomes an indexed access, and the compiler moves the value to scratch memory for it, two trips to memory per
// compression); m: the 16 message words in LDS.  Lane i of each quad returns
// w0 = out[i], w1 = out[4+i], w2 = out[8+i], w3 = out[12+i].
__device__ __forceinline__ void b3_compress_quad(const uint32_t *cv, const uint32_t *m, uint64_t counter,
                                                 uint32_t block_len, uint32_t flags, uint32_t &w0, uint32_t &w1,
                                                 uint32_t &w2, uint32_t &w3) {
  const uint32_t i = threadIdx.x & 3;
  const uint32_t iv = i == 0 ? EXH_B3_IV0 : i == 1 ? EXH_B3_IV1 : i == 2 ? EXH_B3_IV2 : EXH_B3_IV3;
  const uint32_t cva = cv[i], cvb = cv[4 + i];
  uint32_t a = cva, b = cvb, c = iv;
  uint32_t d = i == 0 ? (uint32_t)counter : i == 1 ? (uint32_t)(counter >> 32) : i == 2 ? block_len : flags;
  uint32_t mx[7][2], my[7][2];
#pragma unroll
  for (int r = 0; r < 7; r++) {  // no dependence on the state: issued ahead of the rounds
    // the four lanes' word numbers sit in the nibbles of a compile-time constant: no table in memory to read
    mx[r][0] = m[(b3_lane_words(r, 0) >> (4 * i)) & 15u], my[r][0] = m[(b3_lane_words(r, 1) >> (4 * i)) & 15u];
    mx[r][1] = m[(b3_lane_words(r, 8) >> (4 * i)) & 15u], my[r][1] = m[(b3_lane_words(r, 9) >> (4 * i)) & 15u];
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

// the first 8 output words into the chaining value in LDS (lanes 0-3 hold them; a wavefront's LDS operations
// complete in order, so the next compression reads the new value)
__device__ __forceinline__ void b3_quad_cv(uint32_t w0, uint32_t w1, uint32_t *cv) {
  const uint32_t lane = threadIdx.x & 63;
  if (lane < 4) cv[lane] = w0, cv[4 + lane] = w1;
  __builtin_amdgcn_wave_barrier();
}

// The running state: counters in registers; in LDS (`ring`, RING_WORDS words) the pending block as a 128-byte
// ring (the first 32 words) whose two halves are used alternately, 16 words that stage a squeeze's output, and the
// chaining value (the last 8).  Input is appended by all lanes at once, lane k storing byte k.
constexpr int RING_WORDS = 56;
struct RunB3S {
  uint32_t *cv;  // ring + 48
  uint32_t *ring;
  uint32_t used, half;
  uint64_t counter;
};

__device__ inline void rb3s_load(RunB3S &s, uint32_t *ring, const DevB3S *g) {
  const uint32_t lane = threadIdx.x & 63;
  if (lane < 8) ring[48 + lane] = g->cv[lane];
  if (lane < 16) ring[lane] = g->block[lane], ring[16 + lane] = 0;
  __builtin_amdgcn_wave_barrier();
  s.cv = ring + 48;
  s.ring = ring;
  s.used = g->used, s.half = 0;
  s.counter = ((uint64_t)g->counter_hi << 32) | g->counter_lo;
}
__device__ inline void rb3s_store(const RunB3S &s, DevB3S *g) {
  const uint32_t lane = threadIdx.x & 63;
  if (lane < 8) g->cv[lane] = s.cv[lane];
  if (lane < 16) g->block[lane] = s.ring[16 * s.half + lane];
  g->used = s.used;
  g->counter_lo = (uint32_t)s.counter, g->counter_hi = (uint32_t)(s.counter >> 32);
}

// Append LEN <= 64 bytes, byte k of them held by lane k.  Bytes that do not fit the pending block go
// to the ring's other half (cleared first); the pending block is then full with more input behind it,
// so it is compressed and the halves change roles.  (A wavefront's LDS operations complete in order.)
__device__ inline void rb3s_append_bytes(RunB3S &s, uint32_t byte, uint32_t len) {
  const uint32_t lane = threadIdx.x & 63;
  uint8_t *bytes = reinterpret_cast<uint8_t *>(s.ring);
  if (lane < 16) s.ring[16 * (s.half ^ 1) + lane] = 0;
  __builtin_amdgcn_wave_barrier();
  if (lane < len) {
    const uint32_t o = s.used + lane;
    bytes[o < 64 ? 64 * s.half + o : 64 * (s.half ^ 1) + (o - 64)] = (uint8_t)byte;
  }
  __builtin_amdgcn_wave_barrier();
  if (s.used + len > 64) {
    uint32_t w0, w1, w2, w3;
    b3_compress_quad(s.cv, s.ring + 16 * s.half, s.counter, 64, 0, w0, w1, w2, w3);
    b3_quad_cv(w0, w1, s.cv);
    s.counter++;
    s.half ^= 1;
    s.used = s.used + len - 64;
  } else {
    s.used += len;
  }
}

// absorb(data) for NWORDS little-endian words in LDS: the length as u64 LE, then the bytes
// (src/transcript.lisp:95-100)
__device__ inline void dev_absorb_words(RunB3S &s, const uint32_t *words, uint32_t nwords) {
  const uint32_t lane = threadIdx.x & 63, total = 8 + 4 * nwords;
  for (uint32_t base = 0; base < total; base += 64) {
    const uint32_t g = base + lane;  // this lane's byte of the stream
    uint32_t word = g < 4 ? 4 * nwords : (g < 8 || g >= total) ? 0 : words[(g - 8) >> 2];
    rb3s_append_bytes(s, (word >> (8 * (g & 3))) & 0xff, total - base < 64 ? total - base : 64);
  }
}

// K <= 12 base-field challenges (CHALLENGE-BASE, src/transcript.lisp:159-172): squeeze 4 (missing + 4)
// bytes (at most 64: one output block), keep the 31-bit words below p, repeat until K are kept; each squeeze then absorbs "squeeze" and
// the first min(32, n) bytes of its output (src/transcript.lisp:152-157).  OUT is in LDS.
// `ready` is called by the whole wavefront as soon as the K challenges are in OUT: what follows (absorbing the last
// squeeze's bytes, a compression when they fill the block) is the transcript's own bookkeeping, which whoever waits
// for the challenge need not wait for.
// With `pending` (not null) the bytes the last squeeze leaves to absorb are handed back instead of absorbed: the
// caller absorbs them later (rb3s_flush), before anything else goes through the transcript -- in a round's serial
// part they would stand between the challenge and the fold that waits for it.
struct PendingAppend {
  uint32_t byte, len;  // this lane's byte of the stream; bytes in all (0: nothing pending)
};
__device__ inline void rb3s_flush(RunB3S &s, PendingAppend &pending) {
  if (pending.len) rb3s_append_bytes(s, pending.byte, pending.len);
  pending.len = 0;
}
template <class F>
__device__ inline void dev_challenge(RunB3S &s, int k, uint32_t *out, F ready, PendingAppend *pending = nullptr) {
  const uint32_t lane = threadIdx.x & 63;
  uint32_t *stage = s.ring + 32;
  int have = 0;
  while (have < k) {
    const uint32_t n = 4u * (uint32_t)(k - have + 4);  // at most 64 bytes: one output block
    uint32_t w0, w1, w2, w3;
    b3_compress_quad(s.cv, s.ring + 16 * s.half, 0, s.used, B3_CHUNK_END | B3_ROOT, w0, w1, w2, w3);
    if (lane < 4) stage[lane] = w0, stage[4 + lane] = w1, stage[8 + lane] = w2, stage[12 + lane] = w3;
    __builtin_amdgcn_wave_barrier();
    // "squeeze", then the first min(32, n) bytes of the output
    const uint32_t fed = n < 32 ? n : 32;
    uint32_t byte = 0;
    if (lane < 7)
      byte = (lane < 4 ? 0x65757173u >> (8 * lane) : 0x00657a65u >> (8 * (lane - 4))) & 0xff;
    else if (lane < 7 + fed)
      byte = (stage[(lane - 7) >> 2] >> (8 * ((lane - 7) & 3))) & 0xff;
    const uint32_t cand = lane < n / 4 ? stage[lane] & 0x7fffffffu : P;
    // the candidates below p, in order, as far as needed
    const uint64_t ok = __ballot(cand < P);
    const int rank = __popcll(ok & (((uint64_t)1 << lane) - 1));
    if (cand < P && have + rank < k) out[have + rank] = cand;
    have += __popcll(ok);
    __builtin_amdgcn_wave_barrier();
    if (have >= k) ready();
    if (have >= k && pending) {
      pending->byte = byte, pending->len = 7 + fed;
      return;
    }
    rb3s_append_bytes(s, byte, 7 + fed);
  }
}
__device__ inline void dev_challenge(RunB3S &s, int k, uint32_t *out) {
  dev_challenge(s, k, out, [] {});
}

}  // namespace exh
