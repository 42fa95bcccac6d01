// transcript.hpp -- host side of the proving path: the sequential BLAKE3 mode, the Fiat-Shamir
// transcript and the proof byte format, mirroring the reference's src/blake3.lisp:125-155,
// src/transcript.lisp and src/proofio.lisp (same operations, same bytes).
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

namespace exh {

// status codes shared by the whole C ABI (include/exacta_hip.h)
enum Status : int {
  OK = 0,
  E_PARAM = -1,      // invalid-parameter
  E_DIVZERO = -2,    // field-division-by-zero
  E_SHAPE = -3,      // message-shape-error
  E_EXHAUSTED = -4,  // transcript-exhausted
  E_REJECT = -5,     // verification-failure
  E_MALFORMED = -6,  // malformed-proof
  E_DEVICE = -7,     // a HIP call failed, or no usable GPU
  E_NOMEM = -8,
};

enum MalformedReason : int { MF_NONE = 0, MF_MAGIC, MF_TRUNCATED, MF_TRAILING, MF_TAG, MF_RANGE, MF_RANK, MF_DIMENSION };

void set_error(const std::string &what);
const char *last_error();

// BLAKE3 of a byte string of any length (tree mode), n output bytes (src/blake3.lisp:157-233)
void blake3_hash(const uint8_t *in, uint64_t len, uint8_t *out, uint64_t n);

// The sequential mode of the transcript hash: one chaining value per 64-byte block, output from the
// pending block with CHUNK_END | ROOT (src/blake3.lisp:125-155).
struct B3S {
  uint32_t cv[8];
  uint8_t block[64];
  uint32_t used = 0;
  uint64_t counter = 0;
  B3S();
  void update(const uint8_t *data, uint64_t len);
  void digest(uint8_t *out, uint64_t n) const;
};

struct Message {
  int kind = 0;  // 0: bytes, 1: field array
  std::vector<uint64_t> dims;
  std::vector<uint8_t> bytes;
  std::vector<uint32_t> vals;
  uint64_t size_bytes() const { return kind == 0 ? bytes.size() : 4 * vals.size(); }
};

struct Transcript {
  int D;
  B3S state;
  bool verifier = false;
  std::vector<Message> messages;
  size_t position = 0;
  uint64_t sent_bytes = 0;
  int malformed_reason = MF_NONE;

  Transcript(const uint8_t *label, uint64_t label_len, int degree);
  // a verifier transcript over the messages of a proof; status OK or E_MALFORMED
  int load_proof(const uint8_t *proof, uint64_t len);

  void absorb(const uint8_t *data, uint64_t len);
  // prover: record VALS (reduced mod p) with the given shape; verifier: take the next field array,
  // which must have that shape (rank < 0: any); out (optional) receives the values
  int send(const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out, bool absorb_it = true);
  int send_bytes(const uint8_t *bytes, int64_t len, std::vector<uint8_t> *out, bool absorb_it = true);
  void squeeze(uint8_t *out, uint64_t n);
  void challenge_base(int k, uint32_t *out);
  void challenge(int degree, uint32_t *out) { challenge_base(degree > 0 ? degree : D, out); }
  void challenges(int k, int degree, uint32_t *out) { challenge_base((degree > 0 ? degree : D) * k, out); }
  void challenge_bits(int nbits, int k, uint64_t *out);
  uint64_t grind(int bits);
  int verify_grind(int bits, uint64_t *nonce);
  bool finished() const { return position == messages.size(); }
  std::vector<uint8_t> encode_proof() const;
};

bool check_grind(const uint8_t base[32], uint64_t nonce, int bits);

}  // namespace exh
