// transcript.cpp -- see transcript.hpp.
#include "transcript.hpp"

#include <string.h>

#include "blake3.hpp"

namespace exh {

static thread_local std::string g_error;
void set_error(const std::string &what) { g_error = what; }
const char *last_error() { return g_error.c_str(); }

static inline void put_le(uint64_t v, int size, uint8_t *out) {
  for (int i = 0; i < size; i++) out[i] = (uint8_t)(v >> (8 * i));
}
static inline uint64_t get_le(const uint8_t *b, int size) {
  uint64_t v = 0;
  for (int i = 0; i < size; i++) v |= (uint64_t)b[i] << (8 * i);
  return v;
}
static void words_of(const uint8_t block[64], uint32_t w[16]) {
  for (int i = 0; i < 16; i++) w[i] = (uint32_t)get_le(block + 4 * i, 4);
}

// n bytes of root output from (cv, block words, block length, flags): block i of the output is the
// compression with counter i (src/blake3.lisp:113-123)
static void root_output(const uint32_t cv[8], const uint32_t w[16], uint32_t block_len, uint32_t flags,
                        uint8_t *out, uint64_t n) {
  uint64_t counter = 0;
  for (uint64_t pos = 0; pos < n; pos += 64, counter++) {
    uint32_t o[16];
    b3_compress(cv, w, counter, block_len, flags | B3_ROOT, o, 1);
    for (uint64_t i = pos, j = 0; i < n && j < 64; i++, j++) out[i] = (uint8_t)(o[j >> 2] >> (8 * (j & 3)));
  }
}

// ---- B3S
B3S::B3S() {
  b3_iv(cv);
  memset(block, 0, 64);
}

void B3S::update(const uint8_t *data, uint64_t len) {
  while (len) {
    if (used == 64) {  // a full block is compressed only when more input arrives
      uint32_t w[16];
      words_of(block, w);
      b3_compress(cv, w, counter++, 64, 0, cv, 0);
      memset(block, 0, 64);
      used = 0;
    }
    uint64_t take = len < 64 - used ? len : 64 - used;
    memcpy(block + used, data, take);
    used += (uint32_t)take;
    data += take;
    len -= take;
  }
}

void B3S::digest(uint8_t *out, uint64_t n) const {
  uint32_t w[16];
  words_of(block, w);
  root_output(cv, w, used, B3_CHUNK_END, out, n);
}

// ---- standard BLAKE3 over any length: chunks of 1024 bytes, a stack of subtree chaining values
void blake3_hash(const uint8_t *in, uint64_t len, uint8_t *out, uint64_t n) {
  uint32_t stack[64][8];
  int depth = 0;
  uint64_t nchunks = len == 0 ? 1 : (len + 1023) / 1024;
  uint32_t cv[8], w[16];
  uint32_t last_len = 0, last_flags = 0;
  for (uint64_t c = 0; c < nchunks; c++) {
    const uint8_t *chunk = in + 1024 * c;
    uint64_t clen = len - 1024 * c < 1024 ? len - 1024 * c : 1024;
    uint64_t nblocks = clen == 0 ? 1 : (clen + 63) / 64;
    b3_iv(cv);
    for (uint64_t b = 0; b < nblocks; b++) {
      uint8_t block[64] = {0};
      uint64_t blen = clen - 64 * b < 64 ? clen - 64 * b : 64;
      memcpy(block, chunk + 64 * b, blen);
      words_of(block, w);
      uint32_t flags = (b == 0 ? B3_CHUNK_START : 0u) | (b == nblocks - 1 ? B3_CHUNK_END : 0u);
      if (b == nblocks - 1 && c == nchunks - 1) {  // the last block of the input stays pending
        last_len = (uint32_t)blen;
        last_flags = flags;
        break;
      }
      b3_compress(cv, w, c, (uint32_t)blen, flags, cv, 0);
    }
    if (c == nchunks - 1) break;
    // a finished chunk: merge completed subtrees, one parent per trailing zero bit of the count
    uint32_t merged[8];
    memcpy(merged, cv, 32);
    for (uint64_t count = c + 1; (count & 1) == 0; count >>= 1) {
      uint32_t pw[16], iv[8];
      b3_iv(iv);
      memcpy(pw, stack[--depth], 32);
      memcpy(pw + 8, merged, 32);
      b3_compress(iv, pw, 0, 64, B3_PARENT, merged, 0);
    }
    memcpy(stack[depth++], merged, 32);
  }
  // the root: the pending chunk block, or parents up the stack
  uint32_t rcv[8], rw[16];
  uint64_t rcounter = nchunks - 1;
  uint32_t rlen = last_len, rflags = last_flags;
  memcpy(rcv, cv, 32);
  memcpy(rw, w, 64);
  while (depth > 0) {
    uint32_t child[8];
    b3_compress(rcv, rw, rcounter, rlen, rflags, child, 0);
    b3_iv(rcv);
    memcpy(rw, stack[--depth], 32);
    memcpy(rw + 8, child, 32);
    rcounter = 0;
    rlen = 64;
    rflags = B3_PARENT;
  }
  // root_output uses counter = output block index; the chunk counter of a single-chunk root is 0
  root_output(rcv, rw, rlen, rflags, out, n);
}

// ---- transcript
static const char kDomain[] = "LLM-SUMCHECK-v6-O|";

Transcript::Transcript(const uint8_t *label, uint64_t label_len, int degree) : D(degree) {
  state.update((const uint8_t *)kDomain, sizeof(kDomain) - 1);
  state.update(label, label_len);
}

void Transcript::absorb(const uint8_t *data, uint64_t len) {
  uint8_t l[8];
  put_le(len, 8, l);
  state.update(l, 8);
  state.update(data, len);
}

int Transcript::send(const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out, bool absorb_it) {
  Message *m;
  if (verifier) {
    if (position >= messages.size()) return E_EXHAUSTED;
    m = &messages[position];
    if (m->kind != 1) return E_SHAPE;
    if (rank >= 0) {
      if ((int)m->dims.size() != rank) return E_SHAPE;
      for (int i = 0; i < rank; i++)
        if (m->dims[i] != dims[i]) return E_SHAPE;
    }
    position++;
  } else {
    if (rank < 0 || rank > 8) return E_PARAM;
    messages.emplace_back();
    m = &messages.back();
    m->kind = 1;
    m->dims.assign(dims, dims + rank);
    uint64_t count = 1;
    for (int i = 0; i < rank; i++) count *= dims[i];
    m->vals.resize(count);
    for (uint64_t i = 0; i < count; i++) m->vals[i] = vals[i] % 2130706433u;
  }
  sent_bytes += m->size_bytes();
  if (absorb_it) {
    std::vector<uint8_t> buf(4 * m->vals.size());
    for (size_t i = 0; i < m->vals.size(); i++) put_le(m->vals[i], 4, buf.data() + 4 * i);
    absorb(buf.data(), buf.size());
  }
  if (out) memcpy(out, m->vals.data(), 4 * m->vals.size());
  return OK;
}

int Transcript::send_bytes(const uint8_t *bytes, int64_t len, std::vector<uint8_t> *out, bool absorb_it) {
  Message *m;
  if (verifier) {
    if (position >= messages.size()) return E_EXHAUSTED;
    m = &messages[position];
    if (m->kind != 0) return E_SHAPE;
    if (len >= 0 && m->bytes.size() != (uint64_t)len) return E_SHAPE;
    position++;
  } else {
    if (len < 0) return E_PARAM;
    messages.emplace_back();
    m = &messages.back();
    m->kind = 0;
    m->bytes.assign(bytes, bytes + len);
  }
  sent_bytes += m->size_bytes();
  if (absorb_it) absorb(m->bytes.data(), m->bytes.size());
  if (out) *out = m->bytes;
  return OK;
}

void Transcript::squeeze(uint8_t *out, uint64_t n) {
  state.digest(out, n);
  state.update((const uint8_t *)"squeeze", 7);
  state.update(out, n < 32 ? n : 32);
}

void Transcript::challenge_base(int k, uint32_t *out) {
  int have = 0;
  std::vector<uint8_t> buf;
  while (have < k) {  // 31-bit words below p are kept; squeeze (missing + 4) words at a time
    uint64_t n = 4 * (uint64_t)(k - have + 4);
    buf.resize(n);
    squeeze(buf.data(), n);
    for (uint64_t i = 0; i < n && have < k; i += 4) {
      uint32_t word = (uint32_t)get_le(buf.data() + i, 4) & 0x7fffffffu;
      if (word < 2130706433u) out[have++] = word;
    }
  }
}

void Transcript::challenge_bits(int nbits, int k, uint64_t *out) {
  std::vector<uint8_t> buf(8 * (size_t)k);
  squeeze(buf.data(), buf.size());
  for (int i = 0; i < k; i++) {
    uint64_t w = get_le(buf.data() + 8 * i, 8);
    out[i] = nbits >= 64 ? w : w & (((uint64_t)1 << nbits) - 1);
  }
}

bool check_grind(const uint8_t base[32], uint64_t nonce, int bits) {
  uint8_t in[40], out[8];
  memcpy(in, base, 32);
  put_le(nonce, 8, in + 32);
  blake3_hash(in, 40, out, 8);
  return bits <= 0 || get_le(out, 8) < ((uint64_t)1 << (64 - bits));
}

uint64_t Transcript::grind(int bits) {
  uint8_t base[32], nb[8];
  state.digest(base, 32);
  uint64_t nonce = 0;
  while (!check_grind(base, nonce, bits)) nonce++;
  put_le(nonce, 8, nb);
  send_bytes(nb, 8, nullptr);
  return nonce;
}

int Transcript::verify_grind(int bits, uint64_t *nonce) {
  uint8_t base[32];
  state.digest(base, 32);
  std::vector<uint8_t> nb;
  int st = send_bytes(nullptr, 8, &nb);
  if (st) return st;
  *nonce = get_le(nb.data(), 8);
  return check_grind(base, *nonce, bits) ? OK : E_REJECT;
}

// ---- proof bytes: MAGIC | u32 count | messages (src/proofio.lisp:1-9)
std::vector<uint8_t> Transcript::encode_proof() const {
  std::vector<uint8_t> out;
  auto put = [&](uint64_t v, int size) {
    for (int i = 0; i < size; i++) out.push_back((uint8_t)(v >> (8 * i)));
  };
  const char magic[] = "EXACTPF1";
  out.insert(out.end(), magic, magic + 8);
  put(messages.size(), 4);
  for (const Message &m : messages) {
    if (m.kind == 0) {
      out.push_back(0);
      put(m.bytes.size(), 8);
      out.insert(out.end(), m.bytes.begin(), m.bytes.end());
    } else {
      out.push_back(1);
      out.push_back((uint8_t)m.dims.size());
      for (uint64_t d : m.dims) put(d, 8);
      for (uint32_t v : m.vals) put(v, 4);
    }
  }
  return out;
}

int Transcript::load_proof(const uint8_t *octets, uint64_t end) {
  uint64_t pos = 0;
  messages.clear();
  position = 0;
  auto fail = [&](int reason) {
    malformed_reason = reason;
    messages.clear();
    return (int)E_MALFORMED;
  };
  if (end < 8 || (memcmp(octets, "EXACTPF1", 8) != 0 && memcmp(octets, "SABLEPF1", 8) != 0)) return fail(MF_MAGIC);
  pos = 8;
  if (end - pos < 4) return fail(MF_TRUNCATED);
  uint64_t count = get_le(octets + pos, 4);
  pos += 4;
  for (uint64_t k = 0; k < count; k++) {
    if (end - pos < 1) return fail(MF_TRUNCATED);
    int tag = octets[pos++];
    if (tag == 0) {
      if (end - pos < 8) return fail(MF_TRUNCATED);
      uint64_t len = get_le(octets + pos, 8);
      pos += 8;
      if (len > end - pos) return fail(MF_TRUNCATED);
      Message m;
      m.kind = 0;
      m.bytes.assign(octets + pos, octets + pos + len);
      pos += len;
      messages.push_back(std::move(m));
    } else if (tag == 1) {
      if (end - pos < 1) return fail(MF_TRUNCATED);
      int rank = octets[pos++];
      if (rank > 8) return fail(MF_RANK);
      Message m;
      m.kind = 1;
      unsigned __int128 size = 1;
      const unsigned __int128 cap = (unsigned __int128)1 << 100;
      for (int d = 0; d < rank; d++) {
        if (end - pos < 8) return fail(MF_TRUNCATED);
        m.dims.push_back(get_le(octets + pos, 8));
        pos += 8;
        size = size * m.dims.back();  // exact: a huge shape is rejected as truncated
        if (size > cap) size = cap;
      }
      if (size * 4 > (unsigned __int128)(end - pos)) return fail(MF_TRUNCATED);
      for (uint64_t d : m.dims)
        if (d >= ((uint64_t)1 << 61)) return fail(MF_DIMENSION);
      uint64_t n = (uint64_t)size;
      m.vals.resize(n);
      for (uint64_t i = 0; i < n; i++) {
        uint32_t v = (uint32_t)get_le(octets + pos + 4 * i, 4);
        if (v >= 2130706433u) return fail(MF_RANGE);
        m.vals[i] = v;
      }
      pos += 4 * n;
      messages.push_back(std::move(m));
    } else {
      return fail(MF_TAG);
    }
  }
  if (pos != end) return fail(MF_TRAILING);
  verifier = true;
  malformed_reason = MF_NONE;
  return OK;
}

}  // namespace exh
