/* orc_blake3.c -- BLAKE3 in its two modes, restated from src/blake3.lisp (test oracle; see orc.h). */
#include "orc.h"
#include <string.h>

enum { CHUNK_START = 1, CHUNK_END = 2, PARENT = 4, ROOT = 8, CHUNK_LEN = 1024 };

static const uint32_t IV[8] = {0x6A09E667u, 0xBB67AE85u, 0x3C6EF372u, 0xA54FF53Au,
                               0x510E527Fu, 0x9B05688Cu, 0x1F83D9ABu, 0x5BE0CD19u};
static const uint8_t PERM[16] = {2, 6, 3, 10, 7, 0, 4, 13, 1, 11, 12, 5, 9, 14, 15, 8};

static uint32_t rotr(uint32_t w, int n) { return (w >> n) | (w << (32 - n)); }

#define G(a, b, c, d, x, y)     \
  v[a] = v[a] + v[b] + (x);     \
  v[d] = rotr(v[d] ^ v[a], 16); \
  v[c] = v[c] + v[d];           \
  v[b] = rotr(v[b] ^ v[c], 12); \
  v[a] = v[a] + v[b] + (y);     \
  v[d] = rotr(v[d] ^ v[a], 8);  \
  v[c] = v[c] + v[d];           \
  v[b] = rotr(v[b] ^ v[c], 7);

/* src/blake3.lisp:44-88 */
void orc_blake3_compress(const uint32_t cv[8], const uint32_t m_in[16], uint64_t counter,
                         uint32_t block_len, uint32_t flags, uint32_t out[16]) {
  uint32_t v[16], m[16], t[16];
  memcpy(v, cv, 32);
  memcpy(v + 8, IV, 16);
  v[12] = (uint32_t)counter;
  v[13] = (uint32_t)(counter >> 32);
  v[14] = block_len;
  v[15] = flags;
  memcpy(m, m_in, 64);
  for (int r = 0; r < 7; r++) {
    G(0, 4, 8, 12, m[0], m[1]);
    G(1, 5, 9, 13, m[2], m[3]);
    G(2, 6, 10, 14, m[4], m[5]);
    G(3, 7, 11, 15, m[6], m[7]);
    G(0, 5, 10, 15, m[8], m[9]);
    G(1, 6, 11, 12, m[10], m[11]);
    G(2, 7, 8, 13, m[12], m[13]);
    G(3, 4, 9, 14, m[14], m[15]);
    for (int i = 0; i < 16; i++) t[i] = m[PERM[i]];
    memcpy(m, t, 64);
  }
  for (int i = 0; i < 8; i++) {
    out[i] = v[i] ^ v[i + 8];
    out[i + 8] = v[i + 8] ^ cv[i];
  }
}

static void block_words(const uint8_t block[64], uint32_t w[16]) {
  for (int i = 0; i < 16; i++)
    w[i] = (uint32_t)block[4 * i] | (uint32_t)block[4 * i + 1] << 8 | (uint32_t)block[4 * i + 2] << 16 |
           (uint32_t)block[4 * i + 3] << 24;
}

/* src/blake3.lisp:113-123 */
static void root_output(const uint32_t cv[8], const uint32_t words[16], uint32_t block_len,
                        uint32_t flags, uint8_t *out, uint64_t n) {
  uint64_t counter = 0;
  for (uint64_t pos = 0; pos < n; pos += 64, counter++) {
    uint32_t b[16];
    orc_blake3_compress(cv, words, counter, block_len, flags | ROOT, b);
    for (uint64_t i = pos, j = 0; i < n && j < 64; i++, j++) out[i] = (uint8_t)(b[j / 4] >> (8 * (j % 4)));
  }
}

/* ---- sequential mode, src/blake3.lisp:125-155: a full block is compressed only once more input
   arrives, so the last block, possibly empty, is always pending (FILL-BLOCKS, :99-111) */
void orc_b3s_init(orc_b3s *s) {
  memcpy(s->cv, IV, 32);
  memset(s->block, 0, 64);
  s->used = 0;
  s->counter = 0;
}

void orc_b3s_update(orc_b3s *s, const uint8_t *data, uint64_t len) {
  uint64_t start = 0;
  while (start < len) {
    if (s->used == 64) {
      uint32_t w[16], o[16];
      block_words(s->block, w);
      orc_blake3_compress(s->cv, w, s->counter, 64, 0, o);
      memcpy(s->cv, o, 32);
      s->counter++;
      memset(s->block, 0, 64);
      s->used = 0;
    }
    uint64_t n = len - start;
    if (n > 64 - s->used) n = 64 - s->used;
    memcpy(s->block + s->used, data + start, n);
    s->used += (uint32_t)n;
    start += n;
  }
}

void orc_b3s_digest(const orc_b3s *s, uint8_t *out, uint64_t n) {
  uint32_t w[16];
  block_words(s->block, w);
  root_output(s->cv, w, s->used, CHUNK_END, out, n);
}

/* ---- standard BLAKE3 (tree mode), src/blake3.lisp:157-233 */
typedef struct {
  uint32_t cv[8];
  uint64_t counter;
  uint8_t block[64];
  uint32_t used;
  uint32_t blocks_compressed;
} chunk_t;

typedef struct {
  uint32_t cv[8], words[16];
  uint64_t counter;
  uint32_t block_len, flags;
} node_t;

static void chunk_init(chunk_t *c, uint64_t counter) {
  memcpy(c->cv, IV, 32);
  c->counter = counter;
  memset(c->block, 0, 64);
  c->used = 0;
  c->blocks_compressed = 0;
}
static uint32_t chunk_len(const chunk_t *c) { return 64 * c->blocks_compressed + c->used; }
static uint32_t chunk_start_flag(const chunk_t *c) { return c->blocks_compressed == 0 ? CHUNK_START : 0; }

static void chunk_update(chunk_t *c, const uint8_t *data, uint64_t len) {
  uint64_t start = 0;
  while (start < len) {
    if (c->used == 64) {
      uint32_t w[16], o[16];
      block_words(c->block, w);
      orc_blake3_compress(c->cv, w, c->counter, 64, chunk_start_flag(c), o);
      memcpy(c->cv, o, 32);
      c->blocks_compressed++;
      memset(c->block, 0, 64);
      c->used = 0;
    }
    uint64_t n = len - start;
    if (n > 64 - c->used) n = 64 - c->used;
    memcpy(c->block + c->used, data + start, n);
    c->used += (uint32_t)n;
    start += n;
  }
}

static void chunk_node(const chunk_t *c, node_t *nd) {
  memcpy(nd->cv, c->cv, 32);
  block_words(c->block, nd->words);
  nd->counter = c->counter;
  nd->block_len = c->used;
  nd->flags = chunk_start_flag(c) | CHUNK_END;
}
static void parent_node(const uint32_t left[8], const uint32_t right[8], node_t *nd) {
  memcpy(nd->cv, IV, 32);
  memcpy(nd->words, left, 32);
  memcpy(nd->words + 8, right, 32);
  nd->counter = 0;
  nd->block_len = 64;
  nd->flags = PARENT;
}
static void node_cv(const node_t *nd, uint32_t cv[8]) {
  uint32_t o[16];
  orc_blake3_compress(nd->cv, nd->words, nd->counter, nd->block_len, nd->flags, o);
  memcpy(cv, o, 32);
}

void orc_blake3_hash(const uint8_t *in, uint64_t len, uint8_t *out, uint64_t outlen) {
  chunk_t chunk;
  uint32_t stack[64][8];
  int depth = 0;
  chunk_init(&chunk, 0);
  uint64_t start = 0;
  while (start < len) {
    if (chunk_len(&chunk) == CHUNK_LEN) { /* FINISH-CHUNK, :203-212 */
      node_t nd;
      uint32_t cv[8];
      chunk_node(&chunk, &nd);
      node_cv(&nd, cv);
      for (uint64_t chunks = chunk.counter + 1; (chunks & 1) == 0; chunks >>= 1) {
        node_t pn;
        parent_node(stack[--depth], cv, &pn);
        node_cv(&pn, cv);
      }
      memcpy(stack[depth++], cv, 32);
      chunk_init(&chunk, chunk.counter + 1);
    }
    uint64_t n = len - start;
    if (n > CHUNK_LEN - chunk_len(&chunk)) n = CHUNK_LEN - chunk_len(&chunk);
    chunk_update(&chunk, in + start, n);
    start += n;
  }
  node_t root;
  chunk_node(&chunk, &root);
  while (depth > 0) { /* BLAKE3-DIGEST, :224-229 */
    uint32_t cv[8];
    node_cv(&root, cv);
    parent_node(stack[--depth], cv, &root);
  }
  root_output(root.cv, root.words, root.block_len, root.flags, out, outlen);
}
