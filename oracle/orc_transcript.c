/* orc_transcript.c -- the Fiat-Shamir transcript and the proof byte format, restated from
 * src/transcript.lisp and src/proofio.lisp (test oracle; see orc.h). */
#include "orc.h"
#include <stdlib.h>
#include <string.h>

struct orc_tr {
  int D;
  orc_b3s state;
  int verifier;
  orc_msg *msgs;
  uint64_t nmsgs, cap, pos, sent_bytes;
};

static const char DOMAIN[] = "LLM-SUMCHECK-v6-O|"; /* src/transcript.lisp:24 */
static int g_malformed_reason = 0;
int orc_malformed_reason(void) { return g_malformed_reason; }

static void le_bytes(uint64_t v, int size, uint8_t *out) {
  for (int i = 0; i < size; i++) out[i] = (uint8_t)(v >> (8 * i));
}
static uint64_t le_integer(const uint8_t *b, int size) {
  uint64_t v = 0;
  for (int i = 0; i < size; i++) v |= (uint64_t)b[i] << (8 * i);
  return v;
}

static orc_tr *tr_alloc(const uint8_t *label, uint64_t label_len, int D) {
  if (D != 4 && D != 8) return NULL; /* check-degree, src/field.lisp:105-108 */
  orc_tr *tr = (orc_tr *)calloc(1, sizeof(orc_tr));
  tr->D = D;
  orc_b3s_init(&tr->state); /* src/transcript.lisp:75-84: domain || label, no length prefix */
  orc_b3s_update(&tr->state, (const uint8_t *)DOMAIN, sizeof(DOMAIN) - 1);
  orc_b3s_update(&tr->state, label, label_len);
  return tr;
}

orc_tr *orc_tr_new(const uint8_t *label, uint64_t label_len, int D) { return tr_alloc(label, label_len, D); }

static void msg_free(orc_msg *m) {
  free(m->bytes);
  free(m->vals);
}

void orc_tr_free(orc_tr *tr) {
  if (!tr) return;
  for (uint64_t i = 0; i < tr->nmsgs; i++) msg_free(&tr->msgs[i]);
  free(tr->msgs);
  free(tr);
}

int orc_tr_degree(const orc_tr *tr) { return tr->D; }

static orc_msg *push_msg(orc_tr *tr) {
  if (tr->nmsgs == tr->cap) {
    tr->cap = tr->cap ? 2 * tr->cap : 16;
    tr->msgs = (orc_msg *)realloc(tr->msgs, tr->cap * sizeof(orc_msg));
  }
  orc_msg *m = &tr->msgs[tr->nmsgs++];
  memset(m, 0, sizeof(*m));
  return m;
}

/* src/transcript.lisp:95-100 */
void orc_tr_absorb(orc_tr *tr, const uint8_t *data, uint64_t len) {
  uint8_t l[8];
  le_bytes(len, 8, l);
  orc_b3s_update(&tr->state, l, 8);
  orc_b3s_update(&tr->state, data, len);
}

static void absorb_values(orc_tr *tr, const uint32_t *vals, uint64_t count) {
  uint8_t *buf = (uint8_t *)malloc(4 * count + 1);
  for (uint64_t i = 0; i < count; i++) le_bytes(vals[i], 4, buf + 4 * i);
  orc_tr_absorb(tr, buf, 4 * count);
  free(buf);
}

static uint64_t dims_count(int rank, const uint64_t *dims) {
  uint64_t c = 1;
  for (int i = 0; i < rank; i++) c *= dims[i];
  return c;
}

/* EXCHANGE for field arrays, src/transcript.lisp:102-128 */
static int exchange_field(orc_tr *tr, const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out,
                          int absorb) {
  orc_msg *m;
  if (tr->verifier) {
    if (tr->pos >= tr->nmsgs) return ORC_E_EXHAUSTED;
    m = &tr->msgs[tr->pos];
    if (m->kind != 1) return ORC_E_SHAPE;
    if (rank >= 0) {
      if (m->rank != rank) return ORC_E_SHAPE;
      for (int i = 0; i < rank; i++)
        if (m->dims[i] != dims[i]) return ORC_E_SHAPE;
    }
    tr->pos++;
  } else {
    if (rank < 0 || rank > 8) return ORC_E_PARAM;
    m = push_msg(tr);
    m->kind = 1;
    m->rank = rank;
    for (int i = 0; i < rank; i++) m->dims[i] = dims[i];
    m->count = dims_count(rank, dims);
    m->vals = (uint32_t *)malloc(4 * m->count + 4);
    for (uint64_t i = 0; i < m->count; i++) m->vals[i] = vals[i] % ORC_P; /* to-field-array: canonical */
  }
  tr->sent_bytes += 4 * m->count;
  if (absorb) absorb_values(tr, m->vals, m->count);
  if (out) memcpy(out, m->vals, 4 * m->count);
  return ORC_OK;
}

int orc_tr_send(orc_tr *tr, const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out) {
  return exchange_field(tr, vals, rank, dims, out, 1);
}
int orc_tr_record(orc_tr *tr, const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out) {
  return exchange_field(tr, vals, rank, dims, out, 0);
}

static int exchange_bytes(orc_tr *tr, const uint8_t *bytes, int64_t len, uint8_t *out, uint64_t cap,
                          uint64_t *out_len, int absorb) {
  orc_msg *m;
  if (tr->verifier) {
    if (tr->pos >= tr->nmsgs) return ORC_E_EXHAUSTED;
    m = &tr->msgs[tr->pos];
    if (m->kind != 0) return ORC_E_SHAPE;
    if (len >= 0 && m->count != (uint64_t)len) return ORC_E_SHAPE;
    tr->pos++;
  } else {
    m = push_msg(tr);
    m->kind = 0;
    m->count = (uint64_t)len;
    m->bytes = (uint8_t *)malloc(m->count + 1);
    memcpy(m->bytes, bytes, m->count);
  }
  tr->sent_bytes += m->count;
  if (absorb) orc_tr_absorb(tr, m->bytes, m->count);
  if (out_len) *out_len = m->count;
  if (out) memcpy(out, m->bytes, m->count < cap ? m->count : cap);
  return ORC_OK;
}

int orc_tr_send_bytes(orc_tr *tr, const uint8_t *bytes, int64_t len, uint8_t *out, uint64_t cap,
                      uint64_t *out_len) {
  return exchange_bytes(tr, bytes, len, out, cap, out_len, 1);
}
int orc_tr_record_bytes(orc_tr *tr, const uint8_t *bytes, int64_t len, uint8_t *out, uint64_t cap,
                        uint64_t *out_len) {
  return exchange_bytes(tr, bytes, len, out, cap, out_len, 0);
}

/* src/transcript.lisp:152-157 */
void orc_tr_squeeze(orc_tr *tr, uint8_t *out, uint64_t n) {
  orc_b3s_digest(&tr->state, out, n);
  orc_b3s_update(&tr->state, (const uint8_t *)"squeeze", 7);
  orc_b3s_update(&tr->state, out, n < 32 ? n : 32);
}

/* src/transcript.lisp:159-172 */
void orc_tr_challenge_base(orc_tr *tr, int k, uint32_t *out) {
  int have = 0;
  while (have < k) {
    uint64_t n = 4 * (uint64_t)((k - have) + 4);
    uint8_t *buf = (uint8_t *)malloc(n);
    orc_tr_squeeze(tr, buf, n);
    for (uint64_t i = 0; i < n; i += 4) {
      uint32_t word = (uint32_t)le_integer(buf + i, 4) & 0x7fffffffu;
      if (word < ORC_P && have < k) out[have++] = word;
    }
    free(buf);
  }
}

void orc_tr_challenge(orc_tr *tr, int degree, uint32_t *out) {
  orc_tr_challenge_base(tr, degree > 0 ? degree : tr->D, out);
}
/* one stream of degree * k base challenges (src/transcript.lisp:178-181) */
void orc_tr_challenges(orc_tr *tr, int k, int degree, uint32_t *out) {
  orc_tr_challenge_base(tr, (degree > 0 ? degree : tr->D) * k, out);
}

/* src/transcript.lisp:183-187 */
void orc_tr_challenge_bits(orc_tr *tr, int nbits, int k, uint64_t *out) {
  uint8_t *buf = (uint8_t *)malloc(8 * (size_t)k + 1);
  orc_tr_squeeze(tr, buf, 8 * (uint64_t)k);
  for (int i = 0; i < k; i++) {
    uint64_t w = le_integer(buf + 8 * i, 8);
    out[i] = nbits >= 64 ? w : (w & (((uint64_t)1 << nbits) - 1));
  }
  free(buf);
}

/* src/transcript.lisp:191-209 */
int orc_check_grind(const uint8_t base[32], uint64_t nonce, int bits) {
  uint8_t in[40], out[8];
  memcpy(in, base, 32);
  le_bytes(nonce, 8, in + 32);
  orc_blake3_hash(in, 40, out, 8);
  uint64_t v = le_integer(out, 8);
  return bits == 0 ? 1 : v < ((uint64_t)1 << (64 - bits));
}
uint64_t orc_tr_grind(orc_tr *tr, int bits) {
  uint8_t base[32], nb[8];
  orc_b3s_digest(&tr->state, base, 32);
  uint64_t nonce = 0;
  while (!orc_check_grind(base, nonce, bits)) nonce++;
  le_bytes(nonce, 8, nb);
  orc_tr_send_bytes(tr, nb, 8, NULL, 0, NULL);
  return nonce;
}
int orc_tr_verify_grind(orc_tr *tr, int bits, uint64_t *nonce) {
  uint8_t base[32], nb[8];
  orc_b3s_digest(&tr->state, base, 32);
  int st = orc_tr_send_bytes(tr, NULL, 8, nb, 8, NULL);
  if (st) return st;
  *nonce = le_integer(nb, 8);
  return orc_check_grind(base, *nonce, bits) ? ORC_OK : ORC_E_REJECT;
}

void orc_tr_state_digest(const orc_tr *tr, uint8_t out[32]) { orc_b3s_digest(&tr->state, out, 32); }
int orc_tr_finished(const orc_tr *tr) { return tr->pos == tr->nmsgs; }
uint64_t orc_tr_message_count(const orc_tr *tr) { return tr->nmsgs; }
const orc_msg *orc_tr_message(const orc_tr *tr, uint64_t i) { return i < tr->nmsgs ? &tr->msgs[i] : NULL; }

/* ---- proof bytes, src/proofio.lisp:1-9, 30-49 */
static const char MAGIC[] = "EXACTPF1";
static const char LEGACY[] = "SABLEPF1";

uint64_t orc_tr_encode_proof(const orc_tr *tr, uint8_t *out, uint64_t cap) {
  uint64_t size = 12;
  for (uint64_t i = 0; i < tr->nmsgs; i++) {
    const orc_msg *m = &tr->msgs[i];
    size += m->kind == 0 ? 9 + m->count : 2 + 8 * (uint64_t)m->rank + 4 * m->count;
  }
  if (!out || cap < size) return size;
  uint8_t *p = out;
  memcpy(p, MAGIC, 8);
  p += 8;
  le_bytes(tr->nmsgs, 4, p);
  p += 4;
  for (uint64_t i = 0; i < tr->nmsgs; i++) {
    const orc_msg *m = &tr->msgs[i];
    if (m->kind == 0) {
      *p++ = 0;
      le_bytes(m->count, 8, p);
      p += 8;
      memcpy(p, m->bytes, m->count);
      p += m->count;
    } else {
      *p++ = 1;
      *p++ = (uint8_t)m->rank;
      for (int d = 0; d < m->rank; d++, p += 8) le_bytes(m->dims[d], 8, p);
      for (uint64_t k = 0; k < m->count; k++, p += 4) le_bytes(m->vals[k], 4, p);
    }
  }
  return size;
}

/* DECODE-PROOF, src/proofio.lisp:53-101: every length checked against the remaining input, every
   value against p, dimensions multiplied exactly */
static int decode_proof(orc_tr *tr, const uint8_t *octets, uint64_t end) {
  uint64_t pos = 0;
  g_malformed_reason = ORC_MF_NONE;
#define FAIL(r)               \
  do {                        \
    g_malformed_reason = (r); \
    return ORC_E_MALFORMED;   \
  } while (0)
#define TAKE(n)                                   \
  do {                                            \
    if ((uint64_t)(n) > end - pos) FAIL(ORC_MF_TRUNCATED); \
  } while (0)
  if (end < 8 || (memcmp(octets, MAGIC, 8) != 0 && memcmp(octets, LEGACY, 8) != 0)) FAIL(ORC_MF_MAGIC);
  pos = 8;
  TAKE(4);
  uint64_t count = le_integer(octets + pos, 4);
  pos += 4;
  for (uint64_t k = 0; k < count; k++) {
    TAKE(1);
    int tag = octets[pos++];
    if (tag == 0) {
      TAKE(8);
      uint64_t len = le_integer(octets + pos, 8);
      pos += 8;
      TAKE(len);
      orc_msg *m = push_msg(tr);
      m->kind = 0;
      m->count = len;
      m->bytes = (uint8_t *)malloc(len + 1);
      memcpy(m->bytes, octets + pos, len);
      pos += len;
    } else if (tag == 1) {
      TAKE(1);
      int rank = octets[pos++];
      if (rank > 8) FAIL(ORC_MF_RANK);
      uint64_t dims[8];
      unsigned __int128 size = 1;
      int huge = 0;
      for (int d = 0; d < rank; d++) {
        TAKE(8);
        dims[d] = le_integer(octets + pos, 8);
        pos += 8;
        size *= dims[d];
        if (size > ((unsigned __int128)1 << 100)) huge = 1, size = (unsigned __int128)1 << 100;
      }
      if (huge || size * 4 > (unsigned __int128)(end - pos)) FAIL(ORC_MF_TRUNCATED);
      for (int d = 0; d < rank; d++)
        if (dims[d] >= ((uint64_t)1 << 61)) FAIL(ORC_MF_DIMENSION); /* array-dimension-limit */
      uint64_t n = (uint64_t)size;
      uint32_t *vals = (uint32_t *)malloc(4 * n + 4);
      for (uint64_t i = 0; i < n; i++) {
        uint32_t v = (uint32_t)le_integer(octets + pos + 4 * i, 4);
        if (v >= ORC_P) {
          free(vals);
          FAIL(ORC_MF_RANGE);
        }
        vals[i] = v;
      }
      pos += 4 * n;
      orc_msg *m = push_msg(tr);
      m->kind = 1;
      m->rank = rank;
      memcpy(m->dims, dims, sizeof(dims[0]) * rank);
      m->count = n;
      m->vals = vals;
    } else {
      FAIL(ORC_MF_TAG);
    }
  }
  if (pos != end) FAIL(ORC_MF_TRAILING);
  return ORC_OK;
#undef TAKE
#undef FAIL
}

orc_tr *orc_tr_new_verifier(const uint8_t *label, uint64_t label_len, int D, const uint8_t *proof,
                            uint64_t proof_len, int *status) {
  orc_tr *tr = tr_alloc(label, label_len, D);
  if (!tr) {
    *status = ORC_E_PARAM;
    return NULL;
  }
  *status = decode_proof(tr, proof, proof_len);
  if (*status) {
    orc_tr_free(tr);
    return NULL;
  }
  tr->verifier = 1;
  return tr;
}

int orc_proof_reencode(const uint8_t *proof, uint64_t len, uint8_t *out, uint64_t cap, uint64_t *out_len) {
  int st;
  orc_tr *tr = orc_tr_new_verifier((const uint8_t *)"", 0, 4, proof, len, &st);
  if (!tr) return st;
  *out_len = orc_tr_encode_proof(tr, out, cap);
  orc_tr_free(tr);
  return ORC_OK;
}
