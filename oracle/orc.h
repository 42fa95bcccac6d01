/* orc.h -- CPU oracle for the Exacta/Sable data-parallel proving path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library restates, in plain C, the algorithm of the reference's
 * Common Lisp CPU prover and verifier for the sumcheck / LogUp-GKR / Reed-Solomon / BLAKE3-Merkle /
 * BaseFold path.  It is the checker the GPU library is compared against; only tests, the smoke
 * check and the benchmark's cpu_baseline leg may load it.  Nothing in the shipped library links,
 * loads or calls it.
 *
 * Every value crossing this interface is a canonical residue in [0, p), p = 2^31 - 2^24 + 1, as a
 * little-endian u32; an extension element is D (4 or 8) such words in the reference's tower order
 * (src/field.lisp:8-11).
 *
 * Pinning (what fixes each function without running the reference):
 *   field, tower, lagrange, eq-table, mle     golden vectors :pow :ext :lagrange :eq :mle
 *   BLAKE3 (tree mode), B3S                   golden vectors :blake3 :b3s
 *   transcript, grind, proof bytes            golden vectors :transcript :grind :proofio :proofio-bad
 *   RS roots/twiddles/encode/fold             golden vectors :rs-encode :rs-fold, encode == brute-eval
 *   sumcheck prove/verify (ext tables)        4 whole-proof :sumcheck vectors, byte for byte
 *   sumcheck with base tables / constants     invariants: base == lifted proof bytes, brute-force
 *                                             round sums on tiny n, linearity in the statement,
 *                                             verifier acceptance (no golden bytes exist)
 *   GKR fraction trees, prove-upper,          the reference's frozen GKR cases (tests/tests.lisp:464-483, digest at
 *   verify-upper                              :903): the eight proofs of EXPORT-GKR-CASES (one block and several, one to
 *                                             three lookups, F_p^4 and F_p^8) over the reference's own inputs (SBCL's
 *                                             seeded generator, tests/golden/sbcl_random.py) with the verifier's outputs
 *                                             hash to the SHA-256 the reference holds; also root = sum of leaf fractions,
 *                                             claims = MLE of the parents, forgery rejection
 *   leaf digest, Merkle (with injections),    the reference's frozen commitment cases (tests/tests.lisp:728-758, digest at
 *   cap, combine-columns, dot-pairs,          :905): the reference's scheduler restated over these primitives
 *   fold-table, BaseFold over classes         (tests/golden/pcs_cases.py: units, merge sets, mixed trees, point
 *                                             reductions, segment, finish, query openings) makes the three proofs of
 *                                             EXPORT-PCS-CASES byte for byte; also the :blake3 vectors for every hash
 *                                             shape used, path checks against the cap, fold(encode(m)) =
 *                                             encode(fold(m)), final table = message folded at the challenges
 *   dot-pairs, fold-table, scale-add          their definitions in an independent pure-Python field on small tables;
 *                                             the round identity g(0) + g(1) of the folded tables = g(x)
 *   open-queries (leaves, paths)              numpy indexing of the codewords by the definition; every opened leaf,
 *                                             hashed and walked up its path, lands on the committed cap
 *   opening over several classes, verify-      its BaseFold and trees by the frozen cases above; its own query openings
 *   queries, mixed-height Merkle trees        and the verifier by: prover -> verifier acceptance, rejection of every
 *   queries, mixed-height Merkle trees        flipped opened symbol / path / cap / final-table word, the single-class case
 *                                             being orc_basefold_prove byte for byte, injected levels against a
 *                                             definition-level Python tree
 *   combine-columns                           the definition evaluated with big integers coordinate by
 *                                             coordinate (ext-scale is coordinate-wise, :ext vectors), unit
 *                                             coefficients, linearity; its output opening under BaseFold to
 *                                             the same combination of the columns' evaluations
 */
#ifndef ORC_H
#define ORC_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_P 2130706433u /* 2^31 - 2^24 + 1 */
#define ORC_MAXD 8

/* status codes */
#define ORC_OK 0
#define ORC_E_PARAM (-1)     /* invalid-parameter */
#define ORC_E_DIVZERO (-2)   /* field-division-by-zero */
#define ORC_E_SHAPE (-3)     /* message-shape-error */
#define ORC_E_EXHAUSTED (-4) /* transcript-exhausted */
#define ORC_E_REJECT (-5)    /* verification-failure */
#define ORC_E_MALFORMED (-6) /* malformed-proof; reason in orc_malformed_reason() */

/* malformed-proof reasons (src/conditions.lisp:38-45) */
enum { ORC_MF_NONE = 0, ORC_MF_MAGIC, ORC_MF_TRUNCATED, ORC_MF_TRAILING, ORC_MF_TAG, ORC_MF_RANGE,
       ORC_MF_RANK, ORC_MF_DIMENSION };

/* ---- F_p (src/field.lisp:31-101) */
uint32_t orc_fadd(uint32_t a, uint32_t b);
uint32_t orc_fsub(uint32_t a, uint32_t b);
uint32_t orc_fmul(uint32_t a, uint32_t b);
uint32_t orc_fpow(uint32_t a, uint64_t e);
int orc_finv(uint32_t a, uint32_t *out); /* ORC_E_DIVZERO on 0 (out = 0, the return-zero restart) */

/* ---- tower (src/field.lisp:103-310) */
void orc_ext_add(int D, const uint32_t *a, const uint32_t *b, uint32_t *out);
void orc_ext_sub(int D, const uint32_t *a, const uint32_t *b, uint32_t *out);
void orc_ext_neg(int D, const uint32_t *a, uint32_t *out);
void orc_ext_scale(int D, const uint32_t *a, uint32_t s, uint32_t *out);
void orc_ext_mul(int D, const uint32_t *a, const uint32_t *b, uint32_t *out);
/* MUL* as the loops of src/field.lisp:213-234 for any power-of-two D <= 8 (orc_ext_mul runs the unrolled
   orc_ext_mul4 / orc_ext_mul8 at D = 4, 8: the same residues) */
void orc_ext_mul_plain(int D, const uint32_t *a, const uint32_t *b, uint32_t *out);
void orc_ext_mul4(const uint32_t *a, const uint32_t *b, uint32_t *out);
void orc_ext_mul8(const uint32_t *a, const uint32_t *b, uint32_t *out);
int orc_ext_inv(int D, const uint32_t *a, uint32_t *out);
void orc_ext_eq1(int D, const uint32_t *a, const uint32_t *b, uint32_t *out);
void orc_ext_eq(int D, int k, const uint32_t *as, const uint32_t *bs, uint32_t *out);

/* ---- multilinear helpers (src/field.lisp:312-377) */
void orc_lagrange(int D, int count, const uint32_t *values, const uint32_t *x, uint32_t *out);
void orc_eq_table(int D, int k, const uint32_t *r, uint32_t *out /* D * 2^k */);
void orc_fold_table(int D, uint64_t len, const uint32_t *table, const uint32_t *r, uint32_t *out);
void orc_mle_eval(int D, int k, const uint32_t *values, int stride, const uint32_t *r, uint32_t *out);

/* ---- BLAKE3 (src/blake3.lisp) */
void orc_blake3_compress(const uint32_t cv[8], const uint32_t m[16], uint64_t counter,
                         uint32_t block_len, uint32_t flags, uint32_t out[16]);
void orc_blake3_hash(const uint8_t *in, uint64_t len, uint8_t *out, uint64_t outlen);

typedef struct {
  uint32_t cv[8];
  uint8_t block[64];
  uint32_t used;
  uint64_t counter;
} orc_b3s;
void orc_b3s_init(orc_b3s *s);
void orc_b3s_update(orc_b3s *s, const uint8_t *data, uint64_t len);
void orc_b3s_digest(const orc_b3s *s, uint8_t *out, uint64_t n);

/* ---- transcript and proof bytes (src/transcript.lisp, src/proofio.lisp) */
typedef struct orc_msg {
  int kind; /* 0: byte message, 1: field array */
  int rank;
  uint64_t dims[8];
  uint64_t count; /* bytes, or number of values */
  uint8_t *bytes;
  uint32_t *vals;
} orc_msg;

typedef struct orc_tr orc_tr;
orc_tr *orc_tr_new(const uint8_t *label, uint64_t label_len, int D);
/* a verifier transcript replaying the messages of PROOF; status in *status */
orc_tr *orc_tr_new_verifier(const uint8_t *label, uint64_t label_len, int D, const uint8_t *proof,
                            uint64_t proof_len, int *status);
void orc_tr_free(orc_tr *tr);
int orc_tr_degree(const orc_tr *tr);
void orc_tr_absorb(orc_tr *tr, const uint8_t *data, uint64_t len);
/* prover: record (and absorb) a field array; verifier: take the next one, which must have the
   given shape (rank < 0: any), and copy its values to OUT (may be NULL) */
int orc_tr_send(orc_tr *tr, const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out);
int orc_tr_record(orc_tr *tr, const uint32_t *vals, int rank, const uint64_t *dims, uint32_t *out);
/* byte messages; verifier: LEN < 0 accepts any length; *out_len receives the length */
int orc_tr_send_bytes(orc_tr *tr, const uint8_t *bytes, int64_t len, uint8_t *out, uint64_t cap,
                      uint64_t *out_len);
int orc_tr_record_bytes(orc_tr *tr, const uint8_t *bytes, int64_t len, uint8_t *out, uint64_t cap,
                        uint64_t *out_len);
void orc_tr_squeeze(orc_tr *tr, uint8_t *out, uint64_t n);
void orc_tr_challenge_base(orc_tr *tr, int k, uint32_t *out);
void orc_tr_challenge(orc_tr *tr, int degree, uint32_t *out);
void orc_tr_challenges(orc_tr *tr, int k, int degree, uint32_t *out);
void orc_tr_challenge_bits(orc_tr *tr, int nbits, int k, uint64_t *out);
int orc_check_grind(const uint8_t base[32], uint64_t nonce, int bits);
uint64_t orc_tr_grind(orc_tr *tr, int bits);
int orc_tr_verify_grind(orc_tr *tr, int bits, uint64_t *nonce);
void orc_tr_state_digest(const orc_tr *tr, uint8_t out[32]);
int orc_tr_finished(const orc_tr *tr);
uint64_t orc_tr_message_count(const orc_tr *tr);
const orc_msg *orc_tr_message(const orc_tr *tr, uint64_t i);
/* proof bytes of the messages sent so far: returns the size; writes at most CAP bytes */
uint64_t orc_tr_encode_proof(const orc_tr *tr, uint8_t *out, uint64_t cap);
int orc_malformed_reason(void);
/* decode then re-encode (with the EXACTPF1 magic): round-trip check of the byte format */
int orc_proof_reencode(const uint8_t *proof, uint64_t len, uint8_t *out, uint64_t cap, uint64_t *out_len);

/* ---- Reed-Solomon (src/rs.lisp) */
int orc_root_of_unity(int k, uint32_t *out);
/* levels 0..max(1,n-1)-1 concatenated: level l has 2^(n-1-l) values */
uint64_t orc_twiddles_size(int n);
void orc_twiddles(int n, uint32_t *out);
void orc_domain_points(int n, uint32_t *out);
int orc_rs_encode(const uint32_t *message, int n, uint32_t *codeword /* 2^n */);
void orc_rs_brute_eval(const uint32_t *message, int n, uint32_t *out);
/* fold a codeword of 2m elements of degree D (D = 1: base) on a twiddle level of m values */
void orc_rs_fold(int D, uint64_t m, const uint32_t *codeword, const uint32_t *twiddle_level,
                 const uint32_t *r, uint32_t *out);
/* DOT-PAIRS, src/pcs.lisp:473-483: sum over pairs of pick(e) pick(v) for two tables of len EXT8s; parity 0: even
   entries, 1: odd entries, 2: 2 odd - even */
void orc_dot_pairs(const uint32_t *e, const uint32_t *v, uint64_t len, int parity, uint32_t *out);
/* h[x] += scale * column[x], the per-class table of the opening (src/pcs.lisp:709-716) */
void orc_scale_add(int D, uint64_t len, const uint32_t *scale, const uint32_t *column, uint32_t *h);
/* COMBINE-COLUMNS, src/pcs.lisp:434-441 */
void orc_combine_columns(int D, int ncols, uint64_t len, const uint32_t *columns, const uint32_t *coefficients,
                         uint32_t *out);

/* ---- statements: a sum of monomials, the canonical form of src/forms.lisp:57-78.
   Variable v < T is table v; v >= T is constant v - T.  */
typedef struct {
  int T, C, nterms;
  const uint32_t *coeff;  /* nterms */
  const int32_t *start;   /* nterms + 1 offsets into vars */
  const int32_t *vars;
  /* optionally the form as written, as a postfix program (ARITHMETIC-FORM, src/forms.lisp:113-141): op 0 table,
     1 constant, 2 integer (arg = its residue), 3 +, 4 -, 5 *, 6 unary -; chains reduced left to right.  Only the
     fast path (orc_set_fast) runs it; nops = 0: it evaluates the monomials instead. */
  int nops;
  const int32_t *ops, *args;
} orc_stmt;
int orc_stmt_degree(const orc_stmt *st); /* degree in the tables */
void orc_stmt_eval(const orc_stmt *st, int D, const uint32_t *table_vals /* T*D */,
                   const uint32_t *consts /* C*D */, uint32_t *out);

/* ---- sumcheck (src/sumcheck.lisp) */
void orc_hypercube_sum(const orc_stmt *st, int n, int D, const uint32_t *const *tables,
                       const int32_t *strides, const uint32_t *eq, const uint32_t *consts,
                       uint32_t *out);
/* tables[t]: K * 2^n entries of stride strides[t] (1 or D), block-major; bw: K*D or NULL (K = 1);
   degree < 0: the statement's.  out_folded[t] (if non-NULL) receives K*D words. */
int orc_sumcheck_prove(orc_tr *tr, int n, const orc_stmt *st, const uint32_t *const *tables,
                       const int32_t *strides, const uint32_t *eq, const uint32_t *consts,
                       const uint8_t *label, uint64_t label_len, const uint32_t *bw, int K,
                       int degree, uint32_t *out_chal, uint32_t *out_finals,
                       uint32_t *const *out_folded);
int orc_sumcheck_verify(orc_tr *tr, int n, const orc_stmt *st, const uint32_t *claim,
                        const uint32_t *eq, const uint32_t *consts, int blocks,
                        const uint8_t *label, uint64_t label_len, int degree, uint32_t *out_chal,
                        uint32_t *out_reduced);
int orc_check_final(const orc_stmt *st, int D, const uint32_t *reduced, const uint32_t *finals,
                    const uint32_t *consts);
/* one prover round on the current tables (len entries each): sums at X = 0,2,..,points */
void orc_round_sums(const orc_stmt *st, int D, int points, uint64_t pairs_low, uint64_t n_high,
                    const uint32_t *const *tables, const int32_t *strides, const uint32_t *low,
                    const uint32_t *high, const uint32_t *consts, uint32_t *out /* points*D */);
void orc_fold_flat(int D, uint64_t len, const uint32_t *entries, int stride, const uint32_t *r,
                   uint32_t *out /* D * len/2 */);
/* The same two functions organised for speed (orc_fast.c): the written form as straight-line code, base-field
   lines when the reference would use them, unrolled products, OpenMP threads.  Same words out.
   orc_set_fast(t > 0) makes orc_sumcheck_prove use them with t threads (0: the plain path, the default). */
int orc_round_sums_fast(const orc_stmt *st, int D, int points, uint64_t n_low, uint64_t n_high,
                        const uint32_t *const *tables, const int32_t *strides, const uint32_t *low,
                        const uint32_t *high, const uint32_t *consts, int threads, uint32_t *out);
int orc_fold_flat_fast(int D, uint64_t len, const uint32_t *entries, int stride, const uint32_t *r, int threads,
                       uint32_t *out);
void orc_set_fast(int threads);
int orc_fast_threads(void);
int orc_host_threads(void); /* what OpenMP would use by default */
/* SplitMix64(seed) -> 31-bit words, kept when below p: the seeded synthetic inputs of the benchmarks */
void orc_splitmix_field(uint64_t seed, uint64_t count, uint32_t *out);

/* ---- LogUp-GKR (src/gkr.lisp) */
/* leaves: per lookup l, p = leaves[2l], q = leaves[2l+1], each K*2^n EXTs block-major */
int orc_gkr_prove_upper(orc_tr *tr, int n, int K, int lookups, const uint32_t *const *leaves,
                        const uint8_t *label, uint64_t label_len, uint32_t *out_ri /* (n-1)*D */,
                        uint32_t *out_rb /* lk*D */, uint32_t *out_cp, uint32_t *out_cq);
int orc_gkr_verify_upper(orc_tr *tr, int n, int K, int lookups, const uint8_t *label,
                         uint64_t label_len, uint32_t *out_roots /* lookups*2*D */,
                         uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp, uint32_t *out_cq);
/* one in-block reduction: layer m (K*2^m entries) from layer m+1 */
void orc_gkr_reduce_layer(int D, int K, int m, const uint32_t *p, const uint32_t *q, uint32_t *pp,
                          uint32_t *qq);

/* ---- commitment: leaves, Merkle, BaseFold (src/pcs.lisp:37-101, 271-304, 569-657) */
/* digest of a leaf of ROWS rows of 4 values; previous: 32 bytes or NULL */
void orc_leaf_digest(const uint32_t *rows, uint64_t nrows, const uint8_t *previous, uint8_t out[32]);
void orc_node(const uint8_t left[32], const uint8_t right[32], uint8_t out[32]);
int orc_cap_level(uint64_t leaves);
/* all levels, leaves first, concatenated (2*leaves - 1 digests) */
void orc_merkle_levels(const uint8_t *leaves, uint64_t nleaves, uint8_t *out);
int orc_check_path(const uint8_t h[32], const uint8_t *path, int depth, uint64_t i,
                   const uint8_t *cap);
/* OPEN-QUERIES' leaves and paths of one (unit, class), src/pcs.lisp:721-734; returns the paths' depth */
int orc_open_queries(const uint32_t *codewords, int ncols, int c, const uint8_t *levels, const uint64_t *leaves,
                     int count, uint32_t *out_leaves, uint8_t *out_paths);
/* commit NCOLS columns of 2^c base values: codewords (ncols * 2^(c+1)), leaf digests (2^(c-1) * 32
   bytes), all tree levels, and the cap; returns the cap's row count */
uint64_t orc_commit_columns(const uint32_t *const *columns, int ncols, int c, uint32_t *codewords,
                            uint8_t *levels, uint8_t *cap);
/* BaseFold of one class of 2^nv EXT8s H at the point rr (nv EXT8s), value v = H(rr) */
int orc_basefold_prove(orc_tr *tr, int nv, const uint32_t *rr, const uint32_t *v,
                       const uint32_t *h, int grind_bits, int queries, uint64_t *out_qs,
                       uint32_t *out_chal /* fl*8 */, uint32_t *out_final /* 2^(nv-fl)*8 */);
int orc_basefold_verify(orc_tr *tr, int nv, const uint32_t *rr, const uint32_t *v, int grind_bits,
                        int queries, uint64_t *out_qs);

/* ---- the final opening over several size classes (orc_open.c; src/pcs.lisp:64-95, 581-657, 721-843) */
/* MERKLE-LEVELS with injections: inj[k] (nleaves >> inj_level[k] digests) is hashed into level inj_level[k] */
void orc_merkle_levels_injected(const uint8_t *leaves, uint64_t nleaves, int ninj, const int32_t *inj_level,
                                const uint8_t *const *inj, uint8_t *out);
/* CHECK-PATH with INJECTED-AT: inj_digests[k] (32 bytes) is hashed in after level inj_level[k] */
int orc_check_path_injected(const uint8_t h[32], const uint8_t *path, int depth, uint64_t i, const uint8_t *cap,
                            int ninj, const int32_t *inj_level, const uint8_t *inj_digests);
/* one key of the opening: a size class with its committed columns (a unit of its own with its own tree) */
typedef struct {
  int32_t c, ncols;
  const uint32_t *codewords; /* prover: ncols * 2^(c+1) symbols */
  const uint8_t *levels;     /* prover: the tree's levels, leaves first */
  const uint8_t *cap;        /* verifier: the committed cap */
  const uint32_t *coef;      /* ncols EXT8s: the columns' coefficients in the class's combined column */
  const uint32_t *h;         /* prover: the combined column, 2^c EXT8s */
} orc_open_key;
/* BASEFOLD (classes ascending, the last one nv; class c joins at level nv - c) and OPEN-QUERIES: the claim is
   sum_c H_c(the last c coordinates of rr) = v */
int orc_pcs_open(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr, const uint32_t *v,
                 int grind_bits, int queries, uint64_t *out_qs);
int orc_basefold_classes(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr, const uint32_t *v,
                 int grind_bits, int queries, uint64_t *out_qs);
/* BASEFOLD's verifier side and VERIFY-QUERIES; ORC_E_REJECT when a check fails */
int orc_pcs_verify_opening(orc_tr *tr, int nv, int nkeys, const orc_open_key *keys, const uint32_t *rr,
                           const uint32_t *v, int grind_bits, int queries);

#ifdef __cplusplus
}
#endif
#endif
