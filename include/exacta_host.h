/* exacta_host.h -- C ABI of the host-side mirror of the reference's protocol functions, built into
 * the same libexacta_hip.so.  An SBCL host does not need these (it keeps its own transcript and
 * PROVE); they are the stand-in caller that drives the device sessions where no Lisp exists, with
 * the reference's names, argument meaning and error behaviour, so tests read like the reference's.
 * Conventions as in exacta_hip.h.
 */
#ifndef EXACTA_HOST_H
#define EXACTA_HOST_H
#include <stdint.h>

#include "exacta_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t exh_transcript;

/* ---- field helpers on the host (src/field.lisp), for callers without their own arithmetic */
int exh_ext_mul(int degree_d, const uint32_t *a, const uint32_t *b, uint32_t *out);
int exh_ext_inv(int degree_d, const uint32_t *a, uint32_t *out); /* EXH_E_DIVZERO on zero (out = 0) */
int exh_eq_table(int degree_d, int k, const uint32_t *r, uint32_t *out);

/* ---- BLAKE3 and the transcript (src/blake3.lisp, src/transcript.lisp) */
int exh_blake3(const uint8_t *in, uint64_t len, uint8_t *out, uint64_t out_len);
/* MAKE-TRANSCRIPT, src/transcript.lisp:75-84; proof != NULL: a verifier replaying the proof's
   messages (DECODE-PROOF, src/proofio.lisp:53-101; EXH_E_MALFORMED with the reason in last_error) */
int exh_transcript_new(const uint8_t *label, uint64_t label_len, int degree_d, const uint8_t *proof,
                       uint64_t proof_len, exh_transcript *out);
int exh_transcript_free(exh_transcript tr);
int exh_transcript_absorb(exh_transcript tr, const uint8_t *data, uint64_t len);               /* :95-100 */
int exh_transcript_send(exh_transcript tr, const uint32_t *vals, int rank, const uint64_t *dims,
                        uint32_t *out, int absorb);                                              /* :133-148 */
int exh_transcript_send_bytes(exh_transcript tr, const uint8_t *bytes, int64_t len, uint8_t *out,
                              uint64_t cap, uint64_t *out_len, int absorb);
int exh_transcript_challenge_base(exh_transcript tr, int k, uint32_t *out);                      /* :166-172 */
int exh_transcript_challenge_bits(exh_transcript tr, int nbits, int k, uint64_t *out);          /* :183-187 */
int exh_transcript_grind(exh_transcript tr, int bits, uint64_t *nonce);                          /* :196-201 */
int exh_transcript_verify_grind(exh_transcript tr, int bits, uint64_t *nonce);                   /* :203-209 */
int exh_transcript_digest(exh_transcript tr, uint8_t out[32]);
/* the sequential-mode hash state behind the transcript (src/blake3.lisp:125-134): chaining value,
   pending block (zero beyond *used), bytes pending, blocks compressed -- what exh_sumcheck_run takes */
int exh_transcript_state(exh_transcript tr, uint32_t cv[8], uint8_t block[64], uint32_t *used, uint64_t *counter);
int exh_transcript_finished(exh_transcript tr);
int exh_transcript_message_count(exh_transcript tr, uint64_t *count);
/* ENCODE-PROOF of the messages so far (src/proofio.lisp:45-49): size in *out_len; bytes written when
   cap suffices */
int exh_transcript_proof(exh_transcript tr, uint8_t *out, uint64_t cap, uint64_t *out_len);

/* ---- sumcheck (src/sumcheck.lisp) */
/* HYPERCUBE-SUM, :112-127: the honest claim, computed on the device (a statement wider than one kernel holds: the
   sum of its parts' claims) */
int exh_hypercube_sum(exh_stmt stmt, int degree_d, int n, const exh_table *tables, int n_tables,
                      const uint32_t *eq, const uint32_t *constants, uint32_t *out);
/* PROVE, :512-571.  out_challenges: n * D; out_finals: n_tables * D; out_folded: NULL or n_tables
   pointers to K * D words */
int exh_prove(exh_transcript tr, int n, exh_stmt stmt, const exh_table *tables, int n_tables,
              const uint32_t *eq, const uint32_t *constants, const uint8_t *label, uint64_t label_len,
              const uint32_t *block_weights, int K, int degree, uint32_t *out_challenges, uint32_t *out_finals,
              uint32_t *const *out_folded);
/* VERIFY, :147-163 */
int exh_verify(exh_transcript tr, int n, exh_stmt stmt, const uint32_t *claim, const uint32_t *eq,
               const uint32_t *constants, int blocks, const uint8_t *label, uint64_t label_len, int degree,
               uint32_t *out_challenges, uint32_t *out_reduced);
/* CHECK-FINAL, :165-172 */
int exh_check_final(exh_stmt stmt, int degree_d, const uint32_t *reduced, const uint32_t *finals,
                    const uint32_t *constants);

/* EVALUATE of the statement's form (src/forms.lisp:214-217) at table values (n_tables * D) and constants, as
   VERIFY-DOMAIN applies it to the finals of each block (src/domain.lisp:247-248) */
int exh_stmt_evaluate(exh_stmt stmt, int degree_d, const uint32_t *table_values, const uint32_t *constants,
                      uint32_t *out);

/* ---- LogUp-GKR (src/gkr.lisp) */
/* PROVE-UPPER, :215-272.  leaves: 2 * lookups tables (p, q per lookup) of K * 2^n EXTs */
int exh_gkr_prove_upper(exh_transcript tr, int n, int K, int lookups, const exh_table *leaves,
                        const uint8_t *label, uint64_t label_len, uint32_t *out_ri, uint32_t *out_rb,
                        uint32_t *out_cp, uint32_t *out_cq);
/* Two PROVE-UPPER calls of the same meaning (:215-272), each with a transcript of its own (a lookup's witness
   tree and its table tree, two lookup arguments...), run side by side: the second on a second host thread and a
   second stream, with a workspace of its own.  Their sumchecks are chains of dependent rounds that leave most of
   the device idle, so the pair takes about as long as the longer of the two.  Each tree's results and transcript
   are what the single call gives (the two never touch each other's state); `status` receives each tree's own
   result and the call returns the first that is not EXH_OK.  While launches are being timed (exh_profile_enable)
   the two run one after the other. */
typedef struct exh_gkr_tree {
  exh_transcript tr;
  int n, K, lookups;
  const exh_table *leaves;
  const uint8_t *label;
  uint64_t label_len;
  uint32_t *out_ri, *out_rb, *out_cp, *out_cq;
  int status;
} exh_gkr_tree;
int exh_gkr_prove_upper_pair(exh_gkr_tree *first, exh_gkr_tree *second);
/* VERIFY-UPPER, :91-145 */
int exh_gkr_verify_upper(exh_transcript tr, int n, int K, int lookups, const uint8_t *label, uint64_t label_len,
                         uint32_t *out_roots, uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp,
                         uint32_t *out_cq);

/* ---- commitment (src/pcs.lisp:279-304, 581-657) */
/* PCS-COMMIT of one class: encode + leaves + Merkle + send-bytes of the cap on the transcript */
int exh_pcs_commit(exh_transcript tr, exh_table columns, int ncols, int c, exh_table *codewords,
                   exh_table *levels);
/* BASEFOLD of one class of 2^nv EXT8s h (device) at the point rr (nv EXT8s), value v */
int exh_basefold_prove(exh_transcript tr, int nv, const uint32_t *rr, const uint32_t *v, exh_table h,
                       int grind_bits, int queries, uint64_t *out_qs, uint32_t *out_challenges,
                       uint32_t *out_final);
/* The same with ENCODE-EXT of h (src/pcs.lisp:569-575, 2^(nv+1) EXT8s on the device) supplied by the caller:
   encoding is linear, so when h is COMBINE-COLUMNS of committed columns its codeword is exh_combine_columns of
   their committed codewords with the same coefficients, and BASEFOLD's eight transforms (src/pcs.lisp:598-600)
   are not repeated.  The proof is the same bytes. */
int exh_basefold_prove_encoded(exh_transcript tr, int nv, const uint32_t *rr, const uint32_t *v, exh_table h,
                               exh_table codeword, int grind_bits, int queries, uint64_t *out_qs,
                               uint32_t *out_challenges, uint32_t *out_final);
/* BASEFOLD over several size classes (src/pcs.lisp:581-657 with its CLASSES and H arguments as PCS-FINISH passes
   them, :714-716): classes[k] ascending, the last one nv; hs[k] the class's combined column H_c, 2^classes[k]
   EXT8s on the device, joining at level nv - classes[k] (:590-600, :635-639).  The oracle openings are recorded
   on the transcript as BASEFOLD does; the query openings of the committed trees (OPEN-QUERIES, :721-734) stay with
   the caller, who knows its merge sets. */
int exh_basefold_prove_classes(exh_transcript tr, int nv, int n_classes, const int *classes, const exh_table *hs,
                               const uint32_t *rr, const uint32_t *v, int grind_bits, int queries, uint64_t *out_qs);
int exh_basefold_verify(exh_transcript tr, int nv, const uint32_t *rr, const uint32_t *v, int grind_bits,
                        int queries, uint64_t *out_qs);

/* ---- the final opening over several size classes (src/pcs.lisp:434-441, 581-657, 721-843): one key per class,
   each a unit of its own with its own tree; the classes ascend and the last one is nv.  Merge sets, segments and
   the cross-unit sumcheck around it stay with the caller. */
typedef struct {
  int32_t c, ncols;
  exh_table columns;   /* prover: the class's ncols base columns of 2^c values (as exh_pcs_commit took them) */
  exh_table codewords; /* prover: their codewords (exh_pcs_commit / exh_rs_encode) */
  exh_table levels;    /* prover: the tree's levels (exh_pcs_commit / exh_merkle_commit) */
  const uint32_t *coefficients; /* ncols EXT8s: the columns' coefficients in the class's combined column (UC-COEF) */
  const uint8_t *cap;  /* verifier: the committed cap, 32 * CAP-ROWS(2^(c-1)) bytes */
} exh_open_key;
/* COMBINE-COLUMNS per key, BASEFOLD with class c joining at level nv - c (:590-600, :635-639), OPEN-QUERIES per key
   (:721-734).  The claim: sum_c H_c(the last c coordinates of rr) = v.  out_qs: the query positions */
int exh_pcs_open(exh_transcript tr, int nv, int n_keys, const exh_open_key *keys, const uint32_t *rr, const uint32_t *v,
                 int grind_bits, int queries, uint64_t *out_qs);
/* BASEFOLD's verifier side and VERIFY-QUERIES (:752-843): every opened leaf against its tree's cap, the folding of
   the combined codeword through the oracles down to the final table's codeword.  EXH_E_REJECT when a check fails */
int exh_pcs_verify_opening(exh_transcript tr, int nv, int n_keys, const exh_open_key *keys, const uint32_t *rr,
                           const uint32_t *v, int grind_bits, int queries);
/* MERKLE-LEVELS with injections (:64-77): the levels (a new table, leaves first) of the tree over `leaves` (8-word
   digests), the digests of injected[k] hashed into the nodes of level inject_level[k] (mixed-height trees) */
int exh_merkle_levels_injected(exh_table leaves, int n_injected, const int32_t *inject_level, const exh_table *injected,
                               exh_table *levels);
/* CHECK-PATH with INJECTED-AT (:86-95): 1 when leaf digest h hashes up `path` (depth siblings) from leaf i to
   cap[i >> depth], the digest injected_digests[k] hashed in after level inject_level[k] */
int exh_check_path(const uint8_t h[32], const uint8_t *path, int depth, uint64_t i, const uint8_t *cap, int n_injected,
                   const int32_t *inject_level, const uint8_t *injected_digests);

#ifdef __cplusplus
}
#endif
#endif
