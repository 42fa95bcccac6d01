/* exacta_hip.h -- C ABI of libexacta_hip.so: the MI355X (gfx950) backend for the data-parallel
 * proving path of Exacta/Sable.
 *
 * The reference has no FFI: the boundary is drawn inside its Lisp functions.  Each entry point below
 * names the reference code whose body it replaces (file:line under the reference tree); an SBCL host
 * binds them with sb-alien (define-alien-routine, pinned (unsigned-byte 32) vectors) and keeps its own
 * PROVE / VERIFY / CHECK-FINAL API, statements, transcript and proof format.
 *
 * Conventions
 *   - every field value crossing the boundary is a canonical residue in [0, p), p = 2^31 - 2^24 + 1,
 *     as a little-endian u32; an extension element is D (4 or 8) words in the reference's tower order
 *     (src/field.lisp:8-11); tables are flat, stride 1 (base) or D (src/sumcheck.lisp:53-59);
 *   - host buffers are borrowed for the duration of a call only; device tables live behind handles;
 *   - every function returns EXH_OK or a negative status; exh_last_error() describes the last failure
 *     of the calling thread in the words of the reference's condition classes (src/conditions.lisp);
 *   - one context per process: every entry point takes one process-wide lock, so calls from several threads
 *     are safe and take turns (they never overlap on the device; exh_gkr_prove_upper_pair overlaps its two
 *     proofs itself); handles are shared by all threads; every
 *     call returns after its small result is on the host; nothing calls back into the host language.
 */
#ifndef EXACTA_HIP_H
#define EXACTA_HIP_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EXH_OK 0
#define EXH_E_PARAM (-1)     /* invalid-parameter        (src/conditions.lisp:96-120) */
#define EXH_E_DIVZERO (-2)   /* field-division-by-zero   (src/field.lisp:84-96) */
#define EXH_E_SHAPE (-3)     /* message-shape-error      (src/transcript.lisp:102-114) */
#define EXH_E_EXHAUSTED (-4) /* transcript-exhausted */
#define EXH_E_REJECT (-5)    /* verification-failure     (src/conditions.lisp:12-15) */
#define EXH_E_MALFORMED (-6) /* malformed-proof          (src/conditions.lisp:38-45) */
#define EXH_E_DEVICE (-7)    /* no usable gfx950 device, or a HIP call failed */
#define EXH_E_NOMEM (-8)     /* device memory exhausted */

typedef uint64_t exh_table;   /* a device-resident table */
typedef uint64_t exh_stmt;    /* a compiled statement */
typedef uint64_t exh_session; /* one sumcheck in progress */

/* ---- context */
int exh_init(int device);
void exh_shutdown(void);
const char *exh_last_error(void);
/* wait until everything the library has queued on the device is done */
int exh_synchronize(void);
/* 1 when a kernel generated for the statement is used, 0 when the interpreter kernel is */
int exh_stmt_has_generated_kernel(exh_stmt stmt, int degree_d);
/* ROUND-KERNEL (src/sumcheck.lisp:270-280) compiles a kernel for any statement on first use.  Here the kernels of
   the statements listed at build time are in the library; for any other statement whose tables have at least
   2^20 entries (EXACTA_HIP_RTC_MIN_N changes the 20; EXACTA_HIP_NO_RTC switches this off), the first proof starts
   a compilation of its kernels in the background (hiprtc, seconds to a minute) and runs on the interpreter kernel,
   and proofs begun after the compilation has ended run on the generated kernels: the same bytes either way.  A
   process that ends while a compilation runs ends at once with its exit status (C streams flushed, clean-ups
   registered before the library's first compilation skipped).
   exh_stmt_generate asks for that compilation ahead of a proof, for round polynomials of the given header degree
   (-1: the statement's own).  Returns 1 when the kernels are in place, 0 while they compile (wait = 0), or
   EXH_E_DEVICE with the compiler's log when the compilation failed; with wait != 0 it returns once it has ended.
   A statement too wide for the table groups' kernels (more than 16 table monomials or 36 accumulators) gets the
   kernels of its direct form instead, which evaluate the written form at every wire point (the role of
   COMPILE-FORM, src/forms.lisp:144-186): with them exh_prove proves it in one device-driven session; without them
   (not compiled yet, or EXACTA_HIP_NO_DIRECT=1) in parts proved in step, the same bytes. */
int exh_stmt_generate(exh_stmt stmt, int degree_d, int degree, int wait);
/* 1 when no compilation is running, 0 while one is; with wait != 0 it returns 1 once none is (a host that wants an
   orderly exit calls it before it ends: see above) */
int exh_stmt_generate_idle(int wait);

/* ---- measurement (no counterpart in the reference): with profiling on, every data-parallel kernel
   launch is bracketed by HIP events on the library's stream; entries report the kernel, the round it
   served, its duration and the bytes it had to move (tables read + tables written) */
int exh_profile_enable(int on);
int exh_profile_count(void);
int exh_profile_entry(int index, char *name, int name_cap, int *round, float *ms, uint64_t *alg_bytes);

/* The second roofline's peak, measured (no counterpart in the reference): one launch of `workgroups` workgroups of
   256 threads, every lane running `chains` (8: independent chains, the issue rate; 1: one dependent chain, the
   latency a lone wavefront sees) of the VALU instruction number `op` (0 .. exh_issue_rate_ops() - 1; `name`
   receives its mnemonic) for iterations * 8 links.  Out: the launch's duration, the machine instructions each
   wavefront issued, the device's clock and compute units -- cycles per wavefront instruction and SIMD =
   ms * clock / (instructions_per_wave * wavefronts per SIMD). */
int exh_issue_rate_ops(void);
int exh_issue_rate(int op, int chains, int workgroups, int iterations, char *name, int name_cap, float *ms,
                   double *instructions_per_wave, int *clock_khz, int *compute_units);

/* ---- tables: MAKE-TABLE and the read-back at the end of PROVE (src/sumcheck.lisp:61-70, 564-571) */
int exh_table_upload(const uint32_t *host, uint64_t n_u32, int stride, exh_table *out);
int exh_table_alloc(uint64_t n_u32, int stride, exh_table *out);
/* wrap memory another component already holds on the device (not freed by exh_table_free) */
int exh_table_wrap(void *device_ptr, uint64_t n_u32, int stride, exh_table *out);
int exh_table_download(exh_table table, uint64_t offset_u32, uint32_t *host, uint64_t n_u32);
int exh_table_free(exh_table table);
void *exh_table_device_ptr(exh_table table);
/* seeded synthetic table: SplitMix64(seed), 31-bit words, rejected when >= p (the rule of
   src/transcript.lisp:159-164), generated on the host and uploaded */
int exh_table_random(uint64_t seed, uint64_t n_u32, int stride, exh_table *out);

/* ---- statements: COMPILE-FORM / ROUND-KERNEL (src/forms.lisp:199-212, src/sumcheck.lisp:270-280).
   form: the statement's s-expression text, e.g. "(+ (* alpha t0 t1 t2) (* 3 t1))";
   tables / constants: its variables, in the order the caller passes their values. */
int exh_stmt_compile(const char *form, const char *const *tables, int n_tables, const char *const *constants,
                     int n_constants, exh_stmt *out);
int exh_stmt_degree(exh_stmt stmt); /* STATEMENT-DEGREE, src/sumcheck.lisp:33-35 */
int exh_stmt_free(exh_stmt stmt);

/* ---- one sumcheck, round by round: the call sites inside PROVE (src/sumcheck.lisp:547-563).
   tables: n_tables handles of K * 2^n entries each (block-major); eq: n * D words or NULL;
   block_weights: K * D words or NULL (then K must be 1); constants: n_constants * D words;
   degree < 0: the statement's degree.  One session is open at a time: beginning another (or any
   whole-protocol call) hands the library's scratch arenas on, and the earlier session's calls then fail. */
int exh_sumcheck_begin(exh_stmt stmt, int degree_d, int n, const exh_table *tables, int n_tables,
                       const uint32_t *eq, const uint32_t *block_weights, int K, const uint32_t *constants,
                       int degree, exh_session *out);
/* the round kernel: (apply kernel flat low high constant-values), src/sumcheck.lisp:556;
   out_sums: max(degree,1) * D words, the rows of the round message (X = 0, 2, 3, ...) */
int exh_sumcheck_round(exh_session session, uint32_t *out_sums);
/* FOLD-FLAT-TABLE of every table by the round's challenge, src/sumcheck.lisp:562, 84-104 */
int exh_sumcheck_fold(exh_session session, const uint32_t *r);
/* Every round of a fresh session back to back on the device, the Fiat-Shamir transcript included: the loop
   body of PROVE (src/sumcheck.lisp:546-563) with SEND and CHALLENGE (src/transcript.lisp:116-128, 174-176)
   run by the device on the sequential BLAKE3 state (src/blake3.lisp:125-155) the host's transcript holds after
   absorbing the header (src/sumcheck.lisp:534): cv (8 words), the pending block (64 bytes, zero beyond
   `used`), used, counter.  out_messages: n * max(degree,1) * D words; out_challenges: n * D words.  The host
   sends the messages through its own transcript afterwards and must draw the same challenges.  Statements
   of more than 7 wire points are rejected (use the round-by-round calls). */
int exh_sumcheck_run(exh_session session, const uint32_t *cv, const uint8_t *block, uint32_t used, uint64_t counter,
                     uint32_t *out_messages, uint32_t *out_challenges);
/* finals: n_tables * D words (entry 0 of each folded table); folded: NULL, or n_tables pointers to
   K * D words (src/sumcheck.lisp:564-571).  Ends the session. */
int exh_sumcheck_finish(exh_session session, uint32_t *finals, uint32_t *const *folded);

/* ---- Reed-Solomon, Merkle, BaseFold kernels (src/rs.lisp:60-101, src/pcs.lisp:44-77, 271-304) */
/* ENCODE of ncols columns of 2^c base values each (message table: ncols * 2^c words) into codewords
   of 2^(c+1) words each, bit-reversed order (src/rs.lisp:75-85, src/pcs.lisp:271-273) */
int exh_rs_encode(exh_table messages, int ncols, int c, exh_table *codewords);
/* leaf digests + Merkle levels of a class's codewords (src/pcs.lisp:275-277, 293-302): leaf l holds
   symbols 4l..4l+3 of every column; levels (optional handle out) holds all levels, leaves first, as
   8-word digests; cap: 32 * cap_rows bytes */
int exh_merkle_commit(exh_table codewords, int ncols, int c, exh_table *levels, uint8_t *cap, uint64_t *cap_rows);
/* OPEN-QUERIES' gathers for one (unit, class) (src/pcs.lisp:721-734): out_leaves[count][ncols][4] = LEAF-ROWS
   (src/pcs.lisp:275-277) of leaf leaves[q] < 2^(c-1), the array FIELD-ARRAY-OF-LEAVES (:659-665) records; with
   levels (else 0), out_paths[count][depth][32 bytes] = PATH (src/pcs.lisp:79-84) of the same leaves up to the
   cap level depth = CAP-LEVEL(2^(c-1)) (src/pcs.lisp:57-59), written to out_depth.  The caller derives leaves[q]
   from the query index as (ash q (- c nv)) and records both in the transcript. */
int exh_open_queries(exh_table codewords, int ncols, int c, exh_table levels, const uint64_t *leaves, int count,
                     uint32_t *out_leaves, uint8_t *out_paths, int *out_depth);
/* RS:FOLD of an extension codeword of 2m elements of degree D on twiddle level `level` of the
   2^n_domain tables (src/rs.lisp:93-101) */
int exh_rs_fold(exh_table codeword, int degree_d, uint64_t m, int n_domain, int level, const uint32_t *r,
                exh_table *out);
/* COMBINE-COLUMNS (src/pcs.lisp:434-441): g[x] = sum_k coefficient_k * column_k[x], the extension table BaseFold
   opens, from a class's ncols base columns of len values each (column k at k * len of `columns`, as PCS-COMMIT
   takes them) and ncols coefficients of degree D (canonical, tower order); out: a new table of len elements */
int exh_combine_columns(exh_table columns, int ncols, uint64_t len, int degree_d, const uint32_t *coefficients,
                        exh_table *out);
/* One class's share of a CROSS-ROUNDS round (src/pcs.lisp:485-512): DOT-PAIRS (:473-483) of its tables E and V
   (EXT8s, the same even count) for the parities 0, 1, 2 at once -> out[3][8], and FOLD-TABLE (src/field.lisp:365-370)
   of either by the round's challenge r (degree = the table's) -> a new table of half the length */
int exh_dot_pairs(exh_table e, exh_table v, uint32_t *out);
int exh_fold_table(exh_table table, const uint32_t *r, exh_table *out);
/* exh_dot_pairs for callers that must not allocate device memory while they run (tight serving loops, harnesses
   that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and result as exh_dot_pairs;
   the workgroups' partial sums live in a static 48 KiB device array that each GPU holds until the process ends,
   and the call makes no hipMalloc, hipFree or other allocating call.  Like every entry point it is synchronous
   (it launches on the library's own stream and waits for its 24 words), so it cannot be recorded into a HIP graph.
   Tables of more than 2^26 EXT8s are refused (invalid-parameter).  Calls on one GPU share that GPU's array:
   calls that overlap on one GPU race. */
int exh_dot_pairs_static(exh_table e, exh_table v, uint32_t *out);
/* The opening's table per class (src/pcs.lisp:709-716), one unit at a time: out[x] = h[x] + scale * column[x]
   over extension tables of one shape; h = 0 stands for the table of zeros the sum starts from */
int exh_table_scale_add(exh_table h, const uint32_t *scale, exh_table column, exh_table *out);
/* EQ-TABLE (src/field.lisp:354-363) of the point r (k coordinates of degree D, canonical), as a device table of
   2^k elements: entry x = prod_b (x_b ? r_b : 1 - r_b).  What REDUCE-POINTS pairs with the combined columns
   (src/pcs.lisp:352) before it calls PROVE */
int exh_eq_table_device(int degree_d, int k, const uint32_t *r, exh_table *out);

/* ---- LogUp-GKR layer reductions: FRACTION-TREES (src/gkr.lisp:149-170), one in-block layer:
   p, q: K * 2^(m+1) EXTs each; out_p, out_q: K * 2^m EXTs (children (b,x), (b,x+2^m)) */
int exh_gkr_reduce_layer(exh_table p, exh_table q, int degree_d, int K, int m, exh_table *out_p, exh_table *out_q);

/* ---- the domain layer's device side (src/domain.lisp:288-331).  A column as the domain holds it: base values,
   K 2^n for :FULL (kind 0), K 2^(n-c) for :ROW c (kind 1), K 2^c for :COL c (kind 2), without the factor K when
   shared (MAKE-DOMAIN, src/domain.lisp:36-51) */
typedef struct {
  const char *name;
  int32_t kind, c, shared;
  exh_table data;
} exh_domain_column;
/* TABLE-VALUES (src/domain.lisp:311-321): the sumcheck table of a column's half (0 or 1; -1 for a column with one
   table, which does not depend on the top in-block variable): K blocks of 2^(n-1) base values -> a new table */
int exh_domain_table(const exh_domain_column *column, int half, int n, int K, exh_table *out);
/* DOMAIN-LEAVES (src/domain.lisp:298-309) of one lookup: the forms tag, values[0..n_values) and num (NULL: the
   numerator 1) over the columns' names; z and betas (n_values * D) canonical.  out_p, out_q: new tables of
   K * 2^n EXTs, p = num, q = Z - tag - sum_i beta_i v_i, as PROVE-UPPER takes them */
int exh_domain_leaves(int degree_d, int n, int K, const exh_domain_column *columns, int n_columns, const char *tag,
                      const char *const *values, int n_values, const char *num, const uint32_t *z,
                      const uint32_t *betas, exh_table *out_p, exh_table *out_q);

#ifdef __cplusplus
}
#endif
#endif
