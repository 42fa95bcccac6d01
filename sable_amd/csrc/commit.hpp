// commit.hpp -- the commitment's data-parallel part on the device: rate-1/2 Reed-Solomon encoding
// (src/rs.lisp:60-85), codeword folding (src/rs.lisp:93-101), BLAKE3 leaf digests and Merkle levels
// with caps (src/pcs.lisp:44-77, 271-304) and the BaseFold loop (src/pcs.lisp:581-657).
#pragma once
#include <stdint.h>

#include "transcript.hpp"

namespace exh {

// ncols messages of 2^c base values (contiguous) -> ncols codewords of 2^(c+1) symbols
int rs_encode_columns(const uint32_t *d_messages, int ncols, int c, uint32_t *d_codewords);
// fold a codeword of 2m elements of degree D on level `level` of the 2^n_domain twiddle tables
int rs_fold_device(int D, uint64_t m, int n_domain, int level, const uint32_t *d_codeword, const uint32_t *r,
                   uint32_t *d_out);
// DOT-PAIRS (src/pcs.lisp:473-483) of two device tables of len EXT8s, parities 0, 1, 2 -> out[3][8] (host)
int dot_pairs_device(const uint32_t *d_e, const uint32_t *d_v, uint64_t len, uint32_t *out);
// the same without any allocation (a static device array holds the partial sums); setup: once per device, at init
int dot_pairs_static_setup(int device);
int dot_pairs_static_device(const uint32_t *d_e, const uint32_t *d_v, uint64_t len, uint32_t *out);
// FOLD-TABLE (src/field.lisp:365-370): d_out[i] = in[2i] + r (in[2i+1] - in[2i]) for len extension elements
int fold_table_device(int D, const uint32_t *d_in, uint64_t len, const uint32_t *r, uint32_t *d_out);
// d_out[x] = d_h[x] (null: zero) + scale * d_column[x] over len extension elements (src/pcs.lisp:709-716)
int scale_add_device(int D, const uint32_t *d_h, const uint32_t *d_column, uint64_t len, const uint32_t *scale,
                     uint32_t *d_out);
// COMBINE-COLUMNS (src/pcs.lisp:434-441): d_out[x] = sum_k coef_k * column_k[x]; ncols base columns of len values,
// coefficients canonical on the host (ncols * D words), d_out len * D words
int combine_columns_device(int D, const uint32_t *d_cols, int ncols, uint64_t len, const uint32_t *coef,
                           uint32_t *d_out);
// leaf digests and all Merkle levels (8-word digests, leaves first) of ncols codewords of
// 2^(c+1) symbols; cap: the level max(0, log2(leaves) - 7), as bytes
int merkle_commit_columns(const uint32_t *d_codewords, int ncols, int c, uint32_t *d_levels, uint8_t *cap,
                          uint64_t *cap_rows);
// OPEN-QUERIES' gathers for one (unit, class) (src/pcs.lisp:721-734): the queried leaves' rows of a class's ncols
// codewords of 2^(c+1) symbols (out_leaves: count * ncols * 4 words) and, when d_levels is given, each leaf's
// siblings up to the cap level (out_paths: count * depth * 32 bytes); leaves: count leaf indices below 2^(c-1)
int open_queries_device(const uint32_t *d_codewords, int ncols, int c, const uint32_t *d_levels, const uint64_t *leaves,
                        int count, uint32_t *out_leaves, uint8_t *out_paths, int *out_depth);
// d_cw (optional): ENCODE-EXT of the table (2^(nv+1) EXT8s on the device) when the caller has it already -- by the
// encoder's linearity the same combination of the committed codewords as the table is of the committed columns
int basefold_prove(Transcript &tr, int nv, const uint32_t *rr, const uint32_t *v, const uint32_t *d_h, int grind_bits,
                   int queries, uint64_t *out_qs, uint32_t *out_chal, uint32_t *out_final,
                   const uint32_t *d_cw = nullptr);
int basefold_verify(Transcript &tr, int nv, const uint32_t *rr, const uint32_t *v, int grind_bits, int queries,
                    uint64_t *out_qs);
// BASEFOLD over several size classes (ascending, the last one nv): class c's table d_hs[k] joins at level nv - c
// d_cws (optional): per class its codeword as for basefold_prove, or null entries
int basefold_prove_classes(Transcript &tr, int nv, int ncls, const int *cls, const uint32_t *const *d_hs,
                           const uint32_t *rr, const uint32_t *v, int grind_bits, int queries, uint64_t *out_qs,
                           uint32_t *out_chal, uint32_t *out_final, const uint32_t *const *d_cws = nullptr);
// one key of the final opening: a size class, a unit of its own with its own tree
struct OpenClass {
  int c = 0, ncols = 0;
  const uint32_t *d_columns = nullptr;    // prover: ncols base columns of 2^c values (device)
  const uint32_t *d_codewords = nullptr;  // prover: their codewords (device)
  const uint32_t *d_levels = nullptr;     // prover: the tree's levels (device)
  const uint32_t *coef = nullptr;         // ncols EXT8s (host): the columns' coefficients in the combined column
  const uint8_t *cap = nullptr;           // verifier: the committed cap (host)
};
// COMBINE-COLUMNS per key, BASEFOLD over the classes, OPEN-QUERIES per key (src/pcs.lisp:434-441, 581-657, 721-734)
int pcs_open(Transcript &tr, int nv, int nkeys, const OpenClass *keys, const uint32_t *rr, const uint32_t *v,
             int grind_bits, int queries, uint64_t *out_qs);
// BASEFOLD's verifier side and VERIFY-QUERIES (src/pcs.lisp:752-843), on the host
int pcs_verify_opening(Transcript &tr, int nv, int nkeys, const OpenClass *keys, const uint32_t *rr, const uint32_t *v,
                       int grind_bits, int queries);
// CHECK-PATH with INJECTED-AT (src/pcs.lisp:86-95), on the host
bool check_path_host(const uint8_t *h, const uint8_t *path, int depth, uint64_t i, const uint8_t *cap, int ninj,
                     const int *inj_level, const uint8_t *inj_digests);
// MERKLE-LEVELS with injections (src/pcs.lisp:64-77) from leaf digests on the device: d_levels receives every level,
// leaves first; d_inj[k] (nleaves >> inj_level[k] digests) is hashed into the nodes of level inj_level[k]
int merkle_levels_injected_device(const uint32_t *d_leaves, uint64_t nleaves, int ninj, const int *inj_level,
                                  const uint32_t *const *d_inj, uint32_t *d_levels);

}  // namespace exh
