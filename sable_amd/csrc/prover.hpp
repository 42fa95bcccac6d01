// prover.hpp -- the host side of the protocols over the device sessions: PROVE / VERIFY / CHECK-FINAL
// of the sumcheck with the reference's argument meaning (src/sumcheck.lisp:131-172, 512-571).
#pragma once
#include <stdint.h>

#include <string>

#include "forms.hpp"
#include "sumcheck.hpp"
#include "transcript.hpp"

namespace exh {

// HYPERCUBE-SUM (src/sumcheck.lisp:112-126) of a statement wider than one kernel holds: the sum of its parts' claims
int hypercube_sum_wide(const Statement &st, int D, int n, const uint32_t *const *d_tables, const int *strides,
                       const uint32_t *eq, const uint32_t *consts, uint32_t *out);
// tables: device pointers, K * 2^n entries of stride 1 or D each, block-major.
int sumcheck_prove(Transcript &tr, int n, const Statement &st, const uint32_t *const *d_tables, const int *strides,
                   const uint32_t *eq, const uint32_t *consts, const std::string &label, const uint32_t *bw, int K,
                   int degree, uint32_t *out_chal, uint32_t *out_finals, uint32_t *const *out_folded,
                   uint32_t *d_folded = nullptr, uint64_t d_folded_len = 0);
// (d_folded: the folded tables are also left on the device, table t at d_folded + t * d_folded_len * D, zeros after
// its K entries; with out_finals and out_folded null nothing of them comes to the host)
int sumcheck_verify(Transcript &tr, int n, const Statement &st, const uint32_t *claim, const uint32_t *eq,
                    const uint32_t *consts, int blocks, const std::string &label, int degree, uint32_t *out_chal,
                    uint32_t *out_reduced);
int check_final(const Statement &st, int D, const uint32_t *reduced, const uint32_t *finals, const uint32_t *consts);
void absorb_header(Transcript &tr, const std::string &label, int n, int degree, int blocks);
// the header's bytes: label | n u16 | degree u16 | blocks u32, little-endian (src/sumcheck.lisp:24-27)
std::string header_bytes(const std::string &label, int n, int degree, int blocks);
// the host transcript's hash state as the device transcript keeps it, and back
DevB3S device_state(const Transcript &tr);
int adopt_device_state(Transcript &tr, const DevB3S &state);

}  // namespace exh
