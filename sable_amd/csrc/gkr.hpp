// gkr.hpp -- batched LogUp-GKR fractional sums: the layer reductions on the device and the
// protocol's host side (src/gkr.lisp).
#pragma once
#include <stdint.h>

#include <string>

#include "transcript.hpp"

namespace exh {

// one in-block layer of FRACTION-TREES (src/gkr.lisp:157-170): K blocks of 2^(m+1) children in,
// K blocks of 2^m parents out; all device pointers to EXTs of degree D
int gkr_reduce_layer(int D, int K, int m, const uint32_t *p, const uint32_t *q, uint32_t *pp, uint32_t *qq);

// PROVE-UPPER (src/gkr.lisp:215-272): leaves[2l], leaves[2l+1] = p, q of lookup l on the device
int gkr_prove_upper(Transcript &tr, int n, int K, int lookups, const uint32_t *const *leaves,
                    const std::string &label, uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp,
                    uint32_t *out_cq);
// VERIFY-UPPER (src/gkr.lisp:91-145)
int gkr_verify_upper(Transcript &tr, int n, int K, int lookups, const std::string &label, uint32_t *out_roots,
                     uint32_t *out_ri, uint32_t *out_rb, uint32_t *out_cp, uint32_t *out_cq);

}  // namespace exh
