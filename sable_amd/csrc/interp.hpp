// interp.hpp -- launchers of the interpreter kernels: the round and tail bodies over a run-time descriptor, for
// statements without generated kernels (the reference's GENERIC-ROUND-SUMS analogue, src/sumcheck.lisp:282-311).
#pragma once
#include <hip/hip_runtime.h>

#include "sumcheck_kernels.hpp"

namespace exh {

template <int D>
void launch_interp(const RoundArgs<D> &a, const StmtDesc &d, bool in_base, bool fold, uint32_t grid, hipStream_t s);
template <int D>
void launch_tail_interp(const TailArgs<D> &a, const StmtDesc &d, uint32_t grid, hipStream_t s);
// workgroups of the interpreter's tail kernel a compute unit holds with that much dynamic LDS (-1: unknown)
template <int D>
int tail_interp_blocks_per_cu(uint32_t lds_bytes);

}  // namespace exh
