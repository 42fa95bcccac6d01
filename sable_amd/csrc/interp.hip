// interp.hip -- the interpreter kernels' instantiations.  Compiled once per (degree, kind) with
// -DEXH_INTERP_D=4|8 -DEXH_INTERP_KIND=0|1 (0: the streaming round kernels, 1: the LDS-resident tail), so that the
// slowest compilations of the library run side by side.
#include "interp.hpp"

namespace exh {

#if EXH_INTERP_KIND == 0
template <>
void launch_interp<EXH_INTERP_D>(const RoundArgs<EXH_INTERP_D> &a, const StmtDesc &d, bool in_base, bool fold,
                                 uint32_t grid, hipStream_t s) {
  constexpr int D = EXH_INTERP_D;
  if (in_base && fold)
    hipLaunchKernelGGL((round_kernel_interp<D, true, true>), dim3(grid), dim3(BLOCK), 0, s, a, d);
  else if (in_base)
    hipLaunchKernelGGL((round_kernel_interp<D, true, false>), dim3(grid), dim3(BLOCK), 0, s, a, d);
  else if (fold)
    hipLaunchKernelGGL((round_kernel_interp<D, false, true>), dim3(grid), dim3(BLOCK), 0, s, a, d);
  else
    hipLaunchKernelGGL((round_kernel_interp<D, false, false>), dim3(grid), dim3(BLOCK), 0, s, a, d);
}
#else
template <>
void launch_tail_interp<EXH_INTERP_D>(const TailArgs<EXH_INTERP_D> &a, const StmtDesc &d, uint32_t grid,
                                      hipStream_t s) {
  constexpr int D = EXH_INTERP_D;
  static bool large_lds = false;
  if (a.lds_bytes > TAIL_LDS_BYTES && !large_lds) {
    (void)hipFuncSetAttribute((const void *)tail_kernel_interp<D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              SLICE_LDS_BYTES);
    large_lds = true;
  }
  hipLaunchKernelGGL((tail_kernel_interp<D>), dim3(grid), dim3(BLOCK), a.lds_bytes, s, a, d);
}
template <>
int tail_interp_blocks_per_cu<EXH_INTERP_D>(uint32_t lds_bytes) {
  constexpr int D = EXH_INTERP_D;
  if (lds_bytes > TAIL_LDS_BYTES)
    (void)hipFuncSetAttribute((const void *)tail_kernel_interp<D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              SLICE_LDS_BYTES);
  int blocks = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, (const void *)tail_kernel_interp<D>, BLOCK, lds_bytes) !=
      hipSuccess)
    return -1;
  return blocks;
}
#endif

}  // namespace exh
