// issue_rate.hip -- how fast a SIMD of this part issues the VALU instructions the proving kernels are made of.
//
// The round kernels are bound by HBM bytes and by VALU issue at once, so the second roofline needs a measured
// peak: a kernel of CHAINS independent chains of one instruction (written in assembly, so that the compiler can
// neither fuse nor drop them), ITER iterations, timed with HIP events.  With many resident wavefronts per SIMD
// the figure is the issue rate (cycles per wavefront instruction and SIMD); with one wavefront per SIMD and one
// chain it is the latency between dependent instructions, which bounds the one-wavefront transcript.
// No counterpart in the reference: measurement only.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "blake3.hpp"
#include "context.hpp"

namespace exh {

enum IssueOp : int {
  OP_FMA_F64 = 0,
  OP_ADD_F64,
  OP_MUL_F64,
  OP_MUL_LO_U32,
  OP_MUL_HI_U32,
  OP_MAD_U64_U32,
  OP_ADD_U32,
  OP_SUB_MIN_U32,  // the modular add's tail: two instructions
  OP_XOR_B32,
  OP_ALIGNBIT_B32,
  OP_ADD3_U32,
  OP_FMA_F32,
  OP_ADDC_PAIR,  // a 64-bit add: add with carry-out, add with carry-in (two instructions)
  OP_CVT_F64_U32,
  OP_MIN_U32,
  OP_CNDMASK_B32,    // a select reading a vcc that no instruction near it wrote: 23 cycles each, unlike every real use below
  OP_PERM_B32,       // a rotation by whole bytes as a byte permutation
  OP_ALIGNBYTE_B32,  // the same as a byte alignment of the word with itself
  OP_LSHLREV_B32,
  OP_LSHL_OR_B32,
  OP_XAD_U32,
  OP_CMP_CNDMASK,   // a comparison into vcc and the select that reads it (two instructions)
  OP_CMP_U32,       // the comparison alone
  OP_CNDMASK_SGPR,  // the select reading its mask from a scalar register pair
  OP_CMP_2CNDMASK,  // one comparison, two selects that read it (three instructions)
  OP_CMP_GAP_CNDMASK,  // a comparison, four other instructions, then the select (six instructions)
  OP_CMP_SGPR_CNDMASK,  // the comparison into a scalar register pair and the select reading that (two instructions)
  OP_B3_COMPRESS,  // a BLAKE3 compression as the Merkle kernels run it (compiled code, not assembly): its instructions
                   // (230 v_xor, 224 v_alignbit, 116 v_add, 108 v_add3) in their real order and dependence
  OP_COUNT
};

static const char *const kOpNames[OP_COUNT] = {
    "v_fma_f64",     "v_add_f64",      "v_mul_f64",   "v_mul_lo_u32", "v_mul_hi_u32", "v_mad_u64_u32",
    "v_add_u32",     "v_sub_u32+v_min_u32", "v_xor_b32", "v_alignbit_b32", "v_add3_u32", "v_fma_f32",
    "v_add_co_u32+v_addc_co_u32", "v_cvt_f64_u32", "v_min_u32", "v_cndmask_b32(vcc written once, long before)", "v_perm_b32", "v_alignbyte_b32",
    "v_lshlrev_b32", "v_lshl_or_b32", "v_xad_u32", "v_cmp_lt_u32+v_cndmask_b32", "v_cmp_lt_u32", "v_cndmask_b32(sgpr mask)",
    "v_cmp_lt_u32+2 v_cndmask_b32", "v_cmp_lt_u32+4 v_xor_b32+v_cndmask_b32", "v_cmp_lt_u32(sgpr)+v_cndmask_b32(sgpr)",
    "blake3 compression (678 instructions)"};
static const int kOpInstructions[OP_COUNT] = {1, 1, 1, 1, 1, 1, 1, 2, 1, 1, 1, 1, 2, 1, 1, 1,
                                              1, 1, 1, 1, 1, 2, 1, 1, 3, 6, 2, 678};

constexpr int ISSUE_BLOCK = 256;

template <int OP, int CHAINS>
__global__ __launch_bounds__(ISSUE_BLOCK) void issue_rate_kernel(uint32_t *out, uint32_t iterations, uint32_t ia,
                                                                 uint32_t ib, double fa, double fb) {
  uint32_t u[CHAINS];
  uint64_t w[CHAINS];
  double x[CHAINS];
  float f[CHAINS];
#pragma unroll
  for (int i = 0; i < CHAINS; i++) {
    u[i] = threadIdx.x * 77u + i, w[i] = threadIdx.x + 3u * i, x[i] = (double)(threadIdx.x + i);
    f[i] = (float)(threadIdx.x + i);
  }
  const float ffa = (float)fa, ffb = (float)fb;
  // (the selects below read vcc: written once here, by a vector comparison, as in real code)
  if constexpr (OP == OP_CNDMASK_B32) asm volatile("v_cmp_lt_u32 vcc, %0, %1" : : "v"(u[0]), "v"(ia) : "vcc");
  for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
    for (int rep = 0; rep < 8; rep++) {
#pragma unroll
      for (int i = 0; i < CHAINS; i++) {
        if constexpr (OP == OP_FMA_F64) asm volatile("v_fma_f64 %0, %0, %1, %2" : "+v"(x[i]) : "v"(fa), "v"(fb));
        if constexpr (OP == OP_ADD_F64) asm volatile("v_add_f64 %0, %0, %1" : "+v"(x[i]) : "v"(fa));
        if constexpr (OP == OP_MUL_F64) asm volatile("v_mul_f64 %0, %0, %1" : "+v"(x[i]) : "v"(fa));
        if constexpr (OP == OP_MUL_LO_U32) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(u[i]) : "v"(ia));
        if constexpr (OP == OP_MUL_HI_U32) asm volatile("v_mul_hi_u32 %0, %0, %1" : "+v"(u[i]) : "v"(ia));
        if constexpr (OP == OP_MAD_U64_U32) {
          uint64_t carry;
          asm volatile("v_mad_u64_u32 %0, %1, %2, %3, %0" : "+v"(w[i]), "=&s"(carry) : "v"(u[i]), "v"(ia));
        }
        if constexpr (OP == OP_ADD_U32) asm volatile("v_add_u32 %0, %0, %1" : "+v"(u[i]) : "v"(ia));
        if constexpr (OP == OP_SUB_MIN_U32) {
          uint32_t t;
          asm volatile("v_sub_u32 %1, %0, %2\n\tv_min_u32 %0, %0, %1" : "+v"(u[i]), "=&v"(t) : "v"(ia));
        }
        if constexpr (OP == OP_XOR_B32) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(u[i]) : "v"(ia));
        if constexpr (OP == OP_ALIGNBIT_B32) asm volatile("v_alignbit_b32 %0, %0, %0, 7" : "+v"(u[i]));
        if constexpr (OP == OP_ADD3_U32) asm volatile("v_add3_u32 %0, %0, %1, %2" : "+v"(u[i]) : "v"(ia), "v"(ib));
        if constexpr (OP == OP_FMA_F32) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(f[i]) : "v"(ffa), "v"(ffb));
        if constexpr (OP == OP_ADDC_PAIR) {
          uint32_t lo = (uint32_t)w[i], hi = (uint32_t)(w[i] >> 32);
          asm volatile("v_add_co_u32 %0, vcc, %0, %2\n\tv_addc_co_u32 %1, vcc, %1, %3, vcc"
                       : "+v"(lo), "+v"(hi)
                       : "v"(ia), "v"(ib)
                       : "vcc");
          w[i] = ((uint64_t)hi << 32) | lo;
        }
        if constexpr (OP == OP_CVT_F64_U32) asm volatile("v_cvt_f64_u32 %0, %1" : "=v"(x[i]) : "v"(u[i]));
        if constexpr (OP == OP_MIN_U32) asm volatile("v_min_u32 %0, %0, %1" : "+v"(u[i]) : "v"(ia));
        if constexpr (OP == OP_CNDMASK_B32) asm volatile("v_cndmask_b32 %0, %0, %1, vcc" : "+v"(u[i]) : "v"(ia) : );
        if constexpr (OP == OP_PERM_B32) asm volatile("v_perm_b32 %0, %0, %0, %1" : "+v"(u[i]) : "v"(ib));
        if constexpr (OP == OP_ALIGNBYTE_B32) asm volatile("v_alignbyte_b32 %0, %0, %0, 1" : "+v"(u[i]));
        if constexpr (OP == OP_LSHLREV_B32) asm volatile("v_lshlrev_b32 %0, 7, %0" : "+v"(u[i]));
        if constexpr (OP == OP_LSHL_OR_B32) asm volatile("v_lshl_or_b32 %0, %0, 7, %1" : "+v"(u[i]) : "v"(ia));
        if constexpr (OP == OP_XAD_U32) asm volatile("v_xad_u32 %0, %0, %1, %2" : "+v"(u[i]) : "v"(ia), "v"(ib));
        if constexpr (OP == OP_CMP_CNDMASK)
          asm volatile("v_cmp_lt_u32 vcc, %0, %1\n\tv_cndmask_b32 %0, %0, %2, vcc" : "+v"(u[i]) : "v"(ia), "v"(ib) : "vcc");
        if constexpr (OP == OP_CMP_U32) asm volatile("v_cmp_lt_u32 vcc, %0, %1" : : "v"(u[i]), "v"(ia) : "vcc");
        if constexpr (OP == OP_CMP_2CNDMASK) {
          uint32_t t = u[i];
          asm volatile("v_cmp_lt_u32 vcc, %0, %2\n\tv_cndmask_b32 %0, %0, %3, vcc\n\tv_cndmask_b32 %1, %1, %2, vcc"
                       : "+v"(u[i]), "+v"(t) : "v"(ia), "v"(ib) : "vcc");
          u[i] ^= t;
        }
        if constexpr (OP == OP_CMP_GAP_CNDMASK) {
          uint32_t t = u[i];
          asm volatile("v_cmp_lt_u32 vcc, %0, %2\n\tv_xor_b32 %1, %1, %2\n\tv_xor_b32 %1, %1, %3\n\tv_xor_b32 %1, %1, %2\n\t"
                       "v_xor_b32 %1, %1, %3\n\tv_cndmask_b32 %0, %0, %1, vcc"
                       : "+v"(u[i]), "+v"(t) : "v"(ia), "v"(ib) : "vcc");
        }
        if constexpr (OP == OP_CMP_SGPR_CNDMASK) {
          uint64_t mask;
          asm volatile("v_cmp_lt_u32 %1, %0, %2\n\tv_cndmask_b32 %0, %0, %3, %1" : "+v"(u[i]), "=&s"(mask) : "v"(ia), "v"(ib));
        }
        if constexpr (OP == OP_B3_COMPRESS) {
          if (i == 0) {  // one compression per link, whatever the number of chains: it has four of its own
            uint32_t cv[8], m[16];
#pragma unroll
            for (int k = 0; k < 8; k++) cv[k] = u[0] + k;
#pragma unroll
            for (int k = 0; k < 16; k++) m[k] = ia + k;
            b3_compress(cv, m, 0, 64, 11, cv, 0);
            u[0] = cv[0] ^ cv[1] ^ cv[2] ^ cv[3] ^ cv[4] ^ cv[5] ^ cv[6] ^ cv[7];
          }
        }
        if constexpr (OP == OP_CNDMASK_SGPR) {
          uint64_t mask = 0x5555555555555555ull;
          asm volatile("v_cndmask_b32 %0, %0, %1, %2" : "+v"(u[i]) : "v"(ia), "s"(mask));
        }
      }
    }
  }
  uint32_t s = 0;
#pragma unroll
  for (int i = 0; i < CHAINS; i++) s += u[i] + (uint32_t)w[i] + (uint32_t)(w[i] >> 32) + (uint32_t)x[i] + (uint32_t)f[i];
  out[(size_t)blockIdx.x * ISSUE_BLOCK + threadIdx.x] = s;
}

template <int OP>
static void launch_issue(int chains, uint32_t grid, hipStream_t s, uint32_t *out, uint32_t iterations) {
  if (chains == 1)
    hipLaunchKernelGGL((issue_rate_kernel<OP, 1>), dim3(grid), dim3(ISSUE_BLOCK), 0, s, out, iterations, 12345u, 7u,
                       1.000001, 0.5);
  else
    hipLaunchKernelGGL((issue_rate_kernel<OP, 8>), dim3(grid), dim3(ISSUE_BLOCK), 0, s, out, iterations, 12345u, 7u,
                       1.000001, 0.5);
}

template <int OP = 0>
static void dispatch_issue(int op, int chains, uint32_t grid, hipStream_t s, uint32_t *out, uint32_t iterations) {
  if constexpr (OP < OP_COUNT) {
    if (op == OP)
      launch_issue<OP>(chains, grid, s, out, iterations);
    else
      dispatch_issue<OP + 1>(op, chains, grid, s, out, iterations);
  }
}

// One measurement: `workgroups` workgroups of 256 threads (4 wavefronts, one per SIMD of a compute unit), each
// lane running `chains` (1 or 8) independent chains of instruction `op` for iterations * 8 links.  Out: the
// launch's duration, the machine instructions each wavefront issued, the device's clock and compute units.
int issue_rate(int op, int chains, int workgroups, int iterations, const char **name, float *ms,
               double *instructions_per_wave, int *clock_khz, int *compute_units) {
  Context &c = ctx();
  int status = c.require();
  if (status) return status;
  if (op < 0 || op >= OP_COUNT || (chains != 1 && chains != 8) || workgroups < 1 || workgroups > (1 << 16) ||
      iterations < 1 || iterations > (1 << 20)) {
    set_error("invalid-parameter: issue-rate measurement (op, chains 1 or 8, workgroups, iterations)");
    return E_PARAM;
  }
  uint32_t *out = (uint32_t *)c.pool.alloc((size_t)workgroups * ISSUE_BLOCK * 4);
  if (!out) {
    set_error("device-out-of-memory: issue-rate output");
    return E_NOMEM;
  }
  struct Release {
    Pool &pool;
    void *ptr;
    ~Release() { pool.release(ptr); }
  } release{c.pool, out};
  hipEvent_t e0, e1;
  EXH_HIP(hipEventCreate(&e0));
  EXH_HIP(hipEventCreate(&e1));
  dispatch_issue(op, chains, (uint32_t)workgroups, c.stream, out, 16);  // warm: code object load, clocks
  EXH_HIP(hipStreamSynchronize(c.stream));
  EXH_HIP(hipEventRecord(e0, c.stream));
  dispatch_issue(op, chains, (uint32_t)workgroups, c.stream, out, (uint32_t)iterations);
  EXH_HIP(hipEventRecord(e1, c.stream));
  EXH_HIP(hipStreamSynchronize(c.stream));
  EXH_HIP(hipGetLastError());
  EXH_HIP(hipEventElapsedTime(ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  hipDeviceProp_t prop;
  EXH_HIP(hipGetDeviceProperties(&prop, c.device));
  if (name) *name = kOpNames[op];
  // (a compression is one per link whatever the number of chains)
  if (instructions_per_wave)
    *instructions_per_wave = (double)iterations * 8.0 * (op == OP_B3_COMPRESS ? 1 : chains) * kOpInstructions[op];
  if (clock_khz) *clock_khz = prop.clockRate;
  if (compute_units) *compute_units = prop.multiProcessorCount;
  return OK;
}
int issue_rate_ops() { return OP_COUNT; }

}  // namespace exh
