// wf2_dma.h -- global -> LDS loads for the kernels that feed the matrix cores from LDS tiles.
//
// What an instruction costs a wavefront that is otherwise issuing v_mfma_f32_32x32x2_f32 back to
// back (64 cycles of the matrix pipe each), measured on gfx950 between the MFMAs of such a loop:
//   LDS reads, scalar ALU, s_waitcnt, s_barrier        nothing (latency aside)
//   a vector-ALU instruction                           5 cycles in a run, 12 alone (8 - 16: v_exp_f32,
//                                                      v_max3_f32, v_mov_b64), also when another
//                                                      wavefront of the SIMD issues it
//   a global load, 64-bit address per lane             26 cycles (to registers or to LDS)
//   a global load, scalar base + 32-bit lane offset    5 cycles
// The compiler's own LDS-load builtin always forms the 64-bit address (and a v_lshl_add_u64 per
// instruction to get it), hence this wrapper: the tile loops keep one base per operand in scalar
// registers, advanced on the scalar unit, and per lane only offsets that never change.
#pragma once
#include <stdint.h>

#include "wf2_common.h"

namespace wf2 {

// 64 lanes x 16 bytes from `base` + this lane's byte offset into the 1 KB of LDS that starts at byte
// address `lds_addr`; `lds_addr` and `base` are the same for the whole wavefront.  M0 holds the LDS
// destination: the kernels that use this helper have no other use of M0.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma16(uint32_t lds_addr, uint32_t lane_offset, const float* base) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(lane_offset), "s"(base)
               : "memory", "m0");
#endif
}
#pragma clang diagnostic pop

// byte address within LDS of a pointer into a __shared__ array
__device__ __forceinline__ uint32_t lds_address(const float* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const float*)p;
}

}  // namespace wf2
