// Global -> LDS copy instructions of gfx950, for kernels that order their copies themselves.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aq {

// One global -> LDS copy of 16 bytes per lane (64 lanes fill 1 KiB at lds_base + 16 * lane), written as
// inline asm on purpose.  The compiler knows that the builtin form writes LDS and, unable to tell the
// target from the stages being read, drains EVERY outstanding copy (s_waitcnt vmcnt(0)) before the
// next LDS access; the tile loops need the copies of later blocks in flight while the current block is read and
// order them themselves with counted waits.  Hidden from the compiler, a copy can only make the
// compiler's own waits for ordinary loads stricter, never weaker (completion is in order).
// m0 is reserved by the compiler (it sets it before each of its own uses), so writing it here is safe.
// The source address is a wave-uniform 64-bit base in SGPRs plus a 32-bit byte offset per lane, so the address
// arithmetic of the main loop runs on the scalar unit.
__device__ __forceinline__ void copy16_to_lds(const void* base_uniform, uint32_t lane_offset, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(base_uniform),
                 "s"(__builtin_amdgcn_readfirstlane(lds_base_uniform))
                 : "memory");
}
__device__ __forceinline__ uint32_t lds_offset(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t*)p;
}

}  // namespace aq
