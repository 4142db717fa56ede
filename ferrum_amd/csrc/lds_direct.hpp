// LDS-direct loads (global memory straight into LDS, no register in between) and the hand-counted
// waits that cover them: shared by the streamed GEMV and the rows-resident tile kernel.
#pragma once

#include <cstdint>

#include <hip/hip_runtime.h>

namespace fh {

// A wave-uniform pointer as a 64-bit value the compiler keeps in scalar registers.
__device__ __forceinline__ uint64_t uniform_address(const void* pointer) {
    const uint64_t b = reinterpret_cast<uint64_t>(pointer);
    // (the builtin returns a signed int: each half goes through uint32_t before it is widened)
    const uint32_t low = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint32_t high = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    return ((uint64_t)high << 32) | (uint64_t)low;
}

// LDS-direct load: 16 bytes per lane from `base` + `offset` to LDS address `lds_addr` + 16 * lane.
// `base` is the same for the whole wave and travels in scalar registers, `offset` is a lane's own
// 32-bit byte offset: one vector register and no 64-bit vector arithmetic per load.
// The statement writes M0 (the instruction's LDS base) and cannot declare it: this target rejects
// M0 in a clobber list.  It is sound as long as the compiler keeps no value of its own in M0 across
// the statement, which holds for code that uses none of M0's other clients (s_movrel, GWS and
// sendmsg operands, ds_*_addtid, lane-indexed v_readlane through M0): these kernels have none.
// The load is counted in vmcnt like any vector-memory load and returns no register; the only wait
// that covers it is the author's wait_vmcnt / s_waitcnt vmcnt below, so between such a load and
// the wait that counts it there must be no vector-memory instruction of the compiler's.  The
// build compiles this file to assembly text as well and checks all three facts there
// (ferrum_amd/isa_check.py); it refuses to link a library that breaks one.
__device__ __forceinline__ void lds_load16_at(const void* base, uint32_t offset, uint32_t lds_addr) {
    const uint32_t a = __builtin_amdgcn_readfirstlane(lds_addr);
    const uint64_t sb = uniform_address(base);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(sb), "s"(a) : "memory");
}

// s_waitcnt vmcnt(n), n a wave-uniform run-time value up to 20 (0 beyond)
__device__ __forceinline__ void wait_vmcnt(uint32_t n) {
#define FH_VM(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        FH_VM(1) FH_VM(2) FH_VM(3) FH_VM(4) FH_VM(5) FH_VM(6) FH_VM(7) FH_VM(8)
        FH_VM(9) FH_VM(10) FH_VM(11) FH_VM(12) FH_VM(13) FH_VM(14) FH_VM(15)
        FH_VM(16) FH_VM(17) FH_VM(18) FH_VM(19) FH_VM(20)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef FH_VM
}

}  // namespace fh
