// Direct-to-LDS loads (global memory -> LDS without staging registers) and the explicit waits that go with them,
// shared by the GEMM and the fused-attention kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace brk {
namespace gemm16 {

typedef __attribute__((address_space(3))) unsigned char lds_byte;

// One wave-wide direct-to-LDS load: lane l copies the 16 bytes at
// sbase + voff(l) to LDS byte lds_dst + 16*l.  M0 is written inside the
// statement and not named as clobbered: the compiler treats M0 as reserved and
// rejects it in a clobber list; it holds no compiler-owned value here because
// these kernels contain none of the operations the compiler itself routes
// through M0 (indexed register moves, GWS, messages, lane-indexed reads).
// INVARIANT for whoever adds a kernel that calls dtl_load (or code to one that
// does): it must not contain dynamically indexed register arrays (every array
// index a compile-time constant after unrolling), LDS instructions that take M0
// on this target (none do on gfx9 and later), s_sendmsg, GWS or ds_bpermute-free
// lane-indexed reads (v_readlane with a non-constant lane, v_movrel*).  Check a
// new kernel's assembly for "m0" outside the s_mov_b32 of this statement.
__device__ __forceinline__ void dtl_load(unsigned lds_dst, unsigned voff, const void* sbase) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2"
        :
        : "s"(lds_dst), "v"(voff), "s"(sbase)
        : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmem() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// The 32-bit form: lane l copies the 4 bytes at sbase + voff(l) to LDS byte lds_dst + 4*l (a row of 64 floats per
// wave-wide load).  Same M0 rule as dtl_load.
__device__ __forceinline__ void dtl_load_dword(unsigned lds_dst, unsigned voff, const void* sbase) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %1, %2"
        :
        : "s"(lds_dst), "v"(voff), "s"(sbase)
        : "memory");
}

}  // namespace gemm16
}  // namespace brk
