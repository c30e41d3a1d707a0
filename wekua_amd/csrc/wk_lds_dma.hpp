// Direct global -> LDS loads of gfx950 and the hand-written waits that go with them, shared by the
// kernels that bring their k-slabs straight into LDS (wk_gemm_dma.hip, wk_gemm_ipack.hip).
//
// The loads are issued through inline assembly: the compiler's wait-count pass treats a direct-to-LDS
// load it knows about as a store that any later LDS read may alias and would wait for all of them in
// front of every LDS read, which serialises exactly what these kernels overlap.  The waits that are
// needed are written out instead.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace wk {
namespace lds_dma {

// 16 bytes per lane from global memory (scalar base + 32-bit byte offset per lane) to LDS at
// lds_base + 16 * lane; lds_base is a byte address, the same in every lane.  The LDS base travels in M0,
// which the register allocator writes itself (the "{m0}" operand): a value of its own that it keeps there
// (lane indexing, messages) is then saved and restored around the load like around any other use.  The
// s_nop covers the wait state between a write of M0 and an LDS-DMA instruction that reads it.
__device__ __forceinline__ void dma16(const void *base, uint32_t byte_offset, uint32_t lds_base) {
    asm volatile("s_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(byte_offset), "s"(base), "{m0}"(lds_base)
                 : "memory");
}

// The same with 4 bytes per lane: LDS at lds_base + 4 * lane.  For operands whose rows do not start on
// 16-byte boundaries: every lane names exactly one existing element (or half of one), so nothing is
// read beyond a row, at four times the instructions per byte.
__device__ __forceinline__ void dma4(const void *base, uint32_t byte_offset, uint32_t lds_base) {
    asm volatile("s_nop 0\n\t"
                 "global_load_lds_dword %0, %1"
                 :
                 : "v"(byte_offset), "s"(base), "{m0}"(lds_base)
                 : "memory");
}

template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// wait until at most min(later, MAXN) slabs' loads of this wavefront (PER loads each) are still in flight
template <int PER, int MAXN> __device__ __forceinline__ void wait_vm_slabs(uint32_t later) {
    if constexpr (MAXN <= 0) {
        wait_vm<0>();
    } else {
        if (later >= (uint32_t)MAXN) wait_vm<MAXN * PER>();
        else wait_vm_slabs<PER, MAXN - 1>(later);
    }
}
// f(integral_constant<int, A>) for A = FROM, FROM - 1, ..., 0
template <int FROM, typename F> __device__ __forceinline__ void drain(F &&f) {
    if constexpr (FROM >= 0) {
        f(std::integral_constant<int, FROM>{});
        drain<FROM - 1>(f);
    }
}
// f(integral_constant<int, A>) for A = 0, 1, ..., N - 1
template <int N, int A = 0, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (A < N) {
        f(std::integral_constant<int, A>{});
        static_for<N, A + 1>(f);
    }
}
__device__ __forceinline__ void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }


} // namespace lds_dma
} // namespace wk
