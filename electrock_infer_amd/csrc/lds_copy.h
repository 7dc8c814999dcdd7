// Direct global -> LDS copies (global_load_lds_*) with hand-kept completion counts,
// shared by the tiled GEMM kernels.
#pragma once
#include "common.h"

namespace em {

// M0 is a reserved register that the compiler never keeps live values in here (the
// kernel has no dynamically indexed register arrays); naming it as a clobber documents
// the write and only triggers an advisory warning.
#pragma clang diagnostic ignored "-Winline-asm"

// One wave copies 64 x 16 B from per-lane global addresses to 1 KB of LDS starting at
// the wave-uniform byte address `lds_addr`.  The compiler does not see the LDS write:
// every consumer sits behind wait_dma<>() + block_barrier().
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
// Same copy for data that no other workgroup reads again (weight rows streamed once): the non-temporal
// hint keeps them from displacing reusable lines; plain reads of a stream top out ~15 % lower on this GPU.
__device__ __forceinline__ void dma16_stream(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                 :: "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
// Same copy with the address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit byte
// offset per lane: half the address registers, and stepping through K is scalar arithmetic.
__device__ __forceinline__ void dma16(uint32_t lane_offset, const void* uniform_base, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_offset), "s"(uniform_base), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ void dma16_stream(uint32_t lane_offset, const void* uniform_base, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :: "v"(lane_offset), "s"(uniform_base), "s"(lds_addr) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_dma() {  // at most N of this wave's copies still in flight
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}
// Same for one dword per lane (256 B of LDS per wave): used only to pull lines into L2.
__device__ __forceinline__ void dma4(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                 :: "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ void block_barrier() { asm volatile("s_barrier" ::: "memory"); }


}  // namespace em
