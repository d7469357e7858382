// Direct global -> LDS loads for the operand rings of the grouped GEMM kernels, and the wait-count arithmetic that
// goes with them.
#pragma once
#include "common.h"

namespace mole {

// s_waitcnt immediate that waits for vmcnt <= n and nothing else (gfx9 encoding: vmcnt in bits 3:0
// and 15:14, expcnt 6:4, lgkmcnt 11:8)
constexpr int waitcnt_vm(int n) { return (n & 0xf) | ((n >> 4) << 14) | 0x0070 | 0x0f00; }

// 16 bytes per lane from global memory straight into LDS: lane i of the wave writes LDS bytes
// [lds_off + 16 i, +16).  Issued as inline assembly on purpose: the compiler makes every LDS read
// that follows a global_load_lds it knows about wait for vmcnt(0), which would serialise the ring of
// stages; here the K loop does its own vmcnt accounting (s_waitcnt before each barrier).  M0 is
// reserved by the compiler and nothing else in these kernels uses it.
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_off) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_off) : "memory");
}
// The same with the address split into a wave-uniform 64-bit base (SGPR pair) and a 32-bit per-lane byte
// offset: the K loop then advances the base with scalar adds and spends no VALU work on addresses.
__device__ __forceinline__ void dma16s(const void *sbase, uint32_t voff, uint32_t lds_off) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_off) : "memory");
}
__device__ __forceinline__ const char *uniform_ptr(const void *p) {   // tell the compiler the pointer is wave-uniform
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const char *)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ uint32_t lds_offset_of(const char *p) {
    return (uint32_t)(size_t)(__attribute__((address_space(3))) const char *)p;
}

// Swizzle of the 16-byte piece index of a tile held as [row][4 x 16 B] (64-byte rows: 32 bf16 or 16 fp32 of K),
// chosen so that the 16 rows a ds_read_b128 pass touches (and any 8 aligned rows) fall into distinct bank groups of
// the 64-bank LDS.
__device__ __forceinline__ int swz4(int row) { return (((row >> 1) ^ (row >> 3)) & 1) | ((row >> 1) & 2); }

}  // namespace mole
