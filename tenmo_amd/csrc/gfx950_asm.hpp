// The pieces of the kernels that are written in gfx950 assembly, in one place: the direct global->LDS loads and
// a register keep-alive.  (A CPU build of the kernels, which replays launches thread by thread to check every
// address they touch, defines TENMO_GFX950_ASM_HPP and its own versions of these functions before any source
// includes this header.)
#ifndef TENMO_GFX950_ASM_HPP
#define TENMO_GFX950_ASM_HPP
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tenmo {

// byte address of an LDS object, as the hardware counts it
__device__ __forceinline__ uint32_t lds_address(const float* lds) { return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)lds; }

// One wave-load straight from global memory into LDS: lane L copies the 16 bytes at `src` + `lane_byte_off` (src the
// same in every lane: it lives in scalar registers) to bytes [16L, 16L+16) of the 1 KiB LDS block that starts
// `block_byte_off` bytes into the LDS object `lds` (M0 holds the block's LDS address).  Scalar base + 32-bit lane offset addressing keeps vector ALU work out of the MFMA
// stream: 64-bit per-lane address arithmetic between MFMAs was measured to cost 2 % at 8192^3.
// (M0 is a register the compiler reserves: it sets it itself right before each of its own uses and keeps nothing in it
// across other code, so writing it here needs no declaration — and the compiler rejects one.)
// Issued through inline assembly on purpose: the compiler's wait-count pass otherwise drains every outstanding direct
// load before any later LDS read, which would serialise a ring of stages.  The callers wait for these loads explicitly
// with s_waitcnt vmcnt(n).
__device__ __forceinline__ void direct_load_16B(float* lds, uint32_t block_byte_off, uint32_t lane_byte_off, const float* src) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(lds) + block_byte_off);
    // s_nop 3: the scalar base may have come out of a v_readfirstlane right before this block, and a vector-memory
    // instruction must not read a scalar register within 5 wait states of a vector instruction writing it — the compiler
    // pads its own loads for that, but it does not look inside an asm block (the same padding covers M0: 1 wait state).
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(lane_byte_off), "s"(src) : "memory");
}

// The same for the lanes with `ok` only: the others neither read memory nor write LDS.  The execution mask is narrowed
// inside the assembly block, because under a divergent branch the compiler no longer keeps the block's scalar operands
// in scalar registers.  Everything the block overwrites is declared: s_and_b64 sets SCC, and a block that does not say so
// lets the compiler keep a carry in SCC across it — it then scheduled the s_addc_u32 of a 64-bit address behind this
// block, the high half came out one too large (4 GiB off) and the next load faulted.
__device__ __forceinline__ void direct_load_16B_where(float* lds, uint32_t block_byte_off, uint32_t lane_byte_off, const float* src, bool ok) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(lds) + block_byte_off);
    const uint32_t pred = ok ? 1u : 0u;
    uint64_t saved_exec;
    asm volatile("s_mov_b32 m0, %1\n\t"
                 "s_nop 1\n\t" // with the three instructions below: 5 wait states between code before the block and the load
                 "s_mov_b64 %0, exec\n\t"
                 "v_cmp_ne_u32_e32 vcc, 0, %4\n\t"
                 "s_and_b64 exec, exec, vcc\n\t"
                 "global_load_lds_dwordx4 %2, %3\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved_exec)
                 : "s"(dst), "v"(lane_byte_off), "s"(src), "v"(pred)
                 : "memory", "vcc", "scc");
}

// keeps four accumulator chains alive without a store
template <class V>
__device__ __forceinline__ void keep_alive(const V& a0, const V& a1, const V& a2, const V& a3) {
    asm volatile("" ::"v"(a0), "v"(a1), "v"(a2), "v"(a3));
}

} // namespace tenmo
#endif
