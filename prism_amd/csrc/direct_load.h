// Global memory -> LDS without staging registers (gfx950 global_load_lds_dwordx4).
#pragma once

#include <cstdint>

#include <hip/hip_runtime.h>

namespace prism {

// One wave-wide load of 16 B per lane from global memory straight into LDS: lane l
// reads base + lane_offset(l) and lands at lds_dst + 16 l (1 KiB of contiguous LDS
// per instruction). Written as inline assembly for its addressing mode: a scalar
// base plus a 32-bit vector offset. The compiler's own selection for the
// direct-load builtin builds a 64-bit vector address with vector ALU instructions
// for every load, and a vector ALU instruction between two MFMAs delays the second
// one (about 12 clocks each, measured with one wave per SIMD). M0 carries the LDS
// address; a scalar write of M0 needs one wait state before the load reads it.
//
// The compiler does not see these loads in its wait counts: the caller waits with an
// explicit s_waitcnt (waitcnt_imm below) before the barrier that publishes the data.
__device__ __forceinline__ void direct_load16(const char* base, uint32_t lane_offset, const void* lds_dst) {
    const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (const __attribute__((address_space(3))) void*)lds_dst));
    // M0 is listed as clobbered so that the compiler does not assume a value of its own survives
    // (clang warns that M0 is a reserved register; the kernels here have no other user of it).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
#pragma clang diagnostic pop
}

// The 4-byte form: lane l reads base + lane_offset(l) and lands at lds_dst + 4 l (256 B of contiguous LDS
// per instruction).
__device__ __forceinline__ void direct_load4(const char* base, uint32_t lane_offset, const void* lds_dst) {
    const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (const __attribute__((address_space(3))) void*)lds_dst));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
#pragma clang diagnostic pop
}

// The same load through a buffer descriptor: lane l reads descriptor base + lane_offset(l) +
// scalar_offset. Every dword whose offset (lane + scalar part) is at or beyond the descriptor's
// extent arrives as zero, which is how ragged matrix edges are filled: the extent ends with the
// matrix, and a lane whose element lies outside for another reason (past the row end) passes
// kBeyondExtent as its offset.
typedef int i32x4 __attribute__((ext_vector_type(4)));
constexpr uint32_t kBeyondExtent = 0x80000000u;  // extents here stay below 2 GiB
// Extent of a descriptor that should end `bytes_left` bytes after its base: descriptors hold 32 bits, and
// every offset used here stays below 2 GiB, so anything beyond that is cut to 2 GiB - 1 (kBeyondExtent
// stays out of range).
__host__ __device__ __forceinline__ uint32_t clamped_extent(long long bytes_left) {
    return static_cast<uint32_t>(bytes_left < 0 ? 0 : (bytes_left > 0x7fffffffll ? 0x7fffffffll : bytes_left));
}
// Raw buffer descriptor (stride 0) for `extent_bytes` bytes at `base`: base address, extent, and the
// data-format word of an untyped 32-bit buffer. Wave-uniform by construction (forced into scalar registers).
__device__ __forceinline__ i32x4 buffer_descriptor(const void* base, uint32_t extent_bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    i32x4 d;
    d[0] = __builtin_amdgcn_readfirstlane(static_cast<int>(a & 0xffffffffu));
    d[1] = __builtin_amdgcn_readfirstlane(static_cast<int>((a >> 32) & 0xffffu));
    d[2] = __builtin_amdgcn_readfirstlane(static_cast<int>(extent_bytes));
    d[3] = 0x00020000;
    return d;
}
// A descriptor is wave-uniform by contract; said explicitly, dword by dword, because the operand must be a
// tuple of scalar registers (a descriptor that went through 64-bit arithmetic may otherwise be handed over in
// vector registers, which does not assemble). No instruction results when the value is scalar already.
__device__ __forceinline__ i32x4 scalar_descriptor(i32x4 d) {
#pragma unroll
    for (int c = 0; c < 4; ++c) d[c] = __builtin_amdgcn_readfirstlane(d[c]);
    return d;
}
__device__ __forceinline__ void direct_load16_buffer(i32x4 rsrc, uint32_t lane_offset, uint32_t scalar_offset,
                                                     const void* lds_dst) {
    rsrc = scalar_descriptor(rsrc);
    const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (const __attribute__((address_space(3))) void*)lds_dst));
    // Wave-uniform by contract; said explicitly because the operand must be a scalar register.
    scalar_offset = __builtin_amdgcn_readfirstlane(scalar_offset);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                 :
                 : "v"(lane_offset), "s"(rsrc), "s"(scalar_offset), "s"(lds_addr)
                 : "memory", "m0");
#pragma clang diagnostic pop
}

// The same load in two parts, for loops in which matrix instructions run back to back: M0 is written
// one matrix instruction ahead of the load that reads it. Measured with one wave per SIMD between
// independent 16-clock MFMAs: `s_mov m0; s_nop 0; buffer_load ... lds` in one place holds the next MFMA
// up by 10 clocks (6 for the global_load_lds form), the M0 write alone by none, and the load alone,
// with M0 written one MFMA earlier (which is also the wait state the load needs), by none at six
// instructions between loads and 1 clock at four. Nothing else may write M0 between the two parts: the
// compiler has no use for M0 in these loops (no indexed register access, no spills); the callers'
// kernels are checked for that in the generated code.
__device__ __forceinline__ void set_direct_load_destination(const void* lds_dst) {
    const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (const __attribute__((address_space(3))) void*)lds_dst));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    asm volatile("s_mov_b32 m0, %0" : : "s"(lds_addr) : "memory", "m0");
#pragma clang diagnostic pop
}
// The descriptor and the scalar offset must be in scalar registers already (made so where they are
// computed, away from the loads): a v_readfirstlane here would sit right in front of the load, which would
// then read a scalar register the vector ALU has just written, without the wait states that needs.
__device__ __forceinline__ void direct_load16_buffer_to_destination(i32x4 rsrc, uint32_t lane_offset, uint32_t scalar_offset) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(lane_offset), "s"(rsrc), "s"(scalar_offset) : "memory");
}

// s_waitcnt immediate (gfx9 encoding): at most `vm` vector-memory and `lgkm`
// LDS/scalar operations outstanding; vmcnt[3:0] in bits 3:0 and vmcnt[5:4] in bits
// 15:14, lgkmcnt in bits 11:8, the export counter left at its maximum.
constexpr int kVmMax = 63, kLgkmMax = 15;
constexpr int waitcnt_imm(int vm, int lgkm) {
    return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | ((lgkm & 0xF) << 8);
}

// Workgroup barrier that orders LDS traffic only: waits for this wave's LDS
// operations, not for its outstanding global loads (__syncthreads() waits for
// both, which would drain a software pipeline of loads at every barrier).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

}  // namespace prism
