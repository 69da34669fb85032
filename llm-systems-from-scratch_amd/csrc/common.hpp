// Shared device helpers for the gfx950 (CDNA4) attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define MI355_LDS __attribute__((address_space(3)))

constexpr float kLog2e = 1.4426950408889634f;

// ---- MFMA wrappers -------------------------------------------------------
// 16x16x32 bf16:  A lane l -> row l%16, k = 8*(l/16)+j ; B lane l -> col l%16, k = 8*(l/16)+j
//                 C lane l -> col l%16, rows 4*(l/16)+i (i = 0..3)
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// 32x32x16 bf16:  A lane l -> row l%32, k = 8*(l/32)+j ; B lane l -> col l%32, k = 8*(l/32)+j
//                 C lane l -> col l%32, rows 8*(i/4) + 4*(l/32) + i%4 (i = 0..15)
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// ---- LDS transpose read ----------------------------------------------------
// ds_read_b64_tr_b16: inside each group of 16 lanes, source lane s supplies the
// address of 4 consecutive 16-bit elements; result lane i, element j is element
// (i % 4) of source lane (4*j + i/4).  With source lane s pointing at
// (row r0 + s/4, column c0 + 4*(s%4)) of a row-major tile, lane i receives column
// c0 + i of rows r0 .. r0+3: a 4x16 block read "down the columns".
__device__ __forceinline__ i16x4 lds_read_tr16(const void* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((MI355_LDS i16x4*)p);
}

// Reads through an absolute LDS byte address (what lds_address() returns), for code that shares precomputed
// addresses with hand-written assembly.
template <class T>
__device__ __forceinline__ T lds_load_at(uint32_t addr) {
    return *reinterpret_cast<const MI355_LDS T*>((size_t)addr);
}
__device__ __forceinline__ i16x4 lds_read_tr16_at(uint32_t addr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<MI355_LDS i16x4*>((size_t)addr));
}

__device__ __forceinline__ bf16x8 join_bf16x8(i16x4 lo, i16x4 hi) {
    struct { i16x4 a, b; } t{lo, hi};
    return __builtin_bit_cast(bf16x8, t);
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// two fp32 -> packed bf16 (round to nearest even), low half = a
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    bf16x2 t;
    t[0] = (__bf16)a;
    t[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, t);
}

// 4 fp8-e4m3 (OCP) bytes -> 4 bf16 (exact: e4m3 is a subset of bf16)
__device__ __forceinline__ u32x2 fp8x4_to_bf16x4(uint32_t w) {
    bf16x2 lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
    bf16x2 hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
    u32x2 r;
    r[0] = __builtin_bit_cast(uint32_t, lo);
    r[1] = __builtin_bit_cast(uint32_t, hi);
    return r;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max / sum across the 4 lanes {l, l^16, l^32, l^48}
__device__ __forceinline__ float xor_max_16_32(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
__device__ __forceinline__ float xor_sum_16_32(float v) {
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// Exchange with lane l^32 through v_permlane32_swap.  The instruction swaps the
// upper half of its first operand with the lower half of its second, so feeding
// the same value twice yields {[lo,lo],[hi,hi]}: every lane sees both halves.
// (The two results are copied to scalars before the bit cast: a bit cast applied
// directly to a vector element expression reads element 0 for every index.)
__device__ __forceinline__ void swap32(float v, float& from_lo, float& from_hi) {
    const uint32_t a = __builtin_bit_cast(uint32_t, v);
    auto r = __builtin_amdgcn_permlane32_swap(a, a, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    from_lo = __builtin_bit_cast(float, r0);
    from_hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float xor32_max(float v) {
    float a, b;
    swap32(v, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float xor32_sum(float v) {
    float a, b;
    swap32(v, a, b);
    return a + b;
}

// ---- direct global -> LDS loads ---------------------------------------------
// global_load_lds_dwordx4: every lane supplies its own 16-byte global address; the
// wavefront's 64 x 16 bytes land at lds_base + 16*lane (lds_base is wave-uniform, passed in m0).
// Issued through the compiler's builtin, every later LDS read of the wavefront is treated as a
// possible reader of the landing data and gets `s_waitcnt vmcnt(0)` in front of it, which
// exposes the whole memory latency.  dma_to_lds_16 issues the instruction from inline
// assembly instead: the compiler then places no wait for it at all, and every consumer must
// be preceded by wait_vmcnt<N>() (N = number of younger vector-memory instructions of this
// wavefront allowed to stay in flight) and, across wavefronts, by a barrier.
// gbase: wave-uniform global base address; voff: this lane's byte offset from it (unsigned,
// < 2^32); lds_addr: wave-uniform LDS byte address the wavefront's 1 KiB lands at.
// The LDS address travels in m0 as a declared register operand: the compiler writes m0 itself and knows
// that this statement reads it, so its own uses of m0 elsewhere in a kernel stay correct.  The leading
// s_nop 4 covers two wait-state rules that the compiler cannot apply to an instruction it does not see: one
// state between a write of m0 and an LDS-DMA instruction, and FIVE between a vector instruction that writes a
// scalar register and a vector-memory instruction that reads it as its address -- which is what happens when
// the compiler keeps `gbase` in a spilled scalar register and restores it (v_readlane) directly in front of the
// statement.  (With one state only, a kernel variant with scalar spills fetched from a stale base address.)
__device__ __forceinline__ void dma_to_lds_16(const void* gbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_nop 4\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(gbase), "{m0}"(lds_addr)
                 : "memory");
}
// Logical id of workgroup `bid` of a one-dimensional grid whose ids come in chunks of `chunk` that read the same
// tensor rows (e.g. the query tiles and query heads of one K/V head).  Workgroup ids are dealt round-robin to the 8
// XCDs, each with an L2 of its own; the XCDs take whole chunks in turn, so the workgroups of a chunk are resident on
// one XCD at about the same time, and what one sequence brings is spread over all XCDs however long it is.
// (Ids past the last whole round of eight chunks stay as they are.)
__device__ __forceinline__ int xcd_chunked_id(int bid, int n_wg, int chunk) {
    const int whole = n_wg / (8 * chunk) * (8 * chunk);
    const int xcd = bid % 8, k = bid / 8, turn = k / chunk;
    const int id = (turn * 8 + xcd) * chunk + (k - turn * chunk);
    // (the compiler divides on the vector unit; the result is the same in every lane)
    return __builtin_amdgcn_readfirstlane(bid >= whole ? bid : id);
}

__device__ __forceinline__ uint32_t lds_address(const void* lds_ptr) {
    return (uint32_t)(uintptr_t)(const MI355_LDS void*)lds_ptr;
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

}  // namespace mi355
