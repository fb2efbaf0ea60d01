// Matrix-core (MFMA) helpers for gfx950 and the packed weight layout.
//
// v_mfma_f32_16x16x32_bf16, D[16x16] += A[16x32] * B[32x16], one wave:
//   A[i][k] is held by lane i + 16*(k/8) as element k%8   (8 bf16 = 16 bytes per lane)
//   B[k][j] is held by lane j + 16*(k/8) as element k%8
//   D[i][j] is held by lane j + 16*(i/4) as element i%4   (4 floats per lane)
//
// Packed weights ("P16"): W[N][K] (bf16, row-major [out, in]) is cut into tiles of 16 rows by
// 32 columns; a tile is stored as the 64 lanes' A operands one after another (1 KB), the tiles
// of one k-step (all row blocks) follow each other:
//   packed[(w_tile(nb, kb) * 64 + lane) * 8 + e] = W[16*nb + lane%16][32*kb + 8*(lane/16) + e]
// with NB = ceil(N/16), KB = ceil(K/32) and zeros outside the matrix.  A wave reads a tile with
// one fully coalesced 16-byte load per lane, straight into the registers the MFMA wants.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// Place of tile (row block nb, k-step kb) in a packed matrix of NB row blocks and KB k-steps.
// k-step by k-step: workgroups that each stream their own row blocks then read neighbouring
// kilobytes at any moment, as a plain streaming read does, instead of NB regions far apart.
__host__ __device__ __forceinline__ size_t w_tile(long nb, long kb, long NB, long KB) {
    (void)KB;
    return (size_t)(kb * NB + nb);
}

union frag16 {            // 16 bytes: one lane's share of an MFMA operand
    uint4 u;
    u32x4_t r;
    bf16x8_t v;
    bf16 h[8];
};

__device__ __forceinline__ f32x4_t mfma_16x16x32(const frag16& a, const frag16& b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
}

// v_mfma_f32_32x32x16_bf16, D[32x32] += A[32x16] * B[16x32]:
//   A[i][k] is held by lane i + 32*(k/8) as element k%8;  B[k][j] by lane j + 32*(k/8) as element k%8
//   D[i][j] is held by lane j + 32*((i/4)%2) as element 4*(i/8) + i%4   (16 floats per lane)
typedef float f32x16_t __attribute__((ext_vector_type(16)));
__device__ __forceinline__ f32x16_t mfma_32x32x16(const frag16& a, const frag16& b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}

// A loop whose index is a compile-time constant in the body (f gets IntC<I>): for instructions' immediate fields.
template <int I> struct IntC { static constexpr int value = I; };
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(IntC<I>{});
        static_for<I + 1, N>(f);
    }
}

// An LDS read written as an instruction, for kernels that also load straight into LDS: the compiler
// counts such a load as an LDS access of unknown order and then waits for every pending LDS read
// where one is used, the ones just asked for included; or it keeps so few reads in flight that
// every multiplication waits out the LDS's latency.  The caller places the wait: lds_settle after
// the reads, then lds_use on each value before its first use.
template <int OFFSET> __device__ __forceinline__ void lds_read16(frag16& dst, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst.r) : "v"(addr), "n"(OFFSET));
}
__device__ __forceinline__ void lds_settle() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// Until at most N of the wave's LDS reads are outstanding (they come back in the order they were
// asked for, so the N youngest stay in flight; N up to 15).
template <int N> __device__ __forceinline__ void lds_settle_to() {
    static_assert(N >= 0 && N <= 15, "the counter holds four bits");
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void lds_use(frag16& v) { asm volatile("" : "+v"(v.r)); }
