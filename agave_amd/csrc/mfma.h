// Matrix-core (MFMA) helpers for gfx950 and the packed weight layout.
//
// v_mfma_f32_16x16x32_bf16, D[16x16] += A[16x32] * B[32x16], one wave:
//   A[i][k] is held by lane i + 16*(k/8) as element k%8   (8 bf16 = 16 bytes per lane)
//   B[k][j] is held by lane j + 16*(k/8) as element k%8
//   D[i][j] is held by lane j + 16*(i/4) as element i%4   (4 floats per lane)
//
// Packed weights ("P16"): W[N][K] (bf16, row-major [out, in]) is cut into tiles of 16 rows by
// 32 columns; a tile is stored as the 64 lanes' A operands one after another (1 KB), tiles of
// one row block follow each other along K:
//   packed[((nb * KB + kb) * 64 + lane) * 8 + e] = W[16*nb + lane%16][32*kb + 8*(lane/16) + e]
// with NB = ceil(N/16), KB = ceil(K/32) and zeros outside the matrix.  A wave reads a tile with
// one fully coalesced 16-byte load per lane, straight into the registers the MFMA wants.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

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
