// Two probes of what the machine delivers, for the measurement's "peaks_measured": a streaming
// read of memory far larger than every cache, and a loop of matrix-core instructions on
// operands of normally distributed values (the matrix cores' clock gives way to the power limit
// on such data, so this lies below the published peak, which holds for zeros).  Neither is
// part of the model's path.
#include "common_impl.h"
#include "mfma.h"

// Each workgroup reads tiles b, b + grid, ...; a tile is 256 threads x U loads of 16 bytes, all
// of them asked for before any is used.
template <int U>
__global__ __launch_bounds__(256) void peak_read_kernel(const uint4* __restrict__ p, size_t n_vec, unsigned* sink) {
    const size_t tile = (size_t)256 * U;
    unsigned acc = 0;
    for (size_t t = blockIdx.x; t * tile + tile <= n_vec; t += gridDim.x) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = p[t * tile + (size_t)u * 256 + threadIdx.x];
#pragma unroll
        for (int u = 0; u < U; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345678u) sink[0] = acc;        // (keeps the loads alive; practically never true)
}

extern "C" int agave_peak_read(const void* buf, long bytes, void* sink, int workgroups, hipStream_t stream) {
    AGAVE_CHECK(buf && sink && bytes >= (long)256 * 4 * 16 && workgroups > 0 && workgroups <= 65536,
                "peak_read: needs a buffer of at least 16 KiB and 1..65536 workgroups");
    peak_read_kernel<4><<<workgroups, 256, 0, stream>>>((const uint4*)buf, (size_t)bytes / 16, (unsigned*)sink);
    AGAVE_LAUNCH_CHECK("peak_read");
    return 0;
}

// 512 threads a workgroup (two waves a SIMD), eight independent 32x32 accumulators a wave.
typedef float peak_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 peak_bf16x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(512) void peak_mfma_kernel(const uint4* __restrict__ src, float* __restrict__ out, int iters) {
    union Operand { uint4 u; peak_bf16x8 v; };
    Operand a[4], b[2];
    for (int i = 0; i < 4; ++i) a[i].u = src[i * 512 + threadIdx.x];
    for (int i = 0; i < 2; ++i) b[i].u = src[(4 + i) * 512 + threadIdx.x];
    peak_f32x16 acc[8];
    for (int i = 0; i < 8; ++i)
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc[j * 4 + i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i].v, b[j].v, acc[j * 4 + i], 0, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][15];
    out[(size_t)blockIdx.x * 512 + threadIdx.x] = s;
}

// src: 6 * 512 operands of 16 bytes (bfloat16 values); out: workgroups * 512 floats.
// Multiply-adds done: workgroups * 8 waves * iters * 8 instructions * 32 * 32 * 16.
extern "C" int agave_peak_mfma(const void* src, void* out, int workgroups, int iters, hipStream_t stream) {
    AGAVE_CHECK(src && out && workgroups > 0 && workgroups <= 65536 && iters > 0, "peak_mfma: bad arguments");
    peak_mfma_kernel<<<workgroups, 512, 0, stream>>>((const uint4*)src, (float*)out, iters);
    AGAVE_LAUNCH_CHECK("peak_mfma");
    return 0;
}
