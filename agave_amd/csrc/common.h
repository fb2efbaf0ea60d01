// Shared device helpers for the gfx950 kernels: element types, wave64 reductions,
// error reporting to the host.  Everything is compiled for MI355X only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define AGAVE_WAVE 64
#define AGAVE_PAGE 64          // positions per cache page

// dtype codes shared with the Python side
#define AGAVE_F32 0
#define AGAVE_BF16 1

// ---------------------------------------------------------------- error reporting
// Every entry point returns 0 or a negative code and leaves a message here.
extern "C" const char* agave_last_error();
void agave_set_error(const char* fmt, ...);

#define AGAVE_CHECK(cond, ...)                      \
    do {                                            \
        if (!(cond)) {                              \
            agave_set_error(__VA_ARGS__);           \
            return -1;                              \
        }                                           \
    } while (0)

#define AGAVE_LAUNCH_CHECK(name)                                                   \
    do {                                                                           \
        hipError_t e__ = hipGetLastError();                                        \
        if (e__ != hipSuccess) {                                                   \
            agave_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
            return -2;                                                             \
        }                                                                          \
    } while (0)

// ---------------------------------------------------------------- bfloat16
struct bf16 {
    uint16_t x;
};

__host__ __device__ __forceinline__ float bf16_to_f32(bf16 v) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)v.x) << 16;
    return c.f;
}

// round to nearest, ties to even; NaN stays NaN.  On the device this is one instruction for two
// values (v_cvt_pk_bf16_f32); in software it takes half a dozen, which a product's last step, with
// 128 values a lane, has no time for.
__host__ __device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __bf16 hw_bf16x2 __attribute__((ext_vector_type(2)));
    typedef float hw_f32x2 __attribute__((ext_vector_type(2)));
    const hw_f32x2 v = {lo, hi};
    const hw_bf16x2 r = __builtin_convertvector(v, hw_bf16x2);
    return __builtin_bit_cast(uint32_t, r);
#else
    uint32_t out = 0;
    const float in[2] = {lo, hi};
    for (int i = 0; i < 2; ++i) {
        union { uint32_t u; float f; } c;
        c.f = in[i];
        uint32_t h;
        if ((c.u & 0x7fffffffu) > 0x7f800000u) {
            h = 0x7fc0;
        } else {
            c.u += 0x7fffu + ((c.u >> 16) & 1u);
            h = c.u >> 16;
        }
        out |= h << (16 * i);
    }
    return out;
#endif
}
__host__ __device__ __forceinline__ bf16 f32_to_bf16(float f) {
    bf16 r;
    r.x = (uint16_t)(f32x2_to_bf16x2(f, 0.f) & 0xffffu);
    return r;
}

template <typename T> __device__ __forceinline__ float ld(const T* p);
template <> __device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld<bf16>(const bf16* p) { return bf16_to_f32(*p); }

template <typename T> __device__ __forceinline__ void st(T* p, float v);
template <> __device__ __forceinline__ void st<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st<bf16>(bf16* p, float v) { *p = f32_to_bf16(v); }

// ---------------------------------------------------------------- wave64 reductions
// With the lanes' cross-lane operand modes (DPP): six vector instructions and a read of lane 63,
// where a shuffle is an LDS instruction with its latency each time (six to a reduction).
//   quad_perm, row_half_mirror, row_mirror: every lane gets its row's (16 lanes') result;
//   row_bcast15 to rows 1 and 3, row_bcast31 to rows 2 and 3: lane 63 gets the wave's.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_get(float keep, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, keep), __builtin_bit_cast(int, v),
                                                                 CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_get<0xB1, 0xF>(0.f, v);          // quad_perm [1,0,3,2]
    v += dpp_get<0x4E, 0xF>(0.f, v);          // quad_perm [2,3,0,1]
    v += dpp_get<0x141, 0xF>(0.f, v);         // row_half_mirror
    v += dpp_get<0x140, 0xF>(0.f, v);         // row_mirror
    v += dpp_get<0x142, 0xA>(0.f, v);         // row_bcast15
    v += dpp_get<0x143, 0xC>(0.f, v);         // row_bcast31
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_get<0xB1, 0xF>(v, v));
    v = fmaxf(v, dpp_get<0x4E, 0xF>(v, v));
    v = fmaxf(v, dpp_get<0x141, 0xF>(v, v));
    v = fmaxf(v, dpp_get<0x140, 0xF>(v, v));
    v = fmaxf(v, dpp_get<0x142, 0xA>(v, v));
    v = fmaxf(v, dpp_get<0x143, 0xC>(v, v));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Block-wide reductions for blocks of up to 1024 threads; `red` is 16 floats of LDS.
// Every thread gets the result.  Contains barriers: call from all threads.
__device__ __forceinline__ float block_sum(float v, float* red) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; ++i) r += red[i];
    return r;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < nw; ++i) r = fmaxf(r, red[i]);
    return r;
}
