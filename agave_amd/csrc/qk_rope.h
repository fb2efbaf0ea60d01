// Per-head RMSNorm and rotation of one q or k head by one wave, and the place of a cache row in
// a page that is kept in the matrix cores' tile order.  Shared by the q/k kernel and by the
// decode attention kernel that does this work itself, so that both leave the same bits.
#pragma once
#include "common.h"

#define QK_ROPE_HD_MAX 512
__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return bf16_to_f32(v); }

// What one wave holds of a head's row between asking memory for it and using it: lane l has the
// elements l, l + 64, ... (as they are stored) with their gains, and the frequencies of the pairs
// l, l + 64, ...  NV: groups of 64 elements that the head size needs.
template <typename T, int NV>
struct QkRow {
    T xr[NV];
    float gv[NV], fv[(NV + 1) / 2];
};

// Requests the row, the gains and the frequencies; nothing is waited for here, so a kernel can
// call this first and let the loads travel while it finds out the position.  No load stands
// under a per-lane condition and no loaded value is touched (a conversion would wait for it):
// a lane past the end reads element 0, which nothing uses.  src must be readable for hd elements
// also in a wave that has no work.
template <typename T, int NV>
__device__ __forceinline__ QkRow<T, NV> qk_row_load(const T* src, const float* __restrict__ gain,
                                                    const float* __restrict__ inv_freq, int rot_half, int hd, int lane) {
    QkRow<T, NV> r;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int d = lane + 64 * k;
        r.xr[k] = src[d < hd ? d : 0];
    }
    if (gain) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int d = lane + 64 * k;
            r.gv[k] = gain[d < hd ? d : 0];
        }
    } else {
#pragma unroll
        for (int k = 0; k < NV; ++k) r.gv[k] = 1.f;
    }
    if (rot_half > 0) {
#pragma unroll
        for (int k = 0; k < (NV + 1) / 2; ++k) {
            const int i = lane + 64 * k;
            r.fv[k] = inv_freq[i < rot_half ? i : 0];
        }
    } else {
#pragma unroll
        for (int k = 0; k < (NV + 1) / 2; ++k) r.fv[k] = 0.f;
    }
    return r;
}

// Between a wave's writes to its own part of LDS and its reads of what other lanes wrote there.
// The LDS serves a wave's accesses in order, so no instruction is needed; the compiler must keep
// the order too.
__device__ __forceinline__ void wave_lds_order() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// y[0..hd) (LDS, 32-bit) <- rotate(row * rsqrt(mean(row^2) + eps) * gain) for the row that qk_row_load
// fetched.  has_gain false: no norm; rot_half 0: no rotation.  pf: position times the position
// scale.  y is the calling wave's own; a wave without work passes active = false.
template <typename T, int NV>
__device__ __forceinline__ void qk_row_finish(const QkRow<T, NV>& r, float* y, bool has_gain, float eps, int rot_half,
                                              float pf, int hd, int lane, bool active) {
    float xv[NV];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        xv[k] = to_f32(r.xr[k]);
        ss += (lane + 64 * k < hd) ? xv[k] * xv[k] : 0.f;
    }
    float inv = 1.0f;
    if (active && has_gain) {
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)hd + eps);
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int d = lane + 64 * k;
        if (active && d < hd) y[d] = has_gain ? xv[k] * inv * r.gv[k] : xv[k];
    }
    wave_lds_order();
    // rotation, in place in LDS: y[i], y[i + rot_half] <- rotated pair
#pragma unroll
    for (int k = 0; k < (NV + 1) / 2; ++k) {
        const int i = lane + 64 * k;
        if (active && i < rot_half) {
            const float a = y[i], b2 = y[i + rot_half];
            float s, c;
            sincosf(pf * r.fv[k], &s, &c);
            y[i] = a * c - b2 * s;
            y[i + rot_half] = a * s + b2 * c;
        }
    }
    wave_lds_order();
}

// One wave writes a key row y[0..hd) (LDS) and a value row (in registers: vreg[k] is element
// lane + 64 k) to row `row` of a page in tile
// order: dk, dv are the page's K and V blocks of this kv head.
//   K: tiles [row / 16][d / 32] of 64 lanes x 8: lane (row % 16) + 16 * ((d % 32) / 8), element d % 8
//   V: tiles [d / 16][row / 32] of 64 lanes x 8: lane (d % 16) + 16 * vg, element ve, with the 32 keys
//      of a half page in the order the score accumulators have them
template <typename T, int NV>
__device__ __forceinline__ void store_kv_row_packed_regs(T* dk, T* dv, const float* y, const T (&vreg)[NV], int row,
                                                         int hd, int lane) {
    const int ks_n = (hd + 31) >> 5;
    const int kt = row >> 4, ki = row & 15;
    const int s2 = row >> 5, r32 = row & 31;
    const int vg = (r32 & 15) >> 2, ve = (r32 & 3) + ((r32 >> 4) << 2);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int d = lane + 64 * k;
        if (d < hd) {
            const int ks = d >> 5, g = (d & 31) >> 3, e = d & 7;
            st(dk + ((size_t)(kt * ks_n + ks) * 64 + ki + 16 * g) * 8 + e, y[d]);
            const int dt = d >> 4, j = d & 15;
            dv[((size_t)(dt * 2 + s2) * 64 + j + 16 * vg) * 8 + ve] = vreg[k];
        }
    }
}
