// Sampling over 32-bit logits for gfx950: argmax, temperature / top-k / top-p draws, and the
// repeat penalty.  One workgroup of 1024 threads per row; every sum is taken in a fixed
// order, so a row's result depends only on the row and its parameters.
//
// Reference: src/ops/math.zig:32-50 (argmax, first index on ties), :186-197 (repeat penalty),
// :209-372 (sampleToken): logits * 1/T; top-k keeps values >= the k-th largest (k capped at
// 1024, ties kept); weights exp(x - max), unnormalised; top-p sorts the (at most 1024) largest
// weights, finds the smallest prefix whose mass reaches p * sum and keeps every weight >= the
// last one taken; the draw is the first index whose running sum exceeds u * sum.
#include "common_impl.h"
#include <math.h>

#define SAMPLE_THREADS 1024
#define MAX_CAND 1024

__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// k-th largest (k >= 1, k <= n) of f(i) = x[i] * mult, as an ordered key.  All threads call.
__device__ uint32_t kth_largest_key(const float* __restrict__ x, int n, float mult, int k, uint32_t* hist,
                                    uint32_t* sh) {
    uint32_t prefix = 0, mask = 0;
    uint32_t krem = (uint32_t)k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const uint32_t key = ordered_key(x[i] * mult);
            if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t cum = 0;
            int digit = 0;
            for (int d = 255; d >= 0; --d) {
                if (cum + hist[d] >= krem) {
                    digit = d;
                    break;
                }
                cum += hist[d];
            }
            sh[0] = prefix | ((uint32_t)digit << shift);
            sh[1] = krem - cum;
        }
        __syncthreads();
        prefix = sh[0];
        krem = sh[1];
        mask |= 255u << shift;
        __syncthreads();
    }
    return prefix;
}

// (max value, lowest index holding it) over a row.  All threads call; all get the result.
__device__ void block_argmax(const float* __restrict__ x, int n, float mult, float* red_v, int* red_i, float* out_v,
                             int* out_i) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i] * mult;
        if (idx == 0x7fffffff || v > best) {      // a thread meets its indices in rising order
            best = v;
            idx = i;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(idx, o, 64);
        if (ov > best || (ov == best && oi < idx)) {
            best = ov;
            idx = oi;
        }
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) {
        red_v[w] = best;
        red_i[w] = idx;
    }
    __syncthreads();
    best = red_v[0];
    idx = red_i[0];
    for (int i = 1; i < nw; ++i)
        if (red_v[i] > best || (red_v[i] == best && red_i[i] < idx)) {
            best = red_v[i];
            idx = red_i[i];
        }
    *out_v = best;
    *out_i = idx;
}

// Greedy rows, first pass: the row is cut into ARGMAX_PARTS pieces, one workgroup each, which
// leave (max, lowest index holding it); sample_kernel picks among them.
#define ARGMAX_PARTS 64
__global__ __launch_bounds__(256) void argmax_parts_kernel(const float* __restrict__ logits, long ld,
                                                           const float* __restrict__ params,
                                                           float* __restrict__ part_v, int* __restrict__ part_i, int V) {
    __shared__ float red_v[16];
    __shared__ int red_i[16];
    const int b = blockIdx.y, part = blockIdx.x;
    if (params[b * 4] != 0.f) return;                       // only rows that take the argmax
    const int per = (V + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
    const int lo = part * per;
    int n = V - lo;
    if (n > per) n = per;
    float mx = -INFINITY;
    int idx = 0;
    if (n > 0) {
        block_argmax(logits + (size_t)b * ld + lo, n, 1.0f, red_v, red_i, &mx, &idx);
        idx += lo;
    } else {
        idx = 0x7fffffff;
    }
    if (threadIdx.x == 0) {
        part_v[b * ARGMAX_PARTS + part] = mx;
        part_i[b * ARGMAX_PARTS + part] = idx;
    }
}

// params[b] = {temperature, top_k, top_p, u}
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits, long ld,
                                                                float* __restrict__ work, long ldw,
                                                                const float* __restrict__ params,
                                                                int* __restrict__ out, int V,
                                                                const float* __restrict__ part_v,
                                                                const int* __restrict__ part_i) {
    __shared__ float red[16];
    __shared__ float red_v[16];
    __shared__ int red_i[16];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t sh[2];
    __shared__ float cand[MAX_CAND];
    __shared__ uint32_t n_cand;
    __shared__ float sh_thr;
    __shared__ float incl[SAMPLE_THREADS];
    __shared__ int sh_result;

    const int b = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + (size_t)b * ld;
    float* w = work + (size_t)b * ldw;
    const float temperature = params[b * 4 + 0];
    const int top_k = (int)params[b * 4 + 1];
    const float top_p = params[b * 4 + 2];
    const float u = params[b * 4 + 3];

    float mx;
    int amax;
    if (temperature == 0.f) {
        if (part_v) {                                         // the pieces' winners; ties go to the lowest index
            if (tid < 64) {
                float v = part_v[b * ARGMAX_PARTS + tid];
                int i = part_i[b * ARGMAX_PARTS + tid];
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) {
                    const float ov = __shfl_xor(v, o, 64);
                    const int oi = __shfl_xor(i, o, 64);
                    if (ov > v || (ov == v && oi < i)) {
                        v = ov;
                        i = oi;
                    }
                }
                if (tid == 0) out[b] = i;
            }
            return;
        }
        block_argmax(x, V, 1.0f, red_v, red_i, &mx, &amax);
        if (tid == 0) out[b] = amax;
        return;
    }
    const float inv_t = 1.0f / temperature;

    // top-k: values below the k-th largest are dropped
    float kth = -INFINITY;
    if (top_k > 0 && top_k < V) {
        const int k = top_k < MAX_CAND ? top_k : MAX_CAND;
        kth = key_to_float(kth_largest_key(x, V, inv_t, k, hist, sh));
    }
    block_argmax(x, V, inv_t, red_v, red_i, &mx, &amax);

    // weights and their sum
    float part = 0.f;
    int npos = 0;
    for (int i = tid; i < V; i += blockDim.x) {
        const float v = x[i] * inv_t;
        const float e = (v < kth || v == -INFINITY) ? 0.f : expf(v - mx);
        w[i] = e;
        part += e;
        npos += e > 0.f;
    }
    float sum = block_sum(part, red);
    const int total_pos = (int)(block_sum((float)npos, red) + 0.5f);

    if (top_p < 1.0f && top_p > 0.0f) {
        // the (at most 1024) largest weights, sorted, and the threshold their prefix gives
        uint32_t min_key = 0;
        if (total_pos > MAX_CAND) min_key = kth_largest_key(w, V, 1.0f, MAX_CAND, hist, sh);
        if (tid == 0) n_cand = 0;
        for (int i = tid; i < MAX_CAND; i += blockDim.x) cand[i] = 0.f;
        __syncthreads();
        for (int i = tid; i < V; i += blockDim.x) {
            const float e = w[i];
            if (e > 0.f && ordered_key(e) >= min_key) {
                const uint32_t at = atomicAdd(&n_cand, 1u);
                if (at < MAX_CAND) cand[at] = e;
            }
        }
        __syncthreads();
        // bitonic sort, descending
        for (int size = 2; size <= MAX_CAND; size <<= 1)
            for (int stride = size >> 1; stride > 0; stride >>= 1) {
                const int i = tid;
                const int j = i ^ stride;
                if (i < MAX_CAND && j > i) {
                    const bool desc = (i & size) == 0;
                    const float a = cand[i], c = cand[j];
                    if (desc ? (a < c) : (a > c)) {
                        cand[i] = c;
                        cand[j] = a;
                    }
                }
                __syncthreads();
            }
        if (tid == 0) {
            float cum = 0.f, thr = 0.f;
            const float goal = top_p * sum;
            for (int i = 0; i < MAX_CAND; ++i) {
                const float v = cand[i];
                if (v <= 0.f) break;
                cum += v;
                if (cum >= goal) {
                    thr = v;
                    break;
                }
            }
            sh_thr = thr;
        }
        __syncthreads();
        const float thr = sh_thr;
        part = 0.f;
        for (int i = tid; i < V; i += blockDim.x) {
            float e = w[i];
            if (e < thr) {
                e = 0.f;
                w[i] = 0.f;
            }
            part += e;
        }
        sum = block_sum(part, red);
    }

    // the draw: first index whose running sum exceeds u * sum; contiguous segments per thread
    const int seg = (V + blockDim.x - 1) / blockDim.x;
    const int lo = tid * seg, hi = (lo + seg < V) ? lo + seg : V;
    __syncthreads();     // w[] written by other threads above
    float s = 0.f;
    for (int i = lo; i < hi; ++i) s += w[i];
    incl[tid] = s;
    if (tid == 0) sh_result = V - 1;
    __syncthreads();
    if (tid == 0) {
        float c = 0.f;
        for (int t = 0; t < (int)blockDim.x; ++t) {
            c += incl[t];
            incl[t] = c;
        }
    }
    __syncthreads();
    const float target = u * incl[blockDim.x - 1];
    const float before = tid == 0 ? 0.f : incl[tid - 1];
    if (lo < hi && target < incl[tid] && target >= before) {
        float c = before;
        int pick = hi - 1;
        for (int i = lo; i < hi; ++i) {
            c += w[i];
            if (target < c) {
                pick = i;
                break;
            }
        }
        sh_result = pick;     // exactly one thread's interval holds the target
    }
    __syncthreads();
    if (tid == 0) out[b] = sh_result;
}

// scratch: B * 64 floats followed by B * 64 ints for the greedy rows' first pass, or null.
extern "C" int agave_sample(const float* logits, long ld, float* work, long ldw, const float* params, int* out,
                            int B, int V, float* scratch, hipStream_t stream) {
    AGAVE_CHECK(B >= 0 && V > 0, "sample: bad sizes B=%d V=%d", B, V);
    AGAVE_CHECK(ld >= V && ldw >= V, "sample: a row stride is below the vocabulary");
    AGAVE_CHECK(logits && work && params && out, "sample: null buffer");
    if (B == 0) return 0;
    float* part_v = nullptr;
    int* part_i = nullptr;
    if (scratch && V >= 4096 && B <= 65535) {
        part_v = scratch;
        part_i = reinterpret_cast<int*>(scratch + (size_t)B * ARGMAX_PARTS);
        argmax_parts_kernel<<<dim3(ARGMAX_PARTS, B), 256, 0, stream>>>(logits, ld, params, part_v, part_i, V);
        AGAVE_LAUNCH_CHECK("argmax_parts");
    }
    sample_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, ld, work, ldw, params, out, V, part_v, part_i);
    AGAVE_LAUNCH_CHECK("sample");
    return 0;
}

// ------------------------------------------------------------------ repeat penalty
// For every id a row has generated so far, once per occurrence: a positive logit is divided by
// the penalty, another multiplied.  c occurrences are applied as penalty^c.
__global__ void repeat_penalty_kernel(float* __restrict__ logits, long ld, const int* __restrict__ ids,
                                      const int* __restrict__ cu, const float* __restrict__ penalty, int V) {
    const int b = blockIdx.x;
    const float r = penalty[b];
    if (r == 1.0f) return;
    const int lo = cu[b], hi = cu[b + 1];
    float* x = logits + (size_t)b * ld;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const int id = ids[i];
        if (id < 0 || id >= V) continue;
        bool first = true;
        int count = 0;
        for (int j = lo; j < hi; ++j) {
            if (ids[j] == id) {
                if (j < i) {
                    first = false;
                    break;
                }
                ++count;
            }
        }
        if (!first) continue;
        const float f = powf(r, (float)count);
        const float v = x[id];
        x[id] = v > 0.f ? v / f : v * f;
    }
}

extern "C" int agave_repeat_penalty(float* logits, long ld, const int* ids, const int* cu, const float* penalty,
                                    int B, int V, hipStream_t stream) {
    AGAVE_CHECK(B >= 0 && V > 0 && ld >= V, "repeat_penalty: bad sizes B=%d V=%d ld=%ld", B, V, ld);
    AGAVE_CHECK(logits && ids && cu && penalty, "repeat_penalty: null buffer");
    if (B == 0) return 0;
    repeat_penalty_kernel<<<B, 256, 0, stream>>>(logits, ld, ids, cu, penalty, V);
    AGAVE_LAUNCH_CHECK("repeat_penalty");
    return 0;
}


// ------------------------------------------------------------------ sampled tokens feed the next step
// dst[i] = src[map[i]]: the tokens a step sampled become the next step's input on the device, so
// that the host can launch that step before it has read them.
__global__ void gather_tokens_kernel(const int* __restrict__ src, const int* __restrict__ map, int* __restrict__ dst,
                                     int n, int n_src) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int k = map[i];
    dst[i] = (k >= 0 && k < n_src) ? src[k] : 0;
}

extern "C" int agave_gather_tokens(const int* src, const int* map, int* dst, int n, int n_src, hipStream_t stream) {
    AGAVE_CHECK(n >= 0 && n_src >= 0 && (n == 0 || (src && map && dst)), "gather_tokens: bad sizes or null buffer");
    if (n == 0) return 0;
    gather_tokens_kernel<<<(n + 255) / 256, 256, 0, stream>>>(src, map, dst, n, n_src);
    AGAVE_LAUNCH_CHECK("gather_tokens");
    return 0;
}
