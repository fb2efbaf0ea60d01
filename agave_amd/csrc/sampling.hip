// Sampling over 32-bit logits for gfx950: argmax, temperature / top-k / top-p draws, and the
// repeat penalty.  Small vocabularies: one workgroup of 1024 threads per row; large ones: a row
// is shared among workgroups (see below).  Every sum is taken in a fixed order, so a row's
// result depends only on the row and its parameters.
//
// Reference: src/ops/math.zig:32-50 (argmax, first index on ties), :186-197 (repeat penalty),
// :209-372 (sampleToken): logits * 1/T; top-k keeps values >= the k-th largest (k capped at
// 1024, ties kept); weights exp(x - max), unnormalised; top-p sorts the (at most 1024) largest
// weights, finds the smallest prefix whose mass reaches p * sum and keeps every weight >= the
// last one taken; the draw is the first index whose running sum exceeds u * sum.
#include "common_impl.h"
#include <math.h>

// No multiplication in this file is fused with a following addition: the scaled logit x * 1/T is
// rounded by itself, so that it has the same bits in every kernel here.  Fused into the subtraction
// of the maximum it would differ in its last bit from place to place, and an entry whose weight has
// to equal a threshold that another kernel found (the largest weight, say) would fall below it.
#pragma clang fp contract(off)

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
    // eight loads a thread are asked for before the first is compared (a load and its comparison
    // in turn would be a round trip to memory each); an index past the end reads the last element
    constexpr int U = 8;
    for (int i0 = threadIdx.x; i0 < n; i0 += blockDim.x * U) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * blockDim.x;
            v[u] = x[i < n ? i : n - 1];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * blockDim.x;
            const float val = v[u] * mult;
            if (i < n && (idx == 0x7fffffff || val > best)) {      // a thread meets its indices in rising order
                best = val;
                idx = i;
            }
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

// ------------------------------------------------------------------ large vocabularies: a row shared among workgroups
// One workgroup reads a row of a quarter of a million logits no faster than one compute unit
// pulls data, and the draw needs several passes over the row.  So a row is cut into SP_PARTS
// pieces, one workgroup each, in a handful of small kernels: the pieces' maxima; the pieces'
// sums of weights (rows whose draw ranges over the whole row); for rows with top-k or top-p a
// radix selection of the value of the (at most 1024) largest entries in three rounds of
// histograms (11, 11 and 10 bits of the ordered key), and the collection of those entries; last,
// one workgroup per row decides.  With a filter the kept entries are among the collected ones,
// which are sorted by value (thresholds) and then by index (the draw).  Entries above the value
// of the 1024th largest are collected first and its equals behind them as far as there is room, so
// that a plateau of equal logits can only leave out its own kind; if it does, the thresholds are
// still exact and the draw walks the whole row with them.  Without a filter the piece that
// holds u * sum is found from the pieces' sums and only that piece is read again.
// Words of scratch per row:
#define SP_PARTS 64
#define SP_THREADS 256
#define SP_OFF_MAX 0                          // float[64]: the pieces' maxima
#define SP_OFF_IDX 64                         // int[64]: lowest index holding each
#define SP_OFF_SUM 128                        // float[64]: the pieces' sums of weights
#define SP_OFF_NCAND 192                      // uint: collected entries above the threshold value
#define SP_OFF_NTIE 193                       // uint: entries that equal it
#define SP_OFF_H0 256                         // uint[2048]: histogram of key bits 31..21
#define SP_OFF_H1 (SP_OFF_H0 + 2048)          // uint[2048]: bits 20..10 under the first digit
#define SP_OFF_H2 (SP_OFF_H1 + 2048)          // uint[1024]: bits 9..0 under the first two
#define SP_OFF_CV (SP_OFF_H2 + 1024)          // float[1024]: collected values (scaled logits)
#define SP_OFF_CI (SP_OFF_CV + MAX_CAND)      // int[1024]: their indices
#define SP_ROW_WORDS (SP_OFF_CI + MAX_CAND)
#define SP_HIST_WORDS (SP_OFF_CV - SP_OFF_H0)
static_assert(SP_HIST_WORDS % SP_PARTS == 0, "the pieces' workgroups clear equal shares of the histograms");

extern "C" int agave_sample_scratch_words() { return SP_ROW_WORDS; }

struct RowMode {
    float inv_t, top_p, u;
    int top_k, want;
    bool greedy, use_k, use_p, filt, whole_sum;
};
__device__ __forceinline__ RowMode row_mode(const float* __restrict__ params, int b, int V) {
    RowMode m;
    const float t = params[b * 4 + 0];
    m.top_k = (int)params[b * 4 + 1];
    m.top_p = params[b * 4 + 2];
    m.u = params[b * 4 + 3];
    m.greedy = t == 0.f;
    m.inv_t = m.greedy ? 1.0f : 1.0f / t;
    m.use_k = m.top_k > 0 && m.top_k < V;
    m.use_p = m.top_p < 1.0f && m.top_p > 0.0f;
    m.filt = !m.greedy && (m.use_k || m.use_p);
    m.want = m.use_k ? (m.top_k < MAX_CAND ? m.top_k : MAX_CAND) : MAX_CAND;   // entries to collect
    m.whole_sum = !m.greedy && !m.use_k;         // the sum of weights ranges over the whole row
    return m;
}
__device__ __forceinline__ void part_range(int V, int part, int* lo, int* n) {
    const int per = (V + SP_PARTS - 1) / SP_PARTS;
    *lo = part * per;
    int k = V - *lo;
    *n = k > per ? per : (k > 0 ? k : 0);
}
// the row's maximum from the pieces' (every wave computes it for itself)
__device__ __forceinline__ float sp_row_max(const float* __restrict__ rowf) {
    return wave_max(rowf[SP_OFF_MAX + (threadIdx.x & 63)]);
}

// The pieces' maxima, for every row; also clears what the later kernels add to.
__global__ __launch_bounds__(SP_THREADS) void sp_max_kernel(const float* __restrict__ logits, long ld,
                                                            float* __restrict__ scratch, int V, int clear) {
    __shared__ float red_v[16];
    __shared__ int red_i[16];
    const int b = blockIdx.y, part = blockIdx.x;
    float* rowf = scratch + (size_t)b * SP_ROW_WORDS;
    if (clear) {
        constexpr int SHARE = SP_HIST_WORDS / SP_PARTS;
        for (int i = threadIdx.x; i < SHARE; i += blockDim.x) reinterpret_cast<uint32_t*>(rowf)[SP_OFF_H0 + part * SHARE + i] = 0;
        if (part == 0 && threadIdx.x < 2) reinterpret_cast<uint32_t*>(rowf)[SP_OFF_NCAND + threadIdx.x] = 0;
    }
    int lo, n;
    part_range(V, part, &lo, &n);
    float mx = -INFINITY;
    int idx = 0x7fffffff;
    if (n > 0) {
        block_argmax(logits + (size_t)b * ld + lo, n, 1.0f, red_v, red_i, &mx, &idx);
        idx += lo;
    }
    if (threadIdx.x == 0) {
        rowf[SP_OFF_MAX + part] = mx;
        reinterpret_cast<int*>(rowf)[SP_OFF_IDX + part] = idx;
    }
}

// Calls f(i, x[i] * mult) for the piece's elements, a thread's in rising order, with eight loads
// asked for before the first is used.
template <typename F>
__device__ __forceinline__ void for_piece(const float* __restrict__ x, int n, float mult, F f) {
    constexpr int U = 8;
    for (int i0 = threadIdx.x; i0 < n; i0 += blockDim.x * U) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * blockDim.x;
            v[u] = x[i < n ? i : n - 1];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * blockDim.x;
            if (i < n) f(i, v[u] * mult);
        }
    }
}

__device__ __forceinline__ float weight_of(float v, float mx) { return v == -INFINITY ? 0.f : expf(v - mx); }

// The pieces' sums of exp(v - max), for rows whose sum ranges over the whole row.
__global__ __launch_bounds__(SP_THREADS) void sp_sum_kernel(const float* __restrict__ logits, long ld,
                                                            const float* __restrict__ params,
                                                            float* __restrict__ scratch, int V) {
    __shared__ float red[16];
    const int b = blockIdx.y, part = blockIdx.x;
    const RowMode m = row_mode(params, b, V);
    if (!m.whole_sum) return;
    float* rowf = scratch + (size_t)b * SP_ROW_WORDS;
    const float mx = sp_row_max(rowf) * m.inv_t;
    int lo, n;
    part_range(V, part, &lo, &n);
    float s = 0.f;
    for_piece(logits + (size_t)b * ld + lo, n, m.inv_t, [&](int, float v) { s += weight_of(v, mx); });
    s = block_sum(s, red);
    if (threadIdx.x == 0) rowf[SP_OFF_SUM + part] = s;
}

// From a histogram of `bins` digits (a multiple of 256 * 4; all threads of a 256-thread
// workgroup call): the digit that holds the krem-th largest entry, and how many of that digit's
// entries are still wanted.  sh: 2 words, arr: 256 words of LDS.
__device__ void sp_pick_digit(const uint32_t* __restrict__ hist, int bins, uint32_t krem, uint32_t* digit,
                              uint32_t* krem_out, uint32_t* arr, uint32_t* sh) {
    const int per = bins / SP_THREADS;                    // 8 or 4 digits a thread, consecutive
    uint32_t c[8];
    uint32_t local = 0;
    {
        const uint4 a = *reinterpret_cast<const uint4*>(hist + threadIdx.x * per);
        const uint4 d = per == 8 ? *reinterpret_cast<const uint4*>(hist + threadIdx.x * per + 4) : uint4{0, 0, 0, 0};
        c[0] = a.x; c[1] = a.y; c[2] = a.z; c[3] = a.w; c[4] = d.x; c[5] = d.y; c[6] = d.z; c[7] = d.w;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) local += c[i];
    if (threadIdx.x == 0) {
        sh[0] = 0;
        sh[1] = krem;
    }
    // entries in the digits above this thread's: the total less the running count up to this thread
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    uint32_t run = local;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t t = __shfl_up(run, o, 64);
        if (lane >= o) run += t;
    }
    if (lane == 63) arr[w] = run;
    __syncthreads();
    uint32_t total = 0;
    for (int i = 0; i < SP_THREADS / 64; ++i) {
        if (i < w) run += arr[i];
        total += arr[i];
    }
    const uint32_t above = total - run;
    if (above < krem && krem <= above + local) {          // one thread's digits hold the krem-th largest
        uint32_t cum = above;
        for (int i = per - 1; i >= 0; --i) {
            if (cum + c[i] >= krem) {
                sh[0] = threadIdx.x * per + i;
                sh[1] = krem - cum;
                break;
            }
            cum += c[i];
        }
    }
    __syncthreads();
    *digit = sh[0];
    *krem_out = sh[1];
    __syncthreads();
}

// The prefix that earlier rounds of the selection fixed: key bits above `shift` (ROUND 1: the
// first digit, ROUND 2: the first two, ROUND 3: all three, the threshold key itself).
template <int ROUND>
__device__ void sp_prefix(const uint32_t* __restrict__ row, uint32_t want, uint32_t* prefix, uint32_t* arr,
                          uint32_t* sh, uint32_t* wanted_of_last = nullptr) {
    uint32_t krem = want, d;
    *prefix = 0;
    if (ROUND >= 1) {
        sp_pick_digit(row + SP_OFF_H0, 2048, krem, &d, &krem, arr, sh);
        *prefix = d << 21;
    }
    if (ROUND >= 2) {
        sp_pick_digit(row + SP_OFF_H1, 2048, krem, &d, &krem, arr, sh);
        *prefix |= d << 10;
    }
    if (ROUND >= 3) {
        sp_pick_digit(row + SP_OFF_H2, 1024, krem, &d, &krem, arr, sh);
        *prefix |= d;
    }
    if (wanted_of_last) *wanted_of_last = krem;         // entries still wanted among those with the last digit found
}

// One round of the selection: the histogram of this round's digit over the entries whose key
// agrees with the digits found so far.
template <int ROUND>
__global__ __launch_bounds__(SP_THREADS) void sp_hist_kernel(const float* __restrict__ logits, long ld,
                                                             const float* __restrict__ params,
                                                             float* __restrict__ scratch, int V) {
    __shared__ uint32_t h[2048];
    __shared__ uint32_t arr[SP_THREADS];
    __shared__ uint32_t sh[2];
    const int b = blockIdx.y, part = blockIdx.x;
    const RowMode m = row_mode(params, b, V);
    if (!m.filt) return;
    uint32_t* row = reinterpret_cast<uint32_t*>(scratch + (size_t)b * SP_ROW_WORDS);
    uint32_t prefix;
    sp_prefix<ROUND>(row, (uint32_t)m.want, &prefix, arr, sh);
    constexpr int BINS = ROUND == 2 ? 1024 : 2048;
    constexpr int SHIFT = ROUND == 0 ? 21 : (ROUND == 1 ? 10 : 0);          // this round's digit
    constexpr int ABOVE = ROUND == 0 ? 32 : (ROUND == 1 ? 21 : 10);         // bits from here up are fixed
    for (int i = threadIdx.x; i < BINS; i += blockDim.x) h[i] = 0;
    __syncthreads();
    int lo, n;
    part_range(V, part, &lo, &n);
    for_piece(logits + (size_t)b * ld + lo, n, m.inv_t, [&](int, float v) {
        const uint32_t key = ordered_key(v);
        if (ROUND == 0 || (key >> (ABOVE & 31)) == (prefix >> (ABOVE & 31))) atomicAdd(&h[(key >> SHIFT) & (BINS - 1)], 1u);
    });
    __syncthreads();
    constexpr int OFF = ROUND == 0 ? SP_OFF_H0 : (ROUND == 1 ? SP_OFF_H1 : SP_OFF_H2);
    for (int i = threadIdx.x; i < BINS; i += blockDim.x)
        if (h[i]) atomicAdd(&row[OFF + i], h[i]);
}

// The entries above the threshold key (the want-th largest value; fewer than want of them),
// in any order, then the entries that equal it, as many as still fit MAX_CAND: what is left out
// then equals what was taken.
__global__ __launch_bounds__(SP_THREADS) void sp_collect_kernel(const float* __restrict__ logits, long ld,
                                                                const float* __restrict__ params,
                                                                float* __restrict__ scratch, int V) {
    __shared__ uint32_t arr[SP_THREADS];
    __shared__ uint32_t sh[2];
    const int b = blockIdx.y, part = blockIdx.x;
    const RowMode m = row_mode(params, b, V);
    if (!m.filt) return;
    float* rowf = scratch + (size_t)b * SP_ROW_WORDS;
    uint32_t* row = reinterpret_cast<uint32_t*>(rowf);
    uint32_t thr, ties_wanted;
    sp_prefix<3>(row, (uint32_t)m.want, &thr, arr, sh, &ties_wanted);
    const uint32_t n_above = (uint32_t)m.want - ties_wanted;        // entries above the threshold value
    int lo, n;
    part_range(V, part, &lo, &n);
    for_piece(logits + (size_t)b * ld + lo, n, m.inv_t, [&](int i, float v) {
        const uint32_t key = ordered_key(v);
        if (key >= thr) {
            const uint32_t at = key > thr ? atomicAdd(&row[SP_OFF_NCAND], 1u) : n_above + atomicAdd(&row[SP_OFF_NTIE], 1u);
            if (at < MAX_CAND) {
                rowf[SP_OFF_CV + at] = v;
                reinterpret_cast<int*>(rowf)[SP_OFF_CI + at] = lo + i;
            }
        }
    });
}

// Running sums over the workgroup's threads in thread order: the sum up to and including this
// thread's value is returned, the sum before it goes to *excl (a thread's *excl is bit for bit
// its predecessor's result, so the threads' intervals tile [0, total) exactly); wtot: 16 words of LDS.
__device__ float block_running_sum(float v, float* wtot, float* excl, float* total) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    float s = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(s, o, 64);
        if (lane >= o) s += t;
    }
    float ex = __shfl_up(s, 1, 64);
    if (lane == 0) ex = 0.f;
    __syncthreads();
    if (lane == 63) wtot[w] = s;
    __syncthreads();
    float before = 0.f, tot = 0.f;
    for (int i = 0; i < nw; ++i) {
        if (i == w) before = tot;
        tot += wtot[i];
    }
    *total = tot;
    *excl = lane == 0 ? before : before + ex;
    return before + s;
}

// The pieces' sums: their total (in a fixed order), the piece that holds `target` with what
// remains of it inside that piece, and the last piece with any weight.  Every wave computes it.
__device__ __forceinline__ float sp_parts_total(const float* __restrict__ rowf) {
    return wave_sum(rowf[SP_OFF_SUM + (threadIdx.x & 63)]);
}

// Bitonic sort of the first `span` (a power of two, at most 1024) (key, payload) pairs in LDS;
// all threads of the workgroup call; before(a, pa, c, pc): (a, pa) goes first.
template <typename K, typename P, typename F>
__device__ void sort_pairs(K* key, P* pay, int span, F before) {
    for (int size = 2; size <= span; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const int i = threadIdx.x, j = i ^ stride;
            if (j > i && j < span) {
                const bool up = (i & size) == 0;
                const K a = key[i], c = key[j];
                const P pa = pay[i], pc = pay[j];
                const bool wrong = up ? before(c, pc, a, pa) : before(a, pa, c, pc);
                if (wrong) {
                    key[i] = c;
                    key[j] = a;
                    pay[i] = pc;
                    pay[j] = pa;
                }
            }
            __syncthreads();
        }
}

// Goes through x[0..n) in index order, 4096 elements at a time (loaded side by side, then four
// in a row per thread), with the weight exp(v - mx) of every element whose scaled value v is
// at least kth and whose weight is at least thr (others weigh nothing).  Returns the first
// index whose running sum of weights exceeds rem, or -1 if none does; *sum gets the weights'
// sum up to where the walk ended (all of them when nothing was found), *last_pos the last index
// seen with any weight (-1: none).  All 1024 threads of the workgroup call; chunk: 4096 floats
// of LDS, wtot: 16, sh: 2 ints.  The result is the same in every thread.
__device__ int weights_walk(const float* __restrict__ x, int n, float inv_t, float mx, float kth, float thr, float rem,
                            float* chunk, float* wtot, int* sh, float* sum, int* last_pos) {
    const int tid = threadIdx.x;
    float acc = 0.f;
    int last = -1;
    __syncthreads();
    if (tid == 0) sh[1] = -1;
    __syncthreads();
    for (int c0 = 0; c0 < n; c0 += 4 * SAMPLE_THREADS) {
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int i = c0 + tid + k * SAMPLE_THREADS;
            v[k] = x[i < n ? i : n - 1];
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int i = c0 + tid + k * SAMPLE_THREADS;
            const float sv = v[k] * inv_t;
            float w = (i < n && sv >= kth) ? weight_of(sv, mx) : 0.f;
            if (w < thr) w = 0.f;
            chunk[tid + k * SAMPLE_THREADS] = w;
        }
        __syncthreads();
        float w4[4], s4 = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            w4[k] = chunk[tid * 4 + k];
            s4 += w4[k];
        }
        float total, before;
        const float run = block_running_sum(s4, wtot, &before, &total);
        if (s4 > 0.f && rem < run && rem >= before) {             // this thread's four hold the target
            float c = before;
            int pick = -1, last_k = -1;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                c += w4[k];
                if (w4[k] > 0.f) {
                    last_k = k;
                    if (pick < 0 && rem < c) pick = k;
                }
            }
            if (pick < 0) pick = last_k;         // (the four's own sum rounds differently: their last weight)
            sh[1] = c0 + tid * 4 + pick;
        }
        // the chunk's last index with any weight, should nothing hold the target
        int mine = -1;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (w4[k] > 0.f) mine = c0 + tid * 4 + k;
        __syncthreads();
        if (tid == 0) sh[0] = -1;
        __syncthreads();
        if (mine >= 0) atomicMax(&sh[0], mine);
        __syncthreads();
        if (sh[0] >= 0) last = sh[0];
        if (sh[1] >= 0) break;                   // (uniform: read after a barrier)
        rem -= total;
        acc += total;
    }
    *sum = acc;
    *last_pos = last;
    return sh[1];
}

// One workgroup of 1024 threads per row decides.
__global__ __launch_bounds__(SAMPLE_THREADS) void sp_final_kernel(const float* __restrict__ logits, long ld,
                                                                  const float* __restrict__ params,
                                                                  int* __restrict__ out, int V,
                                                                  float* __restrict__ scratch) {
    __shared__ float cv[MAX_CAND];
    __shared__ int ci[MAX_CAND];
    __shared__ float ce[MAX_CAND];
    __shared__ float wtot[16];
    __shared__ float chunk[4 * SAMPLE_THREADS];
    __shared__ float sh_f[2];
    __shared__ int sh_i[2];
    const int b = blockIdx.x, tid = threadIdx.x;
    const RowMode m = row_mode(params, b, V);
    float* rowf = scratch + (size_t)b * SP_ROW_WORDS;
    if (m.greedy) {                                           // the pieces' winners; ties go to the lowest index
        if (tid < 64) {
            float v = rowf[SP_OFF_MAX + tid];
            int i = reinterpret_cast<const int*>(rowf)[SP_OFF_IDX + tid];
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
    const float mx = sp_row_max(rowf) * m.inv_t;
    bool whole_row = !m.filt;
    if (m.filt) {
        uint32_t n = reinterpret_cast<const uint32_t*>(rowf)[SP_OFF_NCAND] + reinterpret_cast<const uint32_t*>(rowf)[SP_OFF_NTIE];
        const bool overflow = n > MAX_CAND;
        if (n > MAX_CAND) n = MAX_CAND;
        // by falling value (ties: rising index), for the thresholds
        cv[tid] = tid < (int)n ? rowf[SP_OFF_CV + tid] : -INFINITY;
        ci[tid] = tid < (int)n ? reinterpret_cast<const int*>(rowf)[SP_OFF_CI + tid] : 0x7fffffff;
        int span = 2;                                  // the power of two that holds the entries
        while (span < (int)n) span <<= 1;
        __syncthreads();
        sort_pairs(cv, ci, span, [](float a, int ia, float c, int ic) { return a > c || (a == c && ia < ic); });
        float kth = -INFINITY;
        if (m.use_k && m.want <= (int)n) kth = cv[m.want - 1];
        float e = (tid < (int)n && cv[tid] >= kth) ? weight_of(cv[tid], mx) : 0.f;
        float sum, before;
        const float run = block_running_sum(e, wtot, &before, &sum);    // in the order of falling value
        if (!m.use_k) {
            sum = sp_parts_total(rowf);                                 // nothing dropped yet: the whole row's sum
        } else if (overflow && m.use_p) {
            // entries that tie with the last collected one were left out: the sum of what top-k keeps
            // is taken from the row itself
            int none_i;
            weights_walk(logits + (size_t)b * ld, V, m.inv_t, mx, kth, 0.f, INFINITY, chunk, wtot, sh_i, &sum, &none_i);
        }
        if (m.use_p) {
            // the smallest prefix of the sorted weights whose mass reaches top_p * sum; every weight
            // at or above the last one taken stays.  Not reached within the collected entries: nothing is dropped.
            const float goal = m.top_p * sum;
            if (tid == 0) sh_f[0] = 0.f;
            __syncthreads();
            if (e > 0.f && run >= goal && before < goal) sh_f[0] = e;      // at most one thread
            __syncthreads();
            const float thr = sh_f[0];
            if (thr == 0.f && !m.use_k) whole_row = true;
            if (e < thr) e = 0.f;
        }
        if (!whole_row && overflow) {
            // More entries than the collection holds tie with its last one (a thousand equal
            // logits): the thresholds above are still exact, because what was left out equals what
            // was taken; the draw then walks the whole row with them, once for the sum and once
            // for the place (slow, and rare).
            const float kth_v = kth;
            const float thr_w = m.use_p ? sh_f[0] : 0.f;
            const float* x = logits + (size_t)b * ld;
            float total, part_sum;
            int last_pos;
            weights_walk(x, V, m.inv_t, mx, kth_v, thr_w, INFINITY, chunk, wtot, sh_i, &total, &last_pos);
            const int at = weights_walk(x, V, m.inv_t, mx, kth_v, thr_w, m.u * total, chunk, wtot, sh_i, &part_sum, &last_pos);
            if (tid == 0) out[b] = at >= 0 ? at : (last_pos >= 0 ? last_pos : V - 1);
            return;
        }
        if (!whole_row) {
            // by rising index, for the draw: the first kept index whose running sum exceeds u * sum
            ce[tid] = e;
            __syncthreads();
            sort_pairs(ci, ce, span, [](int ia, float, int ic, float) { return ia < ic; });
            e = ce[tid];
            float total;
            const float r2 = block_running_sum(e, wtot, &before, &total);
            const float target = m.u * total;
            if (tid == 0) {
                sh_i[0] = -1;
                sh_i[1] = -1;
            }
            __syncthreads();
            if (e > 0.f) {
                if (target < r2 && target >= before) sh_i[0] = ci[tid];      // the intervals tile: one thread
                atomicMax(&sh_i[1], ci[tid]);                                // rounding at the very end: the last kept index
            }
            __syncthreads();
            if (tid == 0)
                out[b] = sh_i[0] >= 0 ? sh_i[0] : (sh_i[1] >= 0 ? sh_i[1] : reinterpret_cast<const int*>(rowf)[SP_OFF_IDX]);
            return;
        }
        __syncthreads();                               // (the staging memory is used again below)
    }
    // The draw over the whole row: the piece that holds u * sum, then that piece's elements.
    {
        if (tid < 64) {                          // a piece per lane
            const float ps = rowf[SP_OFF_SUM + tid];
            float incl = ps;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const float t = __shfl_up(incl, o, 64);
                if (tid >= o) incl += t;
            }
            float excl = __shfl_up(incl, 1, 64);
            if (tid == 0) excl = 0.f;
            const float total = __shfl(incl, 63, 64);
            const float target = m.u * total;
            const unsigned long long holds = __ballot(ps > 0.f && target < incl && target >= excl);
            const unsigned long long any = __ballot(ps > 0.f);
            int part;
            float rem;
            if (holds) {
                part = __ffsll((long long)holds) - 1;
                rem = target - __shfl(excl, part, 64);
            } else {                             // rounding at the very end: the last piece with any weight, all of it
                part = any ? 63 - __clzll((long long)any) : 0;
                rem = INFINITY;
            }
            if (tid == 0) {
                sh_i[0] = part;
                sh_f[0] = rem;
            }
        }
        __syncthreads();
        const int part = sh_i[0];
        const float rem = sh_f[0];
        int lo, n;
        part_range(V, part, &lo, &n);
        float piece_sum;
        int last_pos;
        const int at = weights_walk(logits + (size_t)b * ld + lo, n, m.inv_t, mx, -INFINITY, 0.f, rem, chunk, wtot, sh_i,
                                    &piece_sum, &last_pos);
        if (tid == 0) out[b] = at >= 0 ? lo + at : (last_pos >= 0 ? lo + last_pos : V - 1);
    }
}

// params[b] = {temperature, top_k, top_p, u}
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits, long ld,
                                                                float* __restrict__ work, long ldw,
                                                                const float* __restrict__ params,
                                                                int* __restrict__ out, int V) {
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
        // first what lies above the 1024th largest weight (fewer than 1024 entries), then its equals
        // as far as there is room: which of them are left out does not matter, they are all the same
        for (int i = tid; i < V; i += blockDim.x) {
            const float e = w[i];
            if (e > 0.f && ordered_key(e) > min_key) cand[atomicAdd(&n_cand, 1u)] = e;
        }
        __syncthreads();
        for (int i = tid; i < V; i += blockDim.x) {
            const float e = w[i];
            if (e > 0.f && ordered_key(e) == min_key) {
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

// scratch: agave_sample_scratch_words() words per row, or null.  With it, rows of a large
// vocabulary are shared among workgroups.  kinds says what the rows need, so that launches
// nothing needs are left out: bit 0: some row draws with a temperature; bit 1: some row has
// top-k or top-p.  (A row decides for itself from params; a set bit that no row needs costs a
// launch, a missing one gives a wrong draw.)
extern "C" int agave_sample(const float* logits, long ld, float* work, long ldw, const float* params, int* out,
                            int B, int V, float* scratch, int kinds, hipStream_t stream) {
    AGAVE_CHECK(B >= 0 && V > 0, "sample: bad sizes B=%d V=%d", B, V);
    AGAVE_CHECK(ld >= V && ldw >= V, "sample: a row stride is below the vocabulary");
    AGAVE_CHECK(logits && work && params && out, "sample: null buffer");
    if (B == 0) return 0;
    if (scratch && V >= 4096 && B <= 65535) {
        const dim3 grid(SP_PARTS, B);
        sp_max_kernel<<<grid, SP_THREADS, 0, stream>>>(logits, ld, scratch, V, (kinds & 2) ? 1 : 0);
        AGAVE_LAUNCH_CHECK("sample (maxima)");
        if (kinds & 1) {
            sp_sum_kernel<<<grid, SP_THREADS, 0, stream>>>(logits, ld, params, scratch, V);
            AGAVE_LAUNCH_CHECK("sample (sums)");
        }
        if (kinds & 2) {
            sp_hist_kernel<0><<<grid, SP_THREADS, 0, stream>>>(logits, ld, params, scratch, V);
            sp_hist_kernel<1><<<grid, SP_THREADS, 0, stream>>>(logits, ld, params, scratch, V);
            sp_hist_kernel<2><<<grid, SP_THREADS, 0, stream>>>(logits, ld, params, scratch, V);
            sp_collect_kernel<<<grid, SP_THREADS, 0, stream>>>(logits, ld, params, scratch, V);
            AGAVE_LAUNCH_CHECK("sample (selection)");
        }
        sp_final_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, ld, params, out, V, scratch);
        AGAVE_LAUNCH_CHECK("sample (draw)");
        return 0;
    }
    sample_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, ld, work, ldw, params, out, V);
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


// ------------------------------------------------------------------ log-probability of the drawn token
// out[b] = logits[b][tok[b]] - log sum_v exp(logits[b][v]): the natural logarithm of the model's
// probability of the token that was drawn, from the row as the sampler saw it (temperature and
// filters are the sampler's own business and leave this number alone).  One workgroup a row; every
// thread keeps a running maximum and a sum relative to it, merged pairwise at the end.
__global__ __launch_bounds__(1024) void token_logprob_kernel(const float* __restrict__ logits, long ld,
                                                             const int* __restrict__ tok, float* __restrict__ out, int V) {
    __shared__ float sm[16], ss[16];
    const float* x = logits + (size_t)blockIdx.x * ld;
    float m = -INFINITY, s = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = x[i];
        if (v > m) {
            s = s * expf(m - v) + 1.0f;          // (m = -inf: s is 0 and stays so)
            m = v;
        } else if (v > -INFINITY) {
            s += expf(v - m);
        }
    }
    // the wave, then the workgroup: (m, s) pairs merge as s1 e^(m1 - m) + s2 e^(m2 - m)
    for (int off = 32; off > 0; off >>= 1) {
        const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(s, off, 64);
        const float mm = fmaxf(m, m2);
        s = (m > -INFINITY ? s * expf(m - mm) : 0.f) + (m2 > -INFINITY ? s2 * expf(m2 - mm) : 0.f);
        m = mm;
    }
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) {
        sm[wave] = m;
        ss[wave] = s;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float mm = -INFINITY;
        for (int w = 0; w < nw; ++w) mm = fmaxf(mm, sm[w]);
        float tot = 0.f;
        for (int w = 0; w < nw; ++w)
            if (sm[w] > -INFINITY) tot += ss[w] * expf(sm[w] - mm);
        const int t = tok[blockIdx.x];
        out[blockIdx.x] = (t >= 0 && t < V && tot > 0.f) ? x[t] - mm - logf(tot) : -INFINITY;
    }
}

extern "C" int agave_token_logprob(const float* logits, long ld, const int* tok, float* out, int B, int V,
                                   hipStream_t stream) {
    AGAVE_CHECK(B >= 0 && V > 0 && ld >= V, "token_logprob: bad sizes B=%d V=%d ld=%ld", B, V, ld);
    AGAVE_CHECK(B == 0 || (logits && tok && out), "token_logprob: null buffer");
    if (B == 0) return 0;
    token_logprob_kernel<<<B, V >= 1024 ? 1024 : 256, 0, stream>>>(logits, ld, tok, out, V);
    AGAVE_LAUNCH_CHECK("token_logprob");
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
