// Plain attention over the paged cache for gfx950, for any even head size and either
// element type: one workgroup per (token, query head), scores and probabilities in 32-bit,
// exact expf, no skipping of small probabilities.  It is the true 32-bit path and the
// fallback for head sizes the MFMA kernels refuse.
//
// Reference: src/backend/kernels/cpu/sdpa.zig:34-88 (scores * scale, softmax, weighted sum
// of V), window bounds as src/ops/attention.zig:92-93 with the callers' convention of
// src/models/gpt_oss.zig:518-519: a query at position p sees keys max(0, p-W+1) .. p.
//
// Cache pages: K [page][kv head][64 rows][hd]; V transposed [page][kv head][hd][64 rows].
// Position j of sequence b lies in page table[b][j/64 - base[b]], row j % 64.
#include "common_impl.h"
#include <math.h>

#define CHUNK 256            // keys per pass = 4 pages
#define ACC_MAX 2            // head_dim <= 512

template <typename T>
__global__ __launch_bounds__(256) void attn_plain_kernel(
    const T* __restrict__ q, long ldq, T* __restrict__ out, long ldo, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, const int* __restrict__ table, int width, const int* __restrict__ base,
    int n_pages, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int nh, int nkv, int hd,
    float scale, int window) {
    __shared__ float qs[512];
    __shared__ float sc[CHUNK];
    __shared__ long page_of[CHUNK / AGAVE_PAGE];
    __shared__ float red[16];

    const int tid = threadIdx.x;
    const int t = blockIdx.x / nh, h = blockIdx.x % nh;
    const int kvh = h / (nh / nkv);
    const int b = tok_seq[t];
    const int p = tok_pos[t];
    const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
    const int pbase = base[b];

    for (int d = tid; d < hd; d += blockDim.x) qs[d] = ld(q + (size_t)t * ldq + (size_t)h * hd + d);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ACC_MAX] = {0.f, 0.f};

    for (int c0 = (lo / AGAVE_PAGE) * AGAVE_PAGE; c0 <= p; c0 += CHUNK) {
        // pages of this chunk
        if (tid < CHUNK / AGAVE_PAGE) {
            const int first = c0 + tid * AGAVE_PAGE;
            long pg = -1;
            const int col = first / AGAVE_PAGE - pbase;
            if (first <= p && col >= 0 && col < width) pg = table[(size_t)b * width + col];
            if (pg >= n_pages) pg = -1;
            page_of[tid] = pg;
        }
        __syncthreads();
        // scores: one key per thread
        const int j = c0 + tid;
        const long pg = page_of[tid / AGAVE_PAGE];
        const bool valid = j >= lo && j <= p && pg >= 0;
        float s = -INFINITY;
        if (valid) {
            const T* kr = k_pages + (((size_t)pg * nkv + kvh) * AGAVE_PAGE + (j % AGAVE_PAGE)) * hd;
            float dot = 0.f;
            for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], ld(kr + d), dot);
            s = dot * scale;
        }
        const float cmax = block_max(s, red);
        const float m_new = fmaxf(m, cmax);
        // m_new is finite whenever any key of this or an earlier chunk was valid
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float pr = valid ? expf(s - m_new) : 0.f;
        sc[tid] = pr;
        const float csum = block_sum(pr, red);      // has barriers: sc[] is visible afterwards
        l = l * alpha + csum;
        m = m_new;
        // weighted sum of V: one output element per thread
#pragma unroll
        for (int a = 0; a < ACC_MAX; ++a) {
            const int d = tid + a * 256;
            if (d < hd) {
                float sum = 0.f;
                for (int pi = 0; pi < CHUNK / AGAVE_PAGE; ++pi) {
                    const long vp = page_of[pi];
                    if (vp < 0) continue;
                    const T* vr = v_pages + (((size_t)vp * nkv + kvh) * hd + d) * AGAVE_PAGE;
                    for (int r = 0; r < AGAVE_PAGE; ++r) {
                        const float w = sc[pi * AGAVE_PAGE + r];
                        if (w != 0.f) sum = fmaf(w, ld(vr + r), sum);   // rows outside the range hold w == 0 and may hold anything
                    }
                }
                acc[a] = acc[a] * alpha + sum;
            }
        }
        __syncthreads();     // sc[] and page_of[] are rewritten by the next chunk
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int a = 0; a < ACC_MAX; ++a) {
        const int d = tid + a * 256;
        if (d < hd) st(out + (size_t)t * ldo + (size_t)h * hd + d, acc[a] * inv);
    }
}

extern "C" int agave_attn_plain(int dtype, const void* q, long ldq, void* out, long ldo, const void* k_pages,
                                const void* v_pages, const int* table, int width, const int* base, int n_pages,
                                const int* tok_seq, const int* tok_pos, int N, int nh, int nkv, int hd, float scale,
                                int window, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh > 0 && nkv > 0 && hd > 0, "attn_plain: bad sizes N=%d nh=%d nkv=%d hd=%d", N, nh, nkv, hd);
    AGAVE_CHECK(nh % nkv == 0, "attn_plain: %d query heads are not a multiple of %d kv heads", nh, nkv);
    AGAVE_CHECK(hd <= 256 * ACC_MAX, "attn_plain: head_dim %d exceeds the supported maximum %d", hd, 256 * ACC_MAX);
    AGAVE_CHECK(ldq >= (long)nh * hd && ldo >= (long)nh * hd, "attn_plain: a row stride is below nh*hd");
    AGAVE_CHECK(window >= 0, "attn_plain: negative window");
    AGAVE_CHECK(q && out && k_pages && v_pages && table && base && tok_seq && tok_pos && width > 0 && n_pages > 0,
                "attn_plain: null buffer or empty table");
    AGAVE_CHECK((long)N * nh < 2147483647L, "attn_plain: too many (token, head) pairs");
    if (N == 0) return 0;
    if (dtype == AGAVE_F32)
        attn_plain_kernel<float><<<N * nh, 256, 0, stream>>>((const float*)q, ldq, (float*)out, ldo, (const float*)k_pages,
                                                             (const float*)v_pages, table, width, base, n_pages, tok_seq,
                                                             tok_pos, nh, nkv, hd, scale, window);
    else if (dtype == AGAVE_BF16)
        attn_plain_kernel<bf16><<<N * nh, 256, 0, stream>>>((const bf16*)q, ldq, (bf16*)out, ldo, (const bf16*)k_pages,
                                                            (const bf16*)v_pages, table, width, base, n_pages, tok_seq,
                                                            tok_pos, nh, nkv, hd, scale, window);
    else
        AGAVE_CHECK(false, "attn_plain: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("attn_plain");
    return 0;
}
