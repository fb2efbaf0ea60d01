// bfloat16 attention over the paged cache on the matrix cores of gfx950 (head sizes in steps
// of 16 up to 256): a decode kernel that splits a sequence's keys over workgroups
// (flash-decoding) with a combine pass, and a prefill kernel for steps that bring many tokens.
// Scores, the running maximum and sum, and the output accumulate in 32-bit; probabilities
// are rounded to bfloat16 only as the operand of the P*V product.
//
// Reference for the arithmetic: src/backend/kernels/cpu/sdpa.zig:34-88, 184-234 (scores *
// scale, max-subtracted softmax, weighted sum of V); window bounds as
// src/ops/attention.zig:92-93 (a query at position p sees keys max(0, p-W+1) .. p).  The
// reference's GPU kernel keeps one workgroup per head with all scores in LDS
// (src/backend/kernels/rocm/sdpa.zig:99-184) and skips probabilities below 1e-6; nothing is
// skipped here.
//
// Packed cache pages (64 positions).  With KS = ceil(hd/32) and the MFMA layouts of mfma.h:
//   K page: tiles [kt 0..3][ks 0..KS-1], tile = 64 lanes x 8: lane (i, g) element e holds
//           K[16*kt + i][32*ks + 8*g + e]   (zero where the column is >= hd)
//   V page: tiles [dt 0..hd/16-1][s 0..1]:  lane (j, g) element e holds V[key][16*dt + j] with
//           key = 32*s + (e < 4 ? 4*g + e : 16 + 4*g + e - 4)
// The odd order of V's keys is the order in which a lane holds the scores of two 16-key tiles
// after S^T = K * Q^T, so probabilities go into the P*V product without leaving their lane.
#include "common_impl.h"
#include "mfma.h"
#include "qk_rope.h"
#include "noalloc.h"
#include <math.h>

#define QT_MAX 4        // most q tiles (of 16 query slots) a wave takes

struct AttnArgs {
    const bf16* q;
    long ldq;
    bf16* out;
    long ldo;
    float* part_o;       // [token][head][split][hd]   (decode with splits)
    float* part_ml;      // [token][head][split][2]
    const uint4* k_pages;
    const uint4* v_pages;
    const int* table;
    int width;
    const int* base;
    int n_pages;
    const int* tok_seq;
    const int* tok_pos;
    const int* cu;       // prefill: first token of each sequence in the step
    int n_seqs;
    int nh, nkv, hd;
    float scale;
    int window;
    int splits, pages_per_split;
    int seq_is_token;    // decode: sequence index == token index
    int table_from_reach; // decode: each table row starts at the first page its token reaches (base[b] == lo / 64)
};

// What the decode kernel needs to do the q/k head norm, the rotation and the cache write of
// the step's own token itself (then AttnArgs::q holds the raw projection).
struct QkFuse {
    const bf16* k_raw;   // null: this run appends nothing
    long ldk;
    const bf16* v_raw;
    long ldv;
    const float* q_gain; // null: no norm
    const float* k_gain;
    float eps_q, eps_k;
    const float* inv_freq;
    int rot_half;
    float pos_scale;
};

// One wave: QT tiles of 16 query slots against the pages [page_lo, page_hi] of one sequence
// and kv head.  Slot j of tile t has position pos[t] (per lane: the lane's column j = lane%16)
// and sees keys lo[t] .. pos[t].
template <int HDT, int QT_MAX_>
struct WaveAttn {
    static constexpr int KS = (HDT + 1) / 2;
    static constexpr int QTM = QT_MAX_;
    f32x4_t o[QTM][HDT];
    float m[QTM], l[QTM];
    frag16 qf[QTM][KS];

    __device__ __forceinline__ void init(int qt) {
#pragma unroll
        for (int t = 0; t < QTM; ++t) {
            m[t] = -INFINITY;
            l[t] = 0.f;
#pragma unroll
            for (int d = 0; d < HDT; ++d) o[t][d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        (void)qt;
    }

    // q_row[t]: pointer to the head's hd values of this lane's slot in tile t, or null
    __device__ __forceinline__ void load_q(const bf16* const* q_row, int qt, int hd, int lane) {
        const int g = lane >> 4;
#pragma unroll
        for (int t = 0; t < QTM; ++t)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int d0 = 32 * ks + 8 * g;
                if (t < qt && q_row[t] != nullptr && d0 < hd)
                    qf[t][ks].u = *reinterpret_cast<const uint4*>(q_row[t] + d0);
                else
                    qf[t][ks].u = uint4{0, 0, 0, 0};
            }
    }

    // PT: pointer (to u32x4_t) to the page's tiles, in global memory or in LDS
    template <typename PT>
    __device__ __forceinline__ void page(PT kp, PT vp, int page_idx,
                                         int qt, int hd, float scale, const int* pos, const int* lo, int lane) {
        const int g = lane >> 4;
        const int hdt = hd >> 4, ks_n = (hd + 31) >> 5;
        f32x4_t st[QTM][4];
#pragma unroll
        for (int t = 0; t < QTM; ++t)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) st[t][kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        // S^T = K * Q^T: rows are keys, columns are query slots
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks < ks_n) {
                    frag16 a;
                    a.r = kp[(kt * ks_n + ks) * 64 + lane];
#pragma unroll
                    for (int t = 0; t < QTM; ++t)
                        if (t < qt) st[t][kt] = mfma_16x16x32(a, qf[t][ks], st[t][kt]);
                }
            }
        frag16 pf[QTM][2];
        float alpha[QTM];
#pragma unroll
        for (int t = 0; t < QTM; ++t) {
            if (t >= qt) continue;
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int key = page_idx * AGAVE_PAGE + kt * 16 + 4 * g + e;
                    float s = st[t][kt][e] * scale;
                    if (key > pos[t] || key < lo[t]) s = -INFINITY;
                    st[t][kt][e] = s;
                    mx = fmaxf(mx, s);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m[t], mx);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;   // a slot may see no key of this page
            alpha[t] = __expf(m[t] - m_safe);
            m[t] = m_new;
            float sum = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float pe = __expf(st[t][kt][e] - m_safe);
                    sum += pe;
                    pf[t][kt >> 1].h[(kt & 1) * 4 + e] = f32_to_bf16(pe);
                }
            l[t] = l[t] * alpha[t] + sum;       // this lane's share; the four lanes of a column meet at the end
        }
        // the output's rows are query slots 4*(lane/16) + e: fetch their factors from the columns
#pragma unroll
        for (int t = 0; t < QTM; ++t) {
            if (t >= qt) continue;
            float a4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) a4[e] = __shfl(alpha[t], 4 * g + e, 64);
#pragma unroll
            for (int d = 0; d < HDT; ++d)
                if (d < hdt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[t][d][e] *= a4[e];
                }
        }
        // O += P * V
#pragma unroll
        for (int d = 0; d < HDT; ++d)
            if (d < hdt) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    frag16 b;
                    b.r = vp[(d * 2 + s) * 64 + lane];
#pragma unroll
                    for (int t = 0; t < QTM; ++t)
                        if (t < qt) o[t][d] = mfma_16x16x32(pf[t][s], b, o[t][d]);
                }
            }
    }

    __device__ __forceinline__ void finish_sums(int qt) {
#pragma unroll
        for (int t = 0; t < QTM; ++t)
            if (t < qt) {
                l[t] += __shfl_xor(l[t], 16, 64);
                l[t] += __shfl_xor(l[t], 32, 64);
            }
    }
};

__device__ __forceinline__ long page_of(const AttnArgs& a, int b, int page_idx) {
    const int col = page_idx - a.base[b];
    if (col < 0 || col >= a.width) return -1;
    const long pg = a.table[(size_t)b * a.width + col];
    return (pg < 0 || pg >= a.n_pages) ? -1 : pg;
}

// ------------------------------------------------------------------ decode: one token per (z), splits over keys
// grid (split, kv head * head chunks, token); 4 waves per workgroup take the split's pages in
// turn and merge in LDS.  Query slots are the heads of the group (16 per chunk).
template <int HDT>
__global__ __launch_bounds__(256, 2) void attn_decode_mfma_kernel(AttnArgs a) {
    extern __shared__ float lds[];            // [4 waves][slots][hd] outputs, then [4][16][2] (max, sum)
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g = lane >> 4;
    const int G = a.nh / a.nkv;
    const int chunks = (G + 15) / 16;
    const int kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
    const int slots = (G - chunk * 16 < 16) ? G - chunk * 16 : 16;
    const int t = blockIdx.z, split = blockIdx.x;
    const int b = a.seq_is_token ? t : a.tok_seq[t];
    // when table rows start at the first page the token reaches, this wave's first page id needs
    // nothing but the grid position: fetch it before anything that waits for the position
    const int col0 = split * a.pages_per_split + wave;
    long pg0 = -1;
    if (a.table_from_reach && col0 < a.width) pg0 = a.table[(size_t)b * a.width + col0];
    const int p = a.tok_pos[t];
    const int lo = a.window > 0 ? (p - a.window + 1 > 0 ? p - a.window + 1 : 0) : 0;
    const int first = lo / AGAVE_PAGE, last = p / AGAVE_PAGE;
    const int page_lo = first + split * a.pages_per_split;
    int page_hi = page_lo + a.pages_per_split - 1;
    if (page_hi > last) page_hi = last;
    const int hd = a.hd, hdt = hd >> 4;
    const int head_j = kvh * G + chunk * 16 + j;                 // this lane's column as a head
    const bool col_ok = j < slots;

    WaveAttn<HDT, 1> w;
    w.init(1);
    const bf16* q_row[1] = {col_ok ? a.q + (size_t)t * a.ldq + (size_t)head_j * hd : nullptr};
    w.load_q(q_row, 1, hd, lane);
    const int pos[1] = {p}, los[1] = {lo};
    const size_t k_stride = (size_t)4 * ((hd + 31) >> 5) * 64, v_stride = (size_t)hdt * 2 * 64;   // uint4 per (page, kv head)
    for (int pi = page_lo + wave; pi <= page_hi; pi += 4) {
        long pg;
        if (a.table_from_reach) {
            const int col = pi - first;
            pg = (col == col0) ? pg0 : (col < a.width ? a.table[(size_t)b * a.width + col] : -1);
            if (pg >= a.n_pages) pg = -1;
        } else {
            pg = page_of(a, b, pi);
        }
        if (pg < 0) continue;
        w.page((const u32x4_t*)(a.k_pages + ((size_t)pg * a.nkv + kvh) * k_stride),
               (const u32x4_t*)(a.v_pages + ((size_t)pg * a.nkv + kvh) * v_stride), pi, 1, hd, a.scale, pos, los, lane);
    }
    w.finish_sums(1);
    // every wave leaves its (unnormalised) rows, maxima and sums in LDS
    float* sm_o = lds;
    float* sm_ml = lds + (size_t)4 * slots * hd;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int slot = 4 * g + e;
        if (slot < slots) {
            float* dst = sm_o + ((size_t)wave * slots + slot) * hd;
#pragma unroll
            for (int d = 0; d < HDT; ++d)
                if (d < hdt) dst[16 * d + j] = w.o[0][d][e];
        }
    }
    if (lane < 16) {
        sm_ml[(wave * 16 + lane) * 2 + 0] = w.m[0];
        sm_ml[(wave * 16 + lane) * 2 + 1] = w.l[0];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < slots * hd; idx += 256) {
        const int slot = idx / hd, d = idx % hd;
        float mm = -INFINITY;
#pragma unroll
        for (int x = 0; x < 4; ++x) mm = fmaxf(mm, sm_ml[(x * 16 + slot) * 2]);
        float acc = 0.f, ll = 0.f;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const float mx = sm_ml[(x * 16 + slot) * 2];
            if (mx != -INFINITY) {
                const float f = __expf(mx - mm);
                acc += sm_o[((size_t)x * slots + slot) * hd + d] * f;
                ll += sm_ml[(x * 16 + slot) * 2 + 1] * f;
            }
        }
        const int head = kvh * G + chunk * 16 + slot;
        if (a.splits == 1) {
            a.out[(size_t)t * a.ldo + (size_t)head * hd + d] = f32_to_bf16(ll > 0.f ? acc / ll : 0.f);
        } else {
            const size_t ps = ((size_t)t * a.nh + head) * a.splits + split;
            a.part_o[ps * hd + d] = acc;
            if (d == 0) {
                a.part_ml[ps * 2 + 0] = mm;
                a.part_ml[ps * 2 + 1] = ll;
            }
        }
    }
}

// out[t][head] = sum_s O_s * exp(m_s - m) / sum_s l_s * exp(m_s - m)
// ------------------------------------------------------------------ decode, streamlined (head sizes 64, 128, 256)
// The same decomposition as attn_decode_mfma_kernel, written for throughput: the unit of work
// is half a page (32 keys: two K tiles per k-step and one V tile per 16 columns of d), the
// loads of the next unit are issued as soon as the registers of the current one are free, the
// output is rescaled only when a running maximum grows by more than 2^8 (otherwise the old
// reference stays: probabilities are bounded by 2^8, which 32-bit sums and bfloat16 operands
// hold without loss), and masks are applied only to units that touch the ends of the range.
#define LAZY_LOG2 8.0f
// FUSED: q arrives as the raw projection; the workgroup normalises and rotates its heads' queries
// itself, and the workgroup whose range holds the token's own position does the same for the key,
// writes key and value into their page and only then reads pages (its own stores are visible to
// it after a workgroup barrier; no other workgroup of this launch reads that row, except those
// of other head chunks of the same kv head, which write the same bytes themselves).
template <int HDT, bool FUSED>
__global__ __launch_bounds__(256) void attn_decode_fast_kernel(AttnArgs a, QkFuse f) {
    constexpr int KS = HDT / 2;
    extern __shared__ float lds[];            // [4 waves][slots][hd] outputs, then [4][16][2] (max, sum);
                                              // FUSED: then [4][hd] floats and [16][hd] bf16 for the queries
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g = lane >> 4;
    const int G = a.nh / a.nkv;
    const int chunks = (G + 15) / 16;
    const int kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
    const int slots = (G - chunk * 16 < 16) ? G - chunk * 16 : 16;
    const int t = blockIdx.z, split = blockIdx.x;
    // the token's sequence and position are asked for first: the page ids wait for them
    const int b = a.seq_is_token ? t : a.tok_seq[t];
    const int p = a.tok_pos[t];
    // The first columns of the table row are asked for before the position is known, a column per
    // lane, and before every other vector load: loads come back in the order they left, so behind
    // the rows of q and k the page ids would wait for those, and the first keys for the page ids.
    int trow = -1;
    if (a.table_from_reach) trow = a.table[(size_t)b * a.width + (lane < a.width ? lane : 0)];
    // FUSED: the first rows of the q/k work are requested next (wave w takes query
    // head w of the chunk; the wave after the last head takes the key and value rows, in case
    // this workgroup turns out to be the one that writes them)
    constexpr int NV = HDT / 4;               // groups of 64 elements in a head
    QkRow<bf16, NV> row0;
    bf16 vreg0[NV];
    const bool row0_q = FUSED && wave < slots, row0_k = FUSED && wave == slots && f.k_raw != nullptr;
    if constexpr (FUSED) {
        constexpr int hd0 = HDT * 16;
        // a wave without a row reads the token's first query head (and nothing uses it); no load
        // stands under a condition, so all of them leave together
        const bf16* src0 = row0_q ? a.q + (size_t)t * a.ldq + (size_t)(kvh * G + chunk * 16 + wave) * hd0
                                  : (row0_k ? f.k_raw + (size_t)t * f.ldk + (size_t)kvh * hd0 : a.q + (size_t)t * a.ldq);
        row0 = qk_row_load<bf16, NV>(src0, row0_q ? f.q_gain : f.k_gain, f.inv_freq, f.rot_half, hd0, lane);
#pragma unroll
        for (int k = 0; k < NV; ++k) vreg0[k] = bf16{0};
        if (row0_k) {
            const bf16* vsrc0 = f.v_raw + (size_t)t * f.ldv + (size_t)kvh * hd0;
#pragma unroll
            for (int k = 0; k < NV; ++k) vreg0[k] = vsrc0[lane + 64 * k];
        }
    }
    // The keys this token sees lie in half pages (units of 32 keys) u_first .. u_last.  The launch's
    // splits share them evenly, whatever the sequence's length (a run of whole pages per split would
    // leave the last splits of a short sequence idle and the waves of a split unequal shares); a
    // workgroup's four waves take its units in turn.  A unit is one round trip to memory, and with
    // as many waves as units nearly every wave makes just one.
    // Which columns of the table row (asked for at the start) this wave needs depends on the
    // position; asking only then would put a second round trip before the first key.
    const int lo = a.window > 0 ? (p - a.window + 1 > 0 ? p - a.window + 1 : 0) : 0;
    const int first = lo / AGAVE_PAGE, last = p / AGAVE_PAGE;
    const int u_first = lo / 32, u_last = p / 32, n_u = u_last - u_first + 1;
    // (32-bit: at most 64 splits times the half pages of a context; a 64-bit division is some hundred instructions)
    const int ua = u_first + (int)((unsigned)(split * n_u) / (unsigned)a.splits);
    const int ub = u_first + (int)((unsigned)((split + 1) * n_u) / (unsigned)a.splits);
    const int u0 = ua + wave;
    const int half = u0 & 1;                                       // (a wave's units are four apart: one half)
    const int n_my = u0 < ub ? (ub - u0 + 3) / 4 : 0;              // units this wave takes
    constexpr int hd = HDT * 16;
    const float scale2 = a.scale * 1.4426950408889634f;          // scores in units of log2

    // queries of this chunk's heads: B operand of S^T = K Q^T
    frag16 qf[KS];
    if constexpr (!FUSED) {
        const bool col_ok = j < slots;
        const bf16* qrow = a.q + (size_t)t * a.ldq + (size_t)(kvh * G + chunk * 16 + j) * hd;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (col_ok) qf[ks].u = *reinterpret_cast<const uint4*>(qrow + 32 * ks + 8 * g);
            else qf[ks].u = uint4{0, 0, 0, 0};
        }
    }
    f32x4_t o[HDT];
#pragma unroll
    for (int d = 0; d < HDT; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_ref = -INFINITY, l = 0.f;

    constexpr size_t k_stride = (size_t)4 * KS * 64, v_stride = (size_t)HDT * 2 * 64;   // uint4 per (page, kv head)
    // a table wider than a wave: the ids of this wave's next pages are fetched together, ahead of
    // any use (a lookup in the loop would stand between every two units)
    constexpr int PG_AHEAD = 10;
    int pg_pre[PG_AHEAD];
    const bool wide = a.table_from_reach && a.width > 64;
#pragma unroll
    for (int i = 0; i < PG_AHEAD; ++i) {
        const int col = ((u0 + 4 * i) >> 1) - first;
        pg_pre[i] = (wide && i < n_my && col < a.width) ? a.table[(size_t)b * a.width + col] : -1;
    }
    auto page_id = [&](int i) -> int {           // page of this wave's i-th unit (page ids fit 31 bits)
        const int pi = (u0 + 4 * i) >> 1;
        int pg;
        if (a.table_from_reach) {
            const int col = pi - first;
            if (!wide) {
                pg = col < a.width ? __builtin_amdgcn_readlane(trow, col) : -1;
            } else if (i < PG_AHEAD) {
                pg = -1;
#pragma unroll
                for (int k = 0; k < PG_AHEAD; ++k)
                    if (k == i) pg = pg_pre[k];
            } else {
                pg = col < a.width ? a.table[(size_t)b * a.width + col] : -1;
            }
            if (pg >= a.n_pages) pg = -1;
        } else {
            pg = (int)page_of(a, b, pi);
        }
        return pg;
    };
    frag16 kb[2][KS], vb[HDT];
    const u32x4_t* kp = nullptr;
    const u32x4_t* vp = nullptr;
    auto load_k = [&]() {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kb[kt][ks].r = kp[((2 * half + kt) * KS + ks) * 64 + lane];
    };
    auto load_v = [&]() {
#pragma unroll
        for (int d = 0; d < HDT; ++d) vb[d].r = vp[(d * 2 + half) * 64 + lane];
    };

    // units: this wave's half of its pages, in order; the next unit's K and V are fetched while this one is used
    int cur_page = 0;
    int pg = n_my > 0 ? page_id(0) : -1;
    bool have = n_my > 0 && pg >= 0;
    if (have) {
        kp = (const u32x4_t*)(a.k_pages + ((size_t)pg * a.nkv + kvh) * k_stride);
        vp = (const u32x4_t*)(a.v_pages + ((size_t)pg * a.nkv + kvh) * v_stride);
    }
    // FUSED: the token's own key and value go into the page of position p, by the workgroup that
    // reads it; the wave whose first page that is waits with its loads until the row is there
    const bool writer = FUSED && f.k_raw != nullptr && split == a.splits - 1;       // (the last split ends with u_last)
    const bool early = !(writer && u0 == u_last);
    if (have && early) {
        load_k();
        load_v();
    }
    if constexpr (FUSED) {
        float* ybuf = lds + (size_t)4 * slots * hd + 4 * 16 * 2 + (size_t)wave * hd;
        bf16* q_s = reinterpret_cast<bf16*>(lds + (size_t)4 * slots * hd + 4 * 16 * 2 + (size_t)4 * hd);
        const float pf = (float)p * f.pos_scale;
        // the token's own key and value go into the page of position p, by the workgroup that reads it
        const int jobs = slots + (writer ? 1 : 0);
        for (int job0 = 0; job0 < jobs; job0 += 4) {
            const int job = job0 + wave;
            const bool active = job < jobs, is_q = job < slots;
            QkRow<bf16, NV> row;
            bf16 vreg[NV];
            if (job0 == 0) {                       // requested at the kernel's start
                row = row0;
#pragma unroll
                for (int k = 0; k < NV; ++k) vreg[k] = vreg0[k];
            } else {
                // (a wave past the last job reads the chunk's first head; the key's job only exists with k_raw)
                const bool k_job = active && !is_q;
                const bf16* src = k_job ? f.k_raw + (size_t)t * f.ldk + (size_t)kvh * hd
                                        : a.q + (size_t)t * a.ldq + (size_t)(kvh * G + chunk * 16 + (active ? job : 0)) * hd;
                row = qk_row_load<bf16, NV>(src, is_q ? f.q_gain : f.k_gain, f.inv_freq, f.rot_half, hd, lane);
#pragma unroll
                for (int k = 0; k < NV; ++k) vreg[k] = bf16{0};
                if (k_job) {
                    const bf16* vsrc = f.v_raw + (size_t)t * f.ldv + (size_t)kvh * hd;
#pragma unroll
                    for (int k = 0; k < NV; ++k) vreg[k] = vsrc[lane + 64 * k];
                }
            }
            qk_row_finish<bf16, NV>(row, ybuf, (is_q ? f.q_gain : f.k_gain) != nullptr, is_q ? f.eps_q : f.eps_k, f.rot_half,
                                    pf, hd, lane, active);
            if (active && is_q) {
                for (int d = lane; d < hd; d += 64) q_s[job * hd + d] = f32_to_bf16(ybuf[d]);
            } else if (active) {
                long wpg;
                if (a.table_from_reach) {
                    const int col = last - first;
                    wpg = col < a.width ? a.table[(size_t)b * a.width + col] : -1;
                    if (wpg >= a.n_pages) wpg = -1;
                } else {
                    wpg = page_of(a, b, last);
                }
                if (wpg >= 0) {
                    bf16* dk = (bf16*)(a.k_pages + ((size_t)wpg * a.nkv + kvh) * ((size_t)4 * KS * 64));
                    bf16* dv = (bf16*)(a.v_pages + ((size_t)wpg * a.nkv + kvh) * ((size_t)HDT * 2 * 64));
                    store_kv_row_packed_regs<bf16, NV>(dk, dv, ybuf, vreg, p % AGAVE_PAGE, hd, lane);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const bool col_ok = j < slots;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (col_ok) qf[ks].u = *reinterpret_cast<const uint4*>(q_s + j * hd + 32 * ks + 8 * g);
            else qf[ks].u = uint4{0, 0, 0, 0};
        }
    }
    if (have && !early) {
        load_k();
        load_v();
    }
    while (have) {
        const int key0 = (u0 + 4 * cur_page) * 32;                // first key of this unit
        // S^T for the unit's two key tiles
        f32x4_t st0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, st1 = st0;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            st0 = mfma_16x16x32(kb[0][ks], qf[ks], st0);
            st1 = mfma_16x16x32(kb[1][ks], qf[ks], st1);
        }
        // where the next unit lies, and its keys (the K registers are free now)
        const int n_page = cur_page + 1;
        bool n_have = n_page < n_my;
        const u32x4_t* nvp = vp;
        if (n_have) {
            const int npg = page_id(n_page);
            if (npg < 0) {
                n_have = false;
            } else {
                kp = (const u32x4_t*)(a.k_pages + ((size_t)npg * a.nkv + kvh) * k_stride);
                nvp = (const u32x4_t*)(a.v_pages + ((size_t)npg * a.nkv + kvh) * v_stride);
            }
        }
        if (n_have) load_k();
        // scores -> probabilities against the running reference
        float s[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s[e] = st0[e] * scale2;
            s[4 + e] = st1[e] * scale2;
        }
        if (key0 < lo || key0 + 31 > p) {                          // a unit at an end of the range: mask
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k0 = key0 + 4 * g + e, k1 = k0 + 16;
                if (k0 > p || k0 < lo) s[e] = -INFINITY;
                if (k1 > p || k1 < lo) s[4 + e] = -INFINITY;
            }
        }
        float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        if (__any(mx > m_ref + LAZY_LOG2)) {                       // rare after the first unit
            const float m_new = fmaxf(m_ref, mx);
            const float f = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
            l *= f;
            float f4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) f4[e] = __shfl(f, 4 * g + e, 64);
#pragma unroll
            for (int d = 0; d < HDT; ++d)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[d][e] *= f4[e];
            m_ref = m_new;
        }
        const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref;
        frag16 pf;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float pe = __builtin_amdgcn_exp2f(s[e] - m_use);
            sum += pe;
            pf.v[e] = (__bf16)pe;
        }
        l += sum;
        // O += P V, then the V registers are free for the next unit
#pragma unroll
        for (int d = 0; d < HDT; ++d) o[d] = mfma_16x16x32(pf, vb[d], o[d]);
        vp = nvp;
        if (n_have) load_v();
        cur_page = n_page;
        have = n_have;
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    // every wave leaves its (unnormalised) rows, references and sums in LDS
    float* sm_o = lds;
    float* sm_ml = lds + (size_t)4 * slots * hd;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int slot = 4 * g + e;
        if (slot < slots) {
            float* dst = sm_o + ((size_t)wave * slots + slot) * hd;
#pragma unroll
            for (int d = 0; d < HDT; ++d) dst[16 * d + j] = o[d][e];
        }
    }
    if (lane < 16) {
        sm_ml[(wave * 16 + lane) * 2 + 0] = m_ref;
        sm_ml[(wave * 16 + lane) * 2 + 1] = l;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < slots * hd; idx += 256) {
        const int slot = idx / hd, d = idx % hd;
        float mm = -INFINITY;
#pragma unroll
        for (int x = 0; x < 4; ++x) mm = fmaxf(mm, sm_ml[(x * 16 + slot) * 2]);
        float acc = 0.f, ll = 0.f;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const float mx = sm_ml[(x * 16 + slot) * 2];
            if (mx != -INFINITY) {
                const float f = __builtin_amdgcn_exp2f(mx - mm);
                acc += sm_o[((size_t)x * slots + slot) * hd + d] * f;
                ll += sm_ml[(x * 16 + slot) * 2 + 1] * f;
            }
        }
        const int head = kvh * G + chunk * 16 + slot;
        if (a.splits == 1) {
            a.out[(size_t)t * a.ldo + (size_t)head * hd + d] = f32_to_bf16(ll > 0.f ? acc / ll : 0.f);
        } else {
            const size_t ps = ((size_t)t * a.nh + head) * a.splits + split;
            a.part_o[ps * hd + d] = acc;
            if (d == 0) {
                a.part_ml[ps * 2 + 0] = mm * 0.6931471805599453f;    // the combine pass works in natural logarithms
                a.part_ml[ps * 2 + 1] = ll;
            }
        }
    }
}

#define COMBINE_MAX_SPLITS 256
__global__ void attn_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                    bf16* __restrict__ out, long ldo, int nh, int hd, int splits) {
    __shared__ float wgt[COMBINE_MAX_SPLITS];
    __shared__ float red[16];
    const int t = blockIdx.x / nh, head = blockIdx.x % nh;
    const size_t slot0 = ((size_t)t * nh + head) * splits;
    // the first splits' partial outputs are requested before anything is waited for (one column
    // per thread when the block is as wide as the head)
    constexpr int PRE = 8;
    float pre[PRE];
    {
        const int d = threadIdx.x < hd ? threadIdx.x : 0;
#pragma unroll
        for (int sp = 0; sp < PRE; ++sp) pre[sp] = sp < splits ? part_o[(slot0 + sp) * hd + d] : 0.f;
    }
    // every split's maximum and sum are fetched at once, one split per thread
    float ms[COMBINE_MAX_SPLITS / 64], ls[COMBINE_MAX_SPLITS / 64];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < COMBINE_MAX_SPLITS / 64; ++i) {
        const int sidx = threadIdx.x + i * blockDim.x;
        const bool in = i * (int)blockDim.x < splits && sidx < splits;
        ms[i] = in ? part_ml[(slot0 + sidx) * 2] : -INFINITY;
        ls[i] = in ? part_ml[(slot0 + sidx) * 2 + 1] : 0.f;
        m = fmaxf(m, ms[i]);
    }
    m = block_max(m, red);
    float l = 0.f;
#pragma unroll
    for (int i = 0; i < COMBINE_MAX_SPLITS / 64; ++i) {
        const int sidx = threadIdx.x + i * blockDim.x;
        const float f = (ms[i] != -INFINITY) ? __expf(ms[i] - m) : 0.f;
        if (sidx < COMBINE_MAX_SPLITS) wgt[sidx] = f;
        l += ls[i] * f;
    }
    l = block_sum(l, red);            // its barriers also publish wgt[]
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float acc = 0.f;
        const float* po = part_o + slot0 * hd + d;
        const bool first = d == (int)threadIdx.x;          // the columns whose first splits are in registers
#pragma unroll
        for (int sp = 0; sp < PRE; ++sp)
            if (sp < splits) acc += (first ? pre[sp] : po[(size_t)sp * hd]) * wgt[sp];
        for (int sp = PRE; sp < splits; ++sp) acc += po[(size_t)sp * hd] * wgt[sp];
        out[(size_t)t * ldo + (size_t)head * hd + d] = f32_to_bf16(acc * inv);
    }
}

// ------------------------------------------------------------------ prefill: 64 positions x QT heads per workgroup
// grid (block of positions, kv head * head chunks, sequence).  The four waves are hw heads
// wide and 4/hw tiles of 16 positions deep; a wave takes QT heads of its tile (slot j of tile t
// is position first + j of head chunk*hw*QT + (wave % hw)*QT + t).  All share the pages: a page's K and V tiles come into LDS once per workgroup, straight from global memory
// (no registers in between), the next page while the current one is being used.
typedef __attribute__((address_space(3))) u32x4_t lds_u32x4;

template <int HDT, int QT>
__global__ __launch_bounds__(256) void attn_prefill_mfma_kernel(AttnArgs a, int qt_heads, int hw) {
    extern __shared__ __attribute__((aligned(16))) uint4 page_lds[];      // [2][K tiles | V tiles][64]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g = lane >> 4;
    const int G = a.nh / a.nkv;
    const int wg_heads = qt_heads * hw;                          // heads a workgroup covers
    const int chunks = (G + wg_heads - 1) / wg_heads;
    const int kvh = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
    const int b = blockIdx.z;
    const int t0 = a.cu[b], n_new = a.cu[b + 1] - t0;
    const int blk_len = (4 / hw) * 16;                           // positions a workgroup covers
    const int blk0 = blockIdx.x * blk_len;
    if (blk0 >= n_new) return;                                   // the whole workgroup leaves
    const int tile0 = blk0 + (wave / hw) * 16;                   // first step-token of this wave's tile
    const int head0 = chunk * wg_heads + (wave % hw) * qt_heads; // first head (within the group) of this wave
    const int qt = (G - head0 < qt_heads) ? (G - head0 > 0 ? G - head0 : 0) : qt_heads;
    const bool wave_on = tile0 < n_new && qt > 0;
    const int hd = a.hd, hdt = hd >> 4, ks_n = (hd + 31) >> 5;
    const bool col_ok = tile0 + j < n_new;
    const int tok = t0 + (col_ok ? tile0 + j : n_new - 1);       // padding columns repeat the last token
    const int p = a.tok_pos[tok];
    const int lo = a.window > 0 ? (p - a.window + 1 > 0 ? p - a.window + 1 : 0) : 0;

    WaveAttn<HDT, QT> w;
    w.init(qt);
    const bf16* q_row[QT];
    int pos[QT], los[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const int head = kvh * G + head0 + t;
        q_row[t] = (t < qt && wave_on) ? a.q + (size_t)tok * a.ldq + (size_t)head * hd : nullptr;
        pos[t] = p;
        los[t] = lo;
    }
    w.load_q(q_row, qt, hd, lane);
    // this wave needs the pages from its first column's lower bound to its last column's position
    const int my_first = __shfl(lo, 0, 64) / AGAVE_PAGE, my_last = __shfl(p, 15, 64) / AGAVE_PAGE;
    // the workgroup: positions are consecutive within the step
    const int p_blk0 = a.tok_pos[t0 + blk0];
    const int blk_n = (n_new - blk0 < blk_len) ? n_new - blk0 : blk_len;
    const int lo_blk = a.window > 0 ? (p_blk0 - a.window + 1 > 0 ? p_blk0 - a.window + 1 : 0) : 0;
    const int page_first = lo_blk / AGAVE_PAGE, page_last = (p_blk0 + blk_n - 1) / AGAVE_PAGE;

    const int n_k = 4 * ks_n, n_v = hdt * 2;                     // tiles (of 64 uint4) per page
    const size_t k_stride = (size_t)n_k * 64, v_stride = (size_t)n_v * 64;
    const int buf_tiles = n_k + n_v;
    auto fetch = [&](int pi, int buf) {
        const long pg = page_of(a, b, pi);
        if (pg < 0) return;
        const uint4* ksrc = a.k_pages + ((size_t)pg * a.nkv + kvh) * k_stride;
        const uint4* vsrc = a.v_pages + ((size_t)pg * a.nkv + kvh) * v_stride;
        for (int ti = wave; ti < buf_tiles; ti += 4) {
            const uint4* src = (ti < n_k) ? ksrc + (size_t)ti * 64 : vsrc + (size_t)(ti - n_k) * 64;
            uint4* dst = page_lds + ((size_t)buf * buf_tiles + ti) * 64;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + lane),
                                             (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
        }
    };

    if (page_first <= page_last) fetch(page_first, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (int pi = page_first; pi <= page_last; ++pi) {
        const int buf = (pi - page_first) & 1;
        if (pi < page_last) fetch(pi + 1, buf ^ 1);
        if (wave_on && pi >= my_first && pi <= my_last && page_of(a, b, pi) >= 0) {
            const lds_u32x4* kl = (const lds_u32x4*)(page_lds + (size_t)buf * buf_tiles * 64);
            const lds_u32x4* vl = kl + (size_t)n_k * 64;
            w.page(kl, vl, pi, qt, hd, a.scale, pos, los, lane);
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }
    if (!wave_on) return;
    w.finish_sums(qt);
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        if (t >= qt) continue;
        const int head = kvh * G + head0 + t;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 4 * g + e;                            // slot (position) this lane's values belong to
            const float lr = __shfl(w.l[t], row, 64);
            if (tile0 + row >= n_new) continue;
            const float inv = lr > 0.f ? 1.0f / lr : 0.f;
            bf16* dst = a.out + (size_t)(t0 + tile0 + row) * a.ldo + (size_t)head * hd;
#pragma unroll
            for (int d = 0; d < HDT; ++d)
                if (d < hdt) dst[16 * d + j] = f32_to_bf16(w.o[t][d][e] * inv);
        }
    }
}

// ------------------------------------------------------------------ the items of a prefill step
// The causal triangle gives a prompt's blocks of positions anything from one page of keys to the
// whole reach, and a prompt of a few thousand tokens has fewer blocks than the chip has compute
// units.  The host therefore cuts the step into *items* of about equal work and lists them with
// the largest first: an item is a block of positions of one sequence and a run of the pages that
// the block sees; a block whose reach is longer than an item may be is cut into several pieces,
// which leave partial results for attn_merge_pieces_kernel.  Workgroups take the items in the
// list's order as compute units free up (grid x = item * kv head chunks + kv head chunk), so the
// last ones to start are the smallest.
struct PrefillItem {
    int seq;          // sequence of the step
    int blk0;         // first of the block's tokens, counted within the sequence's tokens of this step
    int page_first;   // first page (position / 64) of this piece
    int n_pages;      // pages of this piece
    int piece;        // which piece of the block this is
    int n_pieces;     // pieces the block is cut into (1: the item writes the output itself)
};

// out[t][head] from the pieces' partial results, for the tokens of blocks that were cut into
// pieces (tok_pieces[t] > 1; the others were written by their item itself): a wave per (token,
// head), four elements a lane at a time, every load asked for before the first is used.
#define MERGE_MAX_PIECES 4
__global__ __launch_bounds__(256) void attn_merge_pieces_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                const int* __restrict__ tok_pieces,
                                                                bf16* __restrict__ out, long ldo, int nh, int hd,
                                                                int max_pieces, long rows) {
    const int lane = threadIdx.x & 63;
    const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const long t = r / nh;
    const int head = (int)(r % nh);
    const int pieces = tok_pieces[t];
    if (pieces <= 1) return;
    const size_t slot0 = (size_t)r * max_pieces;
    float ms[MERGE_MAX_PIECES], ls[MERGE_MAX_PIECES];
#pragma unroll
    for (int sp = 0; sp < MERGE_MAX_PIECES; ++sp) {
        const int s2 = sp < pieces ? sp : pieces - 1;
        ms[sp] = part_ml[(slot0 + s2) * 2];
        ls[sp] = part_ml[(slot0 + s2) * 2 + 1];
    }
    for (int d0 = lane * 4; d0 < hd; d0 += 256) {
        float4 v[MERGE_MAX_PIECES];
#pragma unroll
        for (int sp = 0; sp < MERGE_MAX_PIECES; ++sp) {
            const int s2 = sp < pieces ? sp : pieces - 1;
            v[sp] = *reinterpret_cast<const float4*>(part_o + (slot0 + s2) * hd + d0);
        }
        float m = -INFINITY;
#pragma unroll
        for (int sp = 0; sp < MERGE_MAX_PIECES; ++sp)
            if (sp < pieces) m = fmaxf(m, ms[sp]);
        float l = 0.f;
        float4 acc = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sp = 0; sp < MERGE_MAX_PIECES; ++sp) {
            const float f = (sp < pieces && ms[sp] != -INFINITY) ? __expf(ms[sp] - m) : 0.f;
            l += ls[sp] * f;
            acc.x += v[sp].x * f;
            acc.y += v[sp].y * f;
            acc.z += v[sp].z * f;
            acc.w += v[sp].w * f;
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        uint2 u;
        u.x = f32x2_to_bf16x2(acc.x * inv, acc.y * inv);
        u.y = f32x2_to_bf16x2(acc.z * inv, acc.w * inv);
        *reinterpret_cast<uint2*>(out + (size_t)t * ldo + (size_t)head * hd + d0) = u;
    }
}

// ------------------------------------------------------------------ prefill, streamlined (head sizes 64, 128, 256)
// The same frame as attn_prefill_mfma_kernel (a workgroup's waves share each page through LDS,
// two pages in flight), with the decode kernel's inner loop: half pages as units, head size
// fixed at compile time, probabilities against a running reference that is renewed only when a
// maximum outgrows it by 2^8, exp2, and masks only on units that touch the diagonal or the
// window's edge; units that no column of the tile can see are skipped.  A wave takes 16
// positions of one head; hw heads of a group sit side by side in a workgroup of NWV waves (4 or
// 8: a page fetched into LDS then serves 64 positions instead of 32, which halves the traffic
// from L2 that bounds this kernel, and two waves share a SIMD).
template <int HDT, int NWV>
__global__ __launch_bounds__(NWV * 64) void attn_prefill_fast_kernel(AttnArgs a, const PrefillItem* __restrict__ items, int nkc,
                                                                   int hw, int max_pieces, int max_item_pages) {
    constexpr int KS = HDT / 2, hd = HDT * 16;
    constexpr int n_k = 4 * KS, n_v = HDT * 2, buf_tiles = n_k + n_v;         // tiles (of 64 uint4) per page
    extern __shared__ __attribute__((aligned(16))) uint4 page_lds[];          // [2][K tiles | V tiles][64]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g = lane >> 4;
    const PrefillItem it = items[blockIdx.x / nkc];
    const int G = a.nh / a.nkv;
    const int chunks = (G + hw - 1) / hw;
    const int kvhc = blockIdx.x % nkc, kvh = kvhc / chunks, chunk = kvhc % chunks;
    const int b = it.seq;
    const int t0 = a.cu[b], n_new = a.cu[b + 1] - t0;
    const int blk0 = it.blk0;                                    // the block is (NWV / hw) * 16 positions long
    const int tile0 = blk0 + (wave / hw) * 16;                   // first step-token of this wave's tile
    const int gh = chunk * hw + wave % hw;                       // this wave's head within the group
    const bool wave_on = tile0 < n_new && gh < G;
    const bool col_ok = tile0 + j < n_new;
    const int tok = t0 + (col_ok ? tile0 + j : n_new - 1);       // padding columns repeat the last token
    const int p = a.tok_pos[tok];
    const int lo = a.window > 0 ? (p - a.window + 1 > 0 ? p - a.window + 1 : 0) : 0;
    const float scale2 = a.scale * 1.4426950408889634f;          // scores in units of log2

    frag16 qf[KS];
    {
        const bf16* qrow = a.q + (size_t)tok * a.ldq + (size_t)(kvh * G + (gh < G ? gh : 0)) * hd;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (wave_on) qf[ks].u = *reinterpret_cast<const uint4*>(qrow + 32 * ks + 8 * g);
            else qf[ks].u = uint4{0, 0, 0, 0};
        }
    }
    f32x4_t o[HDT];
#pragma unroll
    for (int d = 0; d < HDT; ++d) o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_ref = -INFINITY, l = 0.f;

    // positions rise along the tile's columns: the first column has the lowest bounds, the last the highest
    const int p_min = __shfl(p, 0, 64), p_max = __shfl(p, 15, 64);
    const int lo_min = __shfl(lo, 0, 64), lo_max = __shfl(lo, 15, 64);
    const int my_first = lo_min / AGAVE_PAGE, my_last = p_max / AGAVE_PAGE;
    const int page_first = it.page_first;
    int page_last = it.page_first + it.n_pages - 1;

    // The ids of the pages this workgroup goes through, looked up once: a lookup inside the loop
    // is two dependent loads from memory a page, and waiting for them also waits for the next
    // page's loads, which were issued just before and should travel while this page is worked on.
    // (the array holds max_item_pages ids, the most pages that the host says any item has; the bound
    // below keeps the writes inside the array whatever the items in device memory say)
    int* pg_ids = reinterpret_cast<int*>(page_lds + (size_t)2 * buf_tiles * 64);
    if (page_last - page_first >= max_item_pages) page_last = page_first + max_item_pages - 1;
    for (int i = threadIdx.x; i <= page_last - page_first; i += NWV * 64) pg_ids[i] = (int)page_of(a, b, page_first + i);
    __syncthreads();

    constexpr size_t k_stride = (size_t)n_k * 64, v_stride = (size_t)n_v * 64;
    auto fetch = [&](int pi, int buf) {
        const long pg = __builtin_amdgcn_readfirstlane(pg_ids[pi - page_first]);
        if (pg < 0) return;
        const uint4* ksrc = a.k_pages + ((size_t)pg * a.nkv + kvh) * k_stride;
        const uint4* vsrc = a.v_pages + ((size_t)pg * a.nkv + kvh) * v_stride;
        for (int ti = wave; ti < buf_tiles; ti += NWV) {
            const uint4* src = (ti < n_k) ? ksrc + (size_t)ti * 64 : vsrc + (size_t)(ti - n_k) * 64;
            uint4* dst = page_lds + ((size_t)buf * buf_tiles + ti) * 64;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + lane),
                                             (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
        }
    };

    if (page_first <= page_last) fetch(page_first, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (int pi = page_first; pi <= page_last; ++pi) {
        const int buf = (pi - page_first) & 1;
        if (pi < page_last) fetch(pi + 1, buf ^ 1);
        if (wave_on && pi >= my_first && pi <= my_last && pg_ids[pi - page_first] >= 0) {
            // this lane's 16 bytes of the page's first tile; tiles follow each other by 1 KB
            const unsigned kaddr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4*)page_lds +
                                   (unsigned)(buf * buf_tiles * 64 + lane) * 16u;
            if constexpr (HDT == 16) {
                // Which of the page's two units (half pages) some column of the tile sees.
                const bool see0 = !(pi * AGAVE_PAGE > p_max || pi * AGAVE_PAGE + 31 < lo_min);
                const bool see1 = !(pi * AGAVE_PAGE + 32 > p_max || pi * AGAVE_PAGE + 63 < lo_min);
                // A unit's key tiles and its value tiles come from LDS in two batches each, into two sets
                // of registers that take turns: while the multiplications of one batch run, the next
                // batch is on its way, so that the LDS and the matrix cores work at the same time
                // (read whole and then multiplied, the eight waves all read, then all multiply).  The
                // keys of the page's second unit are asked for during the first unit's last
                // multiplications.  The LDS returns a wave's reads in order: a wait for "at most n
                // outstanding" leaves the younger batch in flight.
                constexpr int KH = KS / 2;                            // k-steps per batch of key tiles
                frag16 fa[KS], fb[KS];
                auto read_keys_a = [&](auto halfc) {
                    constexpr int half = decltype(halfc)::value;
                    static_for<0, KH>([&](auto ks) {
                        lds_read16<((2 * half) * KS + ks.value) * 1024>(fa[2 * ks.value], kaddr);
                        lds_read16<((2 * half + 1) * KS + ks.value) * 1024>(fa[2 * ks.value + 1], kaddr);
                    });
                };
                auto read_keys_b = [&](auto halfc) {
                    constexpr int half = decltype(halfc)::value;
                    static_for<0, KH>([&](auto ks) {
                        lds_read16<((2 * half) * KS + KH + ks.value) * 1024>(fb[2 * ks.value], kaddr);
                        lds_read16<((2 * half + 1) * KS + KH + ks.value) * 1024>(fb[2 * ks.value + 1], kaddr);
                    });
                };
                auto unit = [&](auto halfc, bool keys_asked, bool ask_next) {
                    constexpr int half = decltype(halfc)::value;
                    const int key0 = pi * AGAVE_PAGE + 32 * half;
                    if (!keys_asked) {
                        read_keys_a(halfc);
                        read_keys_b(halfc);
                    }
                    lds_settle_to<KS>();                              // the first batch of keys is here
    #pragma unroll
                    for (int i = 0; i < KS; ++i) lds_use(fa[i]);
                    // Head sizes up to 128: four chains of multiplications instead of two (measured at 128:
                    // 55 us instead of 70 for 2,048 tokens and 32 heads; at 256, with chains of 8 and 4, no gain).
                    constexpr bool FOUR_CHAINS = KS > 1 && KS <= 4;
                    f32x4_t st0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, st1 = st0, st0b = st0, st1b = st0;
    #pragma unroll
                    for (int ks = 0; ks < KH; ++ks) {
                        if (FOUR_CHAINS && (ks & 1)) {
                            st0b = mfma_16x16x32(fa[2 * ks], qf[ks], st0b);
                            st1b = mfma_16x16x32(fa[2 * ks + 1], qf[ks], st1b);
                        } else {
                            st0 = mfma_16x16x32(fa[2 * ks], qf[ks], st0);
                            st1 = mfma_16x16x32(fa[2 * ks + 1], qf[ks], st1);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    lds_settle_to<0>();                               // the second batch
    #pragma unroll
                    for (int i = 0; i < KS; ++i) lds_use(fb[i]);
                    static_for<0, KS>([&](auto d) { lds_read16<(n_k + d.value * 2 + half) * 1024>(fa[d.value], kaddr); });
                    __builtin_amdgcn_sched_barrier(0);
    #pragma unroll
                    for (int ks = 0; ks < KH; ++ks) {
                        if (FOUR_CHAINS && ((KH + ks) & 1)) {
                            st0b = mfma_16x16x32(fb[2 * ks], qf[KH + ks], st0b);
                            st1b = mfma_16x16x32(fb[2 * ks + 1], qf[KH + ks], st1b);
                        } else {
                            st0 = mfma_16x16x32(fb[2 * ks], qf[KH + ks], st0);
                            st1 = mfma_16x16x32(fb[2 * ks + 1], qf[KH + ks], st1);
                        }
                    }
                    if (FOUR_CHAINS) {
                        st0 += st0b;
                        st1 += st1b;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, KS>([&](auto d) { lds_read16<(n_k + (KS + d.value) * 2 + half) * 1024>(fb[d.value], kaddr); });
                    __builtin_amdgcn_sched_barrier(0);
                    float s[8];
    #pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s[e] = st0[e] * scale2;
                        s[4 + e] = st1[e] * scale2;
                    }
                    if (key0 + 31 > p_min || key0 < lo_max) {                      // the diagonal or the window's edge
    #pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int k0 = key0 + 4 * g + e, k1 = k0 + 16;
                            if (k0 > p || k0 < lo) s[e] = -INFINITY;
                            if (k1 > p || k1 < lo) s[4 + e] = -INFINITY;
                        }
                    }
                    float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
                    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                    if (__any(mx > m_ref + LAZY_LOG2)) {
                        const float m_new = fmaxf(m_ref, mx);
                        const float f = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
                        l *= f;
                        float f4[4];
    #pragma unroll
                        for (int e = 0; e < 4; ++e) f4[e] = __shfl(f, 4 * g + e, 64);
    #pragma unroll
                        for (int d = 0; d < HDT; ++d)
    #pragma unroll
                            for (int e = 0; e < 4; ++e) o[d][e] *= f4[e];
                        m_ref = m_new;
                    }
                    const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref;
                    frag16 pf;
                    float sum = 0.f;
    #pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float pe = __builtin_amdgcn_exp2f(s[e] - m_use);
                        sum += pe;
                        pf.v[e] = (__bf16)pe;
                    }
                    l += sum;
                    lds_settle_to<KS>();                              // the first batch of values
    #pragma unroll
                    for (int d = 0; d < KS; ++d) {
                        lds_use(fa[d]);
                        o[d] = mfma_16x16x32(pf, fa[d], o[d]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (ask_next) {
                        if constexpr (half == 0) read_keys_a(std::integral_constant<int, 1>{});
                        lds_settle_to<KS>();                          // the second batch of values (the next keys stay in flight)
                    } else {
                        lds_settle_to<0>();
                    }
    #pragma unroll
                    for (int d = 0; d < KS; ++d) {
                        lds_use(fb[d]);
                        o[KS + d] = mfma_16x16x32(pf, fb[d], o[KS + d]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (ask_next) {
                        if constexpr (half == 0) read_keys_b(std::integral_constant<int, 1>{});
                    }
                };
                if (see0) unit(std::integral_constant<int, 0>{}, false, see1);
                if (see1) unit(std::integral_constant<int, 1>{}, see0, false);
            } else {
                // (smaller heads: a unit is too short for batches; measured at 128, two batches were a fifth slower)
                static_for<0, 2>([&](auto halfc) {
                    constexpr int half = decltype(halfc)::value;
                    const int key0 = pi * AGAVE_PAGE + 32 * half;
                    if (key0 > p_max || key0 + 31 < lo_min) return;                // no column sees this unit
                    // all of the unit's key tiles are asked for at once, then multiplied; the value tiles
                    // are asked for before the exponentials and arrive while those are computed
                    frag16 fr[2 * KS > HDT ? 2 * KS : HDT];
                    static_for<0, KS>([&](auto ks) {
                        lds_read16<((2 * half) * KS + ks.value) * 1024>(fr[2 * ks.value], kaddr);
                        lds_read16<((2 * half + 1) * KS + ks.value) * 1024>(fr[2 * ks.value + 1], kaddr);
                    });
                    lds_settle();
    #pragma unroll
                    for (int i = 0; i < 2 * KS; ++i) lds_use(fr[i]);
                    // Head sizes up to 128: four chains of multiplications instead of two (measured at 128:
                    // 55 us instead of 70 for 2,048 tokens and 32 heads; at 256, with chains of 8 and 4, no gain).
                    constexpr bool FOUR_CHAINS = KS > 1 && KS <= 4;
                    f32x4_t st0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, st1 = st0, st0b = st0, st1b = st0;
    #pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        if (FOUR_CHAINS && (ks & 1)) {
                            st0b = mfma_16x16x32(fr[2 * ks], qf[ks], st0b);
                            st1b = mfma_16x16x32(fr[2 * ks + 1], qf[ks], st1b);
                        } else {
                            st0 = mfma_16x16x32(fr[2 * ks], qf[ks], st0);
                            st1 = mfma_16x16x32(fr[2 * ks + 1], qf[ks], st1);
                        }
                    }
                    if (FOUR_CHAINS) {
                        st0 += st0b;
                        st1 += st1b;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, HDT>([&](auto d) { lds_read16<(n_k + d.value * 2 + half) * 1024>(fr[d.value], kaddr); });
                    __builtin_amdgcn_sched_barrier(0);
                    float s[8];
    #pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s[e] = st0[e] * scale2;
                        s[4 + e] = st1[e] * scale2;
                    }
                    if (key0 + 31 > p_min || key0 < lo_max) {                      // the diagonal or the window's edge
    #pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int k0 = key0 + 4 * g + e, k1 = k0 + 16;
                            if (k0 > p || k0 < lo) s[e] = -INFINITY;
                            if (k1 > p || k1 < lo) s[4 + e] = -INFINITY;
                        }
                    }
                    float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
                    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                    if (__any(mx > m_ref + LAZY_LOG2)) {
                        const float m_new = fmaxf(m_ref, mx);
                        const float f = (m_ref == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_ref - m_new);
                        l *= f;
                        float f4[4];
    #pragma unroll
                        for (int e = 0; e < 4; ++e) f4[e] = __shfl(f, 4 * g + e, 64);
    #pragma unroll
                        for (int d = 0; d < HDT; ++d)
    #pragma unroll
                            for (int e = 0; e < 4; ++e) o[d][e] *= f4[e];
                        m_ref = m_new;
                    }
                    const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref;
                    frag16 pf;
                    float sum = 0.f;
    #pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float pe = __builtin_amdgcn_exp2f(s[e] - m_use);
                        sum += pe;
                        pf.v[e] = (__bf16)pe;
                    }
                    l += sum;
                    lds_settle();
    #pragma unroll
                    for (int d = 0; d < HDT; ++d) {
                        lds_use(fr[d]);
                        o[d] = mfma_16x16x32(pf, fr[d], o[d]);
                    }
                });
            }
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }
    if (!wave_on) return;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const int head = kvh * G + gh;
    if (it.n_pieces > 1) {
        // sums as they stand, with the reference they are relative to (in natural logarithms, as the merge reads it)
        if (g == 0 && col_ok) {
            const size_t ps = ((size_t)(t0 + tile0 + j) * a.nh + head) * max_pieces + it.piece;
            a.part_ml[ps * 2 + 0] = m_ref * 0.6931471805599453f;
            a.part_ml[ps * 2 + 1] = l;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 4 * g + e;
            if (tile0 + row >= n_new) continue;
            float* dst = a.part_o + (((size_t)(t0 + tile0 + row) * a.nh + head) * max_pieces + it.piece) * hd;
#pragma unroll
            for (int d = 0; d < HDT; ++d) dst[16 * d + j] = o[d][e];
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int row = 4 * g + e;                                // slot (position) this lane's values belong to
        const float lr = __shfl(l, row, 64);
        if (tile0 + row >= n_new) continue;
        const float inv = lr > 0.f ? 1.0f / lr : 0.f;
        bf16* dst = a.out + (size_t)(t0 + tile0 + row) * a.ldo + (size_t)head * hd;
#pragma unroll
        for (int d = 0; d < HDT; ++d) dst[16 * d + j] = f32_to_bf16(o[d][e] * inv);
    }
}

// ------------------------------------------------------------------ host side
// The partial results of the entry point that allocates nothing (noalloc.h).  In host code this
// name is a stand-in, not a device address: host code only ever uses the address that
// hipGetSymbolAddress gives for the current device, kept per device below.
static __device__ __align__(256) float scratch[AGAVE_NOALLOC_SCRATCH_FLOATS];
#define AGAVE_MAX_DEVICES 64
static float* g_scratch_on_device[AGAVE_MAX_DEVICES] = {};

static int check_common(const char* who, const AttnArgs& a, int N) {
    AGAVE_CHECK(N >= 0 && a.nh > 0 && a.nkv > 0 && a.hd > 0, "%s: bad sizes N=%d nh=%d nkv=%d hd=%d", who, N, a.nh, a.nkv, a.hd);
    AGAVE_CHECK(a.nh % a.nkv == 0, "%s: %d query heads are not a multiple of %d kv heads", who, a.nh, a.nkv);
    AGAVE_CHECK(a.hd % 16 == 0 && a.hd <= 256, "%s: head_dim %d is not a multiple of 16 up to 256", who, a.hd);
    AGAVE_CHECK(a.ldq >= (long)a.nh * a.hd && a.ldo >= (long)a.nh * a.hd, "%s: a row stride is below nh*hd", who);
    AGAVE_CHECK(a.ldq % 8 == 0 && ((uintptr_t)a.q % 16) == 0, "%s: q must be 16-byte aligned with a row stride multiple of 8", who);
    AGAVE_CHECK(a.q && a.out && a.k_pages && a.v_pages && a.table && a.base && a.tok_seq && a.tok_pos && a.width > 0 &&
                    a.n_pages > 0, "%s: null buffer or empty table", who);
    AGAVE_CHECK(a.window >= 0, "%s: negative window", who);
    return 0;
}

// More than the default allowance of LDS for large groups of heads; set once.
static int raise_decode_lds_allowance() {
    static bool raised = false;
    if (raised) return 0;
    const void* fns[] = {(const void*)attn_decode_mfma_kernel<4>, (const void*)attn_decode_mfma_kernel<8>,
                         (const void*)attn_decode_mfma_kernel<16>,
                         (const void*)attn_decode_fast_kernel<4, false>, (const void*)attn_decode_fast_kernel<8, false>,
                         (const void*)attn_decode_fast_kernel<16, false>,
                         (const void*)attn_decode_fast_kernel<4, true>, (const void*)attn_decode_fast_kernel<8, true>,
                         (const void*)attn_decode_fast_kernel<16, true>};
    for (const void* fn : fns)
        AGAVE_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) == hipSuccess,
                    "attn_decode_mfma: cannot raise the LDS allowance");
    raised = true;
    return 0;
}

// FUSED: a.q is the raw q projection and f says how to normalise and rotate it (head sizes 64, 128, 256 only).
// merge: run the pass that merges the splits' partial results into a.out (false: the caller's next
// kernel reads the partial results themselves).
template <bool FUSED>
static int launch_decode(const AttnArgs& a, const QkFuse& f, int N, hipStream_t stream, bool merge = true) {
    const int nh = a.nh, nkv = a.nkv, hd = a.hd, splits = a.splits;
    AGAVE_CHECK(splits >= 1 && splits <= COMBINE_MAX_SPLITS && a.pages_per_split >= 1, "attn_decode_mfma: bad split plan %d x %d", splits, a.pages_per_split);
    AGAVE_CHECK(splits == 1 || (a.part_o && a.part_ml), "attn_decode_mfma: splits need the partial buffers");
    AGAVE_CHECK(N <= 65535, "attn_decode_mfma: %d tokens exceed the grid limit", N);
    AGAVE_CHECK((2l * a.n_pages + 2) * (splits + 1) < (1l << 31), "attn_decode_mfma: %d pages in %d splits exceed 32-bit unit counts", a.n_pages, splits);
    if (N == 0) return 0;
    const int G = nh / nkv;
    dim3 grid(splits, nkv * ((G + 15) / 16), N);
    const int slots = G < 16 ? G : 16;
    size_t lds = ((size_t)4 * slots * hd + 4 * 16 * 2) * sizeof(float);
    if (FUSED) lds += (size_t)4 * hd * sizeof(float) + (size_t)16 * hd * sizeof(bf16);
    AGAVE_CHECK(lds <= 96 * 1024, "attn_decode_mfma: %zu bytes of LDS exceed what a workgroup may take", lds);
    if (raise_decode_lds_allowance()) return -1;
    if (FUSED) {
        AGAVE_CHECK(hd == 64 || hd == 128 || hd == 256, "attn_decode_fused: head_dim %d is not 64, 128 or 256", hd);
        if (hd == 64) attn_decode_fast_kernel<4, true><<<grid, 256, lds, stream>>>(a, f);
        else if (hd == 128) attn_decode_fast_kernel<8, true><<<grid, 256, lds, stream>>>(a, f);
        else attn_decode_fast_kernel<16, true><<<grid, 256, lds, stream>>>(a, f);
    } else if (hd == 64) attn_decode_fast_kernel<4, false><<<grid, 256, lds, stream>>>(a, f);
    else if (hd == 128) attn_decode_fast_kernel<8, false><<<grid, 256, lds, stream>>>(a, f);
    else if (hd == 256) attn_decode_fast_kernel<16, false><<<grid, 256, lds, stream>>>(a, f);
    else if (hd <= 64) attn_decode_mfma_kernel<4><<<grid, 256, lds, stream>>>(a);
    else if (hd <= 128) attn_decode_mfma_kernel<8><<<grid, 256, lds, stream>>>(a);
    else attn_decode_mfma_kernel<16><<<grid, 256, lds, stream>>>(a);
    AGAVE_LAUNCH_CHECK("attn_decode_mfma");
    if (splits > 1 && merge) {
        attn_combine_kernel<<<N * nh, hd >= 256 ? 256 : (hd >= 128 ? 128 : 64), 0, stream>>>(a.part_o, a.part_ml, a.out, a.ldo, nh, hd, splits);
        AGAVE_LAUNCH_CHECK("attn_combine");
    }
    return 0;
}

extern "C" int agave_attn_decode_mfma(const void* q, long ldq, void* out, long ldo, float* part_o, float* part_ml,
                                      const void* k_pages, const void* v_pages, const int* table, int width,
                                      const int* base, int n_pages, const int* tok_seq, const int* tok_pos, int N,
                                      int nh, int nkv, int hd, float scale, int window, int splits,
                                      int pages_per_split, int seq_is_token, int table_from_reach,
                                      hipStream_t stream) {
    AttnArgs a{(const bf16*)q, ldq, (bf16*)out, ldo, part_o, part_ml, (const uint4*)k_pages, (const uint4*)v_pages,
               table, width, base, n_pages, tok_seq, tok_pos, nullptr, 0, nh, nkv, hd, scale, window, splits,
               pages_per_split, seq_is_token, table_from_reach};
    if (check_common("attn_decode_mfma", a, N)) return -1;
    return launch_decode<false>(a, QkFuse{}, N, stream);
}

// The address of `scratch` on the current device, looked up once per device (every GPU holds
// its own copy of the array at its own address).
static int scratch_of_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    AGAVE_CHECK(e == hipSuccess, "attn_noalloc: hipGetDevice failed: %s", hipGetErrorString(e));
    AGAVE_CHECK(dev >= 0 && dev < AGAVE_MAX_DEVICES, "attn_noalloc: device %d is outside 0..%d", dev, AGAVE_MAX_DEVICES - 1);
    if (!g_scratch_on_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        AGAVE_CHECK(e == hipSuccess && p != nullptr, "attn_noalloc: hipGetSymbolAddress failed on device %d: %s", dev,
                    hipGetErrorString(e));
        g_scratch_on_device[dev] = (float*)p;
    }
    *out = g_scratch_on_device[dev];
    return 0;
}

extern "C" int agave_attn_noalloc_init(void) {
    float* p = nullptr;
    if (scratch_of_current_device(&p)) return -1;
    return raise_decode_lds_allowance();
}

extern "C" int agave_attn_decode_mfma_noalloc(const void* q, long ldq, void* out, long ldo, const void* k_pages,
                                              const void* v_pages, const int* table, int width, const int* base,
                                              int n_pages, const int* tok_seq, const int* tok_pos, int N, int nh,
                                              int nkv, int hd, float scale, int window, int splits,
                                              int pages_per_split, int seq_is_token, int table_from_reach,
                                              hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh > 0 && hd > 0 && splits >= 1, "attn_decode_mfma_noalloc: bad sizes N=%d nh=%d hd=%d splits=%d",
                N, nh, hd, splits);
    float* part_o = nullptr;
    float* part_ml = nullptr;
    if (splits > 1) {
        const unsigned long long slots = (unsigned long long)N * nh * splits;
        const unsigned long long need = slots * ((unsigned long long)hd + 2);
        AGAVE_CHECK(need <= AGAVE_NOALLOC_SCRATCH_FLOATS,
                    "attn_decode_mfma_noalloc: %d tokens x %d heads x %d splits x (%d + 2) = %llu floats exceed the "
                    "library's %u; use agave_attn_decode_mfma with buffers of your own",
                    N, nh, splits, hd, need, (unsigned)AGAVE_NOALLOC_SCRATCH_FLOATS);
        float* mine = nullptr;
        if (scratch_of_current_device(&mine)) return -1;
        part_o = mine;                                  // [token][head][split][hd]
        part_ml = mine + slots * hd;                    // [token][head][split][2]
    }
    AttnArgs a{(const bf16*)q, ldq, (bf16*)out, ldo, part_o, part_ml, (const uint4*)k_pages, (const uint4*)v_pages,
               table, width, base, n_pages, tok_seq, tok_pos, nullptr, 0, nh, nkv, hd, scale, window, splits,
               pages_per_split, seq_is_token, table_from_reach};
    if (check_common("attn_decode_mfma_noalloc", a, N)) return -1;
    return launch_decode<false>(a, QkFuse{}, N, stream);
}

// Decode attention that first does the q/k head norm, the rotation and the cache write of each
// sequence's new token (one token per sequence, positions tok_pos): q, k, v are the raw
// projections; k and v null for a run that appends nothing.  leave_partials: with more than one
// split, do not merge the splits' results into `out`; the caller's next kernel reads part_o and
// part_ml itself (gemm_mfma.hip: the output projection that merges while it stages its input).
extern "C" int agave_attn_decode_fused(const void* q, long ldq, const void* k, long ldk, const void* v, long ldv,
                                       const float* q_gain, const float* k_gain, float eps_q, float eps_k,
                                       const float* inv_freq, int rot_half, float pos_scale, void* out, long ldo,
                                       float* part_o, float* part_ml, void* k_pages, void* v_pages, const int* table,
                                       int width, const int* base, int n_pages, const int* tok_seq,
                                       const int* tok_pos, int N, int nh, int nkv, int hd, float scale, int window,
                                       int splits, int pages_per_split, int seq_is_token, int table_from_reach,
                                       int leave_partials, hipStream_t stream) {
    AttnArgs a{(const bf16*)q, ldq, (bf16*)out, ldo, part_o, part_ml, (const uint4*)k_pages, (const uint4*)v_pages,
               table, width, base, n_pages, tok_seq, tok_pos, nullptr, 0, nh, nkv, hd, scale, window, splits,
               pages_per_split, seq_is_token, table_from_reach};
    if (check_common("attn_decode_fused", a, N)) return -1;
    AGAVE_CHECK(!leave_partials || splits > 1, "attn_decode_fused: partial results exist only with more than one split");
    AGAVE_CHECK((k == nullptr) == (v == nullptr), "attn_decode_fused: k and v come together");
    AGAVE_CHECK(!k || (ldk >= (long)nkv * hd && ldv >= (long)nkv * hd), "attn_decode_fused: a k or v row stride is below nkv*hd");
    AGAVE_CHECK(rot_half >= 0 && 2 * rot_half <= hd && (rot_half == 0 || inv_freq), "attn_decode_fused: bad rotation (rotary_dim %d, head_dim %d)", 2 * rot_half, hd);
    QkFuse f{(const bf16*)k, ldk, (const bf16*)v, ldv, q_gain, k_gain, eps_q, eps_k, inv_freq, rot_half, pos_scale};
    return launch_decode<true>(a, f, N, stream, !leave_partials);
}

// A step that brings several tokens per sequence, any head size that is a multiple of 16 up to
// 256 (the general kernel; head sizes 64, 128 and 256 go through agave_attn_prefill_items).
extern "C" int agave_attn_prefill_mfma(const void* q, long ldq, void* out, long ldo, const void* k_pages,
                                       const void* v_pages, const int* table, int width, const int* base,
                                       int n_pages, const int* tok_seq, const int* tok_pos, const int* cu, int n_seqs,
                                       int max_new, int N, int nh, int nkv, int hd, float scale, int window,
                                       hipStream_t stream) {
    AttnArgs a{(const bf16*)q, ldq, (bf16*)out, ldo, nullptr, nullptr, (const uint4*)k_pages, (const uint4*)v_pages,
               table, width, base, n_pages, tok_seq, tok_pos, cu, n_seqs, nh, nkv, hd, scale, window, 1, 0, 0, 0};
    if (check_common("attn_prefill_mfma", a, N)) return -1;
    AGAVE_CHECK(cu && n_seqs > 0 && max_new > 0, "attn_prefill_mfma: needs the sequences' token ranges");
    AGAVE_CHECK(n_seqs <= 65535, "attn_prefill_mfma: %d sequences exceed the grid limit", n_seqs);
    if (N == 0) return 0;
    const int G = nh / nkv;
    const int qt_cap = hd > 128 ? 1 : (hd > 64 ? 2 : QT_MAX);   // heads per wave: what fits the register file
    const int qt_heads = G < qt_cap ? G : qt_cap;
    // the other heads of the group go to other waves of the workgroup
    int hw = 1;
    if (hd > 128) hw = G >= 4 ? 4 : (G >= 2 ? 2 : 1);
    const int wg_heads = qt_heads * hw, blk_len = (4 / hw) * 16;
    const int chunks = (G + wg_heads - 1) / wg_heads;
    AGAVE_CHECK(nkv * chunks <= 65535, "attn_prefill_mfma: too many head chunks");
    dim3 grid((max_new + blk_len - 1) / blk_len, nkv * chunks, n_seqs);
    // two pages (K and V tiles) in LDS
    const size_t lds = (size_t)2 * (4 * ((hd + 31) / 32) + (hd / 16) * 2) * 64 * sizeof(uint4);
    static bool raised = false;
    if (!raised) {
        const void* fns[] = {(const void*)attn_prefill_mfma_kernel<4, QT_MAX>, (const void*)attn_prefill_mfma_kernel<8, 2>,
                             (const void*)attn_prefill_mfma_kernel<16, 1>};
        for (const void* fn : fns)
            AGAVE_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024) == hipSuccess,
                        "attn_prefill_mfma: cannot raise the LDS allowance");
        raised = true;
    }
    if (hd <= 64) attn_prefill_mfma_kernel<4, QT_MAX><<<grid, 256, lds, stream>>>(a, qt_heads, hw);
    else if (hd <= 128) attn_prefill_mfma_kernel<8, 2><<<grid, 256, lds, stream>>>(a, qt_heads, hw);
    else attn_prefill_mfma_kernel<16, 1><<<grid, 256, lds, stream>>>(a, qt_heads, hw);
    AGAVE_LAUNCH_CHECK("attn_prefill_mfma");
    return 0;
}

// A step that brings several tokens per sequence, head sizes 64, 128 and 256, cut into items by
// the host (see PrefillItem).  items: n_items records of six ints in the order in which workgroups
// are to take them; `waves` (4 or 8) waves a workgroup, hw = agave_attn_prefill_items_hw(nh, nkv)
// heads side by side, so a block is (waves / hw) * 16 positions long; max_item_pages: the most
// pages any item has; tok_pieces[t]: pieces the block of token t is cut into (part_o
// [N][nh][max_pieces][hd] and part_ml [N][nh][max_pieces][2] take their partial results when
// max_pieces > 1).
extern "C" int agave_attn_prefill_items_hw(int nh, int nkv) {
    if (nkv <= 0 || nh % nkv != 0) return 0;
    const int G = nh / nkv;
    return G >= 4 ? 4 : (G >= 2 ? 2 : 1);
}

extern "C" int agave_attn_prefill_items(const void* q, long ldq, void* out, long ldo, const void* k_pages,
                                        const void* v_pages, const int* table, int width, const int* base,
                                        int n_pages, const int* tok_seq, const int* tok_pos, const int* cu, int n_seqs,
                                        int N, int nh, int nkv, int hd, float scale, int window, const int* items,
                                        int n_items, int waves, int max_item_pages, const int* tok_pieces,
                                        float* part_o, float* part_ml, int max_pieces, hipStream_t stream) {
    AttnArgs a{(const bf16*)q, ldq, (bf16*)out, ldo, part_o, part_ml, (const uint4*)k_pages, (const uint4*)v_pages,
               table, width, base, n_pages, tok_seq, tok_pos, cu, n_seqs, nh, nkv, hd, scale, window, 1, 0, 0, 0};
    if (check_common("attn_prefill_items", a, N)) return -1;
    AGAVE_CHECK(hd == 64 || hd == 128 || hd == 256, "attn_prefill_items: head_dim %d is not 64, 128 or 256", hd);
    AGAVE_CHECK(waves == 4 || waves == 8, "attn_prefill_items: %d waves a workgroup", waves);
    AGAVE_CHECK(cu && n_seqs > 0 && items && n_items >= 0 && max_item_pages >= 1, "attn_prefill_items: needs sequences and items");
    AGAVE_CHECK(max_pieces >= 1 && max_pieces <= MERGE_MAX_PIECES, "attn_prefill_items: %d pieces", max_pieces);
    AGAVE_CHECK(max_pieces == 1 || (part_o && part_ml && tok_pieces), "attn_prefill_items: pieces need the partial buffers");
    if (N == 0 || n_items == 0) return 0;
    const int hw = agave_attn_prefill_items_hw(nh, nkv);
    const int G = nh / nkv, chunks = (G + hw - 1) / hw, nkc = nkv * chunks;
    AGAVE_CHECK((long)n_items * nkc < (1L << 31), "attn_prefill_items: too many workgroups");
    // two pages (K and V tiles) in LDS, and the ids of the item's pages
    const size_t lds = (size_t)2 * (4 * (hd / 32) + (hd / 16) * 2) * 64 * sizeof(uint4) + (size_t)max_item_pages * sizeof(int);
    AGAVE_CHECK(lds <= 144 * 1024, "attn_prefill_items: items of %d pages do not fit the LDS", max_item_pages);
    static bool raised = false;
    if (!raised) {
        const void* fns[] = {(const void*)attn_prefill_fast_kernel<4, 4>, (const void*)attn_prefill_fast_kernel<8, 4>,
                             (const void*)attn_prefill_fast_kernel<16, 4>, (const void*)attn_prefill_fast_kernel<4, 8>,
                             (const void*)attn_prefill_fast_kernel<8, 8>, (const void*)attn_prefill_fast_kernel<16, 8>};
        for (const void* fn : fns)
            AGAVE_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024) == hipSuccess,
                        "attn_prefill_items: cannot raise the LDS allowance");
        raised = true;
    }
    const unsigned grid = (unsigned)((long)n_items * nkc);
    const PrefillItem* its = reinterpret_cast<const PrefillItem*>(items);
#define PF_LAUNCH(HDT_, NWV_) \
    attn_prefill_fast_kernel<HDT_, NWV_><<<grid, NWV_ * 64, lds, stream>>>(a, its, nkc, hw, max_pieces, max_item_pages)
    if (waves == 8) {
        if (hd == 64) PF_LAUNCH(4, 8);
        else if (hd == 128) PF_LAUNCH(8, 8);
        else PF_LAUNCH(16, 8);
    } else {
        if (hd == 64) PF_LAUNCH(4, 4);
        else if (hd == 128) PF_LAUNCH(8, 4);
        else PF_LAUNCH(16, 4);
    }
#undef PF_LAUNCH
    AGAVE_LAUNCH_CHECK("attn_prefill_items");
    if (max_pieces > 1) {
        AGAVE_CHECK((long)N * nh < (1L << 31) && ldo % 4 == 0 && ((uintptr_t)out % 8) == 0,
                    "attn_prefill_items: the merge needs 8-byte aligned output rows");
        const long rows = (long)N * nh;
        attn_merge_pieces_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, stream>>>(part_o, part_ml, tok_pieces, a.out, a.ldo,
                                                                                 nh, hd, max_pieces, rows);
        AGAVE_LAUNCH_CHECK("attn_merge_pieces");
    }
    return 0;
}
