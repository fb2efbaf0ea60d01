// Row-wise kernels of the decoder for gfx950: embedding with scale, RMSNorm with the
// residual sum, per-head q/k norm + rotation + cache write, GeGLU, casts.
//
// The residual stream is always 32-bit; activations (T) are float or bf16.  Norm sums,
// rotation angles and the residual sum are computed in 32-bit in both cases.
// Reference formulas: src/backend/kernels/cpu/norm.zig:7-40 (x * 1/sqrt(mean x^2 + eps) * g),
// src/backend/kernels/cpu/rope.zig:11-48 (split-half pairs), src/models/gemma3.zig:884-902
// (position scaled before the angle), src/backend/kernels/cpu/activation.zig:69-113 (tanh GELU).
#include "common_impl.h"
#include "qk_rope.h"

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_scale_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                                   float scale, float* __restrict__ out, int e, int vocab) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);   // the host rejects such ids; never read outside
    const T* row = table + (size_t)tok * e;
    float* o = out + (size_t)t * e;
    for (int i = threadIdx.x; i < e; i += blockDim.x) o[i] = ld(row + i) * scale;
}

extern "C" int agave_embed_scale(int dtype, const int* tokens, const void* table, float scale,
                                 float* out, int n_tokens, int e, int vocab, hipStream_t stream) {
    AGAVE_CHECK(n_tokens >= 0 && e > 0 && vocab > 0, "embed_scale: bad sizes N=%d e=%d vocab=%d", n_tokens, e, vocab);
    if (n_tokens == 0) return 0;
    const int threads = e >= 1024 ? 256 : (e >= 256 ? 128 : 64);
    if (dtype == AGAVE_F32)
        embed_scale_kernel<float><<<n_tokens, threads, 0, stream>>>(tokens, (const float*)table, scale, out, e, vocab);
    else if (dtype == AGAVE_BF16)
        embed_scale_kernel<bf16><<<n_tokens, threads, 0, stream>>>(tokens, (const bf16*)table, scale, out, e, vocab);
    else
        AGAVE_CHECK(false, "embed_scale: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("embed_scale");
    return 0;
}

// ------------------------------------------------------------------ residual + norms
//   r = rows ? rows[i] : i                       (row of h and of branch)
//   if branch: h[r] += post_gain ? rmsnorm(branch[r]) * post_gain : branch[r]
//   if out:    out[i] = rmsnorm(h[r]) * pre_gain
// Gains are 32-bit and already hold the "+1" where the architecture has it.
template <typename T>
__global__ void residual_norm_kernel(float* __restrict__ h, const T* __restrict__ branch, long ldb, int n_parts,
                                     long part_stride, const float* __restrict__ post_gain, float post_eps,
                                     T* __restrict__ out, long ldo, const float* __restrict__ pre_gain,
                                     float pre_eps, const int* __restrict__ rows, int e, const float* __restrict__ h_src) {
    __shared__ float red[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    float* hr = h + (size_t)r * e;
    const float* hs = h_src ? h_src + (size_t)r * e : hr;        // where the row is read (it is always written to h)
    float ss_h = 0.f;
    if (branch) {
        const T* br = branch + (size_t)r * ldb;
        // n_parts > 0: the branch is the sum of that many 32-bit slices, part_stride elements apart
        const float* parts = reinterpret_cast<const float*>(branch) + (size_t)r * ldb;
        auto at = [&](int c) {
            if (n_parts == 0) return ld(br + c);
            float v = 0.f;
            for (int p = 0; p < n_parts; ++p) v += parts[(size_t)p * part_stride + c];
            return v;
        };
        float inv = 1.0f;
        if (post_gain) {
            float ss = 0.f;
            for (int c = threadIdx.x; c < e; c += blockDim.x) {
                const float v = at(c);
                ss += v * v;
            }
            ss = block_sum(ss, red);
            inv = 1.0f / sqrtf(ss / (float)e + post_eps);
        }
        for (int c = threadIdx.x; c < e; c += blockDim.x) {
            const float y = post_gain ? at(c) * inv * post_gain[c] : at(c);
            const float hv = hs[c] + y;
            hr[c] = hv;
            ss_h += hv * hv;
        }
    } else if (out || h_src) {
        for (int c = threadIdx.x; c < e; c += blockDim.x) {
            const float hv = hs[c];
            if (h_src) hr[c] = hv;
            ss_h += hv * hv;
        }
    }
    if (out) {
        ss_h = block_sum(ss_h, red);
        const float inv = 1.0f / sqrtf(ss_h / (float)e + pre_eps);
        T* o = out + (size_t)i * ldo;
        for (int c = threadIdx.x; c < e; c += blockDim.x) st(o + c, hr[c] * inv * pre_gain[c]);
    }
}

// The same with the row held in registers (one read of every input, one write of every
// output): for rows of up to threads * 4 * VPT elements whose pointers allow 4-wide accesses.
template <typename T> __device__ __forceinline__ float4 load4(const T* p);
template <> __device__ __forceinline__ float4 load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4<bf16>(const bf16* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    float4 r;
    r.x = __uint_as_float(u.x << 16);
    r.y = __uint_as_float(u.x & 0xffff0000u);
    r.z = __uint_as_float(u.y << 16);
    r.w = __uint_as_float(u.y & 0xffff0000u);
    return r;
}
template <typename T> __device__ __forceinline__ void store4(T* p, float4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16>(bf16* p, float4 v) {
    uint2 u;
    u.x = f32x2_to_bf16x2(v.x, v.y);
    u.y = f32x2_to_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = u;
}

// Loads are written without a per-lane condition around them: under one the compiler splits a
// 16-byte load into four, each in a branch of its own.  A lane past the row's end reads the
// row's start instead; its values are left out of the sums and never stored.  Nothing that was
// loaded is touched before everything has been asked for, so the loads travel together.
__device__ __forceinline__ float sumsq(bool in, float4 v) { return in ? v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w : 0.f; }

template <typename T, int VPT, int PB>          // PB: slices asked for at a time
__global__ void residual_norm_fast_kernel(float* __restrict__ h, const T* __restrict__ branch, long ldb, int n_parts,
                                          long part_stride, const float* __restrict__ post_gain, float post_eps,
                                          T* __restrict__ out, long ldo, const float* __restrict__ pre_gain,
                                          float pre_eps, const int* __restrict__ rows, int e,
                                          const float* __restrict__ h_src) {
    __shared__ float red[16];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    float* hr = h + (size_t)r * e;
    const float* hs = h_src ? h_src + (size_t)r * e : hr;        // where the row is read (it is always written to h)
    const float4 z = float4{0.f, 0.f, 0.f, 0.f};
    float4 hv[VPT], bv[VPT], g1[VPT], g2[VPT], pv[PB][VPT];
    int col[VPT];
    bool in[VPT];
    // a gain that is not there is read from the row itself and not used
    const float* g1p = (branch && post_gain) ? post_gain : hr;
    const float* g2p = out ? pre_gain : hr;
#pragma unroll
    for (int v = 0; v < VPT; ++v) {
        const int c = (threadIdx.x + v * blockDim.x) * 4;
        in[v] = c < e;
        col[v] = in[v] ? c : 0;
        g1[v] = *reinterpret_cast<const float4*>(g1p + col[v]);
        g2[v] = *reinterpret_cast<const float4*>(g2p + col[v]);
        hv[v] = *reinterpret_cast<const float4*>(hs + col[v]);
        bv[v] = z;
    }
    if (branch && n_parts == 0) {
#pragma unroll
        for (int v = 0; v < VPT; ++v) bv[v] = load4(branch + (size_t)r * ldb + col[v]);
    } else if (branch) {
        // the branch is the sum of 32-bit slices (a product that was shared out along its columns)
        for (int p0 = 0; p0 < n_parts; p0 += PB) {
#pragma unroll
            for (int u = 0; u < PB; ++u) {
                const int p = p0 + u < n_parts ? p0 + u : n_parts - 1;
#pragma unroll
                for (int v = 0; v < VPT; ++v)
                    pv[u][v] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(branch) + (size_t)r * ldb +
                                                                col[v] + (size_t)p * part_stride);
            }
#pragma unroll
            for (int u = 0; u < PB; ++u) {
                const bool live = p0 + u < n_parts;
#pragma unroll
                for (int v = 0; v < VPT; ++v) {
                    bv[v].x += live ? pv[u][v].x : 0.f;
                    bv[v].y += live ? pv[u][v].y : 0.f;
                    bv[v].z += live ? pv[u][v].z : 0.f;
                    bv[v].w += live ? pv[u][v].w : 0.f;
                }
            }
        }
    }
    if (branch) {
        float inv = 1.0f;
        if (post_gain) {
            float ss = 0.f;
#pragma unroll
            for (int v = 0; v < VPT; ++v) ss += sumsq(in[v], bv[v]);
            ss = block_sum(ss, red);
            inv = 1.0f / sqrtf(ss / (float)e + post_eps);
        }
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            if (post_gain) {
                hv[v].x += bv[v].x * inv * g1[v].x;
                hv[v].y += bv[v].y * inv * g1[v].y;
                hv[v].z += bv[v].z * inv * g1[v].z;
                hv[v].w += bv[v].w * inv * g1[v].w;
            } else {
                hv[v].x += bv[v].x;
                hv[v].y += bv[v].y;
                hv[v].z += bv[v].z;
                hv[v].w += bv[v].w;
            }
            if (in[v]) *reinterpret_cast<float4*>(hr + col[v]) = hv[v];
        }
    } else if (h_src) {
#pragma unroll
        for (int v = 0; v < VPT; ++v)
            if (in[v]) *reinterpret_cast<float4*>(hr + col[v]) = hv[v];
    }
    if (out) {
        float ss = 0.f;
#pragma unroll
        for (int v = 0; v < VPT; ++v) ss += sumsq(in[v], hv[v]);
        ss = block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)e + pre_eps);
        T* o = out + (size_t)i * ldo;
#pragma unroll
        for (int v = 0; v < VPT; ++v) {
            if (in[v])
                store4(o + col[v], float4{hv[v].x * inv * g2[v].x, hv[v].y * inv * g2[v].y, hv[v].z * inv * g2[v].z,
                                          hv[v].w * inv * g2[v].w});
        }
    }
}

template <typename T>
static bool launch_residual_norm_fast(float* h, const void* branch, long ldb, int n_parts, long part_stride,
                                      const float* post_gain, float post_eps,
                                      void* out, long ldo, const float* pre_gain, float pre_eps, const int* rows,
                                      int n_rows, int e, const float* h_src, hipStream_t stream) {
    const size_t align = sizeof(T) * 4;
    if ((uintptr_t)h_src % 16 != 0) return false;
    if (e % 4 != 0 || e > 16384 || (branch && (ldb % 4 != 0 || (uintptr_t)branch % (n_parts ? 16 : align) != 0)) ||
        (n_parts && part_stride % 4 != 0) ||
        (out && (ldo % 4 != 0 || (uintptr_t)out % align != 0)) || (uintptr_t)h % 16 != 0 ||
        (post_gain && (uintptr_t)post_gain % 16 != 0) || (pre_gain && (uintptr_t)pre_gain % 16 != 0))
        return false;
    // few rows (decode steps): as many threads per row as it has float4, so that every thread's
    // loads are one round trip; many rows: 256 threads with several float4 each
    int threads;
    if (e <= 1024 || (n_rows <= 64 && e <= 4096)) {
        threads = 64 * ((e / 4 + 63) / 64);
    } else {
        // two float4 a thread if 1024 threads cover the row so, else four; no more waves than the row needs
        const int per = e / 4 <= 2048 ? 2 : 4;
        threads = 64 * ((e / 4 + per * 64 - 1) / (per * 64));
    }
    const int vpt = (e / 4 + threads - 1) / threads;
    // more than four slices (the output product's runs of heads): eight at a time when a thread holds one float4 of each
#define RN_FAST(V)                                                                                                    \
    if (n_parts > 4 && V == 1)                                                                                        \
        residual_norm_fast_kernel<T, V, 8><<<n_rows, threads, 0, stream>>>(h, (const T*)branch, ldb, n_parts,        \
                                                                           part_stride, post_gain, post_eps, (T*)out, \
                                                                           ldo, pre_gain, pre_eps, rows, e, h_src);   \
    else                                                                                                              \
    residual_norm_fast_kernel<T, V, 4><<<n_rows, threads, 0, stream>>>(h, (const T*)branch, ldb, n_parts, part_stride,  \
                                                                    post_gain, post_eps,                             \
                                                                    (T*)out, ldo, pre_gain, pre_eps, rows, e, h_src)
    if (vpt <= 1) RN_FAST(1);
    else if (vpt <= 2) RN_FAST(2);
    else RN_FAST(4);
#undef RN_FAST
    return true;
}

// n_parts > 0: branch points at that many 32-bit slices [n_rows][ldb], part_stride elements apart,
// whose sum is the branch (whatever dtype says, which then names out's type alone).
// h_src: the rows are read there instead of from h (and written to h as ever): the residual stream
// as a kernel left it that could not write it in place.
extern "C" int agave_residual_norm(int dtype, float* h, const void* branch, long ldb, int n_parts, long part_stride,
                                   const float* post_gain, float post_eps, void* out, long ldo, const float* pre_gain,
                                   float pre_eps, const int* rows, int n_rows, int e, const float* h_src,
                                   hipStream_t stream) {
    AGAVE_CHECK(n_rows >= 0 && e > 0, "residual_norm: bad sizes rows=%d e=%d", n_rows, e);
    AGAVE_CHECK(h != nullptr, "residual_norm: residual stream is null");
    AGAVE_CHECK(!(h_src && rows), "residual_norm: rows are gathered from the residual stream itself, not from another source");
    AGAVE_CHECK(!out || pre_gain, "residual_norm: output without its gain");
    AGAVE_CHECK(!branch || ldb >= e, "residual_norm: branch row stride %ld < %d", ldb, e);
    AGAVE_CHECK(!out || ldo >= e, "residual_norm: output row stride %ld < %d", ldo, e);
    AGAVE_CHECK(!(rows && branch), "residual_norm: row gather with a branch is not supported");
    AGAVE_CHECK(n_parts >= 0 && n_parts <= 64 && (n_parts == 0 || branch), "residual_norm: %d slices", n_parts);
    if (n_rows == 0 || (!branch && !out)) return 0;
    const int threads = e >= 2048 ? 512 : (e >= 512 ? 256 : 64);
    if (dtype == AGAVE_F32 && launch_residual_norm_fast<float>(h, branch, ldb, n_parts, part_stride, post_gain, post_eps,
                                                              out, ldo, pre_gain, pre_eps, rows, n_rows, e, h_src, stream)) {
    } else if (dtype == AGAVE_BF16 && launch_residual_norm_fast<bf16>(h, branch, ldb, n_parts, part_stride, post_gain,
                                                                     post_eps, out, ldo, pre_gain, pre_eps, rows, n_rows,
                                                                     e, h_src, stream)) {
    } else if (dtype == AGAVE_F32)
        residual_norm_kernel<float><<<n_rows, threads, 0, stream>>>(h, (const float*)branch, ldb, n_parts, part_stride,
                                                                    post_gain, post_eps,
                                                                    (float*)out, ldo, pre_gain, pre_eps, rows, e, h_src);
    else if (dtype == AGAVE_BF16)
        residual_norm_kernel<bf16><<<n_rows, threads, 0, stream>>>(h, (const bf16*)branch, ldb, n_parts, part_stride,
                                                                   post_gain, post_eps,
                                                                   (bf16*)out, ldo, pre_gain, pre_eps, rows, e, h_src);
    else
        AGAVE_CHECK(false, "residual_norm: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("residual_norm");
    return 0;
}

// ------------------------------------------------------------------ q/k head norm + rotation + cache write
// One wave per (token, head); q heads first, then k heads.  A k-head wave also stores the
// matching v head.  Cache pages: K [page][kv head][64 rows][hd], V transposed
// [page][kv head][hd][64 rows]; position p of sequence b lies in page
// table[b][p/64 - base[b]], row p % 64.
#define QK_HD_MAX 512
// NV: groups of 64 elements a head has (1, 2, 4 or 8).  Everything a wave needs is asked for at
// its start: its row with the gains and frequencies, the value row, the position and the
// sequence; the page id follows as soon as those two are there and travels during the arithmetic.
template <typename T, int NV>
__global__ void qk_norm_rope_kv_kernel(const T* q, long ldq, const T* __restrict__ k, long ldk,
                                       const T* __restrict__ v, long ldv, T* q_out, long ldqo,
                                       const float* __restrict__ q_gain, const float* __restrict__ k_gain,
                                       float eps_q, float eps_k, const float* __restrict__ inv_freq,
                                       int rot_half, float pos_scale, const int* __restrict__ tok_seq,
                                       const int* __restrict__ tok_pos, T* __restrict__ k_pages,
                                       T* __restrict__ v_pages, const int* __restrict__ table, int width,
                                       const int* __restrict__ base, int n_pages, int N, int nh, int nkv, int hd,
                                       int packed) {
    __shared__ float buf[4][NV * 64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int heads = nh + nkv;
    const int unit = blockIdx.x * 4 + wave;                 // (the host checks that the units fit 31 bits)
    const bool active = unit < N * heads;
    const int t = active ? unit / heads : 0;
    const int hh = active ? unit % heads : 0;
    const bool is_q = hh < nh;
    const int head = is_q ? hh : hh - nh;
    const T* src = is_q ? q + (size_t)t * ldq + (size_t)head * hd : k + (size_t)t * ldk + (size_t)head * hd;
    const float* gain = is_q ? q_gain : k_gain;
    const float eps = is_q ? eps_q : eps_k;
    float* y = buf[wave];

    const QkRow<T, NV> row = qk_row_load<T, NV>(src, gain, inv_freq, rot_half, hd, lane);
    const int p = tok_pos[t];
    T vreg[NV];
    int b = 0;
    if (!is_q) {                       // a key's wave also takes the value row, and looks its page up
        const T* sv = v + (size_t)t * ldv + (size_t)head * hd;
#pragma unroll
        for (int kk = 0; kk < NV; ++kk) {
            const int d = lane + 64 * kk;
            vreg[kk] = sv[d < hd ? d : 0];
        }
        b = tok_seq[t];
    }
    int col = 0;
    int pg = -1;                       // (kept as it was loaded: widening it would wait for the load here)
    const int row_in_page = p % AGAVE_PAGE;
    if (!is_q) {
        col = p / AGAVE_PAGE - base[b];
        if (col >= 0 && col < width) pg = table[(size_t)b * width + col];
    }
    qk_row_finish<T, NV>(row, y, gain != nullptr, eps, rot_half, (float)p * pos_scale, hd, lane, active);
    if (!active) return;
    if (is_q) {
        T* dst = q_out + (size_t)t * ldqo + (size_t)head * hd;
#pragma unroll
        for (int kk = 0; kk < NV; ++kk) {
            const int d = lane + 64 * kk;
            if (d < hd) st(dst + d, y[d]);
        }
        return;
    }
    if (pg < 0 || pg >= n_pages) return;   // a table the host built wrongly: write nothing
    if (!packed) {
        T* dk = k_pages + (((size_t)pg * nkv + head) * AGAVE_PAGE + row_in_page) * hd;
        T* dv = v_pages + ((size_t)pg * nkv + head) * hd * AGAVE_PAGE + row_in_page;
#pragma unroll
        for (int kk = 0; kk < NV; ++kk) {
            const int d = lane + 64 * kk;
            if (d < hd) {
                st(dk + d, y[d]);
                dv[(size_t)d * AGAVE_PAGE] = vreg[kk];
            }
        }
    } else {
        // matrix-core tile order (see attention_mfma.hip)
        const int ks_n = (hd + 31) >> 5;
        T* dk = k_pages + ((size_t)pg * nkv + head) * (size_t)(AGAVE_PAGE * ks_n * 32);
        T* dv = v_pages + ((size_t)pg * nkv + head) * (size_t)hd * AGAVE_PAGE;
        store_kv_row_packed_regs<T, NV>(dk, dv, y, vreg, row_in_page, hd, lane);
    }
}

template <typename T>
static void launch_qk_norm_rope_kv(int blocks, hipStream_t stream, const void* q, long ldq, const void* k, long ldk,
                                   const void* v, long ldv, void* q_out, long ldqo, const float* q_gain,
                                   const float* k_gain, float eps_q, float eps_k, const float* inv_freq, int rot_half,
                                   float pos_scale, const int* tok_seq, const int* tok_pos, void* k_pages, void* v_pages,
                                   const int* table, int width, const int* base, int n_pages, int N, int nh, int nkv,
                                   int hd, int packed) {
#define QK_LAUNCH(NV_)                                                                                               \
    qk_norm_rope_kv_kernel<T, NV_><<<blocks, 256, 0, stream>>>(                                                      \
        (const T*)q, ldq, (const T*)k, ldk, (const T*)v, ldv, (T*)q_out, ldqo, q_gain, k_gain, eps_q, eps_k, inv_freq, \
        rot_half, pos_scale, tok_seq, tok_pos, (T*)k_pages, (T*)v_pages, table, width, base, n_pages, N, nh, nkv, hd, \
        packed)
    if (hd <= 64) QK_LAUNCH(1);
    else if (hd <= 128) QK_LAUNCH(2);
    else if (hd <= 256) QK_LAUNCH(4);
    else QK_LAUNCH(8);
#undef QK_LAUNCH
}

extern "C" int agave_qk_norm_rope_kv(int dtype, const void* q, long ldq, const void* k, long ldk, const void* v,
                                     long ldv, void* q_out, long ldqo, const float* q_gain, const float* k_gain,
                                     float eps_q, float eps_k, const float* inv_freq, int rot_half, float pos_scale,
                                     const int* tok_seq, const int* tok_pos, void* k_pages, void* v_pages,
                                     const int* table, int width, const int* base, int n_pages, int N, int nh,
                                     int nkv, int hd, int packed, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh >= 0 && nkv >= 0 && hd > 0, "qk_norm_rope_kv: bad sizes N=%d nh=%d nkv=%d hd=%d", N, nh, nkv, hd);
    AGAVE_CHECK(hd <= QK_HD_MAX, "qk_norm_rope_kv: head_dim %d exceeds the supported maximum %d", hd, QK_HD_MAX);
    AGAVE_CHECK(rot_half >= 0 && 2 * rot_half <= hd, "qk_norm_rope_kv: rotary_dim %d exceeds head_dim %d", 2 * rot_half, hd);
    AGAVE_CHECK(rot_half == 0 || inv_freq, "qk_norm_rope_kv: rotation without a frequency table");
    AGAVE_CHECK(nh == 0 || (q && q_out && ldq >= (long)nh * hd && ldqo >= (long)nh * hd), "qk_norm_rope_kv: bad q buffers");
    AGAVE_CHECK(nkv == 0 || (k && v && k_pages && v_pages && table && base && tok_seq && width > 0 && n_pages > 0 &&
                             ldk >= (long)nkv * hd && ldv >= (long)nkv * hd),
                "qk_norm_rope_kv: bad k/v buffers or cache table");
    AGAVE_CHECK(tok_pos != nullptr, "qk_norm_rope_kv: positions are null");
    AGAVE_CHECK(!packed || (dtype == AGAVE_BF16 && hd % 16 == 0), "qk_norm_rope_kv: packed pages need bfloat16 and head_dim %% 16 == 0");
    const long units = (long)N * (nh + nkv);
    if (units == 0) return 0;
    AGAVE_CHECK(units < (1L << 31) - 4, "qk_norm_rope_kv: %ld (token, head) pairs exceed what one launch takes", units);
    const int blocks = (int)((units + 3) / 4);
    if (dtype == AGAVE_F32)
        launch_qk_norm_rope_kv<float>(blocks, stream, q, ldq, k, ldk, v, ldv, q_out, ldqo, q_gain, k_gain, eps_q, eps_k,
                                      inv_freq, rot_half, pos_scale, tok_seq, tok_pos, k_pages, v_pages, table, width,
                                      base, n_pages, N, nh, nkv, hd, packed);
    else if (dtype == AGAVE_BF16)
        launch_qk_norm_rope_kv<bf16>(blocks, stream, q, ldq, k, ldk, v, ldv, q_out, ldqo, q_gain, k_gain, eps_q, eps_k,
                                     inv_freq, rot_half, pos_scale, tok_seq, tok_pos, k_pages, v_pages, table, width,
                                     base, n_pages, N, nh, nkv, hd, packed);
    else
        AGAVE_CHECK(false, "qk_norm_rope_kv: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("qk_norm_rope_kv");
    return 0;
}

// ------------------------------------------------------------------ GeGLU
__device__ __forceinline__ float gelu_tanh(float x) {
    const float c = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x * x * x)));
}

// The gate's activation, by number (the feed-forward part knows the names): 0 gelu, tanh form;
// 1 silu, x / (1 + exp(-x)); 2 gelu with the error function; 3 relu.  Another one is another case
// here; only the tanh form also ends the matrix-core products (gemm_mfma.hip).
#define AGAVE_GATE_ACTS 4
__device__ __forceinline__ float gate_act(float x, int act) {
    switch (act) {
        case 0: return gelu_tanh(x);
        case 1: return x / (1.0f + expf(-x));
        case 2: return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
        default: return x > 0.f ? x : 0.f;
    }
}

template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gate, long ldg, const T* __restrict__ up, long ldu,
                                 T* __restrict__ out, long ldo, long total, int ff, int act) {
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / ff;
        const int c = (int)(idx % ff);
        const float g = ld(gate + r * ldg + c), u = ld(up + r * ldu + c);
        st(out + r * ldo + c, gate_act(g, act) * u);
    }
}

// out = act(gate) * up, row by row
extern "C" int agave_gated_act(int dtype, int act, const void* gate, long ldg, const void* up, long ldu, void* out,
                               long ldo, int n_rows, int ff, hipStream_t stream) {
    AGAVE_CHECK(n_rows >= 0 && ff > 0, "gated_act: bad sizes rows=%d ff=%d", n_rows, ff);
    AGAVE_CHECK(act >= 0 && act < AGAVE_GATE_ACTS, "gated_act: unknown activation %d", act);
    AGAVE_CHECK(ldg >= ff && ldu >= ff && ldo >= ff, "gated_act: a row stride is below %d", ff);
    if (n_rows == 0) return 0;
    const long total = (long)n_rows * ff;
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == AGAVE_F32)
        gated_act_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)gate, ldg, (const float*)up, ldu, (float*)out, ldo, total, ff, act);
    else if (dtype == AGAVE_BF16)
        gated_act_kernel<bf16><<<(int)blocks, 256, 0, stream>>>((const bf16*)gate, ldg, (const bf16*)up, ldu, (bf16*)out, ldo, total, ff, act);
    else
        AGAVE_CHECK(false, "gated_act: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("gated_act");
    return 0;
}

// (the tanh form of gelu under its older name)
extern "C" int agave_geglu(int dtype, const void* gate, long ldg, const void* up, long ldu, void* out, long ldo,
                           int n_rows, int ff, hipStream_t stream) {
    return agave_gated_act(dtype, 0, gate, ldg, up, ldu, out, ldo, n_rows, ff, stream);
}

// ------------------------------------------------------------------ a product's bias
// y[r][c] += bias[c], summed in 32-bit and rounded to y's element type once
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, long ldy, const float* __restrict__ bias, long total, int n_cols) {
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / n_cols;
        const int c = (int)(idx % n_cols);
        T* at = y + r * ldy + c;
        st(at, ld(at) + bias[c]);
    }
}

extern "C" int agave_add_bias(int dtype, void* y, long ldy, const float* bias, int n_rows, int n_cols, hipStream_t stream) {
    AGAVE_CHECK(n_rows >= 0 && n_cols > 0 && ldy >= n_cols, "add_bias: bad sizes rows=%d cols=%d stride=%ld", n_rows, n_cols, ldy);
    AGAVE_CHECK(y != nullptr && bias != nullptr, "add_bias: null tensor");
    if (n_rows == 0) return 0;
    const long total = (long)n_rows * n_cols;
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == AGAVE_F32)
        add_bias_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)y, ldy, bias, total, n_cols);
    else if (dtype == AGAVE_BF16)
        add_bias_kernel<bf16><<<(int)blocks, 256, 0, stream>>>((bf16*)y, ldy, bias, total, n_cols);
    else
        AGAVE_CHECK(false, "add_bias: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("add_bias");
    return 0;
}

// ------------------------------------------------------------------ logits: a factor, and a soft cap
// x <- cap * tanh(scale * x / cap) if cap > 0, scale * x otherwise (32-bit logits, in place)
__global__ void scale_cap_kernel(float* __restrict__ x, long n, float scale, float cap) {
    const float inv = cap > 0.f ? 1.0f / cap : 0.f;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const float v = x[i] * scale;
        x[i] = cap > 0.f ? cap * tanhf(v * inv) : v;
    }
}

extern "C" int agave_scale_cap(float* x, long n, float scale, float cap, hipStream_t stream) {
    AGAVE_CHECK(n >= 0 && cap >= 0.f, "scale_cap: bad arguments n=%ld cap=%g", n, (double)cap);
    AGAVE_CHECK(x != nullptr || n == 0, "scale_cap: null tensor");
    if (n == 0) return 0;
    long blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    scale_cap_kernel<<<(int)blocks, 256, 0, stream>>>(x, n, scale, cap);
    AGAVE_LAUNCH_CHECK("scale_cap");
    return 0;
}

// ------------------------------------------------------------------ rows of the residual stream, as they are
// out[i] = h[rows[i]] (rows null: h[i]) in out's element type: what a model without a final norm
// hands to its output matrix.
template <typename TO>
__global__ void gather_rows_kernel(const float* __restrict__ h, const int* __restrict__ rows, TO* __restrict__ out,
                                   long ldo, int e) {
    const int i = blockIdx.x;
    const float* src = h + (size_t)(rows ? rows[i] : i) * e;
    for (int c = threadIdx.x; c < e; c += blockDim.x) st(out + (size_t)i * ldo + c, src[c]);
}

extern "C" int agave_gather_rows(int dtype_out, const float* h, const int* rows, void* out, long ldo, int n_rows, int e,
                                 hipStream_t stream) {
    AGAVE_CHECK(n_rows >= 0 && e > 0 && ldo >= e, "gather_rows: bad sizes rows=%d e=%d stride=%ld", n_rows, e, ldo);
    AGAVE_CHECK(h != nullptr && out != nullptr, "gather_rows: null tensor");
    if (n_rows == 0) return 0;
    if (dtype_out == AGAVE_F32)
        gather_rows_kernel<float><<<n_rows, 256, 0, stream>>>(h, rows, (float*)out, ldo, e);
    else if (dtype_out == AGAVE_BF16)
        gather_rows_kernel<bf16><<<n_rows, 256, 0, stream>>>(h, rows, (bf16*)out, ldo, e);
    else
        AGAVE_CHECK(false, "gather_rows: unknown dtype %d", dtype_out);
    AGAVE_LAUNCH_CHECK("gather_rows");
    return 0;
}

// ------------------------------------------------------------------ casts
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        st(out + i, ld(in + i));
}

extern "C" int agave_cast(int dtype_in, const void* in, int dtype_out, void* out, long n, hipStream_t stream) {
    AGAVE_CHECK(n >= 0, "cast: negative count");
    if (n == 0) return 0;
    long blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype_in == AGAVE_F32 && dtype_out == AGAVE_BF16)
        cast_kernel<float, bf16><<<(int)blocks, 256, 0, stream>>>((const float*)in, (bf16*)out, n);
    else if (dtype_in == AGAVE_BF16 && dtype_out == AGAVE_F32)
        cast_kernel<bf16, float><<<(int)blocks, 256, 0, stream>>>((const bf16*)in, (float*)out, n);
    else if (dtype_in == AGAVE_F32 && dtype_out == AGAVE_F32)
        cast_kernel<float, float><<<(int)blocks, 256, 0, stream>>>((const float*)in, (float*)out, n);
    else if (dtype_in == AGAVE_BF16 && dtype_out == AGAVE_BF16)
        cast_kernel<bf16, bf16><<<(int)blocks, 256, 0, stream>>>((const bf16*)in, (bf16*)out, n);
    else
        AGAVE_CHECK(false, "cast: unknown dtypes %d -> %d", dtype_in, dtype_out);
    AGAVE_LAUNCH_CHECK("cast");
    return 0;
}
