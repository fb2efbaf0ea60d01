// bfloat16 matrix products on the matrix cores of gfx950: Y[M,N] = X[M,K] * W[N,K]^T with
// 32-bit accumulation, W in the packed layout of mfma.h.
//
//  * pack_w16: row-major W -> packed tiles (optionally interleaving the rows of a stacked
//    [gate; up] matrix so that one lane ends up with gate and up of the same column);
//  * embed_scale_packed: the embedding gather reading rows out of a packed table (tied head);
//  * gemm_skinny: M <= 64 tokens (decode): the weight streams through once at memory speed,
//    K is split over the four waves of a workgroup, partial sums meet in LDS;
//  * gemm_tiled: large M (prefill): 128x128 tiles per workgroup, X staged through LDS.
//
// The reference computes the same products row by row: one workgroup per output row with a
// block reduction (src/backend/kernels/rocm/gemv_bf16.zig:6-24), looped over tokens for a
// batch (src/backend/rocm.zig:1177-1190).
#include "common_impl.h"
#include "mfma.h"

// four consecutive outputs at once (the address is a multiple of four elements)
template <typename T> __device__ __forceinline__ void store4(T* p, float4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16>(bf16* p, float4 v) {
    uint2 u;
    u.x = f32x2_to_bf16x2(v.x, v.y);
    u.y = f32x2_to_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = u;
}

// ------------------------------------------------------------------ packing
// mode 0: packed row p is source row p.
// mode 1: the source is [gate (ff rows); up (ff rows)]; within a block of 16 packed rows, rows
//         4q+0, 4q+1 are gate[8nb+2q], gate[8nb+2q+1] and rows 4q+2, 4q+3 the same two of up.
__global__ void pack_w16_kernel(const bf16* __restrict__ W, long ldw, uint4* __restrict__ P, int N, int K,
                                int NB, int KB, int mode, int ff) {
    const long tile = blockIdx.x;          // source order: nb * KB + kb
    const int nb = (int)(tile / KB), kb = (int)(tile % KB);
    const int lane = threadIdx.x;
    const int i = lane & 15, g = lane >> 4;
    long src = -1;
    if (mode == 0) {
        const int p = nb * 16 + i;
        if (p < N) src = p;
    } else {
        const int q = i >> 2, e = i & 3;
        const int col = 8 * nb + 2 * q + (e & 1);
        if (col < ff) src = (e < 2) ? col : (long)ff + col;
    }
    frag16 f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int k = kb * 32 + g * 8 + e;
        bf16 z;
        z.x = 0;
        f.h[e] = (src >= 0 && k < K) ? W[src * ldw + k] : z;
    }
    P[w_tile(nb, kb, NB, KB) * 64 + lane] = f.u;
}

extern "C" int agave_pack_w16(const void* W, long ldw, void* P, int N, int K, int mode, int ff, hipStream_t stream) {
    AGAVE_CHECK(N > 0 && K > 0 && ldw >= K, "pack_w16: bad sizes N=%d K=%d ldw=%ld", N, K, ldw);
    AGAVE_CHECK(mode == 0 || (mode == 1 && N == 2 * ff), "pack_w16: interleaved mode needs N == 2*ff");
    const int rows = mode == 0 ? N : ff * 2;
    const int NB = mode == 0 ? (N + 15) / 16 : (ff + 7) / 8;
    const int KB = (K + 31) / 32;
    (void)rows;
    AGAVE_CHECK((long)NB * KB < 2147483647L, "pack_w16: too many tiles");
    pack_w16_kernel<<<NB * KB, 64, 0, stream>>>((const bf16*)W, ldw, (uint4*)P, N, K, NB, KB, mode, ff);
    AGAVE_LAUNCH_CHECK("pack_w16");
    return 0;
}

// ------------------------------------------------------------------ embedding from a packed table
__global__ void embed_scale_packed_kernel(const int* __restrict__ tokens, const uint4* __restrict__ P, float scale,
                                          float* __restrict__ out, int e, int vocab, int KB) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const int nb = tok >> 4, i = tok & 15;
    float* o = out + (size_t)t * e;
    // a thread per piece of 8 columns where the row allows it: the row then arrives in one round trip
    for (int piece = threadIdx.x; piece * 8 < e; piece += blockDim.x) {
        const int kb = piece >> 2, g = piece & 3;
        frag16 f;
        f.u = P[w_tile(nb, kb, (vocab + 15) / 16, KB) * 64 + i + 16 * g];
        const int k0 = piece * 8;
        if (k0 + 8 <= e && e % 4 == 0 && ((uintptr_t)out & 15) == 0) {
            *reinterpret_cast<float4*>(o + k0) = float4{bf16_to_f32(f.h[0]) * scale, bf16_to_f32(f.h[1]) * scale,
                                                        bf16_to_f32(f.h[2]) * scale, bf16_to_f32(f.h[3]) * scale};
            *reinterpret_cast<float4*>(o + k0 + 4) = float4{bf16_to_f32(f.h[4]) * scale, bf16_to_f32(f.h[5]) * scale,
                                                            bf16_to_f32(f.h[6]) * scale, bf16_to_f32(f.h[7]) * scale};
        } else {
#pragma unroll
            for (int x = 0; x < 8; ++x)
                if (k0 + x < e) o[k0 + x] = bf16_to_f32(f.h[x]) * scale;
        }
    }
}

extern "C" int agave_embed_scale_packed(const int* tokens, const void* P, float scale, float* out, int n_tokens,
                                        int e, int vocab, hipStream_t stream) {
    AGAVE_CHECK(n_tokens >= 0 && e > 0 && vocab > 0, "embed_scale_packed: bad sizes");
    if (n_tokens == 0) return 0;
    const int pieces = (e + 7) / 8;
    const int threads = pieces >= 1024 ? 1024 : 64 * ((pieces + 63) / 64);
    embed_scale_packed_kernel<<<n_tokens, threads, 0, stream>>>(tokens, (const uint4*)P, scale, out, e, vocab, (e + 31) / 32);
    AGAVE_LAUNCH_CHECK("embed_scale_packed");
    return 0;
}

// ------------------------------------------------------------------ skinny product (decode)
// gelu with the tanh approximation: 0.5 (1 + tanh u) = 1 / (1 + exp(-2u)), u = sqrt(2/pi) (x + 0.044715 x^3);
// the hardware's exp2 and reciprocal (about an ulp each) stand for tanhf, whose many instructions
// a product's last step has no time for
__device__ __forceinline__ float gelu_tanh_f(float x) {
    const float c2 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;        // -2 sqrt(2/pi) log2(e)
    const float e = __builtin_amdgcn_exp2f(c2 * (x + 0.044715f * x * x * x));
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// R: row blocks (of 16 weight rows) per workgroup; MT: tiles of 16 tokens; EPI 0: store, 1: GeGLU;
// NW: waves per workgroup, which share the columns (few row blocks -> many waves each, so
// that a small matrix still has enough loads in flight; the sums meet in LDS, never in memory).
// A wave takes chunks of KS k-steps (tiles of 32 columns): 128 columns for up to 32 tokens, 64 beyond
// (the registers that hold a chunk in flight grow with R and MT).  Every workgroup stages all of X
// once, so with many tokens R grows: X then comes from L2 once per R row blocks.  XR: rows of the
// token tile that are loaded at all (4, 8 or 16 when there is one tile; a workgroup reads as many
// bytes of X as of W when all 16 are loaded, so a step of 8 tokens should not load 16).
template <int R, int MT, int EPI, int NW, typename TC, int XR>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ X, long ldx,
                                                          const uint4* __restrict__ Wp, TC* __restrict__ Y,
                                                          long ldy, int M, int N, int K, int KB, int NB, long part_stride) {
    constexpr int KS = MT <= 2 ? 4 : 2;
    constexpr int ROW = KS * 32 + 8;                                // bf16 per staged X row, 16 bytes of padding
    constexpr int PIECES = KS * 4;                                  // 16-byte pieces per staged row
    constexpr int RPI = 64 / PIECES;                                // rows one load instruction covers
    constexpr int NI = XR / RPI;                                    // load instructions per tile of 16 tokens
    static_assert(XR == 16 || MT == 1, "only a single tile of tokens may be cut short");
    static_assert(XR % RPI == 0 && XR <= 16, "rows of the tile must be whole load instructions");
    // staged X: [wave][MT][16 rows][ROW]; afterwards the same memory holds the waves' partial sums
    constexpr int XS_WAVE = MT * 16 * ROW;                          // bf16 elements
    constexpr int RED_WAVE = R * MT * 64 * 4;                       // floats
    constexpr int LDS_BYTES = (NW * XS_WAVE * 2 > NW * RED_WAVE * 4) ? NW * XS_WAVE * 2 : NW * RED_WAVE * 4;
    static_assert(LDS_BYTES <= 160 * 1024, "the staged tokens or the partial sums do not fit the LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[LDS_BYTES];
    bf16* xs = reinterpret_cast<bf16*>(smem);
    float* red = reinterpret_cast<float*>(smem);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j = lane & 15, g = lane >> 4;
    const int xr = lane / PIECES, xp = lane % PIECES;               // staging: row within an instruction, piece
    const int nb0 = blockIdx.x * R;
    // gridDim.y workgroups share a row block's columns: each takes a run of chunks and leaves its
    // sums in its own slice of Y (partial sums then, which the reader adds up)
    const int n_chunks_all = (KB + KS - 1) / KS;
    const int c_lo = (int)((long)blockIdx.y * n_chunks_all / gridDim.y);
    const int n_chunks = (int)((long)(blockIdx.y + 1) * n_chunks_all / gridDim.y) - c_lo;
    const int n_iter = (n_chunks + NW - 1) / NW;
    Y += (size_t)blockIdx.y * part_stride;

    f32x4_t acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[r][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // S chunks are in flight per wave: the loads of chunk i+S are issued as soon as chunk i has
    // been multiplied, long before they are waited for.
    constexpr int S = (R * MT <= 2 && NW <= 8) ? 3 : 2;      // 16 waves leave 128 registers a lane
    frag16 wreg[S][R][KS];
    uint4 xreg[S][MT][NI];
    bf16* my_xs = xs + wave * XS_WAVE;

    // addresses that do not depend on the chunk; rows past the end repeat the last one (their
    // results are never stored)
    const uint4* wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wrow[r] = Wp + w_tile(nb0 + r < NB ? nb0 + r : NB - 1, 0, NB, KB) * 64 + lane;
    const size_t wstep = (w_tile(0, 1, NB, KB) - w_tile(0, 0, NB, KB)) * 64;        // from a k-step to the next
    const bf16* xrow[MT][NI];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int row = mt * 16 + RPI * i + xr;
            xrow[mt][i] = X + (size_t)(row < M ? row : M - 1) * ldx;
        }

    // Workgroups walk the columns in step: the tiles of a k-step lie side by side in the packed
    // matrix, so what the workgroups read at any moment is one contiguous stretch of memory.
    // Loads are issued without any condition around them (a chunk past the end repeats the last
    // one and is not used): only then can a wait name the loads it needs and leave the younger
    // ones in flight.
#define SK_LOAD(ST, IT)                                                                          \
    {                                                                                            \
        int c_ = (IT) * NW + wave;                    /* chunks are dealt to the waves in turn */ \
        c_ = (c_ < n_chunks ? c_ : n_chunks - 1) + c_lo;                                         \
        _Pragma("unroll") for (int r = 0; r < R; ++r)                                            \
            _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                  \
                const int kb = c_ * KS + ks;           /* past the last tile: any tile, X is zero there */ \
                wreg[ST][r][ks].u = wrow[r][(size_t)(kb < KB ? kb : KB - 1) * wstep];            \
            }                                                                                    \
        const int k_ = c_ * (KS * 32) + xp * 8;         /* past the last column: any piece, zeroed when used */ \
        _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                        \
            _Pragma("unroll") for (int i = 0; i < NI; ++i)                                       \
                xreg[ST][mt][i] = *reinterpret_cast<const uint4*>(xrow[mt][i] + (k_ < K ? k_ : 0)); \
    }
    // The staged rows are this wave's own and LDS serves a wave's accesses in order: no barrier.
#define SK_USE(ST, IT)                                                                           \
    if ((IT) * NW + wave < n_chunks) {                                                           \
        const bool in_ = ((IT) * NW + wave + c_lo) * (KS * 32) + xp * 8 < K;                     \
        _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                        \
            _Pragma("unroll") for (int i = 0; i < NI; ++i)                                       \
                *reinterpret_cast<uint4*>(my_xs + (mt * 16 + RPI * i + xr) * ROW + xp * 8) =     \
                    in_ ? xreg[ST][mt][i] : uint4{0, 0, 0, 0};                                   \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks)                                        \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                  \
                frag16 xb;                                                                       \
                xb.u = *reinterpret_cast<const uint4*>(my_xs + (mt * 16 + j) * ROW + ks * 32 + g * 8); \
                _Pragma("unroll") for (int r = 0; r < R; ++r)                                    \
                    acc[r][mt] = mfma_16x16x32(wreg[ST][r][ks], xb, acc[r][mt]);                 \
            }                                                                                    \
    }

    SK_LOAD(0, 0)
    SK_LOAD(1, 1)
    if constexpr (S == 3) SK_LOAD(2, 2)
    int it = 0;
    for (; it + 2 * S <= n_iter; it += S) {           // steady state: every load is of a chunk that exists
        SK_USE(0, it)
        SK_LOAD(0, it + S)
        SK_USE(1, it + 1)
        SK_LOAD(1, it + 1 + S)
        if constexpr (S == 3) {
            SK_USE(2, it + 2)
            SK_LOAD(2, it + 2 + S)
        }
    }
    // the last chunks: at most S - 1 more loads
    SK_USE(0, it)
    if (it + S < n_iter) SK_LOAD(0, it + S)
    SK_USE(1, it + 1)
    if (it + 1 + S < n_iter) SK_LOAD(1, it + 1 + S)
    if constexpr (S == 3) SK_USE(2, it + 2)
    SK_USE(0, it + S)
    SK_USE(1, it + 1 + S)
#undef SK_LOAD
#undef SK_USE
    __syncthreads();      // the staged rows give way to the partial sums

    // the waves' partial sums meet in LDS
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            *reinterpret_cast<f32x4_t*>(red + ((size_t)wave * R * MT + r * MT + mt) * 256 + lane * 4) = acc[r][mt];
    __syncthreads();
    for (int tile = wave; tile < R * MT; tile += NW) {
        const int r = tile / MT, mt = tile % MT;
        f32x4_t s = *reinterpret_cast<const f32x4_t*>(red + (size_t)tile * 256 + lane * 4);
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            const f32x4_t p = *reinterpret_cast<const f32x4_t*>(red + ((size_t)w * R * MT + tile) * 256 + lane * 4);
            s += p;
        }
        const int m = mt * 16 + j;
        if (m >= M || nb0 + r >= NB) continue;
        if (EPI == 0) {
            const int n = (nb0 + r) * 16 + g * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) st(Y + (size_t)m * ldy + n + e, s[e]);
        } else {
            const int n = (nb0 + r) * 8 + g * 2;      // N counts output columns (ff)
            if (n < N) st(Y + (size_t)m * ldy + n, gelu_tanh_f(s[0]) * s[2]);
            if (n + 1 < N) st(Y + (size_t)m * ldy + n + 1, gelu_tanh_f(s[1]) * s[3]);
        }
    }
}

template <int R, int MT, int EPI, int NW, typename TC, int XR>
static void launch_skinny_nw(const void* X, long ldx, const void* Wp, void* Y, long ldy, int M, int N, int K, int KB,
                             int NB, int splits, hipStream_t stream) {
    const dim3 grid((NB + R - 1) / R, splits);
    gemm_skinny_kernel<R, MT, EPI, NW, TC, XR><<<grid, NW * 64, 0, stream>>>((const bf16*)X, ldx, (const uint4*)Wp, (TC*)Y,
                                                                        ldy, M, N, K, KB, NB, (long)M * ldy);
}

// Waves per workgroup: the fewest that put some 640 waves on the chip.  Every wave keeps two
// or three chunks of loads in flight, which covers the memory's latency with few waves; more
// waves only add to the merge of the sums and deal the chunks less evenly.
static int skinny_waves(int groups, int n_chunks, int max_nw) {
    int nw = 4;
    while (nw < max_nw && (long)groups * nw < 640 && nw < n_chunks) nw *= 2;
    return nw;
}

template <int R, int MT, int EPI, typename TC, int XR>
static void launch_skinny(const void* X, long ldx, const void* Wp, void* Y, long ldy, int M, int N, int K, int KB,
                          int NB, int splits, hipStream_t stream) {
    constexpr int KS = MT <= 2 ? 4 : 2;
    constexpr int MAX_NW = (R * MT <= 2) ? 16 : (R * MT <= 8 ? 8 : 4);
    const int n_chunks = ((KB + KS - 1) / KS) / splits;
    const int groups = (NB + R - 1) / R * splits;
    const int nw = skinny_waves(groups, n_chunks, MAX_NW);
    if (nw == 16) {
        if constexpr (MAX_NW >= 16) launch_skinny_nw<R, MT, EPI, 16, TC, XR>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream);
    } else if (nw == 8) {
        if constexpr (MAX_NW >= 8) launch_skinny_nw<R, MT, EPI, 8, TC, XR>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream);
    } else {
        launch_skinny_nw<R, MT, EPI, 4, TC, XR>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream);
    }
}

// How a product of few tokens is cut into workgroups: r row blocks (of 16 weight rows) by 1/z of
// the columns each.  z > 1 only where the reader takes 32-bit slices that add up to the product.
//
// 256 workgroups run at a time, and a compute unit cannot pull more than some 40 GB/s: the
// workgroups must fill their rounds evenly (1280 row blocks at 4 a workgroup are 320
// workgroups, a quarter of the compute units with twice the others' work, and take a third
// longer than at 5 a workgroup; 160 row blocks leave 96 compute units idle).  Every workgroup
// reads the X columns of its slice, so what comes from L2 besides the weights is X once per
// group of r row blocks, whatever z is: with many tokens, many row blocks a workgroup and many
// slices are better than few of either (X counted half, it comes from L2).  A slice more costs
// its partial sums.  With up to 8 tokens X is small, and the older, measured rule stands.
struct SkinnyCut { int r, z; };
// only_z > 0: the best row blocks for exactly that many slices.
static SkinnyCut cut_skinny(int M, int NB, int KB, int max_z, int only_z = 0) {
    const int mt = (M + 15) / 16;
    auto filled = [](long groups) { return (double)groups / (256.0 * ((groups + 255) / 256)); };
    SkinnyCut cut = {1, 1};
    // (9 to 16 tokens go with the larger batches: several row blocks a workgroup, measured 4 % of a
    // step faster at 16 tokens and 4B sizes, 7 % at 12B sizes, the same at 9 tokens)
    if (M <= 8) {
        cut.r = NB >= 4096 ? 2 : 1;
        const long groups = (NB + cut.r - 1) / cut.r;
        if (only_z > 0) {
            cut.z = only_z;
            return cut;
        }
        if (M < 4 || KB < 128 || filled(groups) >= 0.85) return cut;       // (one or two tokens gain nothing)
        double best = filled(groups) + 0.1;
        for (int z = 2; z <= 4 && z <= max_z && KB / z >= 32; ++z)
            if (filled(groups * z) > best) {
                best = filled(groups * z);
                cut.z = z;
            }
        return cut;
    }
    static const int cand2[] = {1, 2, 4, 5, 0}, cand3[] = {1, 2, 4, 5, 0};
    const int* cand = mt <= 2 ? cand2 : cand3;
    const int n_chunks = (KB + (mt <= 2 ? 4 : 2) - 1) / (mt <= 2 ? 4 : 2);
    double best = 1e30;
    for (int i = 0; cand[i]; ++i) {
        for (int z = only_z > 0 ? only_z : 1; z <= (only_z > 0 ? only_z : (max_z < 8 ? max_z : 8)); ++z) {
            if (only_z == 0 && z > 1 && n_chunks / z < 8) break;
            const long groups = (long)((NB + cand[i] - 1) / cand[i]) * z;
            const double cost = (1.0 + 0.5 * mt / cand[i]) / filled(groups) + 0.03 * (z - 1);
            if (cost < best) {
                best = cost;
                cut = {cand[i], z};
            }
        }
    }
    return cut;
}

template <int EPI, typename TC>
static int dispatch_skinny(const void* X, long ldx, const void* Wp, void* Y, long ldy, int M, int N, int K, int KB,
                           int NB, int splits, hipStream_t stream) {
    const int mt = (M + 15) / 16;
    const int r = cut_skinny(M, NB, KB, splits, splits).r;       // the row blocks that go with this many slices
#define SK_CASE(R_, MT_)                                                                        \
    launch_skinny<R_, MT_, EPI, TC, 16>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream);          \
    break
#define SK_CASE1(R_)                                                                            \
    if (M <= 4) launch_skinny<R_, 1, EPI, TC, 4>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream); \
    else if (M <= 8) launch_skinny<R_, 1, EPI, TC, 8>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream); \
    else launch_skinny<R_, 1, EPI, TC, 16>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream);       \
    break
    switch (mt * 8 + r) {
        case 1 * 8 + 1: SK_CASE1(1);
        case 1 * 8 + 2: SK_CASE1(2);
        case 1 * 8 + 4: SK_CASE(4, 1);
        case 1 * 8 + 5: SK_CASE(5, 1);
        case 2 * 8 + 1: SK_CASE(1, 2);
        case 2 * 8 + 2: SK_CASE(2, 2);
        case 2 * 8 + 4: SK_CASE(4, 2);
        case 2 * 8 + 5: SK_CASE(5, 2);
        case 3 * 8 + 1: SK_CASE(1, 3);
        case 3 * 8 + 2: SK_CASE(2, 3);
        case 3 * 8 + 4: SK_CASE(4, 3);
        case 3 * 8 + 5: SK_CASE(5, 3);
        case 4 * 8 + 1: SK_CASE(1, 4);
        case 4 * 8 + 2: SK_CASE(2, 4);
        case 4 * 8 + 4: SK_CASE(4, 4);
        case 4 * 8 + 5: SK_CASE(5, 4);
        default: AGAVE_CHECK(false, "gemm_skinny: no kernel for %d tokens with %d row blocks a workgroup", M, r);
    }
#undef SK_CASE1
#undef SK_CASE
    return 0;
}

// ------------------------------------------------------------------ one token: the product makes its normalised row itself
// A decode step of one sequence is bound by its kernels' starts and ends (some 4.6 us for the
// norm between two products, which moves a few kilobytes).  Here the product that reads the
// normalised row makes it: h' = h + post(branch), x = pre(h') (two RMS norms, the first one
// optional), for one token.  Every workgroup computes all of x while its first tiles of W are on
// their way from memory and keeps it in LDS; workgroup 0 also writes h' to `h_out`, which must not
// be the memory that the others still read (`h_in`).
//
// What the row is made of is some four times its bytes, read by every workgroup: with one
// workgroup a row block (1280 for gate and up at 4B sizes) that would be as much again as the
// weights.  So there are at most 256 workgroups, one a compute unit, and each takes several row
// blocks one after another: row block b, b + G, b + 2G, ... of G workgroups, so that at any moment
// the workgroups read neighbouring tiles.  The eight waves share a row block's columns in chunks
// of two k-steps, three chunks in flight a wave, across the row blocks' boundaries; a wave's sums
// for a row block go to LDS when it moves on to the next, and meet there at the end.
struct RowNorm {
    const float* h_in;          // [K]
    float* h_out;               // [K], or null without a branch (h' is h then)
    const void* branch;         // [K] in bfloat16 or 32-bit, or 32-bit slices; null: none
    int branch_f32;
    int n_parts;                // 32-bit slices that add up to the branch (0: one tensor)
    long part_stride;
    const float* post_gain;     // null: the branch is added as it is
    float post_eps;
    const float* pre_gain;
    float pre_eps;
};
#define ROW_NORM_MAX_K 6144
#define ROW_NORM_WGS 256
#define ROW_NORM_MAX_SEQ 16        // row blocks a workgroup takes at most (their sums wait in LDS)
#define ROW_NORM_MAX_LDS (ROW_NORM_MAX_SEQ * 8 * 1024 + ROW_NORM_MAX_K * 2)     // the sums and the row: 140 KB of the 160

// NV: pieces of four columns a thread holds of the row (512 threads: K <= 2048 NV); PB: slices of
// the branch asked for ahead of the tiles (the others follow one after another).
template <int EPI, int NV, int PB>
__global__ __launch_bounds__(512) void gemm_row_normed_kernel(RowNorm nz, const uint4* __restrict__ Wp,
                                                             bf16* __restrict__ Y, int N, int K, int KB, int NB) {
    // (three chunks of two k-steps in flight a wave: 6 KB; with 12 or 16 KB a step of the 4B sizes
    // was 3 to 4 % slower, with 2 KB 7 %)
    constexpr int NW = 8, NT = NW * 64, KS = 2, S = 3;
    extern __shared__ __attribute__((aligned(16))) unsigned char rown_smem[];
    const int G = gridDim.x;
    const int n_seq = (NB - (int)blockIdx.x + G - 1) / G;              // row blocks of this workgroup (at least one)
    float* red = reinterpret_cast<float*>(rown_smem);                   // [n_seq][NW][256] sums of the waves
    bf16* xfull = reinterpret_cast<bf16*>(red + (size_t)((NB + G - 1) / G) * NW * 256);   // [K]
    __shared__ float rs[16];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j = lane & 15, g = lane >> 4;
    const int n_chunks = (KB + KS - 1) / KS;
    const int items = n_seq * n_chunks;                                // (row block, chunk), row block by row block
    const int n_iter = (items + NW - 1) / NW;

    // everything the row is made of is asked for before the first tile of W: a wave's loads come
    // back in the order they left, and behind the tiles the few kilobytes from the cache would
    // wait for the tiles from memory
    float4 n_part[PB][NV], n_h[NV], n_g1[NV], n_g2[NV];
    uint2 n_b16[NV];
    const bool has_branch = nz.branch != nullptr;                       // (uniform, like all of nz)
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = (v * NT + (int)threadIdx.x) * 4;
        const int cc = c < K ? c : 0;                  // (a lane past the row's end reads its start and uses nothing of it)
        n_h[v] = *reinterpret_cast<const float4*>(nz.h_in + cc);
        n_g2[v] = *reinterpret_cast<const float4*>(nz.pre_gain + cc);
        n_g1[v] = *reinterpret_cast<const float4*>((nz.post_gain != nullptr ? nz.post_gain : nz.pre_gain) + cc);
        if (has_branch && nz.branch_f32) {
            const float* bp = reinterpret_cast<const float*>(nz.branch) + cc;
            const int last = nz.n_parts > 0 ? nz.n_parts - 1 : 0;
#pragma unroll
            for (int u = 0; u < PB; ++u)              // (a slice that is not there: the last one again, not added)
                n_part[u][v] = *reinterpret_cast<const float4*>(bp + (size_t)(u < last ? u : last) * nz.part_stride);
        } else if (has_branch) {
            n_b16[v] = *reinterpret_cast<const uint2*>(reinterpret_cast<const bf16*>(nz.branch) + cc);
        }
    }

    frag16 wreg[S][KS];
#define RN_LOAD(ST, IT)                                                                          \
    {                                                                                            \
        int i_ = (IT) * NW + wave;                    /* items are dealt to the waves in turn */  \
        i_ = i_ < items ? i_ : items - 1;             /* past the end: the last one again, not used */ \
        const int sq_ = i_ / n_chunks, ch_ = i_ - sq_ * n_chunks;                                \
        const int nb_ = (int)blockIdx.x + G * sq_;                                               \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                      \
            const int kb = ch_ * KS + ks;                                                        \
            wreg[ST][ks].u = Wp[w_tile(nb_, kb < KB ? kb : KB - 1, NB, KB) * 64 + lane];         \
        }                                                                                        \
    }
#pragma unroll
    for (int st = 0; st < S; ++st) RN_LOAD(st, st)

    // the row, while the tiles travel
    {
        const bool writer = blockIdx.x == 0 && nz.h_out != nullptr;
        const int n_sl = nz.n_parts > 0 ? nz.n_parts : 1;
        float ss = 0.f;
        float4 bsum[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int c = (v * NT + (int)threadIdx.x) * 4;
            float4 b = float4{0.f, 0.f, 0.f, 0.f};
            if (has_branch && c < K) {
                if (nz.branch_f32) {
#pragma unroll
                    for (int u = 0; u < PB; ++u)
                        if (u < n_sl) {
                            b.x += n_part[u][v].x; b.y += n_part[u][v].y; b.z += n_part[u][v].z; b.w += n_part[u][v].w;
                        }
                    for (int p = PB; p < n_sl; ++p) {      // more slices than were asked for ahead: one after another
                        const float4 q = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(nz.branch) + c +
                                                                          (size_t)p * nz.part_stride);
                        b.x += q.x; b.y += q.y; b.z += q.z; b.w += q.w;
                    }
                } else {
                    const uint2 u2 = n_b16[v];
                    b = float4{__builtin_bit_cast(float, u2.x << 16), __builtin_bit_cast(float, u2.x & 0xffff0000u),
                               __builtin_bit_cast(float, u2.y << 16), __builtin_bit_cast(float, u2.y & 0xffff0000u)};
                }
            }
            bsum[v] = b;
            ss += b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
        }
        float inv1 = 1.0f;
        if (has_branch && nz.post_gain != nullptr) inv1 = 1.0f / sqrtf(block_sum(ss, rs) / (float)K + nz.post_eps);
        ss = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {                     // h' = h + post(branch)
            const int c = (v * NT + (int)threadIdx.x) * 4;
            float4 h4 = float4{0.f, 0.f, 0.f, 0.f};
            if (c < K) {
                h4 = n_h[v];
                if (has_branch) {
                    const float4 b = bsum[v];
                    if (nz.post_gain != nullptr) {
                        h4.x += b.x * inv1 * n_g1[v].x; h4.y += b.y * inv1 * n_g1[v].y;
                        h4.z += b.z * inv1 * n_g1[v].z; h4.w += b.w * inv1 * n_g1[v].w;
                    } else {
                        h4.x += b.x; h4.y += b.y; h4.z += b.z; h4.w += b.w;
                    }
                    if (writer) *reinterpret_cast<float4*>(nz.h_out + c) = h4;
                }
            }
            n_h[v] = h4;
            ss += h4.x * h4.x + h4.y * h4.y + h4.z * h4.z + h4.w * h4.w;
        }
        // x = pre(h'), rounded to bfloat16 once, as the norm kernel rounds it
        const float inv2 = 1.0f / sqrtf(block_sum(ss, rs) / (float)K + nz.pre_eps);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int c = (v * NT + (int)threadIdx.x) * 4;
            if (c < K)
                store4<bf16>(xfull + c, float4{n_h[v].x * inv2 * n_g2[v].x, n_h[v].y * inv2 * n_g2[v].y,
                                              n_h[v].z * inv2 * n_g2[v].z, n_h[v].w * inv2 * n_g2[v].w});
        }
        // a wave that gets no chunk of some row block leaves zeros there
        for (int i = threadIdx.x; i < n_seq * NW * 64; i += NT)
            reinterpret_cast<f32x4_t*>(red)[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
    }

    f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
    int cur = -1;                                       // the row block (in this workgroup's order) that acc belongs to
    // only lanes 0..15 of a group hold a token's column of the tile; the token is row 0: the others multiply zeros
#define RN_USE(ST, IT)                                                                           \
    if ((IT) * NW + wave < items) {                                                              \
        const int i_ = (IT) * NW + wave;                                                         \
        const int sq_ = i_ / n_chunks, ch_ = i_ - sq_ * n_chunks;                                \
        if (sq_ != cur) {                                                                        \
            if (cur >= 0) *reinterpret_cast<f32x4_t*>(red + ((size_t)(cur * NW + wave) * 64 + lane) * 4) = acc; \
            acc = f32x4_t{0.f, 0.f, 0.f, 0.f};                                                   \
            cur = sq_;                                                                           \
        }                                                                                        \
        _Pragma("unroll") for (int ks = 0; ks < KS; ++ks) {                                      \
            const int k_ = (ch_ * KS + ks) * 32 + g * 8;                                         \
            frag16 xb;                                                                           \
            xb.u = (j == 0 && k_ < K) ? *reinterpret_cast<const uint4*>(xfull + k_) : uint4{0, 0, 0, 0}; \
            acc = mfma_16x16x32(wreg[ST][ks], xb, acc);                                          \
        }                                                                                        \
    }
    // (a load past the last item asks for the last one again and is not used: loads without a
    // condition around them let a wait name the ones it needs and leave the younger ones in flight)
    for (int it = 0; it < n_iter; it += S) {
#pragma unroll
        for (int st = 0; st < S; ++st) {
            RN_USE(st, it + st)
            RN_LOAD(st, it + st + S)
        }
    }
#undef RN_LOAD
#undef RN_USE
    if (cur >= 0) *reinterpret_cast<f32x4_t*>(red + ((size_t)(cur * NW + wave) * 64 + lane) * 4) = acc;
    __syncthreads();

    // the waves' sums meet; the token's outputs are in the lanes with j == 0
    for (int sq = wave; sq < n_seq; sq += NW) {
        f32x4_t s = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < NW; ++w) s += *reinterpret_cast<const f32x4_t*>(red + ((size_t)(sq * NW + w) * 64 + lane) * 4);
        const int nb = (int)blockIdx.x + G * sq;
        if (j != 0 || nb >= NB) continue;
        if (EPI == 0) {
            const int n = nb * 16 + g * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) st(Y + n + e, s[e]);
        } else {
            const int n = nb * 8 + g * 2;                 // N counts output columns (ff)
            if (n < N) st(Y + n, gelu_tanh_f(s[0]) * s[2]);
            if (n + 1 < N) st(Y + n + 1, gelu_tanh_f(s[1]) * s[3]);
        }
    }
}

template <int EPI, int NV, int PB>
static int launch_row_normed(const RowNorm& nz, const void* Wp, void* Y, int N, int K, int KB, int NB, int wgs, size_t lds,
                             hipStream_t stream) {
    static bool raised = false;                 // (once per process: the sums of many row blocks need more than the default 64 KB)
    if (lds > 64 * 1024 && !raised) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_row_normed_kernel<EPI, NV, PB>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, ROW_NORM_MAX_LDS);
        AGAVE_CHECK(e == hipSuccess, "gemm_row_normed: cannot raise the LDS allowance: %s", hipGetErrorString(e));
        raised = true;
    }
    gemm_row_normed_kernel<EPI, NV, PB><<<wgs, 512, lds, stream>>>(nz, (const uint4*)Wp, (bf16*)Y, N, K, KB, NB);
    return 0;
}

// Whether agave_gemm_row_normed takes a product of these sizes (N counts rows of W, or ff with the
// GeGLU epilogue): one token.
extern "C" int agave_gemm_row_normed_ok(int M, int N, int K, int epilogue) {
    if (!(M == 1 && N > 0 && K > 0 && K % 8 == 0 && K <= ROW_NORM_MAX_K)) return 0;
    const long NB = epilogue == 0 ? ((long)N + 15) / 16 : ((long)N + 7) / 8;
    return NB <= (long)ROW_NORM_WGS * ROW_NORM_MAX_SEQ ? 1 : 0;
}

// Y = pre(h_in + post(branch)) W^T in bfloat16 for one token, the residual row h_in + post(branch)
// going to h_out (see RowNorm).  branch null: Y = pre(h_in) W^T, nothing else is written.
extern "C" int agave_gemm_row_normed(const float* h_in, float* h_out, const void* branch, int branch_f32, int n_parts,
                                     long part_stride, const float* post_gain, float post_eps, const float* pre_gain,
                                     float pre_eps, const void* Wp, void* Y, int N, int K, int epilogue,
                                     hipStream_t stream) {
    AGAVE_CHECK(epilogue == 0 || epilogue == 1, "gemm_row_normed: unknown epilogue %d", epilogue);
    AGAVE_CHECK(agave_gemm_row_normed_ok(1, N, K, epilogue),
                "gemm_row_normed: sizes N=%d K=%d (K <= %d, K %% 8 == 0, at most %d row blocks)", N, K, ROW_NORM_MAX_K,
                ROW_NORM_WGS * ROW_NORM_MAX_SEQ);
    AGAVE_CHECK(h_in != nullptr && pre_gain != nullptr && Wp != nullptr && Y != nullptr, "gemm_row_normed: null tensor");
    AGAVE_CHECK(((uintptr_t)h_in % 16) == 0 && ((uintptr_t)pre_gain % 16) == 0 && ((uintptr_t)post_gain % 16) == 0,
                "gemm_row_normed: the residual row and the gains must be 16-byte aligned");
    if (branch != nullptr) {
        AGAVE_CHECK(h_out != nullptr && h_out != h_in && ((uintptr_t)h_out % 16) == 0,
                    "gemm_row_normed: the sum needs 16-byte aligned memory of its own (other workgroups still read h_in)");
        AGAVE_CHECK(((uintptr_t)branch % (branch_f32 ? 16 : 8)) == 0, "gemm_row_normed: the branch must be aligned");
        AGAVE_CHECK(n_parts >= 0 && n_parts <= 64 && (n_parts == 0 || (branch_f32 && part_stride % 4 == 0 && part_stride >= K)),
                    "gemm_row_normed: %d slices (32-bit, a multiple of four elements apart)", n_parts);
    }
    const int KB = (K + 31) / 32;
    const int NB = epilogue == 0 ? (N + 15) / 16 : (N + 7) / 8;
    RowNorm nz;
    nz.h_in = h_in;
    nz.h_out = branch != nullptr ? h_out : nullptr;
    nz.branch = branch;
    nz.branch_f32 = branch_f32;
    nz.n_parts = n_parts;
    nz.part_stride = part_stride;
    nz.post_gain = post_gain;
    nz.post_eps = post_eps;
    nz.pre_gain = pre_gain;
    nz.pre_eps = pre_eps;
    const int wgs = NB < ROW_NORM_WGS ? NB : ROW_NORM_WGS;
    const int max_seq = (NB + wgs - 1) / wgs;
    const size_t lds = (size_t)max_seq * 8 * 256 * sizeof(float) + (size_t)K * sizeof(bf16);
    const bool many = branch != nullptr && branch_f32 && n_parts > 2;       // slices: eight are asked for ahead
    int rc;
#define RN_CASE(EPI_)                                                                                             \
    if (K <= 4096 && !many) rc = launch_row_normed<EPI_, 2, 2>(nz, Wp, Y, N, K, KB, NB, wgs, lds, stream);          \
    else if (K <= 4096) rc = launch_row_normed<EPI_, 2, 8>(nz, Wp, Y, N, K, KB, NB, wgs, lds, stream);              \
    else if (!many) rc = launch_row_normed<EPI_, 3, 2>(nz, Wp, Y, N, K, KB, NB, wgs, lds, stream);                  \
    else rc = launch_row_normed<EPI_, 3, 8>(nz, Wp, Y, N, K, KB, NB, wgs, lds, stream)
    if (epilogue == 1) {
        RN_CASE(1);
    } else {
        RN_CASE(0);
    }
#undef RN_CASE
    if (rc != 0) return rc;
    AGAVE_LAUNCH_CHECK("gemm_row_normed");
    return 0;
}

// How many 32-bit slices a product of M <= 64 tokens is best computed in by a caller that can add
// them up (1: as one product).
extern "C" int agave_gemm_skinny_slices(int M, int N, int K) {
    if (M <= 0 || M > 64 || N <= 0 || K <= 0) return 1;
    return cut_skinny(M, (N + 15) / 16, (K + 31) / 32, 8).z;
}

// N: logical outputs (rows of W, or ff for the GeGLU epilogue); Wp holds NB row blocks.
// splits > 1: Y is 32-bit, [splits][M][ldy]; slice s gets the sums over the s-th run of columns,
// and whoever reads Y adds the slices up (a product with few row blocks and many columns then
// has workgroups enough to keep the memory busy).
extern "C" int agave_gemm_skinny(const void* X, long ldx, const void* Wp, int dt_y, void* Y, long ldy, int M, int N,
                                 int K, int epilogue, int splits, hipStream_t stream) {
    AGAVE_CHECK(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d (M <= 64)", M, N, K);
    AGAVE_CHECK(K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)X % 16) == 0,
                "gemm_skinny: X must be 16-byte aligned with K and its row stride multiples of 8 (K=%d ldx=%ld)", K, ldx);
    AGAVE_CHECK(ldx >= K && ldy >= N, "gemm_skinny: a row stride is too small");
    AGAVE_CHECK(epilogue == 0 || epilogue == 1, "gemm_skinny: unknown epilogue %d", epilogue);
    if (M == 0) return 0;
    const int KB = (K + 31) / 32;
    const int NB = epilogue == 0 ? (N + 15) / 16 : (N + 7) / 8;
    AGAVE_CHECK(splits >= 1 && splits <= 64 && (splits == 1 || splits * 4 <= KB), "gemm_skinny: %d slices for %d columns",
                splits, K);
    AGAVE_CHECK(splits == 1 || (epilogue == 0 && dt_y == AGAVE_F32), "gemm_skinny: partial sums are plain 32-bit sums");
    int rc;
    if (epilogue == 0) {
        if (dt_y == AGAVE_BF16) rc = dispatch_skinny<0, bf16>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, 1, stream);
        else if (dt_y == AGAVE_F32) rc = dispatch_skinny<0, float>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, splits, stream);
        else AGAVE_CHECK(false, "gemm_skinny: unknown output dtype %d", dt_y);
    } else {
        AGAVE_CHECK(dt_y == AGAVE_BF16, "gemm_skinny: the GeGLU epilogue writes bfloat16");
        rc = dispatch_skinny<1, bf16>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, 1, stream);
    }
    if (rc != 0) return rc;
    AGAVE_LAUNCH_CHECK("gemm_skinny");
    return 0;
}



// ------------------------------------------------------------------ output projection from the decode attention's shares
// A decode step over a long cache leaves, for every (token, head, share of the keys), an
// unnormalised output row with its reference and its sum (attention_mfma.hip: part_o
// [token][head][share][hd], part_ml [token][head][share][2] with the reference in natural
// logarithms).  Merging them is a kernel of its own that moves next to nothing; here the
// product that reads the merged rows merges them itself while it stages them:
//   x[t][head] = sum_s part_o[s] * exp(m_s - m) / sum_s l_s * exp(m_s - m),  rounded to bfloat16
// (the arithmetic of attn_combine_kernel; the sums may be taken in another order), then Y = x W^T.
// A workgroup takes R row blocks of W and the columns of `hps` heads; the grid's y counts those
// runs of heads, and Y is one 32-bit slice [M][N] per run: whoever reads Y adds the slices (the
// residual kernel does).  Up to 16 tokens.
#define OPC_MAX_COLS 1024          // columns (hps * hd) a workgroup stages
#define OPC_MAX_SHARES 64
// NKS: k-steps of 32 columns a wave takes (it takes every fourth one of the workgroup's);
// RB: row blocks whose tiles a wave asks for at a time.  Eight waves: four ask for the tiles of W
// (two sets of RB row blocks at once) and multiply, four merge the shares meanwhile.  A wave's
// loads come back in the order they left, and a compute unit serves its waves' loads in the order
// they were asked for: a wave that did both, or merging waves that asked after the others, would
// not see the shares, a few kilobytes from the cache, before all the tiles had come from memory,
// and the merge would start when it should be over.  So the merging waves ask first and a barrier
// holds the others back until they have.  (Measured at 8 tokens, 16 heads of 256 and 3840 rows:
// 11.6 us with four waves doing both, 9.7 us so; the product alone takes 8.2 us and a separate
// merge 4.8 us more.)
template <int NKS, int RB>
__global__ __launch_bounds__(512) void gemm_oproj_combine_kernel(const float* __restrict__ part_o,
                                                                  const float* __restrict__ part_ml,
                                                                  const uint4* __restrict__ Wp, float* __restrict__ Y,
                                                                  int M, int N, int nh, int hd, int shares, int hps, int R,
                                                                  int NB, int KB) {
    extern __shared__ __attribute__((aligned(16))) unsigned char opc_smem[];
    const int cols = hps * hd, row = cols + 8;                    // staged row in bf16, 16 bytes of padding
    bf16* xs = reinterpret_cast<bf16*>(opc_smem);                  // [16][row]
    float* red = reinterpret_cast<float*>(opc_smem);               // afterwards: [4 waves][R][256] partial sums
    const bool merger = threadIdx.x >= 256;
    const int wave = (threadIdx.x >> 6) & 3, lane = threadIdx.x & 63, j = lane & 15, g = lane >> 4;
    const int nb0 = blockIdx.x * R, run = blockIdx.y;
    const int kb0 = run * (cols / 32), kbs = cols / 32;            // this run's k-steps
    const int n_mine = (kbs - wave + 3) / 4;                       // k-steps wave, wave + 4, ...

    // (two sets of registers, each named by a constant: an index known only at run time would send the array to memory)
    frag16 wreg0[RB][NKS], wreg1[RB][NKS];
    auto load_w = [&](frag16 (&wr)[RB][NKS], int r0) {
#pragma unroll
        for (int i = 0; i < NKS; ++i) {           // (a k-step's row blocks lie side by side: asked for one after another)
            // (a k-step this wave does not have: its first one again; a wave without any, which a
            // run of fewer than four k-steps leaves, the run's first, which always exists)
            const int ks = i < n_mine ? wave + 4 * i : (n_mine > 0 ? wave : 0);
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                // (a row block past the workgroup's or the matrix's last: its first one again, from the cache)
                const int nb = (r0 + rr < R && nb0 + r0 + rr < NB) ? nb0 + r0 + rr : nb0;
                wr[rr][i].u = Wp[w_tile(nb, kb0 + ks, NB, KB) * 64 + lane];
            }
        }
    };
    // The merged rows, eight columns an item; rows past the last token are zero.  A thread works
    // out the shares' weights of its (token, head) itself: a few exponentials cost less than a
    // barrier between those who would compute them and those who use them.  A compute unit serves
    // its waves' loads in the order they were asked for, so the merging waves ask first, for two
    // items a thread (which covers 8 tokens by 512 columns), and only then do the others ask for W.
    const int groups = cols / 8, n_items = M * groups;
    if (merger) {
        const int tid = threadIdx.x - 256;
        // A thread holds twelve shares' rows at a time: six of each of two items, or, where every
        // thread has at most one item, twelve of that one (more would not fit its registers).
        constexpr int SB = 6;
        const bool one = n_items <= 256;
        const int k_step = one ? 2 * SB : SB, q_off = one ? SB : 0;
        for (int base = 0; base < n_items; base += 512) {
            float4 lo4[2][SB], hi4[2][SB];
            float2 mls[2][SB];
            const float* po[2];
            const float2* ml[2];
            bool valid[2];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int gi = base + tid + (one ? 0 : 256 * q);
                valid[q] = gi < n_items;
                const int gc = valid[q] ? gi : 0;
                const int m = gc / groups, c0 = (gc % groups) * 8;
                const size_t slot0 = ((size_t)m * nh + run * hps + c0 / hd) * shares;
                po[q] = part_o + slot0 * hd + c0 % hd;
                ml[q] = reinterpret_cast<const float2*>(part_ml) + slot0;
#pragma unroll
                for (int u = 0; u < SB; ++u) {                       // asked for at once
                    const int sh = q * q_off + u;
                    if (sh < shares && valid[q]) {                  // (no load for a share or an item that is not there)
                        lo4[q][u] = *reinterpret_cast<const float4*>(po[q] + (size_t)sh * hd);
                        hi4[q][u] = *reinterpret_cast<const float4*>(po[q] + (size_t)sh * hd + 4);
                        mls[q][u] = ml[q][sh];
                    } else {
                        lo4[q][u] = hi4[q][u] = float4{0.f, 0.f, 0.f, 0.f};
                        mls[q][u] = float2{-INFINITY, 0.f};
                    }
                }
            }
            if (base == 0) __builtin_amdgcn_s_barrier();           // the other waves may ask for W now
            // the reference of each item: the largest of its shares'
            float mx[2];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                mx[q] = -INFINITY;
#pragma unroll
                for (int u = 0; u < SB; ++u) mx[q] = fmaxf(mx[q], mls[q][u].x);
            }
            if (one) mx[0] = mx[1] = fmaxf(mx[0], mx[1]);
#pragma unroll
            for (int q = 0; q < 2; ++q)
                if (valid[q])
                    for (int sh = k_step; sh < shares; ++sh) mx[q] = fmaxf(mx[q], ml[q][sh].x);
            // (one set of sums: the second item starts anew, the second half of one item's shares goes on)
            float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            float l = 0.f;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                if (q == 1 && !one) {
                    l = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
                }
                if (valid[q]) {
                    for (int s0 = q * q_off; s0 < shares; s0 += k_step) {
                        if (s0 >= k_step) {
#pragma unroll
                            for (int u = 0; u < SB; ++u) {
                                const int sh = s0 + u < shares ? s0 + u : shares - 1;
                                lo4[q][u] = *reinterpret_cast<const float4*>(po[q] + (size_t)sh * hd);
                                hi4[q][u] = *reinterpret_cast<const float4*>(po[q] + (size_t)sh * hd + 4);
                                mls[q][u] = ml[q][sh];
                            }
                        }
#pragma unroll
                        for (int u = 0; u < SB; ++u) {
                            const float f = (s0 + u < shares && mls[q][u].x != -INFINITY) ? __expf(mls[q][u].x - mx[q]) : 0.f;
                            l += mls[q][u].y * f;
                            acc[0] += lo4[q][u].x * f; acc[1] += lo4[q][u].y * f; acc[2] += lo4[q][u].z * f; acc[3] += lo4[q][u].w * f;
                            acc[4] += hi4[q][u].x * f; acc[5] += hi4[q][u].y * f; acc[6] += hi4[q][u].z * f; acc[7] += hi4[q][u].w * f;
                        }
                    }
                }
                if (valid[q] && !(one && q == 0)) {
                    const float iv = l > 0.f ? 1.0f / l : 0.f;
                    uint4 packed;
                    packed.x = f32x2_to_bf16x2(acc[0] * iv, acc[1] * iv);
                    packed.y = f32x2_to_bf16x2(acc[2] * iv, acc[3] * iv);
                    packed.z = f32x2_to_bf16x2(acc[4] * iv, acc[5] * iv);
                    packed.w = f32x2_to_bf16x2(acc[6] * iv, acc[7] * iv);
                    const int gi = base + tid + (one ? 0 : 256 * q);
                    *reinterpret_cast<uint4*>(xs + (size_t)(gi / groups) * row + (gi % groups) * 8) = packed;
                }
            }
        }
        for (int gi = n_items + tid; gi < 16 * groups; gi += 256)
            *reinterpret_cast<uint4*>(xs + (size_t)(gi / groups) * row + (gi % groups) * 8) = uint4{0, 0, 0, 0};
    } else {
        __builtin_amdgcn_s_barrier();
        load_w(wreg0, 0);
        if (RB < R) load_w(wreg1, RB);
    }
    __syncthreads();
    // this wave's k-steps of the staged rows, as B operands
    frag16 xb[NKS];
    if (!merger) {
#pragma unroll
        for (int i = 0; i < NKS; ++i) {
            const int ks = i < n_mine ? wave + 4 * i : (n_mine > 0 ? wave : 0);     // (as in load_w: never past the run)
            xb[i].u = *reinterpret_cast<const uint4*>(xs + (size_t)j * row + ks * 32 + g * 8);
        }
    }
    __syncthreads();                                              // the staged rows give way to the partial sums
    auto use_w = [&](const frag16 (&wr)[RB][NKS], int r0) {
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) {
            f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NKS; ++i)
                if (i < n_mine) acc = mfma_16x16x32(wr[rr][i], xb[i], acc);
            if (r0 + rr < R) *reinterpret_cast<f32x4_t*>(red + ((size_t)wave * R + r0 + rr) * 256 + lane * 4) = acc;
        }
    };
    for (int r0 = 0; r0 < R && !merger; r0 += 2 * RB) {
        if (r0 > 0 && r0 + RB < R) load_w(wreg1, r0 + RB);
        use_w(wreg0, r0);
        if (r0 + 2 * RB < R) load_w(wreg0, r0 + 2 * RB);
        if (r0 + RB < R) use_w(wreg1, r0 + RB);
    }
    __syncthreads();
    float* y = Y + (size_t)run * M * N;
    for (int r = threadIdx.x >> 6; r < R; r += 8) {               // (all eight waves add up and write)
        if (nb0 + r >= NB || j >= M) continue;
        f32x4_t sum = *reinterpret_cast<const f32x4_t*>(red + (size_t)r * 256 + lane * 4);
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const f32x4_t part = *reinterpret_cast<const f32x4_t*>(red + ((size_t)w * R + r) * 256 + lane * 4);
            sum += part;
        }
        const int n = (nb0 + r) * 16 + g * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (n + e < N) y[(size_t)j * N + n + e] = sum[e];
    }
}

// Heads a workgroup's run of columns holds, for a product over nh heads of hd columns: the fewest
// that leave at most 8 runs, 4 for one token (the reader adds that many slices); 0 if this kernel does not take
// the sizes (the caller then merges the shares first and runs the ordinary product).
extern "C" int agave_oproj_combine_heads_per_run(int M, int nh, int hd, int shares) {
    if (M <= 0 || M > 16 || nh <= 0 || hd <= 0 || hd % 32 != 0 || shares < 2) return 0;
    // (one token: four runs; the product after the norm then makes its row from half as many slices:
    // 482 -> 486 tokens/s at the 4B sizes, nothing either way at the 12B and 27B sizes)
    const int max_runs = M == 1 ? 4 : 8;
    for (int hps = 1; hps <= nh; ++hps) {
        if (nh % hps != 0 || nh / hps > max_runs) continue;
        if (hps * hd > OPC_MAX_COLS || shares > OPC_MAX_SHARES) return 0;
        return hps;
    }
    return 0;
}

// Y: [nh / hps][M][N] 32-bit slices.
extern "C" int agave_gemm_oproj_combine(const float* part_o, const float* part_ml, const void* Wp, float* Y, int M,
                                        int N, int nh, int hd, int shares, hipStream_t stream) {
    const int hps = agave_oproj_combine_heads_per_run(M, nh, hd, shares);
    AGAVE_CHECK(hps > 0, "gemm_oproj_combine: no kernel for %d tokens, %d heads of %d, %d shares", M, nh, hd, shares);
    AGAVE_CHECK(part_o && part_ml && Wp && Y && N > 0, "gemm_oproj_combine: null tensor or no rows");
    AGAVE_CHECK(((uintptr_t)part_o % 16) == 0 && ((uintptr_t)Y % 16) == 0, "gemm_oproj_combine: unaligned buffers");
    const int runs = nh / hps, cols = hps * hd, K = nh * hd;
    const int NB = (N + 15) / 16, KB = (K + 31) / 32;
    int R = (int)(((long)NB * runs + 255) / 256);                 // some 256 workgroups
    if (R < 1) R = 1;
    if (R > 12) R = 12;
    const size_t staged = (size_t)16 * (cols + 8) * 2;
    const size_t sums = (size_t)4 * R * 256 * 4;
    const size_t lds = staged > sums ? staged : sums;
    AGAVE_CHECK(lds <= 64 * 1024, "gemm_oproj_combine: %zu bytes of LDS", lds);
    const dim3 grid((NB + R - 1) / R, runs);
    const int nks = (cols / 32 + 3) / 4;
    // tiles a wave asks for at a time: RB * NKS, sixteen or so
#define OPC_LAUNCH(NKS_, RB_)                                                                                   \
    gemm_oproj_combine_kernel<NKS_, RB_><<<grid, 512, lds, stream>>>(part_o, part_ml, (const uint4*)Wp, Y, M, N, nh, \
                                                                     hd, shares, hps, R, NB, KB)
    if (nks <= 1) OPC_LAUNCH(1, 12);
    else if (nks <= 2) OPC_LAUNCH(2, 6);
    else if (nks <= 4) OPC_LAUNCH(4, 4);
    else OPC_LAUNCH(8, 2);
#undef OPC_LAUNCH
    AGAVE_LAUNCH_CHECK("gemm_oproj_combine");
    return 0;
}

// ------------------------------------------------------------------ tiled product (prefill)
// A workgroup computes WT*64 weight rows x TT tokens in tiles of 32 x 32
// (v_mfma_f32_32x32x16_bf16) with eight waves (2 x 4, a wave WT x TT/128 tiles): two per SIMD,
// so that one multiplies while the other waits for a stage of loads, at a barrier or for its
// operands, which a single wave per SIMD cannot hide (a third of its time was waiting); they
// read a half more from LDS per flop, which the LDS (256 bytes a clock) has to spare.
// Both operands come into LDS straight from global memory (no registers in between), KT k-steps
// of 32 columns per stage, in a ring of NS buffers: the loads of NS-1 stages ahead are in flight
// while a stage is multiplied.  What a compute unit can load is 64 bytes a clock (a load of one
// kilobyte keeps its address unit busy for 16 cycles), half of which a 256 x 256 tile needs
// when the matrix cores never wait; smaller tiles need more, which is why the largest tile that
// still fills the chip is taken.
// Weight tiles arrive in their packed order (one kilobyte per wave load; a 32-row operand is
// read out of two packed 16-row tiles); token rows are stored with their 16-byte pieces
// permuted so that the rows an MFMA operand reads fall into different banks.
//   WT 4, KT 1, NS 4:  256 x 256 tiles, 128 KB of LDS, the two waves of a SIMD taking turns
//   WT 2, KT 2, NS 3:  128 x 256 and 128 x 128 tiles - more workgroups for smaller products
//   WT 1, KT 2, NS 4:  64 x 128 tiles
// blockIdx.x walks the weight rows, so that workgroups sharing weight rows (ids a multiple of
// the number of row tiles apart) tend to land on the same XCD and find them in its L2.
typedef __attribute__((address_space(3))) u32x4_t tl_lds_u32x4;


template <int WT, int KT, int NS, int EPI, typename TC, int NWV, int TT, bool TURNS>
__global__ __launch_bounds__(NWV * 64, 2) void gemm_tiled_kernel(const bf16* __restrict__ X, long ldx,
                                                         const uint4* __restrict__ Wp, TC* __restrict__ Y, long ldy,
                                                         int M, int N, int K, int KB, int NB, int NBS, long part_stride) {
    // NBS: row blocks of the whole packed matrix (Wp may point at a later row block of it)
    constexpr int CPR = KT * 4;                       // 16-byte pieces per staged token row
    constexpr int RP = 16 / CPR;                      // token rows per 256 bytes of LDS
    constexpr int WTILES = 4 * WT;                    // packed 16-row weight tiles per workgroup
    constexpr int X_BYTES = TT * KT * 64, W_BYTES = WTILES * KT * 1024;      // TT tokens per workgroup
    constexpr int STAGE_BYTES = X_BYTES + W_BYTES;
    constexpr int XB = (TT / 32) / (NWV / 2);         // 32-token tiles per wave
    static_assert(XB >= 1 && XB * (NWV / 2) * 32 == TT, "the waves' token tiles must cover the workgroup's tokens");
    constexpr int X_LOADS = X_BYTES / 1024 / NWV, W_LOADS = W_BYTES / 1024 / NWV;     // per wave and stage
    static_assert(NWV == 4 || NWV == 8, "four or eight waves");
    static_assert(X_LOADS * NWV * 1024 == X_BYTES && W_LOADS * NWV * 1024 == W_BYTES, "whole loads per wave");
    constexpr int LOADS = X_LOADS + W_LOADS;
    static_assert(NS >= 2, "a stage is loaded while another is multiplied");
    extern __shared__ __attribute__((aligned(16))) unsigned char tl_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int wn = wave & 1, wm = wave >> 1;
    const int nbw = blockIdx.x * WTILES;                  // first packed weight tile of this workgroup
    const int m0 = blockIdx.y * TT;                       // first token of this workgroup
    // gridDim.z workgroups share a tile's columns: each takes a run of stages and leaves its sum
    // in its own slice of Y (a buffer of partial sums then, added up by gemm_sum_parts_kernel)
    const int n_stage_all = (KB + KT - 1) / KT;
    const int st0 = (int)((long)blockIdx.z * n_stage_all / gridDim.z);
    const int n_stage = (int)((long)(blockIdx.z + 1) * n_stage_all / gridDim.z);      // one past this workgroup's last stage
    Y += (size_t)blockIdx.z * part_stride;
    const int i32 = lane & 31, kg = lane >> 5;

    f32x16_t acc[WT][XB];
#pragma unroll
    for (int a = 0; a < WT; ++a)
#pragma unroll
        for (int b = 0; b < XB; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    // Staging.  Everything that is the same for a whole wave is kept in scalar registers (the wave's
    // number is made scalar above), so that a load costs the vector unit nothing but its issue: the
    // address is a scalar base, moved from stage to stage, plus a per-lane offset fixed at the start.
    const unsigned char* xbase = (const unsigned char*)(X + (size_t)m0 * ldx);
    unsigned xoff[X_LOADS], xoff_last[X_LOADS];
    const int st_last = n_stage_all - 1;                               // the stage that may hold columns past K
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) {
        const int o = ((wave * X_LOADS + i) * 64 + lane);              // 16-byte slot in the stage
        const int row = o / CPR, pos = o % CPR;                        // LDS row and position this lane's piece lands in
        const int piece = pos ^ ((row / RP) % CPR);                    // which 8 columns of that row it holds
        int mrow = row;
        if (m0 + mrow >= M) mrow = M - 1 - m0;                         // rows past the end repeat the last one (never stored)
        xoff[i] = (unsigned)(((size_t)mrow * ldx + piece * 8) * 2);
        // in the last stage a piece past the last column reads the stage's first columns instead
        // (any valid address: the weights are zero there)
        xoff_last[i] = st_last * (KT * 32) + piece * 8 >= K ? (unsigned)(((size_t)mrow * ldx) * 2) : xoff[i];
    }
    const unsigned woff = lane * 16;
    // load i (of LOADS) of stage st; stages past the last load the last one again and are never multiplied
    auto fetch_one = [&](int st, int i) {
        unsigned char* buf = tl_lds + (size_t)(st % NS) * STAGE_BYTES;
        const int ste = st < st_last ? st : st_last;
        if (i < X_LOADS) {
            const unsigned char* src = xbase + (size_t)ste * (KT * 64);
            const unsigned off = ste == st_last ? xoff_last[i] : xoff[i];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + off),
                                             (__attribute__((address_space(3))) void*)(buf + (wave * X_LOADS + i) * 1024), 16, 0, 0);
        } else {
            const int tt = wave * W_LOADS + (i - X_LOADS);             // tile: row tile tt / KT, k-step tt % KT
            int nb = nbw + tt / KT, kb = ste * KT + tt % KT;
            if (nb >= NB) nb = NB - 1;                                 // rows past the end: never stored
            if (kb >= KB) kb = KB - 1;                                 // k-steps past the end: never multiplied
            const unsigned char* src = (const unsigned char*)(Wp + w_tile(nb, kb, NBS, KB) * 64);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + woff),
                                             (__attribute__((address_space(3))) void*)(buf + X_BYTES + tt * 1024), 16, 0, 0);
        }
    };
    // this lane's operands of one k-step of 16 columns (phase ph of a stage: k-step ph / 2 of 32 columns, its half ph % 2).
    // A 32-row weight operand is made of two packed 16-row tiles: rows 0..15 from the first,
    // 16..31 from the second; the lane holding (row, columns 8*(2h+kg)..) there.
    constexpr int PH = 2 * KT;                                         // phases per stage
    struct Operands { frag16 w[WT]; frag16 x[XB]; };
    // The token rows' 16-byte pieces are permuted by (row / RP) % CPR, which is the same for all of a
    // lane's rows (they are 32 apart), so one address per phase serves them all.
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)tl_lds;
    const unsigned w_lane = lds0 + X_BYTES + (wn * (2 * WT) + (i32 >> 4)) * KT * 1024 + ((i32 & 15) + 16 * kg) * 16;
    unsigned x_lane[PH];
#pragma unroll
    for (int ph = 0; ph < PH; ++ph)
        x_lane[ph] = lds0 + (wm * XB * 32 + i32) * (CPR * 16) + (((ph * 2) ^ kg ^ ((i32 / RP) % CPR)) * 16);
    // The reads are written as instructions, with the waits for them placed by hand: the compiler
    // counts a load that goes straight into LDS as an LDS access of unknown order and would wait for
    // every pending LDS read before each multiplication, the ones just asked for included.
    auto read_operands = [&](Operands& f, int st, auto phc) {
        constexpr int ph = decltype(phc)::value;
        const unsigned buf = (unsigned)(st % NS) * STAGE_BYTES;
        const unsigned wa = w_lane + buf, xa = x_lane[ph] + buf;
        static_for<0, WT>([&](auto a) {
            frag16& dst = f.w[a.value];                                // (operands of asm do not capture by themselves)
            const unsigned addr = wa;
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst.r)
                         : "v"(addr), "n"(2 * a.value * KT * 1024 + (ph >> 1) * 1024 + (ph & 1) * 512));
        });
        static_for<0, XB>([&](auto b) {
            frag16& dst = f.x[b.value];
            const unsigned addr = xa;
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst.r) : "v"(addr), "n"(b.value * 32 * CPR * 16));
        });
    };
    // every read asked for has returned; what uses f comes after this
    auto settle = [&](Operands& f) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int a = 0; a < WT; ++a) asm volatile("" : "+v"(f.w[a].r));
#pragma unroll
        for (int b = 0; b < XB; ++b) asm volatile("" : "+v"(f.x[b].r));
    };

    // The stage loop.  Loads run NS-1 stages ahead and are issued one at a time between the
    // multiplications: in their shadow they cost no time, while all at once they queue up at the
    // address unit, which takes 16 cycles for each, and the matrix cores wait.
    //   TURNS false: every wave reads the operands of a phase from LDS while the phase before it
    //      multiplies; the first phase's are read after the stage's barrier.
    //   TURNS true: the two waves of a SIMD take turns (waves 0-3 and 4-7, half a stage apart): one
    //      reads its operands of a whole stage while the other multiplies, then a barrier, and they
    //      change places.  The matrix cores then always have a wave that does nothing else.
    constexpr int IN_FLIGHT = LOADS * (NS - 2 - (TURNS ? 1 : 0));     // loads that may be outstanding at a barrier
    static_assert(IN_FLIGHT >= 0 && IN_FLIGHT < 64, "the load counter holds 6 bits");
#pragma unroll
    for (int s0 = 0; s0 < NS - 1; ++s0)
#pragma unroll
        for (int i = 0; i < LOADS; ++i) fetch_one(st0 + s0, i);
    auto landed = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70 | (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14));
        // a bare barrier: __syncthreads() would also wait for the loads still wanted in flight
        __builtin_amdgcn_s_barrier();
    };
    // the multiplications of phase ph with this phase's share (or, all = true, all) of the stage's loads between them
    auto multiply = [&](const Operands& o, int st, int ph, int first_load, int end_load) {
        const bool live = KT == 1 || st * KT + (ph >> 1) < KB;
        int li = first_load;
#pragma unroll
        for (int b = 0; b < XB; ++b) {
            if (live) {
#pragma unroll
                for (int a = 0; a < WT; ++a) acc[a][b] = mfma_32x32x16(o.w[a], o.x[b], acc[a][b]);
            }
            if (li < end_load) {
                __builtin_amdgcn_sched_barrier(0);
                fetch_one(st + NS - 1, li++);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (; li < end_load; ++li) fetch_one(st + NS - 1, li);
    };
    if constexpr (TURNS) {
        static_assert(NWV == 8 && NS >= 4, "two waves per SIMD take turns; a stage is in flight behind the awaited one");
        // Slots between barriers: the first group reads stage i in slot 2i and multiplies in slot
        // 2i+1, the second group one slot later; the loads for stage i+NS-1 are issued while stage
        // i is multiplied.  The first group reads stage i+1 in slot 2i+2, so every wave's loads
        // for it must have landed by the end of slot 2i+1, which is where the second group's waves
        // wait, after reading stage i: the loads of the NS-3 stages after i+1, all that are issued
        // by then, may be in flight.  (The first group waits at the same place in its own order,
        // a slot earlier than it would have to.)  A buffer is loaded into again at least a slot
        // after the second group read it.  Both groups pass the same number of barriers.
        const bool second = wave >= 4;
        Operands f[PH];
        landed();
        if (second) __builtin_amdgcn_s_barrier();
        for (int st = st0; st < n_stage; ++st) {
            static_for<0, PH>([&](auto ph) { read_operands(f[ph.value], st, ph); });
#pragma unroll
            for (int ph = 0; ph < PH; ++ph) settle(f[ph]);
            landed();
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int ph = 0; ph < PH; ++ph)
                multiply(f[ph], st, ph, ph * LOADS / PH, ph + 1 == PH ? LOADS : (ph + 1) * LOADS / PH);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            if (!(second && st + 1 == n_stage)) __builtin_amdgcn_s_barrier();
        }
    } else {
        Operands f[2];
        for (int st = st0; st < n_stage; ++st) {
            landed();
            read_operands(f[0], st, IntC<0>{});
            settle(f[0]);
            static_for<0, PH>([&](auto phc) {
                constexpr int ph = decltype(phc)::value;
                if constexpr (ph + 1 < PH) read_operands(f[(ph + 1) & 1], st, IntC<ph + 1>{});
                __builtin_amdgcn_sched_barrier(0);
                multiply(f[ph & 1], st, ph, (ph * LOADS + PH - 1) / PH, ((ph + 1) * LOADS + PH - 1) / PH);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (ph + 1 < PH) settle(f[(ph + 1) & 1]);
            });
        }
    }

    // The loads issued for stages past the last one write into this workgroup's LDS: they must
    // have landed before the workgroup ends and its LDS is given to another (waited for here and
    // not after the stores below, whose completion would take longer to wait for).
    __builtin_amdgcn_s_waitcnt(0x0F70);

    // D[i][j]: this lane holds token j = lane % 32 and rows i = 8*q + 4*kg + e (q, e = 0..3): four
    // consecutive outputs of one token, 32 tokens a store, each in a cache line of its own.  Stored
    // that way the finished tile takes a sixth of the workgroup's time (the same with half the bytes:
    // it is the number of lines touched that counts).  So the tile goes through LDS, which is free
    // now, and leaves it row by row: 16 bytes a lane, whole lines.  The 16-byte pieces of a row are
    // permuted by the token so that the 32 tokens of a store into LDS fall into different banks.
    constexpr int ES = (int)sizeof(TC);
    constexpr int OUT_COLS = EPI == 0 ? WT * 64 : WT * 32;            // columns of Y this workgroup computes
    constexpr int ROW_BYTES = OUT_COLS * ES, CH = ROW_BYTES / 16;     // 16-byte pieces per row
    constexpr bool VIA_LDS = TT * ROW_BYTES <= NS * STAGE_BYTES && CH >= 1 && CH <= 64;
    const int n_base = EPI == 0 ? nbw * 16 : nbw * 8;
    if constexpr (VIA_LDS) {
        constexpr int SWZ = (CH < 32 ? CH : 32) - 1;
        __builtin_amdgcn_s_barrier();                                  // every wave has read its last operands
#pragma unroll
        for (int a = 0; a < WT; ++a) {
#pragma unroll
            for (int b = 0; b < XB; ++b) {
                const int t = (wm * XB + b) * 32 + i32;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int tile = wn * (2 * WT) + 2 * a + (q >> 1);  // packed 16-row tile of these four rows
                    const int r4 = ((2 * q + kg) & 3) * 4;              // their first row inside that tile
                    const float s0 = acc[a][b][4 * q], s1 = acc[a][b][4 * q + 1], s2 = acc[a][b][4 * q + 2],
                                s3 = acc[a][b][4 * q + 3];
                    const int off = (EPI == 0 ? tile * 16 + r4 : tile * 8 + (r4 >> 1)) * ES;     // byte in the row
                    unsigned char* dst = tl_lds + t * ROW_BYTES + (((off >> 4) ^ (t & SWZ)) << 4) + (off & 15);
                    if (EPI == 0) {
                        store4(reinterpret_cast<TC*>(dst), float4{s0, s1, s2, s3});
                    } else {
                        const float v0 = gelu_tanh_f(s0) * s2, v1 = gelu_tanh_f(s1) * s3;
                        *reinterpret_cast<uint32_t*>(dst) = f32x2_to_bf16x2(v0, v1);
                    }
                }
            }
        }
        __syncthreads();
        constexpr int EPC = 16 / ES;                                    // elements per piece
        constexpr int ROWS_PER = 64 / CH;                               // rows one store instruction covers
        const bool whole = (((uintptr_t)Y | (uintptr_t)(ldy * ES)) & 15) == 0;       // pieces are aligned in memory
        const int piece = lane % CH;
#pragma unroll 4
        for (int r = wave * ROWS_PER + lane / CH; r < TT; r += NWV * ROWS_PER) {
            const int m = m0 + r, n = n_base + piece * EPC;
            if (m >= M || n >= N) continue;
            const uint4 v = *reinterpret_cast<const uint4*>(tl_lds + r * ROW_BYTES + ((piece ^ (r & SWZ)) << 4));
            TC* dst = Y + (size_t)m * ldy + n;
            if (whole && n + EPC <= N) {
                *reinterpret_cast<uint4*>(dst) = v;
            } else {
                const TC* e = reinterpret_cast<const TC*>(&v);
#pragma unroll
                for (int i = 0; i < EPC; ++i)
                    if (n + i < N) dst[i] = e[i];
            }
        }
    } else {
#pragma unroll
        for (int a = 0; a < WT; ++a) {
#pragma unroll
            for (int b = 0; b < XB; ++b) {
                const int m = m0 + (wm * XB + b) * 32 + i32;
                if (m >= M) continue;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nb = nbw + wn * (2 * WT) + 2 * a + (q >> 1);
                    if (nb >= NB) continue;
                    const int r4 = ((2 * q + kg) & 3) * 4;
                    const float s0 = acc[a][b][4 * q], s1 = acc[a][b][4 * q + 1], s2 = acc[a][b][4 * q + 2],
                                s3 = acc[a][b][4 * q + 3];
                    static_assert(VIA_LDS || EPI == 0, "only a plain 32-bit tile is too large for the LDS");
                    const int n = nb * 16 + r4;
                    TC* dst = Y + (size_t)m * ldy + n;
                    if (n + 3 < N && (ldy & 3) == 0) {
                        store4(dst, float4{s0, s1, s2, s3});
                    } else {
                        if (n < N) st(dst, s0);
                        if (n + 1 < N) st(dst + 1, s1);
                        if (n + 2 < N) st(dst + 2, s2);
                        if (n + 3 < N) st(dst + 3, s3);
                    }
                }
            }
        }
    }
}

template <int WT, int KT, int NS, int EPI, typename TC, int NWV, int TT, bool TURNS>
static int launch_tiled(const void* X, long ldx, const void* Wp, void* Y, long ldy, int M, int N, int K, int KB, int NB,
                        hipStream_t stream, int splits = 1, long part_stride = 0, int NBS = 0) {
    constexpr int WTILES = 4 * WT;
    const size_t lds = (size_t)NS * (TT * KT * 64 + WTILES * KT * 1024);
    dim3 grid((NB + WTILES - 1) / WTILES, (M + TT - 1) / TT, splits);
    AGAVE_CHECK(grid.y <= 65535, "gemm_tiled: M=%d exceeds the grid limit", M);
    static bool raised = false;
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<WT, KT, NS, EPI, TC, NWV, TT, TURNS>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        AGAVE_CHECK(e == hipSuccess, "gemm_tiled: cannot raise the LDS allowance");
        raised = true;
    }
    gemm_tiled_kernel<WT, KT, NS, EPI, TC, NWV, TT, TURNS><<<grid, NWV * 64, lds, stream>>>((const bf16*)X, ldx, (const uint4*)Wp, (TC*)Y, ldy,
                                                                      M, N, K, KB, NB, NBS > 0 ? NBS : NB, part_stride);
    return 0;
}

// Y[m][n] = sum over the splits' partial sums
template <typename TC>
__global__ void gemm_sum_parts_kernel(const float* __restrict__ part, int splits, long part_stride, TC* __restrict__ Y,
                                      long ldy, int M, int N) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;        // one output each
    if (i >= (long)M * N) return;
    float s = 0.f;
    for (int z = 0; z < splits; ++z) s += part[(size_t)z * part_stride + i];
    st(Y + (size_t)(i / N) * ldy + i % N, s);
}

template <int EPI, typename TC>
static int dispatch_tiled(const void* X, long ldx, const void* Wp, void* Y, long ldy, int M, int N, int K, int KB,
                          int NB, float* part, long part_elems, hipStream_t stream) {
    // The largest tile that still gives some 160 workgroups (a larger tile reads a third less from
    // L2 per flop, which outweighs idle compute units down to about that number); with few tokens
    // or few rows none does, and the tile with the most workgroups is taken.
    //   256 x 256, 128 x 256, 128 x 128, 64 x 128 (weight rows x tokens)
    const long rows16 = (NB + 15) / 16, rows8 = (NB + 7) / 8, rows4 = (NB + 3) / 4;
    const long t256 = (M + 255) / 256, t128 = (M + 127) / 128;
    const long wgs[4] = {rows16 * t256, rows8 * t256, rows8 * t128, rows4 * t128};
    int pick = -1;
    for (int i = 0; i < 4 && pick < 0; ++i)
        if (wgs[i] >= 160) pick = i;
    if (pick < 0) {
        pick = 0;
        for (int i = 1; i < 4; ++i)
            if (wgs[i] > wgs[pick]) pick = i;
    }
    // up to 128 tokens would leave half of a 256-token tile empty: tiles of 128 tokens (a step of 65
    // to 128 tokens 3 to 5 % faster)
    if (pick <= 1 && M <= 128) pick = 2;
    // Still few workgroups and many columns: several workgroups share a tile's columns and leave
    // partial sums (32-bit, in a buffer the caller lends), which a second kernel adds up.
    int splits = 1;
    if (EPI == 0 && part != nullptr && wgs[pick] < 160) {
        const int n_stage = (KB + 1) / 2;                 // the two small tiles take two k-steps a stage
        splits = (int)((256 + wgs[pick] - 1) / wgs[pick]);
        if (splits > 8) splits = 8;
        if (splits > K / (4 * M)) splits = K / (4 * M);       // the partial sums' traffic stays well below the weights'
        while (splits > 1 && (n_stage / splits < 8 || (long)splits * M * N > part_elems)) --splits;
        if (splits < 1) splits = 1;
    }
    if (splits > 1) {
        const long stride = (long)M * N;
        int rc;
        if (pick == 2) rc = launch_tiled<2, 2, 3, 0, float, 8, 128, false>(X, ldx, Wp, part, N, M, N, K, KB, NB, stream, splits, stride);
        else rc = launch_tiled<1, 2, 4, 0, float, 8, 128, false>(X, ldx, Wp, part, N, M, N, K, KB, NB, stream, splits, stride);
        if (rc != 0) return rc;
        AGAVE_LAUNCH_CHECK("gemm_tiled (partial sums)");
        const long total = (long)M * N;
        gemm_sum_parts_kernel<TC><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(part, splits, stride, (TC*)Y, ldy, M, N);
        return 0;
    }
    if (pick == 0) {
        // 256 compute units take 256 tiles at a time.  When the last round would be at most half
        // full, the rows of that round are computed in tiles of half the height instead, in a
        // second launch: all compute units then work for half a round, not half of them for a whole one.
        const long tiles = wgs[0];
        long rows_main = 0;                                // 256-row tiles of the first launch
        if (tiles > 256 && tiles % 256 > 0) {
            // as many whole rows of tiles as fit the whole rounds; the others, if their tiles of half
            // the height fit one round
            rows_main = (tiles / 256) * 256 / t256;
            if (rows_main <= 0 || (rows16 - rows_main) * 2 * t256 > 256) rows_main = 0;
        }
        const long rest = tiles - rows_main * t256;        // 256 x 256 tiles' worth of the second launch
        if (rows_main > 0) {
            const int nb_main = (int)rows_main * 16;
            const int n_main = EPI == 0 ? nb_main * 16 : nb_main * 8;
            int rc = launch_tiled<4, 1, 4, EPI, TC, 8, 256, true>(X, ldx, Wp, Y, ldy, M, n_main, K, KB, nb_main, stream, 1, 0, NB);
            if (rc != 0) return rc;
            // (a quarter of a round or less: tiles of a quarter of the size, which again fill the compute units)
            if (rest <= 64 && (rows16 - rows_main) * 2 * ((M + 127) / 128) <= 256)
                return launch_tiled<2, 2, 3, EPI, TC, 8, 128, false>(X, ldx, (const uint4*)Wp + w_tile(nb_main, 0, NB, KB) * 64,
                                                                     (TC*)Y + n_main, ldy, M, N - n_main, K, KB, NB - nb_main,
                                                                     stream, 1, 0, NB);
            return launch_tiled<2, 2, 3, EPI, TC, 8, 256, false>(X, ldx, (const uint4*)Wp + w_tile(nb_main, 0, NB, KB) * 64,
                                                                 (TC*)Y + n_main, ldy, M, N - n_main, K, KB, NB - nb_main, stream,
                                                                 1, 0, NB);
        }
    }
    switch (pick) {
        case 0: return launch_tiled<4, 1, 4, EPI, TC, 8, 256, true>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
        case 1: return launch_tiled<2, 2, 3, EPI, TC, 8, 256, false>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
        case 2: return launch_tiled<2, 2, 3, EPI, TC, 8, 128, false>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
        default: return launch_tiled<1, 2, 4, EPI, TC, 8, 128, false>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
    }
}

// A product of many tokens whose reader adds 32-bit slices up (the residual kernel does): when
// its 128 x 256 tiles fill the 256 compute units' rounds badly (160 tiles for 2,048 tokens and
// 2,560 rows leave 96 of them idle for the whole product), each tile's columns are shared among
// z workgroups, each of which leaves its sums in a slice of its own.  In units of one tile's
// time the product then takes rounds(tiles * z) / z, and every slice beyond the first costs its
// bytes, written here and read by whoever adds them: some 0.07 of a tile's time at 160 tiles and
// 10,240 columns (measured: down at 2,048 tokens takes 114 us in three slices instead of 136, and
// the kernel that adds them 8 us more), in proportion to the tiles and inversely to the columns.
// Products that run in 256 x 256 tiles are left alone: sliced, they were slower (measured at
// 4,096 and 8,192 tokens, by 4 %; slices of 256 x 256 tiles by 1 to 2 %, except for 168 tiles, a
// round two thirds full, where they gained 2 %).  Shorter prompts gain as much: down at 1,024 tokens takes 59 us
// in three slices of 80 tiles instead of 81 us in 160 tiles of 128 x 128 (a prefill of 384 to
// 1,024 tokens 2 to 5 % less).
struct SlicePlan { int tile; int z; };      // tile: 0 256 x 256, 1 128 x 256, 2 128 x 128, 3 64 x 128 (weight rows x tokens)

static int cut_tiled_slices(int M, int N, int K) {
    const long NB = (N + 15) / 16;
    const long rows16 = (NB + 15) / 16, rows8 = (NB + 7) / 8;
    const long t256 = (M + 255) / 256;
    if (rows16 * t256 >= 160 || rows8 * t256 < 20) return 1;      // 256 x 256 tiles, or next to no tiles at all
    const long t = rows8 * t256;
    // fewer than 160 tiles of 128 x 256 (shorter prompts, which would run in smaller tiles on 160
    // or 240 compute units): only with long runs of columns a slice (down, not o, whose 2,048
    // columns in two slices were no faster)
    const int min_stages = t >= 160 ? 16 : 32;
    // (4,096 columns in two slices of 128 x 256 tiles lose to the one product at 256 and 384 tokens:
    // 3,840 rows 29.8 us against 26.1, 5,376 rows 30.4 and 32.0 against 27.2 and 27.6; the fewer
    // compute units a product keeps busy, the faster each of them runs)
    if (t < 160 && K < 8192) return 1;
    auto rounds = [](long g) { return (double)((g + 255) / 256); };
    const double slice_cost = 0.07 * (10240.0 / K) * ((double)t / 160.0);
    const int n_stage = (K + 63) / 64;
    double best = rounds(t);
    int z_best = 1;
    for (int z = 2; z <= 4; ++z) {
        if (n_stage / z < min_stages) break;
        const double cost = rounds(t * z) / z + (z - 1) * slice_cost;
        if (cost < 0.93 * best) {
            best = cost;
            z_best = z;
        }
    }
    return z_best;
}

static SlicePlan plan_tiled_slices(int M, int N, int K) {
    // Short prompts (up to 128 tiles of 64 x 128: some 400 tokens at 2,560 rows): as many slices of
    // those tiles as fit one round of 256 workgroups, each with at least six stages.  Measured at
    // 2,560 rows, 96 to 384 tokens: 10,240 columns take 17 to 36 us so (4 slices of 128 x 256 tiles:
    // 34 to 40; one product: 28 to 52), 2,048 columns 7 to 11 us (one product and a kernel that adds
    // its shares: 12 to 15).
    {
        const long rows4 = ((N + 15) / 16 + 3) / 4, t128 = (M + 127) / 128;
        const long small = rows4 * t128;
        if (small <= 128) {
            const int n_stage = (K + 63) / 64;
            int z = (int)(256 / small);
            if (z > 8) z = 8;
            while (z > 1 && n_stage / z < 6) --z;
            if (z > 1) return SlicePlan{3, z};
        }
    }
    const int z = cut_tiled_slices(M, N, K);
    // 256 x 256 tiles where the slices of those fill the compute units in one round (down of the 4B
    // sizes at 2,048 tokens: 240 workgroups, 112 us; as 480 of 128 x 256: 119)
    const long NB = (N + 15) / 16;
    const long big = (long)((NB + 15) / 16) * ((M + 255) / 256) * z;
    return SlicePlan{(big > 192 && big <= 256) ? 0 : 1, z};
}

// How many 32-bit slices a product of M > 64 tokens is best computed in by a caller that can
// add them up (1: as one product).
extern "C" int agave_gemm_tiled_slices(int M, int N, int K) {
    if (M <= 64 || N <= 0 || K <= 0 || K % 8 != 0) return 1;
    return plan_tiled_slices(M, N, K).z;
}

// The slices of a product in tiles of a given shape (0: 256 x 256, 1: 128 x 256, 2: 128 x 128,
// 3: 64 x 128, weight rows x tokens).
static int launch_slices(int tile, const void* X, long ldx, const void* Wp, float* Y, int M, int N, int K, int z,
                         hipStream_t stream) {
    const int KB = (K + 31) / 32, NB = (N + 15) / 16;
    const long stride = (long)M * N;
    switch (tile) {
        case 0: return launch_tiled<4, 1, 4, 0, float, 8, 256, true>(X, ldx, Wp, Y, N, M, N, K, KB, NB, stream, z, stride);
        case 1: return launch_tiled<2, 2, 3, 0, float, 8, 256, false>(X, ldx, Wp, Y, N, M, N, K, KB, NB, stream, z, stride);
        case 2: return launch_tiled<2, 2, 3, 0, float, 8, 128, false>(X, ldx, Wp, Y, N, M, N, K, KB, NB, stream, z, stride);
        default: return launch_tiled<1, 2, 4, 0, float, 8, 128, false>(X, ldx, Wp, Y, N, M, N, K, KB, NB, stream, z, stride);
    }
}

static int check_slices_args(const char* who, const void* X, long ldx, int M, int N, int K) {
    AGAVE_CHECK(M > 64 && N > 0 && K > 0, "%s: bad sizes M=%d N=%d K=%d", who, M, N, K);
    AGAVE_CHECK(K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)X % 16) == 0,
                "%s: X must be 16-byte aligned with K and its row stride multiples of 8 (K=%d ldx=%ld)", who, K, ldx);
    AGAVE_CHECK(ldx >= K && ldx < (1L << 22), "%s: bad row stride %ld", who, ldx);
    return 0;
}

// Y: 32-bit [z][M][N], z = agave_gemm_tiled_slices(M, N, K) > 1; slice s gets the sums over the
// s-th run of columns of X W^T.
extern "C" int agave_gemm_tiled_in_slices(const void* X, long ldx, const void* Wp, float* Y, int M, int N, int K,
                                          int z, hipStream_t stream) {
    if (check_slices_args("gemm_tiled_in_slices", X, ldx, M, N, K)) return -1;
    const SlicePlan plan = plan_tiled_slices(M, N, K);
    AGAVE_CHECK(z > 1 && z == plan.z, "gemm_tiled_in_slices: %d slices asked for, %d planned", z, plan.z);
    if (launch_slices(plan.tile, X, ldx, Wp, Y, M, N, K, z, stream) != 0) return -1;
    AGAVE_LAUNCH_CHECK("gemm_tiled_in_slices");
    return 0;
}

// The same with the tile shape and the number of slices given by the caller (tile 0: 256 x 256,
// 1: 128 x 256, 2: 128 x 128, 3: 64 x 128): for tests of every shape and for measurements.  z = 1
// leaves the whole product in the one slice.
extern "C" int agave_gemm_tiled_in_slices_as(const void* X, long ldx, const void* Wp, float* Y, int M, int N, int K,
                                             int tile, int z, hipStream_t stream) {
    if (check_slices_args("gemm_tiled_in_slices_as", X, ldx, M, N, K)) return -1;
    const int n_stage = tile == 0 ? (K + 31) / 32 : (K + 63) / 64;
    AGAVE_CHECK(tile >= 0 && tile <= 3 && z >= 1 && z <= 16 && z <= n_stage, "gemm_tiled_in_slices_as: tile %d in %d slices of %d stages",
                tile, z, n_stage);
    if (launch_slices(tile, X, ldx, Wp, Y, M, N, K, z, stream) != 0) return -1;
    AGAVE_LAUNCH_CHECK("gemm_tiled_in_slices_as");
    return 0;
}

// One product in tiles of a shape the caller names (0: 256 x 256, 1: 128 x 256, 2: 128 x 128,
// 3: 64 x 128), whatever agave_gemm_tiled would choose: for tests of every shape and for measurements.
template <int EPI, typename TC>
static int launch_tile_shape(int tile, const void* X, long ldx, const void* Wp, void* Y, long ldy, int M, int N, int K,
                             int KB, int NB, hipStream_t stream) {
    switch (tile) {
        case 0: return launch_tiled<4, 1, 4, EPI, TC, 8, 256, true>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
        case 1: return launch_tiled<2, 2, 3, EPI, TC, 8, 256, false>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
        case 2: return launch_tiled<2, 2, 3, EPI, TC, 8, 128, false>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
        default: return launch_tiled<1, 2, 4, EPI, TC, 8, 128, false>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
    }
}

extern "C" int agave_gemm_tiled_as(const void* X, long ldx, const void* Wp, int dt_y, void* Y, long ldy, int M, int N,
                                   int K, int epilogue, int tile, hipStream_t stream) {
    AGAVE_CHECK(M > 0 && N > 0 && K > 0 && tile >= 0 && tile <= 3, "gemm_tiled_as: bad sizes M=%d N=%d K=%d or tile %d", M, N, K, tile);
    AGAVE_CHECK(K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)X % 16) == 0,
                "gemm_tiled_as: X must be 16-byte aligned with K and its row stride multiples of 8 (K=%d ldx=%ld)", K, ldx);
    AGAVE_CHECK(ldx >= K && ldy >= N && ldx < (1L << 22), "gemm_tiled_as: bad row strides");
    AGAVE_CHECK((epilogue == 0 && (dt_y == AGAVE_BF16 || dt_y == AGAVE_F32)) || (epilogue == 1 && dt_y == AGAVE_BF16),
                "gemm_tiled_as: epilogue %d with output dtype %d", epilogue, dt_y);
    const int KB = (K + 31) / 32;
    const int NB = epilogue == 0 ? (N + 15) / 16 : (N + 7) / 8;
    int rc;
    if (epilogue == 1) rc = launch_tile_shape<1, bf16>(tile, X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
    else if (dt_y == AGAVE_BF16) rc = launch_tile_shape<0, bf16>(tile, X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
    else rc = launch_tile_shape<0, float>(tile, X, ldx, Wp, Y, ldy, M, N, K, KB, NB, stream);
    if (rc != 0) return rc;
    AGAVE_LAUNCH_CHECK("gemm_tiled_as");
    return 0;
}

// N: logical outputs (rows of W, or ff for the GeGLU epilogue); Wp holds NB row blocks.  part: an
// optional buffer of part_elems floats for partial sums (products with few tiles and many columns
// are then shared out along the columns); null: never.
extern "C" int agave_gemm_tiled(const void* X, long ldx, const void* Wp, int dt_y, void* Y, long ldy, int M, int N,
                                int K, int epilogue, float* part, long part_elems, hipStream_t stream) {
    AGAVE_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    AGAVE_CHECK(K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)X % 16) == 0,
                "gemm_tiled: X must be 16-byte aligned with K and its row stride multiples of 8 (K=%d ldx=%ld)", K, ldx);
    AGAVE_CHECK(ldx >= K && ldy >= N, "gemm_tiled: a row stride is too small");
    AGAVE_CHECK(ldx < (1L << 22), "gemm_tiled: a row stride of %ld elements is beyond the kernel's 32-bit offsets", ldx);
    AGAVE_CHECK(epilogue == 0 || epilogue == 1, "gemm_tiled: unknown epilogue %d", epilogue);
    if (M == 0) return 0;
    const int KB = (K + 31) / 32;
    const int NB = epilogue == 0 ? (N + 15) / 16 : (N + 7) / 8;
    int rc;
    if (epilogue == 0) {
        if (dt_y == AGAVE_BF16) rc = dispatch_tiled<0, bf16>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, part, part_elems, stream);
        else if (dt_y == AGAVE_F32) rc = dispatch_tiled<0, float>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, part, part_elems, stream);
        else AGAVE_CHECK(false, "gemm_tiled: unknown output dtype %d", dt_y);
    } else {
        AGAVE_CHECK(dt_y == AGAVE_BF16, "gemm_tiled: the GeGLU epilogue writes bfloat16");
        rc = dispatch_tiled<1, bf16>(X, ldx, Wp, Y, ldy, M, N, K, KB, NB, nullptr, 0, stream);
    }
    if (rc != 0) return rc;
    AGAVE_LAUNCH_CHECK("gemm_tiled");
    return 0;
}
