// Plain tiled matrix product for gfx950: C[M,N] = A[M,K] * W[N,K]^T with 32-bit
// accumulation, for any M, N, K and any mix of float / bf16 operands.
//
// This is the true 32-bit path of the linear layers (ordinary fused multiply-adds, no
// reduced-precision matrix mode) and the fallback for sizes the MFMA kernels refuse.
// Weights are row-major [out, in] and used as y = W x, as in the reference
// (src/backend/backend.zig:474, 481).
#include "common_impl.h"

#define TM 64
#define TN 64
#define TK 16

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_tn_kernel(const TA* __restrict__ A, long lda,
                                                      const TW* __restrict__ W, long ldw,
                                                      TC* __restrict__ C, long ldc, int M, int N, int K) {
    __shared__ float As[TK][TM + 4];
    __shared__ float Ws[TK][TN + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    // loader: thread -> (row, 4 consecutive k)
    const int lr = tid >> 2, lk = (tid & 3) * 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kk = k0 + lk + i;
            const int am = m0 + lr, wn = n0 + lr;
            As[lk + i][lr] = (am < M && kk < K) ? ld(A + (size_t)am * lda + kk) : 0.f;
            Ws[lk + i][lr] = (wn < N && kk < K) ? ld(W + (size_t)wn * ldw + kk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) st(C + (size_t)m * ldc + n, acc[i][j]);
        }
    }
}

template <typename TA, typename TW, typename TC>
static void launch_gemm(const void* A, long lda, const void* W, long ldw, void* C, long ldc, int M, int N, int K,
                        hipStream_t stream) {
    dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
    gemm_tn_kernel<TA, TW, TC><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, ldw, (TC*)C, ldc, M, N, K);
}

extern "C" int agave_gemm_plain(int dt_a, const void* A, long lda, int dt_w, const void* W, long ldw, int dt_c,
                                void* C, long ldc, int M, int N, int K, hipStream_t stream) {
    AGAVE_CHECK(M >= 0 && N > 0 && K > 0, "gemm_plain: bad sizes M=%d N=%d K=%d", M, N, K);
    AGAVE_CHECK(lda >= K && ldw >= K && ldc >= N, "gemm_plain: a row stride is too small (lda=%ld ldw=%ld ldc=%ld)", lda, ldw, ldc);
    AGAVE_CHECK((M + TM - 1) / TM <= 65535, "gemm_plain: M=%d exceeds the grid limit", M);
    if (M == 0) return 0;
    const int code = dt_a * 4 + dt_w * 2 + dt_c;
    switch (code) {
        case 0: launch_gemm<float, float, float>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 1: launch_gemm<float, float, bf16>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 2: launch_gemm<float, bf16, float>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 3: launch_gemm<float, bf16, bf16>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 4: launch_gemm<bf16, float, float>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 5: launch_gemm<bf16, float, bf16>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 6: launch_gemm<bf16, bf16, float>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        case 7: launch_gemm<bf16, bf16, bf16>(A, lda, W, ldw, C, ldc, M, N, K, stream); break;
        default: AGAVE_CHECK(false, "gemm_plain: unknown dtypes %d %d %d", dt_a, dt_w, dt_c);
    }
    AGAVE_LAUNCH_CHECK("gemm_plain");
    return 0;
}
