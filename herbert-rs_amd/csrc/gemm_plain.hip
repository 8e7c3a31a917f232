// Plain tiled matrix product in float32 arithmetic for any storage types and any sizes:
//   C[m, n] (+)= sum_k A[m, k] * W[n, k]      (weights are [out, in], k contiguous)
// It is the whole matrix path of the float32 mode and the fallback of the bfloat16
// mode for shapes its MFMA kernels refuse. Each output is summed over k ascending by
// one thread with fused multiply-adds, so its value does not depend on M, on the tile
// it falls in, or on what else is in the batch.
// In xigh/herbert-rs: crates/backends/backend_bf16/src/kernels.rs:154-164 (float32 sums over k ascending of
// x[m, k] * float(w[n, k]), no bias); crates/backends/backend_vulkan/shaders/bf16_matmul.comp:31-60.
#include "common.h"

HB_MODULE_ERROR_SLOT()

#define TILE_M 64
#define TILE_N 64
#define TILE_K 16

template <class TA, class TW, class TC, bool ACCUM>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int M, int N,
                  int K, int lda, int ldw, int ldc) {
    __shared__ float As[TILE_K][TILE_M + 1];
    __shared__ float Ws[TILE_K][TILE_N + 1];
    const int tid = threadIdx.x;
    const int tx = tid % 16;   // column group
    const int ty = tid / 16;   // row group
    const int m0 = blockIdx.y * TILE_M;
    const int n0 = blockIdx.x * TILE_N;

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TILE_K) {
        // 64 x 16 elements of each operand, 4 per thread; k runs fastest in memory.
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + i * 256;
            const int kk = e % TILE_K;
            const int rr = e / TILE_K;
            const int k = k0 + kk;
            const int m = m0 + rr;
            const int n = n0 + rr;
            As[kk][rr] = (m < M && k < K) ? hb_to_float(A[(size_t)m * lda + k]) : 0.f;
            Ws[kk][rr] = (n < N && k < K) ? hb_to_float(W[(size_t)n * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TILE_K; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty + 16 * i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n >= N) continue;
            const size_t idx = (size_t)m * ldc + n;
            if (ACCUM)
                C[idx] = hb_from_float<TC>(hb_to_float(C[idx]) + acc[i][j]);
            else
                C[idx] = hb_from_float<TC>(acc[i][j]);
        }
    }
}

template <class TA, class TW, class TC>
static void launch(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                   int accumulate, hipStream_t stream) {
    dim3 grid((N + TILE_N - 1) / TILE_N, (M + TILE_M - 1) / TILE_M);
    if (accumulate)
        gemm_plain_kernel<TA, TW, TC, true><<<grid, 256, 0, stream>>>(
            (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda, ldw, ldc);
    else
        gemm_plain_kernel<TA, TW, TC, false><<<grid, 256, 0, stream>>>(
            (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda, ldw, ldc);
}

// C[M, N] (+)= A[M, K] * W[N, K]^T with row strides lda, ldw, ldc (in elements).
extern "C" int hb_gemm_plain(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                             int M, int N, int K, int lda, int ldw, int ldc, int accumulate,
                             hipStream_t stream) {
    HB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: empty problem (M=%d, N=%d, K=%d)", M, N, K);
    HB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: a row stride is smaller than its row");
    HB_REQUIRE((M + TILE_M - 1) / TILE_M <= 65535, "gemm: M=%d exceeds the grid", M);
    const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
    switch (key) {
        case 0: launch<float, float, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 1: launch<float, float, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 2: launch<float, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 3: launch<float, bf16, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 4: launch<bf16, float, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 5: launch<bf16, float, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 6: launch<bf16, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 7: launch<bf16, bf16, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        default: HB_REQUIRE(false, "gemm: unknown dtypes (%d, %d, %d)", a_dtype, w_dtype, c_dtype);
    }
    HB_CHECK_LAUNCH("gemm_plain");
    return 0;
}
