// Plain matrix product  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N])  with 32-bit multiply-add
// on the vector units: no matrix-core mode, no reduced precision.  It is the linear layer
// of the float32 path, and takes bfloat16 operands (products and sums still 32-bit) where
// a 32-bit result is wanted from bfloat16 weights.  Any M, N, K.
#include "common.h"

#define TILE_M 64
#define TILE_N 64
#define TILE_K 16

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_fma_kernel(TOut* __restrict__ C, const TIn* __restrict__ A,
                                                       const TIn* __restrict__ W,
                                                       const TIn* __restrict__ bias, int M, int N, int K,
                                                       int lda, int ldc) {
    __shared__ float As[TILE_K][TILE_M + 4];
    __shared__ float Ws[TILE_K][TILE_N + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * TILE_M, n0 = blockIdx.x * TILE_N;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    float acc[4][4] = {};
    // each thread stages 4 elements of A and 4 of W per K step: row = tid / 4, k = (tid % 4) * 4 ..
    const int lr = tid / 4, lk = (tid % 4) * 4;
    for (int k0 = 0; k0 < K; k0 += TILE_K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int am = m0 + lr, wn = n0 + lr;
            As[lk + i][lr] = (am < M && k < K) ? to_f32(A[(size_t)am * lda + k]) : 0.f;
            Ws[lk + i][lr] = (wn < N && k < K) ? to_f32(W[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TILE_K; ++k) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][tm + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[k][tn + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + tm + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += to_f32(bias[n]);
            C[(size_t)m * ldc + n] = from_f32<TOut>(v);
        }
    }
}

extern "C" {

// in_dtype / out_dtype: 0 = float32, 1 = bfloat16.  Supported: (0,0), (1,1), (1,0).
int llms_gemm_fma(int in_dtype, int out_dtype, void* C, const void* A, const void* W, const void* bias,
                  int M, int N, int K, int lda, int ldc, hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_fma: sizes must be positive");
    LLMS_REQUIRE(lda >= K && ldc >= N, "gemm_fma: leading dimensions too small");
    dim3 grid((N + TILE_N - 1) / TILE_N, (M + TILE_M - 1) / TILE_M);
    LLMS_REQUIRE(grid.y <= 65535, "gemm_fma: too many rows for one launch");
    if (in_dtype == 0 && out_dtype == 0) {
        gemm_fma_kernel<float, float><<<grid, 256, 0, stream>>>((float*)C, (const float*)A, (const float*)W,
                                                                (const float*)bias, M, N, K, lda, ldc);
    } else if (in_dtype == 1 && out_dtype == 1) {
        gemm_fma_kernel<bf16, bf16><<<grid, 256, 0, stream>>>((bf16*)C, (const bf16*)A, (const bf16*)W,
                                                              (const bf16*)bias, M, N, K, lda, ldc);
    } else if (in_dtype == 1 && out_dtype == 0) {
        gemm_fma_kernel<bf16, float><<<grid, 256, 0, stream>>>((float*)C, (const bf16*)A, (const bf16*)W,
                                                               (const bf16*)bias, M, N, K, lda, ldc);
    } else {
        LLMS_REQUIRE(false, "gemm_fma: unsupported dtype pair");
    }
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
