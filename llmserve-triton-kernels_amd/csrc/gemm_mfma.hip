// bfloat16 matrix products on the gfx950 matrix cores:  C[M,N] = A[M,K] * W[N,K]^T (+ bias),
// 32-bit accumulation, result stored as bfloat16 or float.  Both operands are contiguous
// along K, which is how the matrix instructions want them: a lane holds 8 consecutive k of
// one row (one 16-byte load).
//
//   gemm_skinny  M <= 64: the weight is read once, straight from global memory into the matrix
//                instruction; a workgroup owns 16 output features and its 8 waves split K; their
//                partial sums meet in LDS in a fixed order.
//   gemm_tile    any M: 128x128 tiles through double-buffered LDS, 4 waves of 64x64.
// (The product for up to 16 rows, with its fused epilogues, is gemm_stream.hip.)
//
// K must be a multiple of 8 and rows 16-byte aligned (the host checks); M, N are arbitrary.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

template <typename TOut>
__device__ __forceinline__ void store_out(TOut* p, float v);
template <>
__device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_out<bf16>(bf16* p, float v) { p->bits = f32_to_bf16_bits(v); }

// ------------------------------------------------------------------------------ skinny
#define SK_WAVES 8
#define SK_UNROLL 4

// v_mfma_f32_16x16x32_bf16: lane l holds A[i = l%16][k = 8*(l/16) .. +7], B[k = same][j = l%16];
// result D[i = 4*(l/16) + r][j = l%16], r = 0..3.  Here i = output feature n, j = row m of X.
template <int MB, typename TOut>
__global__ __launch_bounds__(SK_WAVES* LLMS_WAVE) void gemm_skinny_kernel(
    TOut* __restrict__ C, const bf16* __restrict__ X, const bf16* __restrict__ W, const bf16* __restrict__ bias,
    int M, int N, int K, int ldx, int ldc) {
    __shared__ float red[SK_WAVES][MB][LLMS_WAVE][4];
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE;
    const int r16 = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int n = n0 + r16;
    const bool n_ok = n < N;
    const bf16* wrow = W + (size_t)(n_ok ? n : 0) * K;
    const int ksteps = (K + 31) / 32;
    f32x4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const uint4 zero = make_uint4(0, 0, 0, 0);

    // k-steps are dealt to the waves round-robin, so the 8 waves of a workgroup read one
    // contiguous 512-byte stretch of each of the 16 weight rows at a time
    for (int ks0 = wave; ks0 < ksteps; ks0 += SK_WAVES * SK_UNROLL) {
        uint4 wv[SK_UNROLL];
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int k = (ks0 + u * SK_WAVES) * 32 + g * 8;
            wv[u] = (n_ok && k < K) ? *reinterpret_cast<const uint4*>(wrow + k) : zero;
        }
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int k = (ks0 + u * SK_WAVES) * 32 + g * 8;
            if ((ks0 + u * SK_WAVES) < ksteps) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const int m = mb * 16 + r16;
                    const uint4 xv = (m < M && k < K) ? *reinterpret_cast<const uint4*>(X + (size_t)m * ldx + k) : zero;
                    acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wv[u]), as_bf16x8(xv), acc[mb], 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][mb][lane][r] = acc[mb][r];
    __syncthreads();
    // 256*MB outputs; consecutive threads take consecutive features of one row
    for (int idx = threadIdx.x; idx < 256 * MB; idx += SK_WAVES * LLMS_WAVE) {
        const int nl = idx % 16, ml = (idx / 16) % 16, mb = idx / 256;
        const int m = mb * 16 + ml, nn = n0 + nl;
        if (m >= M || nn >= N) continue;
        const int src_lane = (nl / 4) * 16 + ml, r = nl % 4;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) s += red[w][mb][src_lane][r];
        if (bias) s += bf16_bits_to_f32(bias[nn].bits);
        store_out<TOut>(C + (size_t)m * ldc + nn, s);
    }
}

// ------------------------------------------------------------------------------ tiled
#define TL_BM 128
#define TL_BN 128
#define TL_BK 32
#define TL_LD 40  // LDS row stride in elements: 32 + 8 of padding against bank conflicts

// v_mfma_f32_32x32x16_bf16: lane l holds A[i = l%32][k = 8*(l/32) .. +7], B[k = same][j = l%32];
// result D[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32], r = 0..15.  Here i = row m, j = feature n.
template <typename TOut>
__global__ __launch_bounds__(256) void gemm_tile_kernel(TOut* __restrict__ C, const bf16* __restrict__ A,
                                                        const bf16* __restrict__ W, const bf16* __restrict__ bias,
                                                        int M, int N, int K, int lda, int ldc, int tiles_m) {
    __shared__ __attribute__((aligned(16))) uint16_t As[2][TL_BM * TL_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][TL_BN * TL_LD];
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of tiles
    // (M fastest), so the tiles that share a weight slab share an L2.
    const int nblk = gridDim.x, pid = blockIdx.x;
    const int full = nblk / 8, rem = nblk % 8, xcd = pid % 8;
    const int t = xcd * full + min(xcd, rem) + pid / 8;
    const int m0 = (t % tiles_m) * TL_BM, n0 = (t / tiles_m) * TL_BN;

    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int wm = (wave % 2) * 64, wn = (wave / 2) * 64;
    const int l32 = lane % 32, g = lane / 32;
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;  // a struct (uint4) held in an array is copied
    const u32x4 zero = {0, 0, 0, 0};                              // through private memory by the compiler

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // staging: 512 chunks of 8 elements per operand tile, two per thread
    u32x4 ra[2], rb[2];
    const int crow[2] = {tid / 4, (tid + 256) / 4};
    const int ckc = (tid % 4) * 8;
    auto load_global = [&](int k0) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int k = k0 + ckc;
            const int am = m0 + crow[c], wn_ = n0 + crow[c];
            ra[c] = (am < M && k < K) ? *reinterpret_cast<const u32x4*>(A + (size_t)am * lda + k) : zero;
            rb[c] = (wn_ < N && k < K) ? *reinterpret_cast<const u32x4*>(W + (size_t)wn_ * K + k) : zero;
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            *reinterpret_cast<u32x4*>(&As[buf][crow[c] * TL_LD + ckc]) = ra[c];
            *reinterpret_cast<u32x4*>(&Bs[buf][crow[c] * TL_LD + ckc]) = rb[c];
        }
    };

    const int ktiles = (K + TL_BK - 1) / TL_BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < ktiles; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < ktiles) load_global((kt + 1) * TL_BK);
#pragma unroll
        for (int s = 0; s < TL_BK / 16; ++s) {
            bf16x8 af[2], bfr[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = as_bf16x8(*reinterpret_cast<const uint4*>(&As[buf][(wm + i * 32 + l32) * TL_LD + s * 16 + g * 8]));
                bfr[i] = as_bf16x8(*reinterpret_cast<const uint4*>(&Bs[buf][(wn + i * 32 + l32) * TL_LD + s * 16 + g * 8]));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < ktiles) store_lds(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn + j * 32 + l32;
            if (n >= N) continue;
            const float b = bias ? bf16_bits_to_f32(bias[n].bits) : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm + i * 32 + 8 * (r / 4) + 4 * g + (r % 4);
                if (m < M) store_out<TOut>(C + (size_t)m * ldc + n, acc[i][j][r] + b);
            }
        }
}

// ------------------------------------------------------------------------------ launchers
static int check_common(const void* C, const void* A, const void* W, int M, int N, int K, int lda, int ldc) {
    LLMS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: sizes must be positive");
    LLMS_REQUIRE(K % 8 == 0 && lda % 8 == 0, "gemm_bf16: K and the row stride of A must be multiples of 8");
    LLMS_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_bf16: A and W must be 16-byte aligned");
    LLMS_REQUIRE(lda >= K && ldc >= N, "gemm_bf16: leading dimensions too small");
    LLMS_REQUIRE(C != nullptr, "gemm_bf16: no output");
    return LLMS_OK;
}

template <typename TOut>
static void launch_skinny(TOut* C, const bf16* X, const bf16* W, const bf16* bias, int M, int N, int K, int ldx,
                          int ldc, hipStream_t stream) {
    const dim3 grid((N + 15) / 16), block(SK_WAVES * LLMS_WAVE);
    const int mb = (M + 15) / 16;
    if (mb == 1) gemm_skinny_kernel<1, TOut><<<grid, block, 0, stream>>>(C, X, W, bias, M, N, K, ldx, ldc);
    else if (mb == 2) gemm_skinny_kernel<2, TOut><<<grid, block, 0, stream>>>(C, X, W, bias, M, N, K, ldx, ldc);
    else if (mb == 3) gemm_skinny_kernel<3, TOut><<<grid, block, 0, stream>>>(C, X, W, bias, M, N, K, ldx, ldc);
    else gemm_skinny_kernel<4, TOut><<<grid, block, 0, stream>>>(C, X, W, bias, M, N, K, ldx, ldc);
}

extern "C" {

// out_dtype: 0 = float32, 1 = bfloat16.  M <= 64.
int llms_gemm_bf16_skinny(int out_dtype, void* C, const void* X, const void* W, const void* bias, int M, int N,
                          int K, int ldx, int ldc, hipStream_t stream) {
    if (int e = check_common(C, X, W, M, N, K, ldx, ldc)) return e;
    LLMS_REQUIRE(M <= 64, "gemm_bf16_skinny: M must be <= 64");
    LLMS_REQUIRE(out_dtype == 0 || out_dtype == 1, "gemm_bf16_skinny: out_dtype must be 0 or 1");
    if (out_dtype == 0)
        launch_skinny<float>((float*)C, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, N, K, ldx, ldc, stream);
    else
        launch_skinny<bf16>((bf16*)C, (const bf16*)X, (const bf16*)W, (const bf16*)bias, M, N, K, ldx, ldc, stream);
    LLMS_LAUNCH_CHECK();
}

int llms_gemm_bf16_tile(int out_dtype, void* C, const void* A, const void* W, const void* bias, int M, int N, int K,
                        int lda, int ldc, hipStream_t stream) {
    if (int e = check_common(C, A, W, M, N, K, lda, ldc)) return e;
    LLMS_REQUIRE(out_dtype == 0 || out_dtype == 1, "gemm_bf16_tile: out_dtype must be 0 or 1");
    const int tiles_m = (M + TL_BM - 1) / TL_BM, tiles_n = (N + TL_BN - 1) / TL_BN;
    const long long blocks = (long long)tiles_m * tiles_n;
    LLMS_REQUIRE(blocks < (1ll << 31), "gemm_bf16_tile: too many tiles");
    if (out_dtype == 0)
        gemm_tile_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((float*)C, (const bf16*)A, (const bf16*)W,
                                                                      (const bf16*)bias, M, N, K, lda, ldc, tiles_m);
    else
        gemm_tile_kernel<bf16><<<(unsigned)blocks, 256, 0, stream>>>((bf16*)C, (const bf16*)A, (const bf16*)W,
                                                                     (const bf16*)bias, M, N, K, lda, ldc, tiles_m);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
