// bfloat16 matrix product for few rows (decoding):  C[M,N] = X[M,K] * W[N,K]^T, 32-bit sums on the gfx950
// matrix cores, built around reading the weight once at memory speed.
//
// A workgroup owns 16 weight rows and 16 rows of X; its 4 waves take the K chunks (ST_KC = 128 or 512 wide) in turn.
// (More than 16 rows of X, up to 64: one workgroup per block of 16 rows; the workgroups that share weight
// rows get consecutive places on the same XCD, so the weights cross HBM once and come from that XCD's L2
// for the others.)  One load instruction of a wave covers whole 256-byte pieces of 4 weight rows (coalesced,
// non-temporal; with chunks of 512 it is 1 KB of one row); the loads of a chunk are in flight before anything waits,
// and the next chunk's loads are issued before the arithmetic of this one.  The chunk goes through a wave-private, XOR-swizzled LDS tile to reach
// the layout of v_mfma_f32_16x16x32_bf16 (lane l: A[i = l%16][k = 8*(l/16) .. +7], here i = weight row; B likewise
// with j = row m of X; D[i = 4*(l/16) + r][j = l%16]).  The waves' partial sums meet in LDS in a fixed order.
// With chunks of 512 (64 KB of LDS) two workgroups fit a CU; a CU takes only so many bytes a microsecond however
// much a wave has in flight, so what counts is that every CU has work at every moment: with chunks of 128 (16 KB)
// eight workgroups fit, a launch of 704 or 2,000 tiles no longer runs in rounds, and a step of the 7B shape at
// batch 8 went from 3.98 to 3.73 ms.  A launch of at most a workgroup per CU keeps the chunks of 512.
//
// Because a launch costs more than most of these products take, what surrounds the product is fused in:
//   SWIGLU    the 16 rows are 8 gate rows and the 8 up rows of the same features; the epilogue writes
//             bf16(bf16(silu(bf16(gate))) * bf16(up)) (src/llmserve/model/llama.py:120).
//   ROPE_QKV  the 16 rows are 8 rows of one head and their 8 rotary partners (i, i + D/2); the epilogue
//             rotates q and k (src/llmserve/model/llama.py:31-54), writes q, and stores k and v at the
//             tokens' slots of the paged cache (values transposed inside a page).
// Which weight rows a workgroup takes is only an index map, so the weights keep their stacked layout
// ([q; k; v], [gate; up]) and the same tensors serve the library product used for more rows.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// 16-byte load that is not kept in the caches: weights are read once per step.
__device__ __forceinline__ uint4 load_streaming(const void* p) {
    return __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}

__device__ __forceinline__ float bfr(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

template <typename TOut>
__device__ __forceinline__ void store_out(TOut* p, float v);
template <>
__device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_out<bf16>(bf16* p, float v) { p->bits = f32_to_bf16_bits(v); }

#define ST_WAVES 4
#define EPI_PLAIN 0
#define EPI_SWIGLU 1
#define EPI_ROPE_QKV 2

struct StreamArgs {
    void* C;
    int ldc;
    const bf16* X;
    int ldx;
    const bf16* W;
    const bf16* bias;
    int M, N, K;
    int num_tiles;  // tiles of 16 weight rows (8 features for the gated and rotary epilogues)
    int k_splits;   // workgroups that share a tile's K (blockIdx.y); each stores its partial sums, 32-bit, in C[split]
    // SWIGLU
    int inter;
    // ROPE_QKV
    int n_heads, n_kv_heads, head_dim, block_size;
    const float* inv_freq;
    const int* positions;
    const int* slots;
    bf16* k_pool;
    bf16* v_pool;
};

// 8 packed bfloat16 -> floats
__device__ __forceinline__ void unpack8(uint4 v, float (&f)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = bf16_bits_to_f32((uint16_t)(w[j] & 0xffffu));
        f[2 * j + 1] = bf16_bits_to_f32((uint16_t)(w[j] >> 16));
    }
}

__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename TOut, int EPI, int ST_KC, int NW>  // ST_KC: width of a chunk of K, 128 or 512; NW: waves, 4 or 8
__global__ __launch_bounds__(NW* LLMS_WAVE) void gemm_stream_kernel(const StreamArgs a) {
    __shared__ uint4 lds[NW * 16 * (ST_KC / 8)];  // per wave 16 rows x ST_KC / 8 pieces of 16 bytes
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE;
    const int r16 = lane % 16, g = lane / 16;
    // Workgroups go round the 8 XCDs; tile t lives on XCD t % 8, its blocks of 16 rows of X next to each other
    const int m_blocks = (a.M + 15) / 16;
    const int xcd = blockIdx.x % 8, place = blockIdx.x / 8;
    const int tile_id = (place / m_blocks) * 8 + xcd;
    const int m0 = (place % m_blocks) * 16;
    if (tile_id >= a.num_tiles) return;
    const int M = a.M, N = a.N, K = a.K;
    const uint4 zero = make_uint4(0, 0, 0, 0);

    // ---- which 16 weight rows this workgroup owns (-1: none)
    const int D = a.head_dim;
    int rot_tiles = 0, spt = 1;
    if (EPI == EPI_ROPE_QKV) {
        spt = D / 16;
        rot_tiles = (a.n_heads + a.n_kv_heads) * spt;
    }
    auto weight_row = [&](int i) -> int {
        if (EPI == EPI_SWIGLU) {
            const int f = tile_id * 8 + (i & 7);
            return f < a.inter ? (i < 8 ? f : a.inter + f) : -1;
        } else if (EPI == EPI_ROPE_QKV) {
            if (tile_id < rot_tiles) {
                const int h = tile_id / spt, s = tile_id % spt;
                return h * D + 8 * s + (i & 7) + (i < 8 ? 0 : D / 2);
            }
            return (a.n_heads + a.n_kv_heads) * D + (tile_id - rot_tiles) * 16 + i;
        } else {
            const int n = tile_id * 16 + i;
            return n < N ? n : -1;
        }
    };

    uint4* tile = lds + wave * 16 * (ST_KC / 8);
    // this workgroup's chunks of K: all of them, or its share when K is split over workgroups
    const int all_chunks = (K + ST_KC - 1) / ST_KC;
    const int shares = (K + 511) / 512;  // K is shared out in pieces of 512, whatever the chunk
    const int per_split = (shares + a.k_splits - 1) / a.k_splits * (512 / ST_KC);
    const int split = blockIdx.y, c_begin = split * per_split;
    const int chunks = min(all_chunks, c_begin + per_split);
    constexpr int LPR = ST_KC / 8;        // lanes that cover a row's piece of a chunk (16 bytes each)
    constexpr int RPL = LLMS_WAVE / LPR;  // rows per load instruction
    constexpr int NLOAD = 16 / RPL;       // load instructions per chunk
    constexpr int KSTEPS = ST_KC / 32;    // matrix instructions per chunk
    uint4 wreg[NLOAD];
    auto load_weights = [&](int c) {
        const int kl = c * ST_KC + 8 * (lane % LPR);
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int n = weight_row(i * RPL + lane / LPR);
            wreg[i] = (n >= 0 && kl < K) ? load_streaming(a.W + (size_t)n * K + kl) : zero;
        }
    };
    if (c_begin + wave < chunks) load_weights(c_begin + wave);

    const bool m_ok = m0 + r16 < M;
    const bf16* xrow = a.X + (size_t)(m_ok ? m0 + r16 : 0) * a.ldx;

    // what the rotary epilogue needs of its token (thread -> row idx / 8 or idx / 16 of X) is asked for now: after
    // the last barrier it would cost a trip to memory at the end of the kernel
    int epi_pos = 0, epi_slot = -1, epi_slot_v = -1;
    float epi_freq = 0.f;
    if (EPI == EPI_ROPE_QKV) {
        const int m8 = m0 + (int)threadIdx.x / 8, m16 = m0 + (int)threadIdx.x / 16;
        if (threadIdx.x < 128 && m8 < M) {
            if (a.inv_freq) epi_pos = a.positions[m8];
            if (a.slots) epi_slot = a.slots[m8];
            if (a.inv_freq && tile_id < rot_tiles) epi_freq = a.inv_freq[8 * (tile_id % spt) + (int)threadIdx.x % 8];
        }
        if (a.slots && m16 < M) epi_slot_v = a.slots[m16];
    }

    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int c = c_begin + wave; c < chunks; c += NW) {
        const int k0 = c * ST_KC;
        uint4 xreg[KSTEPS];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const int k = k0 + 32 * s + 8 * g;
            // (a branch, not a select: written as `cond ? load : zero` the load is issued for every lane, also for
            // the rows that do not exist, and the step at batch 8 takes 1.35 instead of 1.05 ms)
            if (m_ok && k < K)
                xreg[s] = *reinterpret_cast<const uint4*>(xrow + k);
            else
                xreg[s] = zero;
        }
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            const int row = i * RPL + lane / LPR;
            tile[row * LPR + ((lane % LPR) ^ row)] = wreg[i];
        }
        if (c + NW < chunks) load_weights(c + NW);  // the registers are free again
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const uint4 av = tile[r16 * LPR + ((4 * s + g) ^ r16)];
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av), as_bf16x8(xreg[s]), acc, 0, 0, 0);
        }
    }
    __syncthreads();  // every wave is done with its tile; the memory now carries the partial sums
    float* red = reinterpret_cast<float*>(lds);  // [wave][lane][4]; acc[r] = D[row 4g + r][m = r16]
#pragma unroll
    for (int r = 0; r < 4; ++r) red[(wave * LLMS_WAVE + lane) * 4 + r] = acc[r];
    __syncthreads();
    // sum of the 4 waves for weight row i (0..15) of this tile and row m0 + ml of X, wave 0 first
    auto total_of = [&](int i, int ml) -> float {
        const int src_lane = (i / 4) * 16 + ml, r = i % 4;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[(w * LLMS_WAVE + src_lane) * 4 + r];
        return s;
    };
    const int idx = threadIdx.x;
    TOut* C = reinterpret_cast<TOut*>(a.C) + (size_t)split * M * a.ldc;  // (one result, or one array of partial sums per split)

    if (EPI == EPI_PLAIN) {
        const int i = idx % 16, ml = idx / 16, m = m0 + ml, n = tile_id * 16 + i;  // consecutive threads: consecutive features
        if (idx < 256 && m < M && n < N) {
            float s = total_of(i, ml);
            if (a.bias && split == 0) s += bf16_bits_to_f32(a.bias[n].bits);
            store_out<TOut>(C + (size_t)m * a.ldc + n, s);
        }
    } else if (EPI == EPI_SWIGLU) {
        const int j = idx % 8, ml = idx / 8, m = m0 + ml, f = tile_id * 8 + j;
        if (idx < 128 && m < M && f < a.inter) {
            const float gate = bfr(total_of(j, ml)), up = bfr(total_of(j + 8, ml));
            store_out<TOut>(C + (size_t)m * a.ldc + f, bfr(gate / (1.f + expf(-gate))) * up);
        }
    } else {
        const int nh = a.n_heads, nkv = a.n_kv_heads, bs = a.block_size;
        if (tile_id < rot_tiles) {
            const int j = idx % 8, ml = idx / 8, m = m0 + ml;
            if (idx < 128 && m < M) {
                const int h = tile_id / spt, s = tile_id % spt, d = 8 * s + j;
                float lo = total_of(j, ml), hi = total_of(j + 8, ml);
                if (a.bias) {
                    lo += bf16_bits_to_f32(a.bias[h * D + d].bits);
                    hi += bf16_bits_to_f32(a.bias[h * D + d + D / 2].bits);
                }
                lo = bfr(lo);  // the projection's result is bfloat16 before it is rotated
                hi = bfr(hi);
                float ra = lo, rb = hi;
                if (a.inv_freq) {
                    const float2 angle = rotary_angle((float)epi_pos, epi_freq);
                    const float2 r = rotate_pair(lo, hi, angle.y, angle.x);
                    ra = r.x;
                    rb = r.y;
                }
                if (h < nh) {
                    store_out<TOut>(C + (size_t)m * a.ldc + h * D + d, ra);
                    store_out<TOut>(C + (size_t)m * a.ldc + h * D + d + D / 2, rb);
                } else {
                    const int slot = epi_slot;
                    if (slot >= 0) {
                        const int page = slot / bs, off = slot % bs;
                        bf16* dst = a.k_pool + (((size_t)page * nkv + (h - nh)) * bs + off) * D;
                        dst[d].bits = f32_to_bf16_bits(ra);
                        dst[d + D / 2].bits = f32_to_bf16_bits(rb);
                    }
                }
            }
        } else {
            const int i = idx % 16, ml = idx / 16, m = m0 + ml;
            const int slot = epi_slot_v;
            if (idx < 256 && m < M && slot >= 0) {
                const int f = (tile_id - rot_tiles) * 16 + i;  // feature among the value heads
                float v = total_of(i, ml);
                if (a.bias) v += bf16_bits_to_f32(a.bias[(nh + nkv) * D + f].bits);
                const int kvh = f / D, d = f % D, page = slot / bs, off = slot % bs;
                a.v_pool[(((size_t)page * nkv + kvh) * D + d) * bs + off].bits = f32_to_bf16_bits(v);
            }
        }
    }
}

// 17 to 64 rows against a short, wide weight (o_proj, down_proj): K is cut into slices of 512 and a workgroup
// (blockIdx.y = slice) keeps that slice of all rows of X in LDS, where its 4 waves, each with 16 weight rows of its
// own, read it as the second operand; with one workgroup per block of 16 rows (above) every workgroup would pull
// its weights through L2 again.  The weights come straight from memory in the matrix instruction's layout (a lane
// reads 16 bytes of row l%16 at element 8*(l/16) of each k-step: 64 bytes per row and instruction, and the 16
// instructions of a wave use every byte of the 1 KB it touches per row), all 16 loads in flight before the first
// product.  Every slice leaves 32-bit partial sums P[slice][M][N]; the norm kernel that follows adds them up.
#define SL_KC 512
#define SL_PITCH (SL_KC * 2 + 16)  // bytes per row of X in LDS: the 16 rows of an operand fall into different banks

template <int MB>  // blocks of 16 rows of X
__global__ __launch_bounds__(ST_WAVES* LLMS_WAVE) void gemm_slices_kernel(const bf16* __restrict__ X, int ldx,
                                                                         const bf16* __restrict__ W,
                                                                         float* __restrict__ P, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) char x_lds[MB * 16 * SL_PITCH];
    constexpr int THREADS = ST_WAVES * LLMS_WAVE;
    constexpr int PIECES = MB * 16 * (SL_KC / 8) / THREADS;  // 16-byte pieces of the slice per thread
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE, r16 = lane % 16, g = lane / 16;
    const int slice = blockIdx.y, k0 = slice * SL_KC;
    // the slice of X (addresses clamped, what lies outside is zeroed when it is stored)
    uint4 xr[PIECES];
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int idx = p * THREADS + tid, row = idx / (SL_KC / 8), k = k0 + (idx % (SL_KC / 8)) * 8;
        const bool ok = row < M && k < K;
        xr[p] = *reinterpret_cast<const uint4*>(X + (size_t)(ok ? row : 0) * ldx + (ok ? k : 0));
    }
    // this wave's 16 weight rows x 512 (clamped likewise: what they meet in X is zero)
    const int tile = blockIdx.x * ST_WAVES + wave, n = tile * 16 + r16;
    const bf16* wrow = W + (size_t)(n < N ? n : N - 1) * K;
    uint4 wr[16];
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        const int k = k0 + 32 * s + 8 * g;
        wr[s] = load_streaming(wrow + (k < K ? k : 0));
    }
    __builtin_amdgcn_sched_barrier(0);  // all loads are issued before anything waits for the first
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int idx = p * THREADS + tid, row = idx / (SL_KC / 8), piece = idx % (SL_KC / 8);
        if (!(row < M && k0 + piece * 8 < K)) xr[p] = make_uint4(0, 0, 0, 0);
        *reinterpret_cast<uint4*>(x_lds + row * SL_PITCH + piece * 16) = xr[p];
    }
    __syncthreads();
    f32x4 acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[b] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 16; ++s) {
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const uint4 xv = *reinterpret_cast<const uint4*>(x_lds + (16 * b + r16) * SL_PITCH + 64 * s + 16 * g);
            acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wr[s]), as_bf16x8(xv), acc[b], 0, 0, 0);
        }
    }
    // acc[b][r] = D[weight row 4g + r][row 16b + r16 of X]
    float* out = P + (size_t)slice * M * N;
    const int n0 = tile * 16 + 4 * g;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = 16 * b + r16;
        if (m >= M || n0 >= N) continue;
        if (n0 + 3 < N && N % 4 == 0) {
            *reinterpret_cast<f32x4*>(out + (size_t)m * N + n0) = acc[b];
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n0 + r < N) out[(size_t)m * N + n0 + r] = acc[b][r];
        }
    }
}

// A launch with a workgroup or less per CU gets chunks of 512 (16 KB in flight per wave: all a lone workgroup can
// do for its CU), a larger one chunks of 128 (eight workgroups per CU, no rounds); up to three workgroups per CU
// and 16 rows these have 8 waves, which doubles what the launch has in flight (TinyLlama's down_proj: 7.4 to 6.5
// microseconds at batch 1, 7.5 to 7.2 at batch 8; with more workgroups or more rows the same was slower: the
// 7B shape's o_proj with 1,024 workgroups 9.0 to 9.8).
#define ST_FEW_WORKGROUPS 256

template <typename TOut, int EPI>
static void launch_stream(unsigned tiles, const StreamArgs& a, hipStream_t stream) {
    const dim3 grid(tiles, a.k_splits);
    if ((long long)tiles * a.k_splits <= ST_FEW_WORKGROUPS)
        gemm_stream_kernel<TOut, EPI, 512, 4><<<grid, 4 * LLMS_WAVE, 0, stream>>>(a);
    else if ((long long)tiles * a.k_splits <= 3 * ST_FEW_WORKGROUPS && a.M <= 16)
        gemm_stream_kernel<TOut, EPI, 128, 8><<<grid, 8 * LLMS_WAVE, 0, stream>>>(a);
    else
        gemm_stream_kernel<TOut, EPI, 128, 4><<<grid, 4 * LLMS_WAVE, 0, stream>>>(a);
}

extern "C" {

// epilogue: 0 plain (C [M,N] + bias), 1 gated (W = [gate; up] of `inter` rows each, C [M, inter]),
// 2 rotary q/k/v (W = [q; k; v], C = q [M, n_heads*head_dim], k and v stored at `slots` when given).
// out_dtype: 0 float32, 1 bfloat16.
// k_splits > 1 (plain epilogue, float32): K is shared out to k_splits workgroups per tile, a short wide matrix
// then fills the chip; C is [k_splits][M][ldc], partial sums that the caller adds up (bias in the first).
int llms_gemm_stream(int out_dtype, int epilogue, void* C, int ldc, const void* X, int ldx, const void* W,
                     const void* bias, int M, int N, int K, int inter, int n_heads, int n_kv_heads, int head_dim,
                     int block_size, const float* inv_freq, const int* positions, const int* slots, void* k_pool,
                     void* v_pool, int k_splits, hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_stream: needs 1 <= M <= 64 and positive sizes");
    LLMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldx >= K, "gemm_stream: K and the row stride of X must be multiples of 8");
    LLMS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_stream: X and W must be 16-byte aligned");
    LLMS_REQUIRE(C != nullptr && (out_dtype == 0 || out_dtype == 1), "gemm_stream: bad output");
    LLMS_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm_stream: epilogue must be 0, 1 or 2");
    LLMS_REQUIRE(k_splits >= 1 && k_splits <= 16, "gemm_stream: k_splits must be in 1..16");
    LLMS_REQUIRE(k_splits == 1 || (epilogue == EPI_PLAIN && out_dtype == 0),
                 "gemm_stream: K is split for plain 32-bit partial sums only");
    StreamArgs a = {C, ldc, (const bf16*)X, ldx, (const bf16*)W, (const bf16*)bias, M, N, K, 0, k_splits, inter, n_heads,
                    n_kv_heads, head_dim, block_size, inv_freq, positions, slots, (bf16*)k_pool, (bf16*)v_pool};
    unsigned grid;
    if (epilogue == EPI_PLAIN) {
        LLMS_REQUIRE(ldc >= N, "gemm_stream: ldc too small");
        grid = (N + 15) / 16;
    } else if (epilogue == EPI_SWIGLU) {
        LLMS_REQUIRE(inter > 0 && inter % 8 == 0 && N == 2 * inter && bias == nullptr && ldc >= inter,
                     "gemm_stream: the gated epilogue needs N = 2*inter, inter % 8 == 0, no bias");
        grid = inter / 8;
    } else {
        LLMS_REQUIRE(n_heads > 0 && n_kv_heads > 0 && head_dim >= 16 && head_dim % 16 == 0 &&
                         N == (n_heads + 2 * n_kv_heads) * head_dim && ldc >= n_heads * head_dim,
                     "gemm_stream: the rotary epilogue needs head_dim % 16 == 0 and N = (heads + 2 kv heads) * head_dim");
        LLMS_REQUIRE(positions != nullptr || inv_freq == nullptr, "gemm_stream: rotation needs positions");
        LLMS_REQUIRE(slots == nullptr || (k_pool && v_pool && block_size > 0), "gemm_stream: slots given without pools");
        grid = (n_heads + n_kv_heads) * (head_dim / 16) + n_kv_heads * head_dim / 16;
    }
    a.num_tiles = (int)grid;
    grid = ((grid + 7) / 8) * 8 * ((M + 15) / 16);  // every XCD gets whole tiles with all their row blocks
#define ST_EPI(E)                                                   \
    if (out_dtype == 0) launch_stream<float, E>(grid, a, stream);   \
    else launch_stream<bf16, E>(grid, a, stream);
    if (epilogue == EPI_PLAIN) { ST_EPI(EPI_PLAIN) }
    else if (epilogue == EPI_SWIGLU) { ST_EPI(EPI_SWIGLU) }
    else { ST_EPI(EPI_ROPE_QKV) }
#undef ST_EPI
    LLMS_LAUNCH_CHECK();
}

// P[slice][M][N] (float32, contiguous) = X[:, slice] * W[:, slice]^T for the ceil(K / 512) slices of K; their sum in
// order is X * W^T.  For 17 to 64 rows (fewer are taken too) against a weight that is short and wide.
int llms_gemm_slices(void* P, const void* X, int ldx, const void* W, int M, int N, int K, hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_slices: needs 1 <= M <= 64 and positive sizes");
    LLMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldx >= K, "gemm_slices: K and the row stride of X must be multiples of 8");
    LLMS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)P % 16) == 0,
                 "gemm_slices: X, W and P must be 16-byte aligned");
    const int slices = (K + SL_KC - 1) / SL_KC, tiles = (N + 15) / 16;
    LLMS_REQUIRE(slices <= 65535, "gemm_slices: K too large");
    const dim3 grid((tiles + ST_WAVES - 1) / ST_WAVES, slices);
    const bf16* x = (const bf16*)X;
    const bf16* w = (const bf16*)W;
    switch ((M + 15) / 16) {
        case 1: gemm_slices_kernel<1><<<grid, ST_WAVES * LLMS_WAVE, 0, stream>>>(x, ldx, w, (float*)P, M, N, K); break;
        case 2: gemm_slices_kernel<2><<<grid, ST_WAVES * LLMS_WAVE, 0, stream>>>(x, ldx, w, (float*)P, M, N, K); break;
        case 3: gemm_slices_kernel<3><<<grid, ST_WAVES * LLMS_WAVE, 0, stream>>>(x, ldx, w, (float*)P, M, N, K); break;
        default: gemm_slices_kernel<4><<<grid, ST_WAVES * LLMS_WAVE, 0, stream>>>(x, ldx, w, (float*)P, M, N, K); break;
    }
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
