// bfloat16 matrix product for up to 64 rows (decoding) with one workgroup per compute unit:
//   C[M,N] = f(X)[M,K] * W[N,K]^T, 32-bit sums on the gfx950 matrix cores.
// Two kernels: gemm_decode_kernel (up to 16 rows, which stay in LDS; described first) and gemm_decode_rows_kernel
// (the rows in registers: 17 to 64 rows of up to 2,048 columns, 9 to 16 rows whose K is too long for LDS, and K
// shared out to sets of workgroups that leave partial sums; described where it stands).
//
// A decode step is a chain of short launches; what each of them costs beyond the bytes of its weight is what it
// does before its first load is out, the rows of X that every workgroup pulls in, and every launch that only
// norms or adds.  Here a compute unit gets one workgroup of 16 waves, which owns an equal share of the weight rows
// (every unit reads the same number of bytes) and whose waves share K out in chunks of 128 for good: wave w takes
// chunks w, w + 16, ... of every tile.  So the part of X a wave needs is the same for all its tiles: it loads its
// chunks of the rows that exist (a load instruction per 4 rows), once, and leaves them in LDS, where the matrix
// instruction's second operand is read from.  Because X enters a compute unit once, what is done to X on the way
// in is paid once per unit as well: the RMSNorm of the rows (src/llmserve/model/llama.py:18-28; the workgroup
// holds whole rows, so the sum of squares is a reduction over what its waves hold) is part of the prologue, and a
// layer needs no norm kernel.  The weights go through a wave-private, XOR-swizzled LDS tile to reach the layout of
// v_mfma_f32_16x16x32_bf16, as in gemm_stream.hip.
//
// Memory answers a wave in the order it asked, and a compute unit's address unit takes 16 cycles per 16-byte load
// instruction whether the lanes' addresses exist or not.  So the small things are asked for first (rows of X, the
// norm's weight, what the epilogue needs), then the weights; no load instruction is issued in vain (a tile is 8 or
// 16 rows, a template parameter, and so is the number of tiles in flight), and after the rows of X none is issued
// under a condition: the compiler counts the loads issued after the one it waits for, and where paths differ in
// that count it waits for all.  Lanes whose row or column does not exist load through the buffer descriptor from
// beyond its end, which brings zeros and touches no memory.
//
// Epilogues (the waves' partial sums meet in LDS in the order of the waves):
//   PLAIN     C = sums (+ bias), float32 or bfloat16.
//   SWIGLU    W = [gate; up]; C[m, f] = bf16(silu(bf16(gate))) * bf16(up)   (src/llmserve/model/llama.py:120).
//   ROPE_QKV  W = [q; k; v]; q and k rotated (src/llmserve/model/llama.py:31-54), q written, k and v stored at the
//             tokens' slots of the paged cache (values transposed inside a page).
//   RESIDUAL  residual[m, n] = bf16(residual[m, n] + bf16(sums)) in place: the layer's residual sum
//             (src/llmserve/model/llama.py:131-135), so that the next product's prologue finds whole rows to norm.
// What is shared out to the workgroups are units: a weight row (PLAIN, RESIDUAL), a feature's gate and up rows
// (SWIGLU), a rotary pair (i, i + D/2) of a query or key head or two value rows (ROPE_QKV).  A tile is up to 16
// rows of the matrix instruction: 8 or 16 units, or 8 units with their partners in rows 8 to 15.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define GD_NW 16     // waves of a workgroup
#define GD_KC 128    // elements of K per item
#define GD_MAX_XC 3  // chunks of K per wave
#define GD_MAX_K (GD_NW * GD_MAX_XC * GD_KC)
// LDS: the waves' tiles (later their partial sums), the rows' sums of squares, then the rows of X
#define GD_LDS_TILES (GD_NW * 16 * (GD_KC / 8) * 16)
#define GD_LDS_SQ (16 * GD_NW * 4)
#define GD_LDS_X_MAX (160 * 1024 - GD_LDS_TILES - GD_LDS_SQ)

#define GD_PLAIN 0
#define GD_SWIGLU 1
#define GD_ROPE_QKV 2
#define GD_RESIDUAL 3

struct DecodeGemmArgs {
    const bf16* W;
    const bf16* X;
    const bf16* bias;
    const bf16* norm_weight;  // given: the rows of X are normed on the way in (K is the width of the norm)
    float eps;
    void* C;
    int ldc, ldx;
    int M, N, K;
    int units;      // what the workgroups share out: workgroup w takes units_each (+1 for the first units_more)
    int units_each, units_more;
    int groups;     // groups of NT tiles the workgroup with the most tiles has
    int x_rows;     // rows of X kept in LDS: 8 or 16
    int x_pitch;    // bytes from row to row there: all chunks of K and 16 more (rows then start in different banks)
    int inter;  // SWIGLU
    int n_heads, n_kv_heads, head_dim, block_size;  // ROPE_QKV
    // ceil(2^32 / (head_dim / 2)): a unit's head by one multiply (exact while unit * head_dim < 2^32, which the
    // entry point checks); log2 of the page size, or -1 if it is no power of 2
    unsigned half_inv;
    int bs_shift;
    const float* inv_freq;
    const float* angles;  // [M][head_dim / 2] (sine, cosine): given, it stands for positions and inv_freq
    const int* positions;
    const int* slots;
    bf16* k_pool;
    bf16* v_pool;
    bf16* residual;  // RESIDUAL
    int ldr;
    // 17 to 64 rows, plain 32-bit output: K shared out to k_parts sets of wgs_per_part workgroups, part p taking the
    // columns from p * k_each on (k_each a multiple of 128) and leaving its sums at C + p * part_stride; a norm adds the
    // parts up.  ldw is the row stride of W (K of the whole weight).
    int ldw, k_parts, k_each, wgs_per_part;
    long long part_stride;
};

__device__ __forceinline__ bf16x8 gd_as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }
// Loads through a buffer descriptor: an offset beyond the buffer's end (GD_NOWHERE) brings zeros and touches no
// memory, so rows and columns that do not exist need no branch.  Weights are read once per step: non-temporal.
#define GD_NOWHERE 0x80000000u
__device__ __forceinline__ __amdgpu_buffer_rsrc_t gd_buffer(const void* p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 gd_load(__amdgpu_buffer_rsrc_t b, unsigned offset) {
    return __builtin_amdgcn_raw_buffer_load_b128(b, offset, 0, 0);
}
__device__ __forceinline__ u32x4 gd_load_streaming(__amdgpu_buffer_rsrc_t b, unsigned offset) {
    return __builtin_amdgcn_raw_buffer_load_b128(b, offset, 0, 2);
}
__device__ __forceinline__ float gd_bfr(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
// c + a.lo * b.lo + a.hi * b.hi of two packed pairs of bfloat16, in 32-bit (one instruction)
__device__ __forceinline__ float gd_dot2(uint32_t a, uint32_t b, float c) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}

template <typename TOut>
__device__ __forceinline__ void gd_store(TOut* p, float v);
template <>
__device__ __forceinline__ void gd_store<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void gd_store<bf16>(bf16* p, float v) { p->bits = f32_to_bf16_bits(v); }

// Weight row behind row i (0..15) of the tile of `upt` units that starts at unit u0 (-1: none).
template <int EPI>
__device__ __forceinline__ int gd_weight_row(const DecodeGemmArgs& a, int u0, int u_end, int upt, int i) {
    if (EPI == GD_PLAIN || EPI == GD_RESIDUAL) {
        const int n = u0 + i;
        return i < upt && n < u_end ? n : -1;
    }
    const int u = u0 + (i & 7);
    if (u >= u_end) return -1;
    const bool hi = i >= 8;
    if (EPI == GD_SWIGLU) return hi ? a.inter + u : u;
    const int D = a.head_dim, half = D / 2, rot_units = (a.n_heads + a.n_kv_heads) * half;
    if (u < rot_units) {
        const int h = (int)__umulhi((unsigned)u, a.half_inv), j = u - h * half;
        return h * D + j + (hi ? half : 0);
    }
    return (a.n_heads + a.n_kv_heads) * D + (u - rot_units) + (hi ? a.n_kv_heads * half : 0);
}

// What a thread needs from memory to finish one place (a unit or row of the weight, a row of X): asked for early,
// whether the place exists or not (from nowhere if it does not), used after the waves' sums have met.
struct GdFinish {
    int pos, slot;
    float freq;
    float sn, cs;
    unsigned res;
};

struct GdFinishBuffers {
    __amdgpu_buffer_rsrc_t pos, slot, freq, angles, res;
};

__device__ __forceinline__ GdFinishBuffers gd_finish_buffers(const DecodeGemmArgs& a) {
    GdFinishBuffers b;
    b.pos = gd_buffer(a.positions, a.positions ? (unsigned)a.M * 4 : 0u);
    b.slot = gd_buffer(a.slots, a.slots ? (unsigned)a.M * 4 : 0u);
    b.freq = gd_buffer(a.inv_freq, a.inv_freq ? (unsigned)a.head_dim * 2 : 0u);
    b.angles = gd_buffer(a.angles, a.angles ? (unsigned)a.M * a.head_dim * 4 : 0u);
    b.res = gd_buffer(a.residual, a.residual ? (unsigned)(((size_t)(a.M - 1) * a.ldr + a.N) * 2) : 0u);
    return b;
}

// `u`: the unit (pairs) or weight row (plain, residual) of the place, `m` its row of X; `live`: the place exists.
template <int EPI>
__device__ __forceinline__ void gd_ask(const DecodeGemmArgs& a, const GdFinishBuffers& b, bool live, int m, int u, GdFinish& f) {
    if (EPI == GD_ROPE_QKV) {
        const int half = a.head_dim / 2;
        f.slot = (int)__builtin_amdgcn_raw_buffer_load_b32(b.slot, live ? (unsigned)m * 4 : GD_NOWHERE, 0, 0);
        if (!a.slots) f.slot = -1;
        const bool rot = live && u < (a.n_heads + a.n_kv_heads) * half;
        // the angle's sine and cosine from the step's table, or position and frequency to work them out here
        // (every load is issued either way, from nowhere where it is not wanted, so that their number is known)
        const bool table = a.angles != nullptr;
        const int i_rot = u - (int)__umulhi((unsigned)u, a.half_inv) * half;  // u % half
        f.pos = (int)__builtin_amdgcn_raw_buffer_load_b32(b.pos, rot && !table ? (unsigned)m * 4 : GD_NOWHERE, 0, 0);
        f.freq = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(b.freq, rot && !table ? (unsigned)i_rot * 4 : GD_NOWHERE, 0, 0));
        typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
        const u32x2 sc = __builtin_amdgcn_raw_buffer_load_b64(b.angles, rot && table ? (unsigned)(m * half + i_rot) * 8 : GD_NOWHERE, 0, 0);
        f.sn = __uint_as_float(sc[0]);
        f.cs = __uint_as_float(sc[1]);
    }
    if (EPI == GD_RESIDUAL)
        f.res = __builtin_amdgcn_raw_buffer_load_b16(b.res, live ? (unsigned)(m * a.ldr + u) * 2 : GD_NOWHERE, 0, 0);
}

// PLAIN, RESIDUAL: the sum `s` of weight row n and row m of X.
template <typename TOut, int EPI>
__device__ __forceinline__ void gd_finish_row(const DecodeGemmArgs& a, int m, int n, float s, const GdFinish& f,
                                              size_t part_offset = 0) {
    if (a.bias) s += bf16_bits_to_f32(a.bias[n].bits);
    if (EPI == GD_PLAIN)
        gd_store<TOut>(reinterpret_cast<TOut*>(a.C) + part_offset + (size_t)m * a.ldc + n, s);
    else
        a.residual[(size_t)m * a.ldr + n].bits = f32_to_bf16_bits(bf16_bits_to_f32((uint16_t)f.res) + gd_bfr(s));
}

// SWIGLU, ROPE_QKV: the sums `lo` and `hi` of unit u's two weight rows and row m of X.
template <typename TOut, int EPI>
__device__ __forceinline__ void gd_finish_pair(const DecodeGemmArgs& a, int m, int u, float lo, float hi, const GdFinish& f) {
    if (EPI == GD_SWIGLU) {
        const float gate = gd_bfr(lo), up = gd_bfr(hi);
        gd_store<TOut>(reinterpret_cast<TOut*>(a.C) + (size_t)m * a.ldc + u, gd_bfr(gate / (1.f + expf(-gate))) * up);
        return;
    }
    const int nh = a.n_heads, nkv = a.n_kv_heads, D = a.head_dim, half = D / 2, bs = a.block_size;
    const int rot_units = (nh + nkv) * half;
    if (a.bias) {
        lo += bf16_bits_to_f32(a.bias[gd_weight_row<EPI>(a, u, u + 1, 8, 0)].bits);
        hi += bf16_bits_to_f32(a.bias[gd_weight_row<EPI>(a, u, u + 1, 8, 8)].bits);
    }
    lo = gd_bfr(lo);  // the projection's result is bfloat16 before it is rotated
    hi = gd_bfr(hi);
    const int slot = f.slot;
    const int page = a.bs_shift >= 0 ? slot >> a.bs_shift : slot / bs, off = slot - page * bs;  // (used where slot >= 0)
    if (u < rot_units) {
        const int h = (int)__umulhi((unsigned)u, a.half_inv), d = u - h * half;
        float ra = lo, rb = hi;
        if (a.inv_freq || a.angles) {
            const float2 angle = a.angles ? make_float2(f.sn, f.cs) : rotary_angle((float)f.pos, f.freq);
            const float2 r = rotate_pair(lo, hi, angle.y, angle.x);
            ra = r.x;
            rb = r.y;
        }
        if (h < nh) {
            TOut* q = reinterpret_cast<TOut*>(a.C) + (size_t)m * a.ldc + h * D + d;
            gd_store<TOut>(q, ra);
            gd_store<TOut>(q + half, rb);
        } else if (slot >= 0) {
            bf16* dst = a.k_pool + (((size_t)page * nkv + (h - nh)) * bs + off) * D;
            dst[d].bits = f32_to_bf16_bits(ra);
            dst[d + half].bits = f32_to_bf16_bits(rb);
        }
    } else if (slot >= 0) {
        // features f_lo and f_hi among the value heads: a page holds [kv head][dimension][token], and kv head times
        // D plus dimension is the feature itself
        const int f_lo = u - rot_units, f_hi = f_lo + nkv * half;
        a.v_pool[((size_t)page * nkv * D + f_lo) * bs + off].bits = f32_to_bf16_bits(lo);
        a.v_pool[((size_t)page * nkv * D + f_hi) * bs + off].bits = f32_to_bf16_bits(hi);
    }
}

// XC: chunks of K a wave holds (ceil(K / 128 / 16)); LPI: load instructions per item, each 4 rows of 256 bytes (a
// tile is 4 LPI rows); NT: tiles of a group, whose partial sums meet in LDS together (the items of a group,
// NT * XC, are unrolled).
template <typename TOut, int EPI, int XC, int LPI, int NT>
__global__ __launch_bounds__(GD_NW* LLMS_WAVE) void gemm_decode_kernel(const DecodeGemmArgs a) {
    constexpr int NW = GD_NW;
    constexpr bool PAIRS = EPI == GD_SWIGLU || EPI == GD_ROPE_QKV;
    static_assert(!PAIRS || LPI == 4, "units with partners fill rows 0..7 and 8..15");
    constexpr int UPT = PAIRS ? 8 : 4 * LPI;  // units per tile
    constexpr int ITEMS = NT * XC;            // items (tile, chunk) of a group
    // items in flight per wave; a divisor of ITEMS, so that an item has the same place in the ring in every group
    constexpr int RING = ITEMS == 4 ? (XC == 1 ? 4 : 2) : (ITEMS < 3 ? ITEMS : 3);
    static_assert(ITEMS % RING == 0, "the ring must go round a whole number of times per group");
    constexpr int THREADS = NW * LLMS_WAVE;
    constexpr int PLACES = PAIRS ? 128 : 16 * UPT;  // (unit or row, row of X) pairs of a tile: one thread each
    constexpr int EPI_ROUNDS = (NT * PLACES + THREADS - 1) / THREADS;
    extern __shared__ __attribute__((aligned(16))) char gd_lds[];
    u32x4* lds = reinterpret_cast<u32x4*>(gd_lds);                      // per wave 16 rows x 16 pieces of 16 bytes
    float* red = reinterpret_cast<float*>(gd_lds);                       // later [tile of the group][wave][lane][4]
    float* sq_lds = reinterpret_cast<float*>(gd_lds + GD_LDS_TILES);     // [row][wave]
    char* x_lds = gd_lds + GD_LDS_TILES + GD_LDS_SQ;                     // [row][x_pitch bytes]
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int r16 = lane % 16, g = lane / 16;
    const int M = a.M, K = a.K, n_chunks = (K + GD_KC - 1) / GD_KC;
    const int wg = blockIdx.x;
    const int u_begin = wg * a.units_each + min(wg, a.units_more);
    const int u_last = u_begin + a.units_each + (wg < a.units_more ? 1 : 0);

    // ---- first what is small and needed early: this wave's chunks of the rows of X that exist (lane (g, p) brings
    // piece p of 16 bytes of rows g, g + 4, ...), and the norm's weight for the same columns
    u32x4 xf[4][XC], nwf[XC];
    const __amdgpu_buffer_rsrc_t x_buf = gd_buffer(a.X, (unsigned)(((size_t)(M - 1) * a.ldx + K) * 2));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (4 * i < M) {
#pragma unroll
            for (int j = 0; j < XC; ++j) {
                const int row = g + 4 * i, k = (wave + NW * j) * GD_KC + 8 * r16;
                xf[i][j] = gd_load(x_buf, row < M && k < K ? (unsigned)(row * a.ldx + k) * 2 : GD_NOWHERE);
            }
        }
    }
    if (a.norm_weight) {
        const __amdgpu_buffer_rsrc_t nw_buf = gd_buffer(a.norm_weight, (unsigned)K * 2);
#pragma unroll
        for (int j = 0; j < XC; ++j) nwf[j] = gd_load(nw_buf, (unsigned)((wave + NW * j) * GD_KC + 8 * r16) * 2);
        // The sum of squares waits for the rows of every wave: no wave asks for weights before every wave has asked
        // for its rows, or the last wave's rows would queue behind the others' weights.
        __builtin_amdgcn_s_barrier();
    }

    // ---- what a thread needs from memory to finish its places of a group of tiles
    const GdFinishBuffers fin_bufs = gd_finish_buffers(a);
    auto place_of = [&](int e, int& te, int& idx) {  // round e of this thread: tile of the group, place in the tile
        const int p = e * THREADS + tid;
        te = p / PLACES;
        idx = p % PLACES;
    };
    auto ask_finish = [&](int tile0, GdFinish(&f)[EPI_ROUNDS]) {
#pragma unroll
        for (int e = 0; e < EPI_ROUNDS; ++e) {
            int te, idx;
            place_of(e, te, idx);
            const int per = PAIRS ? 8 : UPT;
            const int m = idx / per, u = u_begin + (tile0 + te) * UPT + idx % per;
            gd_ask<EPI>(a, fin_bufs, te < NT && m < M && u < u_last, m, u, f[e]);
        }
    };
    GdFinish fin[EPI_ROUNDS];
    ask_finish(0, fin);

    // ---- then the stream of weights
    u32x4 ring[RING][LPI];
    const __amdgpu_buffer_rsrc_t w_buf = gd_buffer(a.W, (unsigned)((size_t)a.N * K * 2));
    // loads of item q of the group that starts at tile `tile0` (tile q / XC, this wave's chunk q % XC)
    auto issue = [&](u32x4(&w)[LPI], int tile0, int q) {
        const int c = wave + NW * (q % XC), kl = c * GD_KC + 8 * (lane % 16);
        const int u0 = u_begin + (tile0 + q / XC) * UPT;
#pragma unroll
        for (int i = 0; i < LPI; ++i) {
            const int n = gd_weight_row<EPI>(a, u0, u_last, UPT, i * 4 + lane / 16);
            w[i] = gd_load_streaming(w_buf, n >= 0 && kl < K ? (unsigned)(n * K + kl) * 2 : GD_NOWHERE);
        }
    };
    // (a wave issues in order and waits when the memory pipeline is full: with all its loads asked for here it
    // would get to the norm of its rows only after the pipeline has taken them all)
    issue(ring[0], 0, 0);

    // ---- the rows of X, normed if asked, go to LDS: only this wave reads its chunks there
    if (a.norm_weight) {
        // sum of squares of a row: the lane's elements, the 16 lanes that hold the row's pieces of a chunk, then the
        // waves (in their order)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (4 * i < M) {
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < XC; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) ss = gd_dot2(xf[i][j][e], xf[i][j][e], ss);
                // (within the 16 lanes: shifts by 1, 2, 4, 8 lanes with zeros coming in; the last lane has the sum)
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x111, 0xf, 0xf, true));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x112, 0xf, 0xf, true));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x114, 0xf, 0xf, true));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x118, 0xf, 0xf, true));
                if (r16 == 15) sq_lds[(g + 4 * i) * NW + wave] = ss;
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // (LDS writes done; the weights stay in flight across the barrier)
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (4 * i < M) {
                float total = 0.f;
#pragma unroll
                for (int w = 0; w < NW; w += 4) {
                    const f32x4 part = *reinterpret_cast<const f32x4*>(sq_lds + (g + 4 * i) * NW + w);
                    total += part[0];
                    total += part[1];
                    total += part[2];
                    total += part[3];
                }
                const float inv = rsqrtf(total / (float)K + a.eps);
                // y = weight * bf16(x * inv)  (cast before the weight, as the reference does)
#pragma unroll
                for (int j = 0; j < XC; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t xv = xf[i][j][e], wv = nwf[j][e];
                        const uint32_t y = pack_bf16x2(__uint_as_float(xv << 16) * inv, __uint_as_float(xv & 0xffff0000u) * inv);
                        // bf16 x bf16 is exact in 32-bit: a dot product with the partner's half zeroed is the product
                        xf[i][j][e] = pack_bf16x2(gd_dot2(y, wv & 0xffffu, 0.f), gd_dot2(y, wv & 0xffff0000u, 0.f));
                    }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (4 * i < a.x_rows) {  // (rows between M and x_rows: zeros; columns beyond K: zeros, which meet the weights' zeros)
#pragma unroll
            for (int j = 0; j < XC; ++j)
                if (wave + NW * j < n_chunks)  // (a row has room for the chunks that exist)
                    *reinterpret_cast<u32x4*>(x_lds + (g + 4 * i) * a.x_pitch + (wave + NW * j) * (GD_KC * 2) + 16 * r16) =
                        4 * i < M ? xf[i][j] : (u32x4){0u, 0u, 0u, 0u};
        }
    }

#pragma unroll
    for (int q = 1; q < RING; ++q) issue(ring[q], 0, q);

    u32x4* tile = lds + wave * 16 * (GD_KC / 8);
    const char* x_mine = x_lds + (r16 & (a.x_rows - 1)) * a.x_pitch + wave * (GD_KC * 2) + 16 * g;
    // one item: the chunk goes through the wave's LDS tile into the operand layout, then 4 matrix instructions
    auto stage = [&](const u32x4(&w)[LPI]) {
#pragma unroll
        for (int i = 0; i < LPI; ++i) {
            const int row = i * 4 + lane / 16;
            tile[row * 16 + ((lane % 16) ^ row)] = w[i];
        }
    };
    auto multiply = [&](f32x4& acc, int j) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const u32x4 av = tile[r16 * 16 + ((4 * s + g) ^ r16)];  // (rows beyond 4 LPI: whatever lies there)
            const u32x4 xv = *reinterpret_cast<const u32x4*>(x_mine + j * (NW * GD_KC * 2) + 64 * s);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gd_as_bf16x8(av), gd_as_bf16x8(xv), acc, 0, 0, 0);
        }
    };
    // the items of one group; `more`: another group follows, whose first items are asked for as the ring frees.  The
    // partial sums take the place of the waves' tiles once every wave is done with its own.
    auto run_group = [&](int tile0, const bool more) {
        f32x4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < ITEMS; ++q) {
            const bool live = wave + NW * (q % XC) < n_chunks;  // (a chunk beyond K: its loads brought zeros)
            if (live) stage(ring[q % RING]);
            if (q + RING < ITEMS) issue(ring[q % RING], tile0, q + RING);  // the registers are free again
            else if (more) issue(ring[q % RING], tile0 + NT, q + RING - ITEMS);
            if (live) multiply(acc[q / XC], q % XC);
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < NT; ++t) *reinterpret_cast<f32x4*>(red + ((t * NW + wave) * LLMS_WAVE + lane) * 4) = acc[t];
    };
    auto finish_group = [&](int tile0) {
        __syncthreads();
#pragma unroll
        for (int e = 0; e < EPI_ROUNDS; ++e) {
            int te, idx;
            place_of(e, te, idx);
            const int eu0 = u_begin + (tile0 + te) * UPT;  // first unit of the tile
            if (te >= NT) continue;
            // sum of the waves for row i (0..15) of the tile and row ml of X, wave 0 first
            auto total_of = [&](int i, int ml) -> float {
                const int src_lane = (i / 4) * 16 + ml, r = i % 4;
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) s += red[((te * NW + w) * LLMS_WAVE + src_lane) * 4 + r];
                return s;
            };
            if (!PAIRS) {
                const int i = idx % UPT, m = idx / UPT, n = eu0 + i;
                if (m < M && n < u_last) gd_finish_row<TOut, EPI>(a, m, n, total_of(i, m), fin[e]);
            } else {
                const int j = idx % 8, m = idx / 8, u = eu0 + j;
                if (m < M && u < u_last) gd_finish_pair<TOut, EPI>(a, m, u, total_of(j, m), total_of(j + 8, m), fin[e]);
            }
        }
    };
    // Every workgroup walks as many groups as the one with the most tiles (tiles that do not exist are zeros from
    // nowhere and are written nowhere); the last group is apart because nothing follows it.
    int tile0 = 0;
    for (int gr = 0; gr + 1 < a.groups; ++gr, tile0 += NT) {
        run_group(tile0, true);
        finish_group(tile0);
        ask_finish(tile0 + NT, fin);
        __syncthreads();  // the sums are read before the next tiles overwrite them
    }
    run_group(tile0, false);
    finish_group(tile0);
}

// 17 to 64 rows of X (RB blocks of 16): the same sharing out of weight rows and of K, with 8 waves that have
// twice the registers.  A wave keeps its chunks of all rows of X in registers (asked for as whole lines, then
// turned into the operand layout through the wave's LDS tile), and every chunk of weights it stages meets RB blocks
// of rows: RB matrix instructions per fragment read from LDS.  X enters a compute unit once, as much as the unit's
// share of a large weight; with one workgroup per block of 16 rows it would enter four times as many workgroups.
// Where the sums go to a norm (plain 32-bit output), K may be shared out as well: k_parts sets of workgroups, each
// with all of N and a part of K, leave one array of partial sums each, and a compute unit pulls 1/k_parts of X.
// With 16 waves and one block of rows the same kernel takes 9 to 16 rows whose K is too long for LDS (up to 6,144: three
// chunks of 16 rows are 48 of a wave's 128 registers).
#define GR_NW 8

template <typename TOut, int EPI, int XC, int RB, int NT, bool NORM, int NW = GR_NW, int LPI = 4>
__global__ __launch_bounds__(NW* LLMS_WAVE) void gemm_decode_rows_kernel(const DecodeGemmArgs a) {
    static_assert(!NORM || RB == 1, "the norm on the way in is for up to 16 rows");
    static_assert(NW == GR_NW || (NW == 16 && RB == 1), "16 waves have registers for one block of rows");
    constexpr bool PAIRS = EPI == GD_SWIGLU || EPI == GD_ROPE_QKV;
    static_assert(!PAIRS || LPI == 4, "units with partners fill rows 0..7 and 8..15");
    constexpr int UPT = PAIRS ? 8 : 4 * LPI;  // units per tile (rows of the tile beyond them hold whatever lies in LDS)
    constexpr int ITEMS = NT * XC;
    constexpr int RING = ITEMS % 2 == 0 ? 2 : (ITEMS < 3 ? ITEMS : 3);  // (1, 2, 3, 4, 6 items: 1, 2, 3, 2, 2)
    static_assert(ITEMS % RING == 0, "the ring must go round a whole number of times per group");
    constexpr int THREADS = NW * LLMS_WAVE;
    constexpr int PLACES = UPT * RB * 16;  // (unit or row, row of X) pairs of a tile: one thread each
    constexpr int EPI_ROUNDS = (NT * PLACES + THREADS - 1) / THREADS;
    __shared__ u32x4 lds[NW * 16 * (GD_KC / 8)];         // per wave 16 rows x 16 pieces of 16 bytes
    __shared__ __attribute__((aligned(16))) float red[NT * NW * RB * LLMS_WAVE * 4];  // [tile of the group][wave][block of rows][lane][4]
    float* sq_lds = red;  // the norm's sums of squares, [row][wave], before the first sums of the product
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int r16 = lane % 16, g = lane / 16;
    const int part = (int)blockIdx.x / a.wgs_per_part, wg = (int)blockIdx.x - part * a.wgs_per_part;
    const int k_from = part * a.k_each;
    const int M = a.M, K = min(a.K - k_from, a.k_each), n_chunks = (K + GD_KC - 1) / GD_KC;  // (this part's columns)
    const int u_begin = wg * a.units_each + min(wg, a.units_more);
    const int u_last = u_begin + a.units_each + (wg < a.units_more ? 1 : 0);

    // ---- this wave's chunks of all rows of X, asked for as whole 256-byte pieces of 4 rows per instruction (every
    // compute unit reads the same rows from L2 at this moment: half as many requests as 64-byte pieces would be);
    // they reach the operand layout (lane (r16, g): X[16 rb + r16][c*128 + 32 s + 8 g ..+7]) through the wave's
    // LDS tile further down
    u32x4 xr[XC][RB][4];
    const __amdgpu_buffer_rsrc_t x_buf = gd_buffer(a.X + k_from, (unsigned)(((size_t)(M - 1) * a.ldx + K) * 2));
#pragma unroll
    for (int j = 0; j < XC; ++j)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 16 * rb + 4 * i + lane / 16, k = (wave + NW * j) * GD_KC + 8 * (lane % 16);
                xr[j][rb][i] = gd_load(x_buf, row < M && k < K ? (unsigned)(row * a.ldx + k) * 2 : GD_NOWHERE);
            }
    u32x4 nwf[NORM ? XC : 1];
    if (NORM) {
        const __amdgpu_buffer_rsrc_t nw_buf = gd_buffer(a.norm_weight, (unsigned)K * 2);
#pragma unroll
        for (int j = 0; j < XC; ++j) nwf[j] = gd_load(nw_buf, (unsigned)((wave + NW * j) * GD_KC + 8 * (lane % 16)) * 2);
        __builtin_amdgcn_s_barrier();  // (no wave asks for weights before every wave has asked for its rows)
    }

    const GdFinishBuffers fin_bufs = gd_finish_buffers(a);
    auto place_of = [&](int e, int& te, int& idx) {
        const int p = e * THREADS + tid;
        te = p / PLACES;
        idx = p % PLACES;
    };
    auto ask_finish = [&](int tile0, GdFinish(&f)[EPI_ROUNDS]) {
#pragma unroll
        for (int e = 0; e < EPI_ROUNDS; ++e) {
            int te, idx;
            place_of(e, te, idx);
            const int m = idx / UPT, u = u_begin + (tile0 + te) * UPT + idx % UPT;
            gd_ask<EPI>(a, fin_bufs, te < NT && m < M && u < u_last, m, u, f[e]);
        }
    };
    GdFinish fin[EPI_ROUNDS];
    ask_finish(0, fin);

    u32x4 ring[RING][LPI];
    const __amdgpu_buffer_rsrc_t w_buf = gd_buffer(a.W + k_from, (unsigned)(((size_t)(a.N - 1) * a.ldw + K) * 2));
    auto issue = [&](u32x4(&w)[LPI], int tile0, int q) {
        const int c = wave + NW * (q % XC), kl = c * GD_KC + 8 * (lane % 16);
        const int u0 = u_begin + (tile0 + q / XC) * UPT;
#pragma unroll
        for (int i = 0; i < LPI; ++i) {
            const int n = gd_weight_row<EPI>(a, u0, u_last, UPT, i * 4 + lane / 16);
            w[i] = gd_load_streaming(w_buf, n >= 0 && kl < K ? (unsigned)(n * a.ldw + kl) * 2 : GD_NOWHERE);
        }
    };
#pragma unroll
    for (int q = 0; q < RING; ++q) issue(ring[q], 0, q);

    // ---- the norm of the rows, if asked: as in the kernel above (there the rows go to LDS afterwards, here they
    // stay in registers), under the cover of the weights in flight
    if (NORM) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (16 * rb + 4 * i >= M) continue;  // (rows that do not exist are zeros and stay zeros)
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < XC; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) ss = gd_dot2(xr[j][rb][i][e], xr[j][rb][i][e], ss);
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x111, 0xf, 0xf, true));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x112, 0xf, 0xf, true));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x114, 0xf, 0xf, true));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x118, 0xf, 0xf, true));
                if (r16 == 15) sq_lds[(16 * rb + 4 * i + g) * NW + wave] = ss;
            }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // (LDS writes done; the weights stay in flight across the barrier)
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (16 * rb + 4 * i >= M) continue;
                float total = 0.f;
#pragma unroll
                for (int w = 0; w < NW; w += 4) {
                    const f32x4 part = *reinterpret_cast<const f32x4*>(sq_lds + (16 * rb + 4 * i + g) * NW + w);
                    total += part[0];
                    total += part[1];
                    total += part[2];
                    total += part[3];
                }
                const float inv = rsqrtf(total / (float)K + a.eps);
#pragma unroll
                for (int j = 0; j < XC; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t xv = xr[j][rb][i][e], wv = nwf[j][e];
                        const uint32_t y = pack_bf16x2(__uint_as_float(xv << 16) * inv, __uint_as_float(xv & 0xffff0000u) * inv);
                        xr[j][rb][i][e] = pack_bf16x2(gd_dot2(y, wv & 0xffffu, 0.f), gd_dot2(y, wv & 0xffff0000u, 0.f));
                    }
            }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_s_barrier();  // (every wave has read the sums of squares before the product's sums go there)
    }

    u32x4* tile = lds + wave * 16 * (GD_KC / 8);
#pragma unroll
    for (int j = 0; j < XC; ++j)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = i * 4 + lane / 16;
                tile[row * 16 + ((lane % 16) ^ row)] = xr[j][rb][i];
            }
#pragma unroll
            for (int s_ = 0; s_ < 4; ++s_) xr[j][rb][s_] = tile[r16 * 16 + ((4 * s_ + g) ^ r16)];
        }
    auto run_group = [&](int tile0, const bool more) {
        f32x4 acc[RB];  // (of the tile under way: its sums go to LDS when its last chunk is in)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < ITEMS; ++q) {
            const bool live = wave + NW * (q % XC) < n_chunks;  // (a chunk beyond K: its loads brought zeros)
            if (live) {
#pragma unroll
                for (int i = 0; i < LPI; ++i) {
                    const int row = i * 4 + lane / 16;
                    tile[row * 16 + ((lane % 16) ^ row)] = ring[q % RING][i];
                }
            }
            if (q + RING < ITEMS) issue(ring[q % RING], tile0, q + RING);  // the registers are free again
            else if (more) issue(ring[q % RING], tile0 + NT, q + RING - ITEMS);
            if (live) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const u32x4 av = tile[r16 * 16 + ((4 * s + g) ^ r16)];
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb)
                        acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gd_as_bf16x8(av), gd_as_bf16x8(xr[q % XC][rb][s]), acc[rb], 0, 0, 0);
                }
            }
            if (q % XC == XC - 1) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    *reinterpret_cast<f32x4*>(red + ((((q / XC) * NW + wave) * RB + rb) * LLMS_WAVE + lane) * 4) = acc[rb];
                    acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
                }
            }
        }
    };
    auto finish_group = [&](int tile0) {
        __syncthreads();
#pragma unroll
        for (int e = 0; e < EPI_ROUNDS; ++e) {
            int te, idx;
            place_of(e, te, idx);
            if (te >= NT) continue;
            const int i = idx % UPT, m = idx / UPT, u = u_begin + (tile0 + te) * UPT + i;
            // sum of the waves for row i (0..15) of the tile and row m of X, wave 0 first
            auto total_of = [&](int row) -> float {
                const int src_lane = (row / 4) * 16 + m % 16, r = row % 4;
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) sum += red[(((te * NW + w) * RB + m / 16) * LLMS_WAVE + src_lane) * 4 + r];
                return sum;
            };
            if (m >= M || u >= u_last) continue;
            if (!PAIRS) gd_finish_row<TOut, EPI>(a, m, u, total_of(i), fin[e], (size_t)(part * a.part_stride));
            else gd_finish_pair<TOut, EPI>(a, m, u, total_of(i), total_of(i + 8), fin[e]);
        }
    };
    int tile0 = 0;
    for (int gr = 0; gr + 1 < a.groups; ++gr, tile0 += NT) {
        run_group(tile0, true);
        finish_group(tile0);
        ask_finish(tile0 + NT, fin);
        __syncthreads();  // the sums are read before the next tiles overwrite them
    }
    run_group(tile0, false);
    finish_group(tile0);
}

// 17 to 64 rows: K up to 2,048 (a wave's two chunks of 64 rows are 128 registers).
#define GR_GO(XC, RB, NT)                                                                                  \
    do {                                                                                                   \
        a.groups = (tiles + NT - 1) / NT;                                                                  \
        gemm_decode_rows_kernel<TOut, EPI, XC, RB, NT, NORM><<<grid, GR_NW * LLMS_WAVE, 0, stream>>>(a);   \
    } while (0)

template <typename TOut, int EPI, int RB, bool NORM = false>
static void gd_launch_rows_one_chunk(int tiles, unsigned grid, DecodeGemmArgs& a, hipStream_t stream) {
    const int groups = (tiles + 3) / 4, nt = (tiles + groups - 1) / groups;
    if (nt == 1) GR_GO(1, RB, 1);
    else if (nt == 2) GR_GO(1, RB, 2);
    else if (nt == 3) GR_GO(1, RB, 3);
    else GR_GO(1, RB, 4);
}

template <typename TOut, int EPI, int RB, bool NORM = false>
static void gd_launch_rows_two_chunks(int tiles, unsigned grid, DecodeGemmArgs& a, hipStream_t stream) {
    if (tiles == 1) GR_GO(2, RB, 1);
    else if constexpr (RB == 4) {  // (three tiles of 64 rows of two chunks would not fit the registers)
        if (tiles % 2) GR_GO(2, RB, 1);
        else GR_GO(2, RB, 2);
    }
    // three tiles a group, or two where that leaves fewer tiles that do not exist in the last group
    else if ((tiles + 2) / 3 * 3 - tiles <= (tiles + 1) / 2 * 2 - tiles) GR_GO(2, RB, 3);
    else GR_GO(2, RB, 2);
}

// 17 to 32 rows of a longer K (up to 4,096): three or four chunks of two blocks of rows are up to 128 of a wave's 256
// registers.  Two tiles a group, one where there is only one.
template <typename TOut, int EPI, int XC>
static void gd_launch_rows_long_k(int tiles, unsigned grid, DecodeGemmArgs& a, hipStream_t stream) {
    constexpr bool NORM = false;
    if (tiles == 1) GR_GO(XC, 2, 1);
    else GR_GO(XC, 2, 2);
}
#undef GR_GO

// 9 to 16 rows whose K does not fit LDS: 16 waves, two or three chunks each.  LPI = 2: tiles of 8 weight rows, for a
// share whose last tile of 16 would be half empty (two load instructions less per chunk, and with three chunks a group
// of one tile whose ring of three fits the registers).
template <typename TOut, int EPI, bool NORM, int LPI>
static void gd_launch_rows_16_waves(int chunks, int tiles, unsigned grid, DecodeGemmArgs& a, hipStream_t stream) {
#define GR_GO16(XC, NT)                                                                                          \
    do {                                                                                                         \
        a.groups = (tiles + NT - 1) / NT;                                                                        \
        gemm_decode_rows_kernel<TOut, EPI, XC, 1, NT, NORM, 16, LPI><<<grid, 16 * LLMS_WAVE, 0, stream>>>(a);    \
    } while (0)
    if (chunks <= 32) {
        if (tiles == 1) GR_GO16(2, 1);
        else GR_GO16(2, 2);
    } else {
        if constexpr (LPI == 2) {
            if (tiles == 1) {
                GR_GO16(3, 1);
                return;
            }
        }
        GR_GO16(3, 2);  // (a ring of three whole chunks beside three chunks of X would not fit the registers: two tiles
                        // a group, of which the second may not exist, and a ring of two)
    }
#undef GR_GO16
}

template <typename TOut, int EPI>
static int gd_launch_rows(int chunks, int rows, int tiles, bool low, unsigned grid, DecodeGemmArgs& a, hipStream_t stream) {
    if (rows <= 16) {
        if (low) {
            if constexpr (EPI == GD_PLAIN || EPI == GD_RESIDUAL) {
                if (a.norm_weight) gd_launch_rows_16_waves<TOut, EPI, true, 2>(chunks, tiles, grid, a, stream);
                else gd_launch_rows_16_waves<TOut, EPI, false, 2>(chunks, tiles, grid, a, stream);
            }
        } else if (a.norm_weight) gd_launch_rows_16_waves<TOut, EPI, true, 4>(chunks, tiles, grid, a, stream);
        else gd_launch_rows_16_waves<TOut, EPI, false, 4>(chunks, tiles, grid, a, stream);
        return LLMS_OK;
    }
    if (chunks > 2 * GR_NW) {  // (17 to 32 rows: checked by the caller)
        if (chunks <= 3 * GR_NW) gd_launch_rows_long_k<TOut, EPI, 3>(tiles, grid, a, stream);
        else gd_launch_rows_long_k<TOut, EPI, 4>(tiles, grid, a, stream);
        return LLMS_OK;
    }
    if (chunks <= GR_NW) {  // (no norm on the way in beyond 16 rows: checked by the caller)
        if (rows <= 32) gd_launch_rows_one_chunk<TOut, EPI, 2>(tiles, grid, a, stream);
        else gd_launch_rows_one_chunk<TOut, EPI, 4>(tiles, grid, a, stream);
    } else {
        if (rows <= 32) gd_launch_rows_two_chunks<TOut, EPI, 2>(tiles, grid, a, stream);
        else gd_launch_rows_two_chunks<TOut, EPI, 4>(tiles, grid, a, stream);
    }
    return LLMS_OK;
}

// `tiles`: tiles of the workgroup with the most units; `lds_bytes`: what the kernel needs of LDS.
template <typename TOut, int EPI, int LPI>
static int gd_launch(int chunks, int tiles, unsigned grid, unsigned lds_bytes, DecodeGemmArgs& a, hipStream_t stream) {
#define GD_GO(XC, NT)                                                                                            \
    do {                                                                                                         \
        static bool large_lds_allowed = false;                                                                   \
        if (!large_lds_allowed) {                                                                                \
            LLMS_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_decode_kernel<TOut, EPI, XC, LPI, NT>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));         \
            large_lds_allowed = true;                                                                            \
        }                                                                                                        \
        a.groups = (tiles + NT - 1) / NT;                                                                        \
        gemm_decode_kernel<TOut, EPI, XC, LPI, NT><<<grid, GD_NW * LLMS_WAVE, lds_bytes, stream>>>(a);           \
    } while (0)
    if (chunks <= GD_NW) {
        // tiles of a group: as few groups as possible, and then as few tiles that do not exist
        const int groups = (tiles + 3) / 4, nt = (tiles + groups - 1) / groups;
        if (nt == 1) GD_GO(1, 1);
        else if (nt == 2) GD_GO(1, 2);
        else if (nt == 3) GD_GO(1, 3);
        else GD_GO(1, 4);
    } else if (chunks <= 2 * GD_NW) {
        if (tiles % 2) GD_GO(2, 1);
        else GD_GO(2, 2);
    } else {
        GD_GO(3, 1);
    }
#undef GD_GO
    return LLMS_OK;
}

extern "C" {

// Whether up to 16 rows of K elements stay in LDS beside the tiles (8 of them up to 8 rows, else 16).
static bool gd_rows_fit_lds(int M, int K) {
    return (M <= 8 ? 8 : 16) * ((K + GD_KC - 1) / GD_KC * (GD_KC * 2) + 16) <= GD_LDS_X_MAX;
}

// Whether M rows of K elements fit: up to 16 rows in LDS, or where K is too long for that in the registers of 16
// waves, three chunks of 128 each; 17 to 64 rows in the registers of 8 waves, two chunks each (four up to 32 rows).
int llms_gemm_decode_fits(int M, int K) {
    if (M <= 0 || M > 64 || K <= 0 || K > GD_MAX_K) return 0;
    if (M > 32) return K <= 2 * GR_NW * GD_KC;
    if (M > 16) return K <= 4 * GR_NW * GD_KC;
    return 1;
}

// epilogue: 0 plain (C [M,N] + bias; out_dtype 0 float32, 1 bfloat16), 1 gated (W = [gate; up] of `inter` rows each,
// C [M, inter] bfloat16), 2 rotary q/k/v (W = [q; k; v], C = q [M, n_heads*head_dim] bfloat16, k and v stored at
// `slots` when given; the angles as position times inv_freq, or their sines and cosines as `angles` [M][head_dim / 2][2],
// or neither: no rotation), 3 residual (residual[M, N] += X W^T in place, bfloat16; C unused).
// norm_weight (bfloat16 [K]) given: the rows of X are replaced by RMSNorm(X) * norm_weight with `eps` on the way in.
// workgroups: how many share the work out (the caller passes the number of compute units).
// k_parts > 1 (17 to 64 rows, plain 32-bit sums): K is shared out as well, to k_parts sets of workgroups, and C is
// [k_parts][M][ldc]: partial sums for a norm to add up.
int llms_gemm_decode(int out_dtype, int epilogue, void* C, int ldc, const void* X, int ldx, const void* W,
                     const void* bias, const void* norm_weight, float eps, int M, int N, int K, int inter,
                     int n_heads, int n_kv_heads, int head_dim, int block_size, const float* inv_freq,
                     const float* angles, const int* positions, const int* slots, void* k_pool, void* v_pool,
                     void* residual, int ldr, int workgroups, int k_parts, hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_decode: needs 1 <= M <= 64 and positive sizes");
    LLMS_REQUIRE((long long)N * K < (1ll << 30) && (long long)M * ldx < (1ll << 30), "gemm_decode: operands of 2 GB or more");
    const int x_rows = M <= 8 ? 8 : 16, x_pitch = (K + GD_KC - 1) / GD_KC * (GD_KC * 2) + 16;
    LLMS_REQUIRE(k_parts >= 1 && k_parts <= 16, "gemm_decode: k_parts must be 1..16");
    const int k_each = k_parts == 1 ? K : ((K + GD_KC - 1) / GD_KC + k_parts - 1) / k_parts * GD_KC;  // columns of a part
    LLMS_REQUIRE(llms_gemm_decode_fits(M, k_each), "gemm_decode: the rows of X do not fit a compute unit (see llms_gemm_decode_fits)");
    LLMS_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldx >= K, "gemm_decode: K and the row stride of X must be multiples of 8");
    // (norming 32 rows in every compute unit was built and measured: 4 microseconds of vector arithmetic in the
    // prologue, more than the norm kernel it saves)
    LLMS_REQUIRE(M <= 16 || norm_weight == nullptr, "gemm_decode: more than 16 rows are taken as they are (no norm on the way in)");
    LLMS_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)norm_weight % 16) == 0,
                 "gemm_decode: X, W and the norm's weight must be 16-byte aligned");
    LLMS_REQUIRE(epilogue >= 0 && epilogue <= 3, "gemm_decode: epilogue must be 0..3");
    LLMS_REQUIRE(out_dtype == 1 || (out_dtype == 0 && epilogue == GD_PLAIN), "gemm_decode: 32-bit output goes with the plain epilogue");
    LLMS_REQUIRE(workgroups > 0 && workgroups <= 4096, "gemm_decode: bad number of workgroups");
    DecodeGemmArgs a = {(const bf16*)W, (const bf16*)X, (const bf16*)bias, (const bf16*)norm_weight, eps, C, ldc, ldx,
                        M, N, K, 0, 0, 0, 0, x_rows, x_pitch, inter, n_heads, n_kv_heads, head_dim, block_size, 0u, -1, inv_freq, angles, positions, slots,
                        (bf16*)k_pool, (bf16*)v_pool, (bf16*)residual, ldr, K, 1, K, 0, 0};
    if (epilogue == GD_PLAIN) {
        LLMS_REQUIRE(C != nullptr && ldc >= N, "gemm_decode: bad output");
        a.units = N;
    } else if (epilogue == GD_RESIDUAL) {
        LLMS_REQUIRE(residual != nullptr && ldr >= N, "gemm_decode: the residual epilogue needs the residual rows");
        LLMS_REQUIRE((long long)M * ldr < (1ll << 30), "gemm_decode: residual rows of 2 GB or more");
        a.units = N;
    } else if (epilogue == GD_SWIGLU) {
        LLMS_REQUIRE(C != nullptr && inter > 0 && N == 2 * inter && bias == nullptr && ldc >= inter,
                     "gemm_decode: the gated epilogue needs N = 2*inter and no bias");
        a.units = inter;
    } else {
        LLMS_REQUIRE(C != nullptr && n_heads > 0 && n_kv_heads > 0 && head_dim >= 4 && head_dim % 2 == 0 &&
                         (n_kv_heads * head_dim) % 2 == 0 && N == (n_heads + 2 * n_kv_heads) * head_dim &&
                         ldc >= n_heads * head_dim,
                     "gemm_decode: the rotary epilogue needs an even head_dim of 4 or more and N = (heads + 2 kv heads) * head_dim");
        LLMS_REQUIRE(positions != nullptr || inv_freq == nullptr, "gemm_decode: rotation needs positions");
        LLMS_REQUIRE(angles == nullptr || ((uintptr_t)angles % 8) == 0, "gemm_decode: the table of angles must be 8-byte aligned");
        LLMS_REQUIRE(slots == nullptr || (k_pool && v_pool && block_size > 0), "gemm_decode: slots given without pools");
        a.units = (n_heads + n_kv_heads) * (head_dim / 2) + n_kv_heads * head_dim / 2;
        LLMS_REQUIRE((long long)a.units * head_dim < (1ll << 32), "gemm_decode: too many heads for the rotary epilogue");
        a.half_inv = (unsigned)(((1ull << 32) + head_dim / 2 - 1) / (head_dim / 2));
        a.bs_shift = block_size > 0 && (block_size & (block_size - 1)) == 0 ? __builtin_ctz((unsigned)block_size) : -1;
    }
    if (k_parts > 1) {  // C is [k_parts][M][ldc] floats
        LLMS_REQUIRE(M > 16 && epilogue == GD_PLAIN && out_dtype == 0 && bias == nullptr && norm_weight == nullptr,
                     "gemm_decode: K is shared out only for 17 to 64 rows with plain 32-bit sums (no bias, no norm)");
        a.k_parts = k_parts;
        a.k_each = k_each;
        LLMS_REQUIRE((long long)(k_parts - 1) * a.k_each < K, "gemm_decode: more parts than K has chunks of 128");
        a.part_stride = (long long)M * ldc;
    }
    const int per_part = workgroups / k_parts > 0 ? workgroups / k_parts : 1;
    const unsigned wgs = (unsigned)(per_part < a.units ? per_part : a.units);  // workgroups that share the units out
    const unsigned grid = wgs * (unsigned)k_parts;
    a.wgs_per_part = (int)wgs;
    a.units_each = a.units / (int)wgs;
    a.units_more = a.units % (int)wgs;
    const int most = a.units_each + (a.units_more ? 1 : 0);  // units of the largest share
    const int chunks = (a.k_each + GD_KC - 1) / GD_KC;
    const unsigned lds = GD_LDS_TILES + GD_LDS_SQ + (unsigned)(x_rows * x_pitch);
    int rc;
    if (M > 16 || !gd_rows_fit_lds(M, K)) {  // the rows in registers: tiles of 16 weight rows (8 units with partners)
        const bool pairs = epilogue == GD_SWIGLU || epilogue == GD_ROPE_QKV;
        // up to 16 rows, units without partners: tiles of 8 weight rows where the last tile of 16 would be half empty
        const bool low = M <= 16 && !pairs && ((most + 7) / 8) % 2 == 1;
        const int tiles = pairs || low ? (most + 7) / 8 : (most + 15) / 16;
        if (epilogue == GD_SWIGLU) rc = gd_launch_rows<bf16, GD_SWIGLU>(chunks, M, tiles, low, grid, a, stream);
        else if (epilogue == GD_ROPE_QKV) rc = gd_launch_rows<bf16, GD_ROPE_QKV>(chunks, M, tiles, low, grid, a, stream);
        else if (epilogue == GD_RESIDUAL) rc = gd_launch_rows<bf16, GD_RESIDUAL>(chunks, M, tiles, low, grid, a, stream);
        else if (out_dtype == 0) rc = gd_launch_rows<float, GD_PLAIN>(chunks, M, tiles, low, grid, a, stream);
        else rc = gd_launch_rows<bf16, GD_PLAIN>(chunks, M, tiles, low, grid, a, stream);
    } else if (epilogue == GD_SWIGLU) rc = gd_launch<bf16, GD_SWIGLU, 4>(chunks, (most + 7) / 8, grid, lds, a, stream);
    else if (epilogue == GD_ROPE_QKV) rc = gd_launch<bf16, GD_ROPE_QKV, 4>(chunks, (most + 7) / 8, grid, lds, a, stream);
    else {
        // tiles of 8 rows where the last tile of 16 would be half empty (a share of up to 8 rows, of 17 to 24, ...):
        // two load instructions less per chunk
        const bool low = ((most + 7) / 8) % 2 == 1;
        const int tiles = low ? (most + 7) / 8 : (most + 15) / 16;
        if (epilogue == GD_RESIDUAL) {
            if (low) rc = gd_launch<bf16, GD_RESIDUAL, 2>(chunks, tiles, grid, lds, a, stream);
            else rc = gd_launch<bf16, GD_RESIDUAL, 4>(chunks, tiles, grid, lds, a, stream);
        } else if (out_dtype == 0) {
            if (low) rc = gd_launch<float, GD_PLAIN, 2>(chunks, tiles, grid, lds, a, stream);
            else rc = gd_launch<float, GD_PLAIN, 4>(chunks, tiles, grid, lds, a, stream);
        } else {
            if (low) rc = gd_launch<bf16, GD_PLAIN, 2>(chunks, tiles, grid, lds, a, stream);
            else rc = gd_launch<bf16, GD_PLAIN, 4>(chunks, tiles, grid, lds, a, stream);
        }
    }
    if (rc != LLMS_OK) return rc;
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
