// bfloat16 causal attention over the paged cache on the gfx950 matrix cores, for prompts,
// portions of prompts and decoded tokens alike.
//
// A wave owns a *column group*: up to 16 (token, query head) pairs of one request that share
// one KV head (for 8 heads per KV head: 2 tokens x 8 heads; for 1: 16 tokens; for 16: 1 token),
// and walks that request's keys in tiles of 32 through its block table:
//   S^T[key, col] = K[key, :] . Q[col, :]      v_mfma_f32_16x16x32_bf16, A = key rows straight from
//                                              the cache, B = queries held in registers
//   online softmax per column in 32-bit        (max, sum, rescale), masked by position and window
//   O^T[d, col] += V^T[d, key] . P^T[key, col] A = values, which the cache stores transposed inside
//                                              a page, so 8 keys of one dimension are one 16-byte load
// The row-to-key assignment of the two S^T tiles is chosen so that each lane ends up with 8 consecutive
// keys, which is what the B operand of the second product wants: no exchange between lanes.
//
// Two kernels, two arrangements of the waves of a workgroup:
//   attn_mfma_kernel (decoding): one column group; its key tiles are dealt to the 4 or 8 waves, which load
//     their operands straight from the cache (nothing goes through LDS on the way to the matrix instruction),
//     and optionally to `num_splits` workgroups whose partial results a second kernel merges.
//   attn_prompt_kernel (prompts): consecutive column groups of one request want the same keys and share
//     each tile through LDS, one or two groups per wave; without a window, each wave has a twin that takes every
//     other tile for the same columns, or (a short portion behind a long prefix) the keys of a block are shared
//     out to `num_splits` workgroups.
// All merges run in a fixed order, so a token's result does not depend on the batch around it.
//
// Needs block_size % 8 == 0, head_dim % 16 == 0 and <= 256, 16-byte aligned rows.
#include "common.h"
#include "attention_mfma.h"

#include <algorithm>
#include <mutex>
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
// 16 bytes on their way from memory to LDS, as a vector the compiler keeps in registers (an array of two uint4, a
// struct, that is filled in one place and emptied in another it copied through memory)
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    return pack_bf16x2(lo, hi);
}

// Keep elements [first, last) of 8 packed bfloat16, zero the rest.
__device__ __forceinline__ uint4 keep_elements(uint4 v, int first, int last) {
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = (2 * i >= first && 2 * i < last) ? 0x0000ffffu : 0u;
        const uint32_t hi = (2 * i + 1 >= first && 2 * i + 1 < last) ? 0xffff0000u : 0u;
        w[i] &= (lo | hi);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

struct AttnArgs {
    bf16* out;
    int out_stride;
    const bf16* q;
    int q_stride;
    const bf16* k_pool;
    const bf16* v_pool;
    const int* block_tables;
    const int* table_rows;  // row of block_tables of each request (null: the request's own index)
    int max_blocks;
    const int* cu_seqlens;
    const int* context_lens;
    int seq_begin;
    int n_heads, n_kv_heads, block_size, window;
    float scale;
    int num_splits;
    float* ws_o;   // [token, head, split, D]
    float* ws_ml;  // [token, head, split, 2]
    // decoding with num_splits > 1: one counter per column group (request, KV head, block of heads, group of tokens),
    // zero between launches.  Non-null: the workgroups of a group count themselves here and the last to arrive adds
    // the shares up (no merge kernel).
    unsigned* arrive;
    // token rows of the step that q, out and the workspace have: a column whose row lies beyond them (cu_seqlens on
    // the device that disagree with what the caller sized its tensors by) is left out, not written past the end
    int row_end;
    // prompts with twins: the first workgroup of every CU (the first `first_blocks` values of blockIdx.y) takes one
    // of the longest blocks of tokens, shortest of them first; the rest follow from the longest remaining one down
    int first_blocks;
    // decoding, every request of the launch with exactly one new token: the row of request seq_begin + i is
    // one_token_from + i, which saves a workgroup the wait for cu_seqlens before it can ask for its queries (-1: not so)
    int one_token_from;
};

// 2^x by the hardware's own instruction.  Scores are kept in units of log2(e) (scale_log2 = scale * log2 e), so
// that a weight is one multiply-add and one exponential.
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ const bf16* page_ptr(const bf16* base, int page, uint32_t page_stride) {
    return base + (uint64_t)(uint32_t)page * page_stride;  // one 32 x 32 -> 64 bit multiply-add
}

// Maximum and sum over the four lanes l, l^16, l^32, l^48 that share a column, with gfx950's row swaps
// (v_permlane32_swap, v_permlane16_swap: the upper half / the odd rows of 16 lanes of one operand change
// places with the lower half / the even rows of the other), which stay in the vector unit; a lane shuffle
// would go through LDS four times per tile.
// (the maximum as the instruction itself: fmaxf would first pass each swapped value, whose origin the compiler
// cannot see, through an instruction of its own that quiets a signalling NaN, four more per tile and column group)
__device__ __forceinline__ float max_of_swapped(unsigned a, unsigned b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

__device__ __forceinline__ float column_max(float x) {
    const unsigned xi = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const unsigned mi = __float_as_uint(max_of_swapped(a[0], a[1]));
    const auto b = __builtin_amdgcn_permlane16_swap(mi, mi, false, false);
    return max_of_swapped(b[0], b[1]);
}

__device__ __forceinline__ float column_sum(float x) {
    const unsigned xi = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const unsigned si = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane16_swap(si, si, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// One tile of 32 keys for CG column groups of 16 columns that share the keys: scores, online softmax, weighted
// values.
//   kf[u][s]: key rows of score tile u (row i = key 8*(i/4) + 4u + i%4), k-step s;  vf[m]: the lane's 8 keys
//   (jk .. jk+7) of value dimensions 16m + col, already zero where the key is outside the group's range;
//   qf[cg][s]: the lane's column of queries.  acc[cg][m][r] = O^T[16m + 4g + r][col], the column's reference
//   for its weights (times log2 e; its running maximum or a little less) and the sum of its weights are updated in
//   place; the sum as the lane's own share of it (the caller adds the four lanes of a column up once, at the end:
//   column_sum).  MASKED = false: every key of the tile is visible to every column of the wave (the caller
//   knows), which saves the comparisons.  The groups go through each stage side by side, not one group after the
//   other: their chains (matrix product, maximum, exponentials, matrix product) do not depend on each other, and
//   a wave that alternates between them waits less for each.
//   fill_values(): called once the score products are issued, may bring vf in then (it is read after the softmax):
//   what it asks LDS for arrives while the vector unit is busy, and does not stand in the way of the key rows.
#define STALE_MAX 8.f  // by how much (in powers of two) a column's maximum may pass the reference before a rescale
template <int DB, int KS, bool MASKED, int CG, class FillValues>
__device__ __forceinline__ void attend_tile_groups(f32x4 (&acc)[CG][DB], float (&m_run)[CG], float (&l_run)[CG],
                                                   const uint4 (&kf)[2][KS], uint4 (&vf)[DB], const uint4 (&qf)[CG][KS],
                                                   int jk, const int (&lo_col)[CG], const int (&p_col)[CG], float scale_log2,
                                                   FillValues fill_values) {
    f32x4 s_acc[CG][2];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            s_acc[cg][u] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s)
                s_acc[cg][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf[u][s]), as_bf16x8(qf[cg][s]), s_acc[cg][u], 0, 0, 0);
        }
    fill_values();
    // the lane holds its column's scores for the keys jk .. jk+7; the other 24 keys sit in the 3 other lane groups
    float sc[CG][8], t_max[CG], m_safe[CG];
    bool grew = false;
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        float tmax = -INFINITY;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sc[cg][e] = s_acc[cg][e / 4][e % 4];
            if (MASKED) {
                const int key = jk + e;
                if (!(key >= lo_col[cg] && key <= p_col[cg])) sc[cg][e] = -INFINITY;
            }
            tmax = fmaxf(tmax, sc[cg][e]);
        }
        t_max[cg] = tmax;  // of the lane's 8 keys
        grew = grew || tmax * scale_log2 > m_run[cg] + STALE_MAX;  // (scale > 0; also a column's first key: -inf + x = -inf)
    }
    // m_run is the reference the weights are taken against, not necessarily the maximum: while no score has passed
    // its column's reference by more than STALE_MAX (a factor of 2^STALE_MAX in the weights and sums, far inside
    // the range of 32-bit and bfloat16 numbers, and the same relative precision), nothing is rescaled, and the
    // maximum over the column's four lanes is not even formed.  The quotient at the end does not depend on the
    // reference.
    if (__builtin_amdgcn_ballot_w64(grew) != 0) {
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
            const float m_new = fmaxf(m_run[cg], column_max(t_max[cg]) * scale_log2);
            const float m_ref = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
            const float corr = exp2_fast(m_run[cg] - m_ref);  // 1 where the maximum stayed; 0 while the column has seen no key
            l_run[cg] *= corr;
#pragma unroll
            for (int m = 0; m < DB; ++m)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[cg][m][r] *= corr;
            m_run[cg] = m_new;
        }
    }
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) m_safe[cg] = (MASKED && m_run[cg] == -INFINITY) ? 0.f : m_run[cg];
    uint4 pf[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        float psum;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sc[cg][e] = exp2_fast(fmaf(sc[cg][e], scale_log2, -m_safe[cg]));
            psum = e == 0 ? sc[cg][0] : psum + sc[cg][e];
        }
        l_run[cg] += psum;  // (the lane's share: the four lanes of a column are added up once, by whoever reads the sum)
        pf[cg] = make_uint4(pack_bf16(sc[cg][0], sc[cg][1]), pack_bf16(sc[cg][2], sc[cg][3]), pack_bf16(sc[cg][4], sc[cg][5]),
                            pack_bf16(sc[cg][6], sc[cg][7]));
    }
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
        for (int m = 0; m < DB; ++m)
            acc[cg][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf[m]), as_bf16x8(pf[cg]), acc[cg][m], 0, 0, 0);
}

// The same for one column group (decoding).
template <int DB, int KS, bool MASKED>
__device__ __forceinline__ void attend_tile(f32x4 (&acc)[DB], float& m_run, float& l_run, const uint4 (&kf)[2][KS],
                                            const uint4 (&vf)[DB], const uint4 (&qf)[KS], int jk, int lo_col, int p_col,
                                            float scale_log2) {
    float m1[1] = {m_run}, l1[1] = {l_run};
    const int lo1[1] = {lo_col}, p1[1] = {p_col};
    attend_tile_groups<DB, KS, MASKED, 1>(reinterpret_cast<f32x4 (&)[1][DB]>(acc), m1, l1, kf, const_cast<uint4 (&)[DB]>(vf),
                                          reinterpret_cast<const uint4 (&)[1][KS]>(qf), jk, lo1, p1, scale_log2, [] {});
    m_run = m1[0];
    l_run = l1[0];
}

// 8 bytes to or from memory past the caches that other XCDs do not see (an L2 belongs to one XCD): what one
// workgroup leaves for another inside a kernel goes this way, with a relaxed atomic access at agent scope, which
// the compiler turns into a store that is written through and a load that does not hit a stale line.  No fence:
// a release at agent scope writes a whole L2 back and costs more than the kernel (9 to 130 microseconds a
// launch where this costs 1.5 to 3).
__device__ __forceinline__ void store_across(float* p, float a, float b) {
    const unsigned long long v = ((unsigned long long)__float_as_uint(b) << 32) | __float_as_uint(a);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float2 load_across(const float* p) {
    const unsigned long long v =
        __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__uint_as_float((unsigned)v), __uint_as_float((unsigned)(v >> 32)));
}

// The last workgroup of a column group adds the shares of all its workgroups up, split 0 first, with the arithmetic
// of attn_merge_kernel (the same bits).  SMAX >= num_splits: every load of a thread is asked for before the first
// is used (a split beyond the last is the last once more, with weight 0).
template <int DB, int SMAX>
__device__ __forceinline__ void merge_shares(const AttnArgs& a, size_t item0, bool col_ok, int wave, int nw, int g,
                                             bf16* orow) {
    constexpr int D = DB * 16;
    if (!col_ok) return;
    const int S = a.num_splits;
    float2 ml[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) ml[s] = load_across(a.ws_ml + 2 * (item0 + min(s, S - 1)));
    float m_tot = -INFINITY;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) m_tot = fmaxf(m_tot, ml[s].x);
    float w[SMAX], l_tot = 0.f;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        w[s] = (s < S && ml[s].x != -INFINITY) ? exp2_fast(ml[s].x - m_tot) : 0.f;
        if (s < S && ml[s].x != -INFINITY) l_tot += ml[s].y * w[s];
    }
    const float inv = 1.f / l_tot;
    for (int m = wave; m < DB; m += nw) {
        float2 lo[SMAX], hi[SMAX];
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            const float* share = a.ws_o + (item0 + min(s, S - 1)) * D + 16 * m + 4 * g;
            lo[s] = load_across(share);
            hi[s] = load_across(share + 2);
        }
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            if (s < S && ml[s].x != -INFINITY) {
                o.x += lo[s].x * w[s];
                o.y += lo[s].y * w[s];
                o.z += hi[s].x * w[s];
                o.w += hi[s].y * w[s];
            }
        }
        uint2 pk;
        pk.x = pack_bf16(o.x * inv, o.y * inv);
        pk.y = pack_bf16(o.z * inv, o.w * inv);
        *reinterpret_cast<uint2*>(orow + 16 * m + 4 * g) = pk;
    }
}

template <int DB, int NW>  // blocks of 16 dimensions of a head; waves of the workgroup (4 or 8), which share the keys
__global__ __launch_bounds__(NW* LLMS_WAVE) void attn_mfma_kernel(const AttnArgs a) {
    constexpr int D = DB * 16;
    constexpr int KS = (D + 31) / 32;  // k-steps of the score product
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE;
    const int col = lane % 16, g = lane / 16;

    const int G = a.n_heads / a.n_kv_heads;
    const int HG = G < 16 ? G : 16;       // heads of one column group
    const int TPG = 16 / HG;              // tokens of one column group
    const int HB = (G + HG - 1) / HG;     // column groups needed to cover a KV head's query heads
    const int kvh = blockIdx.y / HB, hb = blockIdx.y % HB;
    const int b = a.seq_begin + blockIdx.z;
    const bool one_each = a.one_token_from >= 0;
    const int tok0 = one_each ? a.one_token_from + (int)blockIdx.z : a.cu_seqlens[b];
    const int n_new = one_each ? 1 : a.cu_seqlens[b + 1] - tok0;
    const int ctx = a.context_lens[b];
    // (asked for together with the lengths: one trip to memory earlier than where the block table is first needed)
    const int table_row = a.table_rows ? a.table_rows[b] : b;
    // The request's first 64 page ids are asked for before its length is known (whatever the length, they are the
    // ones most launches need; entries beyond the request's own blocks are never used): with a table that has a row
    // per request and one token each, a workgroup's lengths, page ids and queries are one trip to memory.
    const int* table = a.block_tables + (size_t)table_row * a.max_blocks;
    int blk_base = 0, pages_reg = table[min(lane, a.max_blocks - 1)];

    const int tile = blockIdx.x / a.num_splits, split = blockIdx.x % a.num_splits;
    const int t_first = tile * TPG;  // first token (within the request's new tokens) of this group

    // this lane's column
    const int c_tok = t_first + col / HG, c_head_in = hb * HG + col % HG;
    const bool col_ok = col < HG * TPG && c_tok < n_new && c_head_in < G && tok0 + c_tok < a.row_end;
    const int head = kvh * G + c_head_in;
    // queries of this lane's column: Q[col][32s + 8g .. +7]; asked for before the request's length is here where
    // the rows are known without it
    const uint4 zero = make_uint4(0, 0, 0, 0);
    uint4 qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int d = 32 * s + 8 * g;
        qf[s] = (col_ok && d < D)
                    ? *reinterpret_cast<const uint4*>(a.q + (size_t)(tok0 + c_tok) * a.q_stride + (size_t)head * D + d)
                    : zero;
    }
    if (t_first >= n_new || ctx <= 0) return;  // (uniform over the workgroup)

    const int p_col = col_ok ? ctx - n_new + c_tok : -1;  // absolute position of the column's token
    const int lo_col = (a.window > 0 && p_col - a.window + 1 > 0) ? p_col - a.window + 1 : 0;
    // key range of the whole group
    const int t_last = min(t_first + TPG, n_new) - 1;
    const int p_max = ctx - n_new + t_last;
    const int p_min = ctx - n_new + t_first;
    const int lo_min = (a.window > 0 && p_min - a.window + 1 > 0) ? p_min - a.window + 1 : 0;
    const int j_begin = lo_min & ~31;
    const int n_tiles = (p_max - j_begin) / 32 + 1;

    f32x4 acc[DB];
#pragma unroll
    for (int m = 0; m < DB; ++m) acc[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    const uint32_t page_stride = (uint32_t)a.n_kv_heads * a.block_size * D;
    const bf16* k_base = a.k_pool + (size_t)kvh * a.block_size * D;
    const bf16* v_base = a.v_pool + (size_t)kvh * a.block_size * D;
    const float scale_log2 = a.scale * 1.44269504088896341f;
    // first and last tile whose 32 keys every column of the group sees
    const int lo_max = (a.window > 0 && p_max - a.window + 1 > 0) ? p_max - a.window + 1 : 0;

    // this workgroup's share of the tiles, dealt to its waves
    const int per_split = (n_tiles + a.num_splits - 1) / a.num_splits;
    const int t_begin = split * per_split + wave;
    const int t_end = min(n_tiles, (split + 1) * per_split);
    constexpr int t_step = NW;
    // The request's page ids are held in registers, 64 blocks at a time (lane l: block blk_base + l), and
    // handed around with lane shuffles, so finding a key's page costs no memory access in the loop.
    const int bs_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1;
    auto block_of = [&](int key) { return bs_shift >= 0 ? key >> bs_shift : key / a.block_size; };
    const int last_blk = block_of(p_max);
    auto load_pages = [&](int base) {
        if (base == blk_base) return;  // (uniform over the wave; the first 64 are there from the start)
        blk_base = base;
        pages_reg = table[min(base + lane, last_blk)];
    };
    // Operands of one tile of 32 keys starting at j0: key rows for the scores (rows of tile u are the keys
    // j0 + 8*(i/4) + 4u + i%4) and, for every block of 16 dimensions, the values of the lane's 8 keys
    // j0 + 8g .. +7.  Every load is unconditional (addresses are clamped to the last key of the group, which
    // exists), so the number of loads in flight is known and the arithmetic of one tile overlaps the loads of
    // the next.  Key rows beyond p_max hold real keys whose scores the mask discards; values outside
    // [lo_min, p_max], which may be stale or never written, are zeroed after the load.
    auto fetch_tile = [&](int j0, uint4 (&kf)[2][KS], uint4 (&vf)[DB]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int key = min(j0 + 8 * (col / 4) + 4 * u + (col % 4), p_max);  // `col` is the row index i here
            const int blk = block_of(key);
            const int page = __shfl(pages_reg, blk - blk_base, LLMS_WAVE);
            const bf16* krow = page_ptr(k_base, page, page_stride) + (uint32_t)((key - blk * a.block_size) * D);
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const int d = 32 * s + 8 * g;
                kf[u][s] = *reinterpret_cast<const uint4*>(krow + (d < D ? d : 0));
            }
        }
        const int jk = min(j0 + 8 * g, p_max & ~7);
        const int blk = block_of(jk);
        const int page = __shfl(pages_reg, blk - blk_base, LLMS_WAVE);
        const bf16* vrow = page_ptr(v_base, page, page_stride) + (uint32_t)(jk - blk * a.block_size + col * a.block_size);
#pragma unroll
        for (int m = 0; m < DB; ++m) vf[m] = *reinterpret_cast<const uint4*>(vrow + (uint32_t)(16 * m * a.block_size));
    };
    auto load_tile = [&](int j0, uint4 (&kf)[2][KS], uint4 (&vf)[DB]) {
        const int blk_first = block_of(j0);
        if (blk_first < blk_base || block_of(min(j0 + 31, p_max)) >= blk_base + LLMS_WAVE) load_pages(blk_first);
        fetch_tile(j0, kf, vf);
    };
    // scores, softmax and weighted values of the tile that starts at key j0
    auto attend = [&](int j0, const uint4 (&kf)[2][KS], uint4 (&vf)[DB]) {
        // (queries beyond head_dim are zero, so a key chunk loaded from a clamped address adds nothing)
        const int jk = j0 + 8 * g;
        if (j0 >= lo_max && j0 + 31 <= p_min) {  // (uniform over the wave; columns without a token are discarded)
            attend_tile<DB, KS, false>(acc, m_run, l_run, kf, vf, qf, jk, lo_col, p_col, scale_log2);
        } else {
            const int first = lo_min - jk, last = p_max + 1 - jk;
#pragma unroll
            for (int m = 0; m < DB; ++m) vf[m] = keep_elements(vf[m], first, last);
            attend_tile<DB, KS, true>(acc, m_run, l_run, kf, vf, qf, jk, lo_col, p_col, scale_log2);
        }
    };

    // Few tiles per wave (a decoded token behind a context of some hundred keys: up to AHEAD each, whose pages one
    // register per lane holds): every tile's operands are asked for at once, so the wave's way through memory is
    // one trip and not one per tile.  Every wave issues the same loads (a tile it does not have is the workgroup's
    // last once more, which some other wave brings in anyway), so the compiler knows how many are in flight when
    // it waits for the first.
    constexpr int AHEAD = DB <= 4 ? 3 : DB <= 8 ? 2 : 1;  // (what the registers hold beside the sums)
    const int t_first_here = split * per_split;
    const bool at_once = t_end > t_first_here && t_end - t_first_here <= AHEAD * NW &&
                         block_of(min(j_begin + 32 * t_end - 1, p_max)) - block_of(j_begin + 32 * t_first_here) < LLMS_WAVE;
    if (at_once) {
        load_pages(block_of(j_begin + 32 * t_first_here));
        uint4 kfa[AHEAD][2][KS], vfa[AHEAD][DB];
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) fetch_tile(j_begin + 32 * min(t_begin + i * NW, t_end - 1), kfa[i], vfa[i]);
#pragma unroll
        for (int i = 0; i < AHEAD; ++i)
            if (t_begin + i * NW < t_end) attend(j_begin + 32 * (t_begin + i * NW), kfa[i], vfa[i]);
    } else {
        // the next tile's operands are requested before this tile's arithmetic starts
        uint4 kf_next[2][KS], vf_next[DB];
        if (t_begin < t_end) {
            load_pages(block_of(j_begin + 32 * t_begin));
            load_tile(j_begin + 32 * t_begin, kf_next, vf_next);
        }
        for (int t = t_begin; t < t_end; t += t_step) {
            uint4 kf[2][KS], vf[DB];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int s = 0; s < KS; ++s) kf[u][s] = kf_next[u][s];
#pragma unroll
            for (int m = 0; m < DB; ++m) vf[m] = vf_next[m];
            if (t + t_step < t_end) load_tile(j_begin + 32 * (t + t_step), kf_next, vf_next);
            attend(j_begin + 32 * t, kf, vf);
        }
    }

    // acc[m][r] = O^T[d = 16m + 4g + r][col]
    // ---- the waves' partial results meet in LDS: every wave leaves its own, then the blocks of 16 dimensions
    // are dealt to the waves, each of which adds the partial results up in the order of the waves
    // (the number of waves is the kernel's own: with a count read at run time every step of the sums below was a
    // branch and a wait of its own, 1.3 microseconds for what is now a few loads and one wait)
    __shared__ float sh_acc[NW][DB][LLMS_WAVE][4];
    __shared__ float sh_m[NW][16], sh_l[NW][16];
    constexpr int nw = NW;
#pragma unroll
    for (int m = 0; m < DB; ++m)
        *reinterpret_cast<float4*>(sh_acc[wave][m][lane]) = make_float4(acc[m][0], acc[m][1], acc[m][2], acc[m][3]);
    l_run = column_sum(l_run);  // (until here every lane kept its own share of its column's sum)
    if (g == 0) {
        sh_m[wave][col] = m_run;
        sh_l[wave][col] = l_run;
    }
    __syncthreads();
    float m_tot = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) m_tot = fmaxf(m_tot, sh_m[w][col]);
    const float m_safe = (m_tot == -INFINITY) ? 0.f : m_tot;
    float weight[NW], l_tot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        weight[w] = exp2_fast(sh_m[w][col] - m_safe);  // 0 for a wave that saw no key
        l_tot += sh_l[w][col] * weight[w];
    }
    const size_t item = ((size_t)(tok0 + c_tok) * a.n_heads + head) * a.num_splits + split;
    for (int m = wave; m < DB; m += nw) {
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float4 p = *reinterpret_cast<const float4*>(sh_acc[w][m][lane]);
            o.x += p.x * weight[w];
            o.y += p.y * weight[w];
            o.z += p.z * weight[w];
            o.w += p.w * weight[w];
        }
        if (!col_ok) continue;
        if (a.num_splits == 1) {
            const float inv = 1.f / l_tot;
            uint2 pk;
            pk.x = pack_bf16(o.x * inv, o.y * inv);
            pk.y = pack_bf16(o.z * inv, o.w * inv);
            *reinterpret_cast<uint2*>(a.out + (size_t)(tok0 + c_tok) * a.out_stride + (size_t)head * D + 16 * m + 4 * g) = pk;
        } else if (a.arrive) {
            store_across(a.ws_o + item * D + 16 * m + 4 * g, o.x, o.y);
            store_across(a.ws_o + item * D + 16 * m + 4 * g + 2, o.z, o.w);
        } else {
            *reinterpret_cast<float4*>(a.ws_o + item * D + 16 * m + 4 * g) = o;
        }
    }
    if (a.num_splits > 1 && wave == 0 && g == 0 && col_ok) {
        if (a.arrive) {
            store_across(a.ws_ml + item * 2, m_tot, l_tot);
        } else {
            a.ws_ml[item * 2] = m_tot;
            a.ws_ml[item * 2 + 1] = l_tot;
        }
    }
    if (a.num_splits > 1 && a.arrive) {  // (the same in every thread of the launch)
        // A thread's stores have been taken by memory before its workgroup is counted; the one that finds all
        // others counted reads their shares.  Nobody waits for anybody: a workgroup that is not the last leaves.
        __shared__ unsigned is_last;
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned* counter = a.arrive + ((size_t)blockIdx.z * gridDim.y + blockIdx.y) * (gridDim.x / a.num_splits) + tile;
            const unsigned before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = before + 1 == (unsigned)a.num_splits;
            if (is_last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero again for the next launch
        }
        __syncthreads();
        if (!is_last) return;
        const size_t item0 = ((size_t)(tok0 + c_tok) * a.n_heads + head) * a.num_splits;
        bf16* orow = a.out + (size_t)(tok0 + c_tok) * a.out_stride + (size_t)head * D;
        if (a.num_splits <= 2) merge_shares<DB, 2>(a, item0, col_ok, wave, nw, g, orow);
        else if (a.num_splits <= 4) merge_shares<DB, 4>(a, item0, col_ok, wave, nw, g, orow);
        else if (a.num_splits <= 8) merge_shares<DB, 8>(a, item0, col_ok, wave, nw, g, orow);
        else merge_shares<DB, 16>(a, item0, col_ok, wave, nw, g, orow);
    }
}

// Prompt portions: a block of WB * CG consecutive column groups of one request and KV head per workgroup, CG per
// wave.  The waves walk the same keys, so each tile of 32 keys is fetched once per workgroup: every thread brings
// 16-byte pieces of the key rows and of the (page-transposed) value rows into LDS, double-buffered, and the waves
// read their matrix operands from there.  Key rows are stored in the order the score product wants them (row
// 16u + i holds key 8*(i/4) + 4u + i%4, padded by one chunk per row against bank conflicts); values keep their
// [dimension][key] order.  With CG = 2 every key and value fragment that a wave reads from LDS serves 32 columns
// instead of 16: with head_dim 128 the LDS reads were what the loop waited for (twice the matrix instructions'
// time), with head_dim 64 it was instruction issue, of which the reads and the loop's own work are a third.
//
// TWIN (no window, no splits): the workgroup has 2 WB waves and a round of the loop brings two tiles; wave w and
// its twin w + WB own the same columns, the one takes the first tile of every round, the other the second, and
// the twin's sums are merged into the other's through LDS at the end, first tile first.  The causal triangle gives
// the last tokens of a prompt the most keys: the chain of dependent rounds of the longest block is halved this way,
// a SIMD always has two waves to switch between (four up to head_dim 64, where two workgroups share a CU), and the
// blocks are handed out in an order (see `rank` below) in which a CU that was given a long one gets a short one
// beside or after it.
template <int DB, bool TWIN, int CG, int WB>
__global__ __launch_bounds__((TWIN ? 2 : 1) * WB * LLMS_WAVE, (TWIN && DB <= 4) ? 4 : 1) void attn_prompt_kernel(const AttnArgs a) {
    constexpr int D = DB * 16;
    constexpr int KS = (D + 31) / 32;
    constexpr int KCH = D / 8;          // 16-byte chunks of a key row
    constexpr int KROW = KCH + 1;       // padded row stride in chunks
    constexpr int TW = TWIN ? 2 : 1;    // tiles per round of the loop
    constexpr int K_TILE = 32 * KROW, V_TILE = D * 4;  // chunks of a tile in LDS
    // two buffers of TW key tiles, then two of TW value tiles; at the end the twins' sums pass through the same memory
    __shared__ uint4 lds_raw[2 * TW * (K_TILE + V_TILE)];
    uint4* const k_lds = lds_raw;                     // [buffer][tile of the round][row][chunk]
    uint4* const v_lds = lds_raw + 2 * TW * K_TILE;   // [buffer][tile of the round][dimension][4 chunks of 8 keys]
    const int tid = threadIdx.x, wave = tid / LLMS_WAVE, lane = tid % LLMS_WAVE;
    const int col = lane % 16, g = lane / 16;
    const int twin = __builtin_amdgcn_readfirstlane(wave / WB);  // which tile of a round this wave takes

    const int G = a.n_heads / a.n_kv_heads;
    const int HG = G < 16 ? G : 16, TPG = 16 / HG, HB = (G + HG - 1) / HG;
    const int head_block = TWIN ? blockIdx.x : blockIdx.y;
    const int kvh = head_block / HB, hb = head_block % HB;
    const int b = a.seq_begin + blockIdx.z;
    const int tok0 = a.cu_seqlens[b], n_new = a.cu_seqlens[b + 1] - tok0;
    const int ctx = a.context_lens[b];
    // (asked for together with the lengths: one trip to memory earlier than where the block table is first needed)
    const int table_row = a.table_rows ? a.table_rows[b] : b;
    const int BLK = WB * CG * TPG;  // tokens of a block: WB waves with CG column groups each
    int wg_first;                   // first token (within the request's new tokens) of the workgroup's block
    if (TWIN) {
        // rank 0: the last block of the prompt, which sees the most keys.  Workgroups are handed out in the order
        // of blockIdx.y: the first on every CU get the longest blocks, and the CU that was given the shortest of
        // these gets the longest of the rest
        const int blocks = (n_new + BLK - 1) / BLK, by = blockIdx.y;
        const int rank = by < a.first_blocks ? a.first_blocks - 1 - by : by;
        if (rank >= blocks || ctx <= 0) return;
        wg_first = (blocks - 1 - rank) * BLK;
    } else {
        wg_first = ((int)blockIdx.x / a.num_splits) * BLK;
        if (wg_first >= n_new || ctx <= 0) return;
    }
    // Without twins the keys of a block may be shared out to num_splits workgroups (blockIdx.x % num_splits), whose
    // partial results attn_merge adds up: a short portion with a long prefix has few blocks and many keys.
    const int n_splits = TWIN ? 1 : a.num_splits, split = TWIN ? 0 : (int)blockIdx.x % a.num_splits;

    // this wave's CG column groups: consecutive tokens, the same heads
    const int w_first = wg_first + (wave % WB) * CG * TPG;
    const bool wave_on = w_first < n_new;
    const int c_head_in = hb * HG + col % HG, head = kvh * G + c_head_in;
    int c_tok[CG], p_col[CG], lo_col[CG];
    bool col_ok[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        c_tok[cg] = w_first + cg * TPG + col / HG;
        col_ok[cg] = wave_on && col < HG * TPG && c_tok[cg] < n_new && c_head_in < G && tok0 + c_tok[cg] < a.row_end;
        p_col[cg] = col_ok[cg] ? ctx - n_new + c_tok[cg] : -1;
        lo_col[cg] = (a.window > 0 && p_col[cg] - a.window + 1 > 0) ? p_col[cg] - a.window + 1 : 0;
    }
    // key range of the whole workgroup
    const int p_max = ctx - n_new + min(wg_first + BLK, n_new) - 1;
    const int p_min = ctx - n_new + wg_first;
    const int lo_min = (a.window > 0 && p_min - a.window + 1 > 0) ? p_min - a.window + 1 : 0;
    const int j_begin = lo_min & ~31;
    const int n_rounds = ((p_max - j_begin) / 32 + TW) / TW;  // of TW tiles each

    const uint4 zero = make_uint4(0, 0, 0, 0);
    uint4 qf[CG][KS];
    f32x4 acc[CG][DB];
    float m_run[CG], l_run[CG];
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int d = 32 * s + 8 * g;
            qf[cg][s] = (col_ok[cg] && d < D) ? *reinterpret_cast<const uint4*>(a.q + (size_t)(tok0 + c_tok[cg]) * a.q_stride +
                                                                                (size_t)head * D + d)
                                              : zero;
        }
#pragma unroll
        for (int m = 0; m < DB; ++m) acc[cg][m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        m_run[cg] = -INFINITY;
        l_run[cg] = 0.f;
    }

    const int* table = a.block_tables + (size_t)table_row * a.max_blocks;
    const uint32_t page_stride = (uint32_t)a.n_kv_heads * a.block_size * D;
    const bf16* k_base = a.k_pool + (size_t)kvh * a.block_size * D;
    const bf16* v_base = a.v_pool + (size_t)kvh * a.block_size * D;
    const float scale_log2 = a.scale * 1.44269504088896341f;
    // the tiles whose 32 keys every column of this wave sees: up to the wave's first token, from the window's
    // start of its last one
    const int w_last = min(w_first + CG * TPG, n_new) - 1;
    const int w_pmin = ctx - n_new + w_first, w_pmax = ctx - n_new + w_last;
    const int w_lo_max = (a.window > 0 && w_pmax - a.window + 1 > 0) ? w_pmax - a.window + 1 : 0;
    // key / block_size by one multiply with ceil(2^32 / block_size): exact below 2^32 / block_size keys (the
    // entry point refuses longer block tables)
    const uint32_t bs_magic = 0xFFFFFFFFu / (uint32_t)a.block_size + 1u;
    auto block_of = [&](int key) { return (int)__umulhi((uint32_t)key, bs_magic); };

    // A round is 4 TW groups of 8 consecutive keys, one per wave: inside a page the key rows of a group are one
    // contiguous piece of 16 D bytes, and its values are 16 bytes per dimension, so everything a wave asks for in a
    // round lies in one page.  The page, the group's place in it and the two base addresses are therefore the same
    // for all lanes and are worked out by the scalar unit; a lane adds its constant offset.  Groups are clamped to
    // the one that holds the workgroup's last key (which exists), so every round can be asked for, also one past
    // the last: key rows past the last key may hold anything (their scores are masked), values outside
    // [lo_min, p_max] are zeroed on their way into LDS (not earlier: that would wait for the load).  The page is
    // read from the block table a round before the group is asked for, and that a round before it goes into LDS:
    // three rounds in flight, nothing waited for inside the loop.
    static_assert(WB == 4, "a wave per group of 8 keys: 4 to a tile");
    constexpr int PER_LANE = (D + LLMS_WAVE - 1) / LLMS_WAVE;  // 16-byte pieces of a group per lane (keys and values alike)
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    // Rounds between asking for a group and putting it into LDS: one where the keys of a KV head stay in L2, two
    // with wide heads (a head's keys and values are then megabytes, the trip goes to memory and takes longer than a
    // round); each round in flight has registers of its own.
    constexpr int AHEAD = DB > 4 ? 2 : 1;
    u32x4 kreg0[PER_LANE], vreg0[PER_LANE], kreg1[PER_LANE], vreg1[PER_LANE];  // (the second set only with AHEAD == 2)
    constexpr std::integral_constant<int, 0> SET0{};
    constexpr std::integral_constant<int, 1> SET1{};
    int page_ahead = 0;
    auto group_key_of = [&](int j0) { return min(j0 + 8 * wave_s, p_max & ~7); };  // first key of this wave's group
    // (the block table does not change while the kernel runs: read as constant memory, which is what lets the
    // scalar unit fetch it; as an ordinary load it would come back through the vector memory queue, and moving it
    // to a scalar register would wait for the key and value pieces queued before it)
    typedef const int __attribute__((address_space(4))) * ConstInts;
    const ConstInts table_c = (ConstInts)(uintptr_t)table;
    auto ask_pages = [&](int j0) { page_ahead = table_c[block_of(group_key_of(j0))]; };
    // (the register set is named by a type, std::integral_constant<int, 0 or 1>: an array passed by reference would
    // be kept in memory by the compiler)
    auto load_round = [&](int j0, auto set) __attribute__((always_inline)) {  // after ask_pages(j0)
        auto& kreg = *[&]() { if constexpr (decltype(set)::value == 1) return &kreg1; else return &kreg0; }();
        auto& vreg = *[&]() { if constexpr (decltype(set)::value == 1) return &vreg1; else return &vreg0; }();
        const int jg = group_key_of(j0), in_page = jg - block_of(jg) * a.block_size;
        const bf16* kg = page_ptr(k_base, page_ahead, page_stride) + (uint32_t)(in_page * D);
        const bf16* vg = page_ptr(v_base, page_ahead, page_stride) + (uint32_t)in_page;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            const int p = min(lane + LLMS_WAVE * i, D - 1);  // (D % 64 != 0: the upper lanes repeat the last piece)
            kreg[i] = *reinterpret_cast<const u32x4*>(kg + 8 * p);
            vreg[i] = *reinterpret_cast<const u32x4*>(vg + (uint32_t)(p * a.block_size));
        }
    };
    auto store_round = [&](int buf, int j0, auto set) __attribute__((always_inline)) {
        auto& kreg = *[&]() { if constexpr (decltype(set)::value == 1) return &kreg1; else return &kreg0; }();
        auto& vreg = *[&]() { if constexpr (decltype(set)::value == 1) return &vreg1; else return &vreg0; }();
        const int jk = j0 + 8 * wave_s;                       // (not clamped: what the group stands for)
        const bool inside = jk >= lo_min && jk + 7 <= p_max;  // (the same for the wave)
        const int tile = wave_s / 4, kg4 = wave_s % 4;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            const int p = lane + LLMS_WAVE * i;
            if (p < D) {
                uint4 values = make_uint4(vreg[i][0], vreg[i][1], vreg[i][2], vreg[i][3]);
                if (!inside) values = keep_elements(values, lo_min - jk, p_max + 1 - jk);
                const int q = p / KCH, ch = p % KCH;             // key 8 kg4 + q of the tile = 8a + 4u + b2
                const int row = (q >> 2) * 16 + kg4 * 4 + (q & 3);  // -> row 16u + 4a + b2
                *reinterpret_cast<u32x4*>(&k_lds[(buf * TW + tile) * K_TILE + row * KROW + ch]) = kreg[i];
                v_lds[(buf * TW + tile) * V_TILE + p * 4 + kg4] = values;  // [dimension][4 chunks of 8 keys]
            }
        }
    };

    const int per_split = (n_rounds + n_splits - 1) / n_splits;
    const int r_lo = split * per_split, r_hi = min(n_rounds, r_lo + per_split);  // this workgroup's rounds (maybe none)
    auto first_key = [&](int r) { return j_begin + 32 * TW * r; };
    // round r_lo + i is fetched into register set i % AHEAD and goes into LDS buffer i % 2
    ask_pages(first_key(r_lo));
    load_round(first_key(r_lo), SET0);
    ask_pages(first_key(r_lo + 1));
    if (AHEAD == 2) {
        load_round(first_key(r_lo + 1), SET1);
        ask_pages(first_key(r_lo + 2));
    }
    store_round(0, first_key(r_lo), SET0);
    // The queries have arrived by now (they were asked for before the first round, which has just been stored).
    // Saying so here, outside the loop, keeps the wait for them out of it: inside, a wait for loads from memory
    // would also wait for the rounds that are being fetched ahead.
#pragma unroll
    for (int cg = 0; cg < CG; ++cg)
#pragma unroll
        for (int s = 0; s < KS; ++s)
            asm volatile("" : "+v"(qf[cg][s].x), "+v"(qf[cg][s].y), "+v"(qf[cg][s].z), "+v"(qf[cg][s].w));
    load_round(first_key(r_lo + AHEAD), SET0);
    ask_pages(first_key(r_lo + AHEAD + 1));
    __syncthreads();
    // One round: `buf` is its LDS buffer, `set` names the registers that hold the round after it.
    auto one_round = [&](int r, int buf, auto set) __attribute__((always_inline)) {
        const int j0 = j_begin + 32 * (TW * r + twin);  // this wave's tile of the round
        const bool busy = wave_on && j0 <= w_pmax;  // (a tile beyond the wave's last position adds nothing)
        // the next round into the other buffer (last read before the previous barrier), a later one asked for, and the
        // pages of the one after that: by the twins before they read their fragments from LDS, by the others after
        // their tile, so that the two waves of a SIMD are not at the same stage at the same time (one multiplies
        // while the other computes exponentials) and the reads of the one half of the waves have LDS to themselves
        // while the other half still fetches
        auto fetch_ahead = [&]() {
            if (r + 1 < r_hi) store_round(buf ^ 1, first_key(r + 1), set);
            load_round(first_key(r + 1 + AHEAD), set);
            ask_pages(first_key(r + 2 + AHEAD));
        };
        if (TWIN && twin == 1) fetch_ahead();
        uint4 kf[2][KS], vf[DB];
        if (busy) {
            const uint4* kt = k_lds + (buf * TW + twin) * K_TILE;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int s = 0; s < KS; ++s) {
                    const int ch = 4 * s + g;
                    kf[u][s] = kt[(16 * u + col) * KROW + (ch < KCH ? ch : 0)];  // (beyond head_dim the queries are zero)
                }
        }
        if (!TWIN) fetch_ahead();  // (while the fragments are on their way)
        if (busy) {
            const bool all_seen = j0 >= w_lo_max && j0 + 31 <= w_pmin;  // (uniform over the wave; columns without a token are discarded)
            // the same keys and values for each of the wave's column groups; the values are asked for after the keys' products
            const uint4* vt = v_lds + (buf * TW + twin) * V_TILE;
            auto read_values = [&]() {
#pragma unroll
                for (int m = 0; m < DB; ++m) vf[m] = vt[(16 * m + col) * 4 + g];
            };
            if (all_seen) attend_tile_groups<DB, KS, false, CG>(acc, m_run, l_run, kf, vf, qf, j0 + 8 * g, lo_col, p_col, scale_log2, read_values);
            else attend_tile_groups<DB, KS, true, CG>(acc, m_run, l_run, kf, vf, qf, j0 + 8 * g, lo_col, p_col, scale_log2, read_values);
        }
        if (TWIN && twin == 0) fetch_ahead();
        __syncthreads();
    };
    // two rounds per turn, so that buffers and register sets are known by name: round r_lo + i goes into LDS from
    // set i % AHEAD, which then takes round i + AHEAD
    for (int r = r_lo; r < r_hi; r += 2) {
        one_round(r, 0, std::integral_constant<int, AHEAD - 1>{});
        if (r + 1 < r_hi) one_round(r + 1, 1, SET0);
    }
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) l_run[cg] = column_sum(l_run[cg]);  // (every lane kept its own share of its column's sum)
    if constexpr (TWIN) {
        // The twin's share (second tile of every round) joins the first wave's, one column group at a time:
        // [item][twin wave][lane] floats in the memory of the tiles, which nobody reads any more.
        float* share = reinterpret_cast<float*>(lds_raw);
        constexpr int ITEMS = 4 * DB + 2;
        const int slot = (wave % WB) * LLMS_WAVE + lane;
#pragma unroll
        for (int cg = 0; cg < CG; ++cg) {
            if (cg > 0) __syncthreads();  // (the group before has been read)
            if (twin == 1) {
                share[slot] = m_run[cg];
                share[WB * LLMS_WAVE + slot] = l_run[cg];
#pragma unroll
                for (int m = 0; m < DB; ++m)
#pragma unroll
                    for (int r = 0; r < 4; ++r) share[(2 + 4 * m + r) * WB * LLMS_WAVE + slot] = acc[cg][m][r];
            }
            __syncthreads();
            if (twin == 0) {
                const float m_b = share[slot], l_b = share[WB * LLMS_WAVE + slot];
                const float m_tot = fmaxf(m_run[cg], m_b);
                const float w_a = m_run[cg] == -INFINITY ? 0.f : exp2_fast(m_run[cg] - m_tot);
                const float w_b = m_b == -INFINITY ? 0.f : exp2_fast(m_b - m_tot);
                l_run[cg] = l_run[cg] * w_a + l_b * w_b;
                m_run[cg] = m_tot;
#pragma unroll
                for (int m = 0; m < DB; ++m)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc[cg][m][r] = acc[cg][m][r] * w_a + share[(2 + 4 * m + r) * WB * LLMS_WAVE + slot] * w_b;
            }
        }
        static_assert(ITEMS * WB * LLMS_WAVE * sizeof(float) <= sizeof(lds_raw), "the twins' shares must fit the tiles' memory");
        if (twin == 1) return;
    }
#pragma unroll
    for (int cg = 0; cg < CG; ++cg) {
        if (!col_ok[cg]) continue;
        if (n_splits > 1) {  // the share of this workgroup, as the decode kernel leaves its own
            const size_t item = ((size_t)(tok0 + c_tok[cg]) * a.n_heads + head) * n_splits + split;
#pragma unroll
            for (int m = 0; m < DB; ++m)
                *reinterpret_cast<float4*>(a.ws_o + item * D + 16 * m + 4 * g) =
                    make_float4(acc[cg][m][0], acc[cg][m][1], acc[cg][m][2], acc[cg][m][3]);
            if (g == 0) {
                a.ws_ml[item * 2] = m_run[cg];
                a.ws_ml[item * 2 + 1] = l_run[cg];
            }
            continue;
        }
        const float inv = 1.f / l_run[cg];
        bf16* orow = a.out + (size_t)(tok0 + c_tok[cg]) * a.out_stride + (size_t)head * D;
#pragma unroll
        for (int m = 0; m < DB; ++m) {
            uint2 w;
            w.x = pack_bf16(acc[cg][m][0] * inv, acc[cg][m][1] * inv);
            w.y = pack_bf16(acc[cg][m][2] * inv, acc[cg][m][3] * inv);
            *reinterpret_cast<uint2*>(orow + 16 * m + 4 * g) = w;
        }
    }
}

// Merge of the splits of every (token, head), split 0 first: a thread per token, head and 4 dimensions (blockIdx.x:
// token, blockIdx.y: which blockDim.x of the token's heads * head_dim / 4 pieces).
__global__ __launch_bounds__(256) void attn_merge_kernel(bf16* __restrict__ out, int out_stride, const float* __restrict__ ws_o,
                                                         const float* __restrict__ ws_ml, int token_begin, int n_heads,
                                                         int head_dim, int num_splits) {
    const int token = token_begin + blockIdx.x;
    const int q4 = head_dim / 4;
    const int idx = blockIdx.y * blockDim.x + threadIdx.x;
    if (idx < n_heads * q4) {
        const int head = idx / q4, d = 4 * (idx % q4);
        const size_t item0 = ((size_t)token * n_heads + head) * num_splits;
        const float2* ml = reinterpret_cast<const float2*>(ws_ml) + item0;  // (maximum, sum) of each split
        float m_tot = -INFINITY;
#pragma unroll 4
        for (int s = 0; s < num_splits; ++s) m_tot = fmaxf(m_tot, ml[s].x);
        float l_tot = 0.f;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
        for (int s = 0; s < num_splits; ++s) {
            const float2 v = ml[s];
            const float4 p = *reinterpret_cast<const float4*>(ws_o + (item0 + s) * head_dim + d);
            if (v.x != -INFINITY) {  // (a split that saw no key of this column)
                const float w = exp2_fast(v.x - m_tot);
                l_tot += v.y * w;
                o.x += p.x * w;
                o.y += p.y * w;
                o.z += p.z * w;
                o.w += p.w * w;
            }
        }
        const float inv = 1.f / l_tot;
        uint2 pk;
        pk.x = pack_bf16(o.x * inv, o.y * inv);
        pk.y = pack_bf16(o.z * inv, o.w * inv);
        *reinterpret_cast<uint2*>(out + (size_t)token * out_stride + (size_t)head * head_dim + d) = pk;
    }
}

// Column groups per wave of the prompt kernel: two share every key and value fragment a wave reads from LDS
// (half the LDS reads and loop overhead per column), as long as the accumulators of both fit the registers and
// the launch still has a workgroup for every CU.
#define PROMPT_CG_MAX(N) ((N) <= 8 ? 2 : 1)
#define PROMPT_WB 4  // waves per block of tokens (2 was tried with 2 column groups each: slower)
#define PROMPT_FULL_CHIP 256  // workgroups below which one column group per wave is kept

#define PROMPT_TWIN_MAX_DB 12  // widest head (in blocks of 16 dimensions) whose 8 waves with twins fit the registers

template <int DB, int CG>
static void launch_prompt_cg(dim3 grid, bool twin, const AttnArgs& a, hipStream_t stream) {
    if constexpr (DB <= PROMPT_TWIN_MAX_DB) {  // (wider heads are never given twins, so those kernels are not built)
        if (twin) {
            attn_prompt_kernel<DB, true, CG, PROMPT_WB><<<grid, 2 * PROMPT_WB * LLMS_WAVE, 0, stream>>>(a);
            return;
        }
    }
    attn_prompt_kernel<DB, false, CG, PROMPT_WB><<<grid, PROMPT_WB * LLMS_WAVE, 0, stream>>>(a);
}

// Few tokens (decoding): small workgroups, so that the merge reaches many CUs; many tokens: 256 threads each.
static void launch_merge(void* out, int out_stride, const float* ws_o, const float* ws_ml, int token_begin, int n_tokens,
                         int n_heads, int head_dim, int num_splits, hipStream_t stream) {
    const int threads = n_tokens <= 64 ? 64 : 256, pieces = n_heads * (head_dim / 4);
    attn_merge_kernel<<<dim3(n_tokens, (pieces + threads - 1) / threads), threads, 0, stream>>>(
        (bf16*)out, out_stride, ws_o, ws_ml, token_begin, n_heads, head_dim, num_splits);
}

static int launch_prompt(int db, int cg, dim3 grid, bool twin, const AttnArgs& a, hipStream_t stream) {
#define ATT_CASE(N)                                                                       \
    case N:                                                                               \
        if (cg == 2 && PROMPT_CG_MAX(N) == 2) launch_prompt_cg<N, PROMPT_CG_MAX(N)>(grid, twin, a, stream); \
        else launch_prompt_cg<N, 1>(grid, twin, a, stream);                             \
        break;
    switch (db) {
        ATT_CASE(1) ATT_CASE(2) ATT_CASE(3) ATT_CASE(4) ATT_CASE(5) ATT_CASE(6) ATT_CASE(7) ATT_CASE(8)
        ATT_CASE(9) ATT_CASE(10) ATT_CASE(11) ATT_CASE(12) ATT_CASE(13) ATT_CASE(14) ATT_CASE(15) ATT_CASE(16)
        default:
            LLMS_REQUIRE(false, "attention_mfma: head_dim must be a multiple of 16 up to 256");
    }
#undef ATT_CASE
    return LLMS_OK;
}

// CUs of the current device (asked once per device).
static int compute_units(int* out) {
    static int cached[64];
    int dev = -1;
    LLMS_HIP_CHECK(hipGetDevice(&dev));
    LLMS_REQUIRE(dev >= 0 && dev < 64, "attention_mfma: device index out of range");
    if (cached[dev] == 0) {
        int n = 0;
        LLMS_HIP_CHECK(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
        LLMS_REQUIRE(n > 0, "attention_mfma: the device reports no compute units");
        cached[dev] = n;
    }
    *out = cached[dev];
    return LLMS_OK;
}

static int launch_attn(int db, dim3 grid, int threads, const AttnArgs& a, hipStream_t stream) {
#define ATT_CASE(N)                                                                                  \
    case N:                                                                                          \
        if (threads == 8 * LLMS_WAVE && N <= 10) attn_mfma_kernel<N, (N <= 10 ? 8 : 4)><<<grid, 8 * LLMS_WAVE, 0, stream>>>(a); \
        else attn_mfma_kernel<N, 4><<<grid, 4 * LLMS_WAVE, 0, stream>>>(a);                          \
        break;
    switch (db) {
        ATT_CASE(1) ATT_CASE(2) ATT_CASE(3) ATT_CASE(4) ATT_CASE(5) ATT_CASE(6) ATT_CASE(7) ATT_CASE(8)
        ATT_CASE(9) ATT_CASE(10) ATT_CASE(11) ATT_CASE(12) ATT_CASE(13) ATT_CASE(14) ATT_CASE(15) ATT_CASE(16)
        default:
            LLMS_REQUIRE(false, "attention_mfma: head_dim must be a multiple of 16 up to 256");
    }
#undef ATT_CASE
    return LLMS_OK;
}

extern "C" {

// Attention for the requests [seq_begin, seq_begin + n_seqs) of a step.  max_new: most new tokens any of
// them brings.  split_waves = 0: prompt portions (attn_prompt_kernel);
// split_waves = 1 deals the keys of each column group to `waves` (4 or 8) waves and
// `num_splits` workgroups (decoding); split_waves = 0 with num_splits > 1 shares the keys of each block of prompt
// tokens out to that many workgroups (no window then); with num_splits > 1 the caller provides ws_o [tokens * heads * splits * D] and
// ws_ml [tokens * heads * splits * 2] floats, indexed by absolute token row.  `arrive` (may be null): n_arrive
// counters in device memory, all zero, which the kernel leaves zero: decoding with 2 to 16 splits then adds the
// shares up in the workgroup that finishes last instead of in a second kernel.
int llms_attention_mfma(void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                        const int* cu_seqlens,
                        const int* context_lens, int seq_begin, int n_seqs, int max_new, int token_begin,
                        int n_tokens, int n_heads, int n_kv_heads, int head_dim, int block_size, int window,
                        float scale, int split_waves, int num_splits, int waves, float* ws_o, float* ws_ml,
                        unsigned* arrive, int n_arrive, hipStream_t stream) {
    LLMS_REQUIRE(n_seqs > 0 && max_new > 0 && n_heads > 0 && n_kv_heads > 0, "attention_mfma: sizes must be positive");
    LLMS_REQUIRE(n_heads % n_kv_heads == 0, "attention_mfma: n_heads must be a multiple of n_kv_heads");
    LLMS_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256, "attention_mfma: head_dim must be a multiple of 16 up to 256");
    LLMS_REQUIRE(block_size > 0 && block_size % 8 == 0, "attention_mfma: block_size must be a multiple of 8");
    LLMS_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0, "attention_mfma: row strides must keep 16-byte (q) and 8-byte (out) alignment");
    LLMS_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 && ((uintptr_t)v_pool % 16) == 0 &&
                     ((uintptr_t)out % 8) == 0, "attention_mfma: pointers must be 16-byte aligned");
    LLMS_REQUIRE(window >= 0 && max_blocks > 0, "attention_mfma: bad window or max_blocks");
    LLMS_REQUIRE(num_splits >= 1, "attention_mfma: num_splits must be >= 1");
    LLMS_REQUIRE(scale > 0.f, "attention_mfma: scale must be positive");
    LLMS_REQUIRE((long long)n_kv_heads * block_size * head_dim < (1ll << 31), "attention_mfma: a page is too large");
    LLMS_REQUIRE(split_waves == 0 || split_waves == 1, "attention_mfma: split_waves is 0 or 1");
    LLMS_REQUIRE(waves == 4 || (split_waves > 0 && waves == 8), "attention_mfma: 4 waves, or 8 when the waves share the keys");
    LLMS_REQUIRE(waves == 4 || head_dim <= 160, "attention_mfma: 8 waves take head_dim up to 160");
    LLMS_REQUIRE(split_waves > 0 || num_splits == 1 || window == 0, "attention_mfma: portions with a window are not split");
    LLMS_REQUIRE(num_splits == 1 || (ws_o && ws_ml && ((uintptr_t)ws_o % 16) == 0 && ((uintptr_t)ws_ml % 8) == 0),
                 "attention_mfma: splits need a (16-byte aligned) workspace");
    LLMS_REQUIRE(n_seqs <= 65535, "attention_mfma: too many requests for one launch");
    const int G = n_heads / n_kv_heads, HG = G < 16 ? G : 16, TPG = 16 / HG, HB = (G + HG - 1) / HG;
    const int groups = (max_new + TPG - 1) / TPG;
    AttnArgs a = {(bf16*)out, out_stride, (const bf16*)q, q_stride, (const bf16*)k_pool, (const bf16*)v_pool,
                  block_tables, table_rows, max_blocks, cu_seqlens, context_lens, seq_begin, n_heads, n_kv_heads, block_size,
                  window, scale, num_splits, ws_o, ws_ml, nullptr, token_begin + n_tokens, 0, -1};
    // (at most one token each and as many tokens as requests: every request has exactly one, in the order of the requests)
    if (split_waves > 0 && max_new == 1 && n_tokens == n_seqs) a.one_token_from = token_begin;
    LLMS_REQUIRE(n_kv_heads * HB <= 65535, "attention_mfma: too many heads");
    LLMS_REQUIRE((unsigned long long)max_blocks * block_size * block_size <= 0xFFFFFFFFull,
                 "attention_mfma: block table too long for this page size (keys * block_size must stay below 2^32)");
    LLMS_REQUIRE(arrive == nullptr || ((uintptr_t)arrive % 4 == 0 && n_arrive > 0), "attention_mfma: bad counters");
    if (split_waves > 0) {
        dim3 grid(groups * num_splits, n_kv_heads * HB, n_seqs);
        if (arrive && num_splits > 1 && num_splits <= 16 && (long long)groups * grid.y * grid.z <= n_arrive) a.arrive = arrive;
        if (int e = launch_attn(head_dim / 16, grid, waves * LLMS_WAVE, a, stream)) return e;
        if (num_splits > 1 && a.arrive == nullptr) {
            hipError_t e1 = hipGetLastError();
            if (e1 != hipSuccess) {
                fprintf(stderr, "llmserve kernel launch failed: %s\n", hipGetErrorString(e1));
                return LLMS_ERR_LAUNCH;
            }
            launch_merge(out, out_stride, ws_o, ws_ml, token_begin, n_tokens, n_heads, head_dim, num_splits, stream);
        }
    } else {
        // twins (8 waves, two tiles a round) where a workgroup per CU is left that way; wider heads would not fit
        // the registers of 8 waves, a window or splits have their own arrangement
        bool twin = window == 0 && head_dim <= 16 * PROMPT_TWIN_MAX_DB && num_splits == 1;
        auto grid_for = [&](int cg) {
            const int per_block = PROMPT_WB * cg;  // column groups of a block of tokens
            return dim3((groups + per_block - 1) / per_block * num_splits, n_kv_heads * HB, n_seqs);
        };
        auto workgroups = [](dim3 g) { return (long long)g.x * g.y * g.z; };
        int cg = PROMPT_CG_MAX(head_dim / 16);
        dim3 grid = grid_for(cg);
        if (cg == 2 && workgroups(grid) < PROMPT_FULL_CHIP * (twin && head_dim <= 64 ? 2 : 1)) grid = grid_for(cg = 1);
        if (twin && workgroups(grid) < PROMPT_FULL_CHIP) twin = false;  // a short portion: workgroups for more CUs matter more
        if (twin) {  // heads in x, blocks of tokens in y: the order in which workgroups are handed out
            LLMS_REQUIRE(grid.x <= 65535, "attention_mfma: too many tokens per request for one launch");
            grid = dim3(grid.y, grid.x, grid.z);
            int cus = 0;
            if (int e = compute_units(&cus)) return e;
            // The first workgroup of every CU: the longest blocks, shortest of them first; then from the longest
            // remaining block down.  Where a CU holds one workgroup, the CU that is free first takes the longest of
            // the rest; where it holds two (head_dim up to 64: the registers of 16 waves and two sets of tiles fit),
            // the second lands on the CUs in the order of the first (measured), so each CU gets a long and a
            // short one that add up to the same.
            a.first_blocks = n_seqs == 1 ? (int)std::min<long long>(grid.y, cus / grid.x) : 0;
        }
        if (int e = launch_prompt(head_dim / 16, cg, grid, twin, a, stream)) return e;
        if (num_splits > 1) {
            hipError_t e1 = hipGetLastError();
            if (e1 != hipSuccess) {
                fprintf(stderr, "llmserve kernel launch failed: %s\n", hipGetErrorString(e1));
                return LLMS_ERR_LAUNCH;
            }
            launch_merge(out, out_stride, ws_o, ws_ml, token_begin, n_tokens, n_heads, head_dim, num_splits, stream);
        }
    }
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------
// Decoding with the keys of a request shared out to several workgroups, without a workspace from the caller:
// the partial results go through a fixed array in device memory that this library owns.  Every GPU the library
// runs on holds its own copy of the array (at its own address) until the process ends.
static __device__ __align__(256) unsigned char scratch[LLMS_ATTN_SCRATCH_BYTES];

#define LLMS_MAX_DEVICES 64
static void* scratch_ptr[LLMS_MAX_DEVICES];  // device address of `scratch` on each GPU (null: not asked yet)
static std::mutex scratch_mutex;

// The array's address on the current device.  In host code `scratch` is only a handle for the runtime, never
// an address a kernel could use: the address comes from hipGetSymbolAddress, once per device.
static int scratch_of_current_device(unsigned char** out) {
    int dev = -1;
    LLMS_HIP_CHECK(hipGetDevice(&dev));
    LLMS_REQUIRE(dev >= 0 && dev < LLMS_MAX_DEVICES, "attention_decode_noalloc: device index out of range");
    std::lock_guard<std::mutex> hold(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        LLMS_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        LLMS_REQUIRE(p != nullptr && ((uintptr_t)p % 256) == 0, "attention_decode_noalloc: no aligned device address for the scratch array");
        scratch_ptr[dev] = p;
    }
    *out = static_cast<unsigned char*>(scratch_ptr[dev]);
    return LLMS_OK;
}

extern "C" {

int llms_attention_decode_noalloc(void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                                  const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                                  const int* cu_seqlens, const int* context_lens, int seq_begin, int n_seqs,
                                  int token_begin, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                  int block_size, int window, float scale, int num_splits, int waves,
                                  hipStream_t stream) {
    LLMS_REQUIRE(num_splits >= 2, "attention_decode_noalloc: num_splits must be >= 2 (one split needs no scratch: use attention_mfma)");
    LLMS_REQUIRE(token_begin >= 0 && n_tokens > 0 && n_heads > 0 && head_dim > 0 && head_dim % 16 == 0,
                 "attention_decode_noalloc: sizes must be positive, head_dim a multiple of 16");
    // partial results are indexed by absolute token row, as in attention_mfma: [row][head][split][D] sums, then
    // [row][head][split][2] (maximum, sum of weights)
    const unsigned long long items = (unsigned long long)(token_begin + n_tokens) * n_heads * num_splits;
    const unsigned long long o_bytes = items * head_dim * sizeof(float);  // (a multiple of 64)
    const unsigned long long ml_bytes = items * 2 * sizeof(float);
    if (o_bytes + ml_bytes > LLMS_ATTN_SCRATCH_BYTES) {
        fprintf(stderr, "llmserve kernel argument error: attention_decode_noalloc: %llu rows x heads x splits need %llu bytes "
                        "of scratch, the fixed array has %u\n", items, o_bytes + ml_bytes, (unsigned)LLMS_ATTN_SCRATCH_BYTES);
        return LLMS_ERR_ARG;
    }
    unsigned char* base = nullptr;
    if (int e = scratch_of_current_device(&base)) return e;
    float* ws_o = reinterpret_cast<float*>(base);
    float* ws_ml = reinterpret_cast<float*>(base + o_bytes);
    // Nothing in the array has to start at zero: the merge reads, for every token row of the launch, exactly the
    // entries the attention kernel has just written (a request without keys writes nothing and its rows of `out`
    // are meaningless, as with a caller's workspace).
    return llms_attention_mfma(out, out_stride, q, q_stride, k_pool, v_pool, block_tables, table_rows, max_blocks,
                               cu_seqlens, context_lens, seq_begin, n_seqs, /*max_new=*/1, token_begin, n_tokens, n_heads,
                               n_kv_heads, head_dim, block_size, window, scale, /*split_waves=*/1, num_splits, waves, ws_o,
                               ws_ml, /*arrive=*/nullptr, 0, stream);
}

}  // extern "C"
