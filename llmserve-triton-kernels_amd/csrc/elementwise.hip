// Row-wise kernels of the decoder: embedding gather, (residual add +) RMSNorm,
// rotary position encoding fused with the paged key/value store, SiLU(gate)*up.
// Every kernel exists for float and for bfloat16 storage; statistics, angles and the
// residual sum are always computed in 32-bit.
#include "common.h"

// ------------------------------------------------------------------ embedding gather
// out[n, :] = table[ids[n], :].  An id outside [0, vocab) yields a row of NaN, so a bad
// token shows in the logits and never reads outside the table.
template <typename T>
__global__ void embed_gather_kernel(T* __restrict__ out, const T* __restrict__ table,
                                    const int* __restrict__ ids, int hidden, int vocab) {
    const int n = blockIdx.x;
    const int id = ids[n];
    T* o = out + (size_t)n * hidden;
    if ((unsigned)id >= (unsigned)vocab) {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_f32<T>(__uint_as_float(0x7fc00000u));
        return;
    }
    const T* src = table + (size_t)id * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = src[i];
}

// ------------------------------------------------------------------ RMSNorm
// For output row r (source row s = rows ? rows[r] : r):
//   v = x[s] (+ delta[s], summed in 32-bit and rounded once to T)
//   if resid_out: resid_out[s] = v                    (may alias x)
//   out[r] = weight * T(v * rsqrt(mean(v^2) + eps))   (cast before the weight, as the
//            reference does: src/llmserve/model/llama.py:24-28)
template <typename T>
__global__ void rmsnorm_kernel(T* __restrict__ out, const T* x, const T* __restrict__ delta, T* resid_out,
                               const T* __restrict__ weight, const int* __restrict__ rows, float eps,
                               int hidden, const float* __restrict__ parts, int n_parts, size_t part_stride) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int s = rows ? rows[r] : r;
    const T* xs = x + (size_t)s * hidden;
    const T* ds = delta ? delta + (size_t)s * hidden : nullptr;
    T* rs = resid_out ? resid_out + (size_t)s * hidden : nullptr;
    // delta as partial sums in 32-bit (a product whose K was split): added up in order, rounded as the product
    // would have rounded its result
    const float* ps = parts ? parts + (size_t)s * hidden : nullptr;
    auto delta_at = [&](int i) -> float {
        if (ds) return to_f32(ds[i]);
        float d = 0.f;
        for (int p = 0; p < n_parts; ++p) d += ps[(size_t)p * part_stride + i];
        return round_to<T>(d);
    };
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = to_f32(xs[i]);
        if (ds || ps) v = round_to<T>(v + delta_at(i));
        if (rs) rs[i] = from_f32<T>(v);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    T* o = out + (size_t)r * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v;
        if (rs) {
            v = to_f32(rs[i]);  // written by this same thread above
        } else {
            v = to_f32(xs[i]);
            if (ds || ps) v = round_to<T>(v + delta_at(i));
        }
        o[i] = from_f32<T>(to_f32(weight[i]) * round_to<T>(v * inv));
    }
}

// d[0..7] += the 8 consecutive floats at `ps` of each of n_parts arrays, part_stride elements apart, in the order of
// the arrays; the loads of four arrays are in flight together (one after the other, each would wait for memory).
__device__ __forceinline__ void sum_parts8(float (&d)[8], const float* __restrict__ ps, int n_parts, size_t part_stride) {
    for (int p0 = 0; p0 < n_parts; p0 += 4) {
        float4 a[4], b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float* src = ps + (size_t)min(p0 + j, n_parts - 1) * part_stride;  // (clamped: loaded, not added)
            a[j] = *reinterpret_cast<const float4*>(src);
            b[j] = *reinterpret_cast<const float4*>(src + 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (p0 + j < n_parts) {
                d[0] += a[j].x; d[1] += a[j].y; d[2] += a[j].z; d[3] += a[j].w;
                d[4] += b[j].x; d[5] += b[j].y; d[6] += b[j].z; d[7] += b[j].w;
            }
        }
    }
}

// The same for bfloat16 rows of hidden % 8 == 0 and hidden <= 8 * RV_CHUNKS * blockDim: every thread keeps
// its elements in registers (16-byte loads and stores), so the row is read once.
#define RV_CHUNKS 4
__global__ void rmsnorm_bf16_vec_kernel(bf16* __restrict__ out, const bf16* x, const bf16* __restrict__ delta,
                                        bf16* resid_out, const bf16* __restrict__ weight,
                                        const int* __restrict__ rows, float eps, int hidden,
                                        const float* __restrict__ parts, int n_parts, size_t part_stride) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int s = rows ? rows[r] : r;
    const uint4* xs = reinterpret_cast<const uint4*>(x + (size_t)s * hidden);
    const uint4* ds = delta ? reinterpret_cast<const uint4*>(delta + (size_t)s * hidden) : nullptr;
    uint4* rs = resid_out ? reinterpret_cast<uint4*>(resid_out + (size_t)s * hidden) : nullptr;
    const int nchunks = hidden / 8;
    float v[RV_CHUNKS][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < RV_CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nchunks) {
            const uint4 xv = xs[i];
            const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
            uint32_t dw[4] = {0, 0, 0, 0};
            if (ds) {
                const uint4 dv = ds[i];
                dw[0] = dv.x; dw[1] = dv.y; dw[2] = dv.z; dw[3] = dv.w;
            } else if (parts) {  // partial sums in 32-bit, added up in order and rounded as the product would have
                float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                const float* ps = parts + (size_t)s * hidden + 8 * i;
                sum_parts8(d, ps, n_parts, part_stride);
#pragma unroll
                for (int j = 0; j < 4; ++j) dw[j] = pack_bf16x2(d[2 * j], d[2 * j + 1]);
            }
            uint32_t ow[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float lo = bf16_bits_to_f32((uint16_t)(xw[j] & 0xffffu)), hi = bf16_bits_to_f32((uint16_t)(xw[j] >> 16));
                if (ds || parts) {
                    lo = bf16_bits_to_f32(f32_to_bf16_bits(lo + bf16_bits_to_f32((uint16_t)(dw[j] & 0xffffu))));
                    hi = bf16_bits_to_f32(f32_to_bf16_bits(hi + bf16_bits_to_f32((uint16_t)(dw[j] >> 16))));
                }
                v[c][2 * j] = lo;
                v[c][2 * j + 1] = hi;
                ss += lo * lo + hi * hi;
                ow[j] = pack_bf16x2(lo, hi);
            }
            if (rs) rs[i] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        }
    }
    // the norm's weight is asked for before the barriers of the sum, behind which it would cost a trip to memory
    const uint4* ws = reinterpret_cast<const uint4*>(weight);
    uint4 wreg[RV_CHUNKS];
#pragma unroll
    for (int c = 0; c < RV_CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nchunks) wreg[c] = ws[i];
    }
    ss = block_sum(ss, red);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    uint4* o = reinterpret_cast<uint4*>(out + (size_t)r * hidden);
#pragma unroll
    for (int c = 0; c < RV_CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nchunks) {
            const uint4 wv = wreg[c];
            const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
            uint32_t ow[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float lo = bf16_bits_to_f32((uint16_t)(ww[j] & 0xffffu)) * round_to<bf16>(v[c][2 * j] * inv);
                const float hi = bf16_bits_to_f32((uint16_t)(ww[j] >> 16)) * round_to<bf16>(v[c][2 * j + 1] * inv);
                ow[j] = pack_bf16x2(lo, hi);
            }
            o[i] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        }
    }
}

// ------------------------------------------------------------------ rotary encoding + cache store
// qkv row n = [q heads | k heads | v heads], head_dim wide each.
//   q, k: x' = x*cos + rotate_half(x)*sin with pairs (i, i + D/2) and angle
//         float(position) * inv_freq[i]  (src/llmserve/model/llama.py:31-54), computed in
//         32-bit and rounded once.  q is rotated in place.  inv_freq == nullptr: no rotation.
//   Without pools (k_pool == nullptr) k is rotated in place as well and nothing is stored.  With pools
//   k' goes to k_pool[page, kv_head, offset, :], v to v_pool[page, kv_head, :, offset]
//   (values transposed inside a page so that attention reads keys of one dimension
//   contiguously), page = slot / block_size, offset = slot % block_size.  slot < 0: no store.
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, const float* __restrict__ inv_freq,
                                  const int* __restrict__ positions, const int* __restrict__ slots,
                                  T* __restrict__ k_pool, T* __restrict__ v_pool, int n_heads,
                                  int n_kv_heads, int head_dim, int block_size) {
    const int n = blockIdx.x;
    const int half = head_dim / 2;
    const int row_width = (n_heads + 2 * n_kv_heads) * head_dim;
    T* row = qkv + (size_t)n * row_width;
    const float pos = (float)positions[n];
    const int slot = slots ? slots[n] : -1;
    const int page = slot >= 0 ? slot / block_size : 0;
    const int off = slot >= 0 ? slot % block_size : 0;

    // rotate q heads in place and k heads into the pool: one thread per (head, pair)
    const int rot_heads = n_heads + n_kv_heads;
    for (int t = threadIdx.x; t < rot_heads * half; t += blockDim.x) {
        const int h = t / half, i = t % half;
        T* x = row + (size_t)h * head_dim;
        float a = to_f32(x[i]), b = to_f32(x[i + half]);
        float ra = a, rb = b;
        if (inv_freq) {
            const float2 angle = rotary_angle(pos, inv_freq[i]);
            const float2 r = rotate_pair(a, b, angle.y, angle.x);
            ra = r.x;
            rb = r.y;
        }
        if (h < n_heads || k_pool == nullptr) {
            x[i] = from_f32<T>(ra);
            x[i + half] = from_f32<T>(rb);
        } else if (slot >= 0) {
            const int kvh = h - n_heads;
            T* dst = k_pool + (((size_t)page * n_kv_heads + kvh) * block_size + off) * head_dim;
            dst[i] = from_f32<T>(ra);
            dst[i + half] = from_f32<T>(rb);
        }
    }
    if (slot >= 0) {
        const T* v = row + (size_t)(n_heads + n_kv_heads) * head_dim;
        for (int t = threadIdx.x; t < n_kv_heads * head_dim; t += blockDim.x) {
            const int kvh = t / head_dim, d = t % head_dim;
            v_pool[(((size_t)page * n_kv_heads + kvh) * head_dim + d) * block_size + off] = v[t];
        }
    }
}

// bfloat16, head_dim % 16 == 0: the token's head_dim/2 sines and cosines are computed once per workgroup (the angle
// depends on the token and on i only; computed per element they cost more than the kernel's memory traffic); a
// thread takes 8 consecutive pairs (i .. i+7 and their partners at + head_dim/2) of one head with 16-byte loads and
// stores.  A workgroup is a chain of trips to memory (slot and position, the row, the run's slots, the values), so
// the row's first pieces are asked for before the angles are worked out, and a head's pieces while the head
// before it is rotated.
//
// Values: a page holds them transposed (a dimension's keys side by side), so a token alone leaves them in 2-byte
// stores.  G tokens (16, or 8 where the page size is no multiple of 16; 0: never) that lie side by side in one page,
// the first at a multiple of G, are a run: the run's workgroups share its KV heads out, and for a head a workgroup
// brings the G tokens' values through LDS, so that every thread stores 16 bytes of one dimension and a wave's
// stores are one contiguous piece where the page is G tokens wide.  Every workgroup of a run finds the same answer
// from the same G slots.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
#define ROPE_TILE_PAD 8  // elements between the rows of the LDS tile, so that a row starts at a multiple of 16 bytes

template <int G>
__global__ __launch_bounds__(256) void rope_store_bf16_vec_kernel(bf16* __restrict__ qkv, const float* __restrict__ inv_freq,
                                                                  const int* __restrict__ positions,
                                                                  const int* __restrict__ slots, bf16* __restrict__ k_pool,
                                                                  bf16* __restrict__ v_pool, int n_tokens, int n_heads,
                                                                  int n_kv_heads, int head_dim, int block_size) {
    // Workgroups go round the 8 XCDs; 16 consecutive tokens go to one XCD, so that what they write into the same
    // lines of a page meets in one L2.
    const int xcd = blockIdx.x % 8, place = blockIdx.x / 8;
    const int n = (place / 16) * 128 + xcd * 16 + place % 16;
    if (n >= n_tokens) return;
    const int tid = threadIdx.x;
    const int half = head_dim / 2, chunks = half / 8;
    const int row_width = (n_heads + 2 * n_kv_heads) * head_dim;
    bf16* row = qkv + (size_t)n * row_width;
    const int slot = slots ? slots[n] : -1;
    const int page = slot >= 0 ? slot / block_size : 0;
    const int off = slot >= 0 ? slot % block_size : 0;
    const int c = tid % chunks, h0 = tid / chunks, h_step = blockDim.x / chunks;
    const int rot_heads = n_heads + n_kv_heads;
    const bool rotates = h0 < h_step && h0 < rot_heads;  // (threads past the last whole group of `chunks` have no head)
    u32x4 av = {0, 0, 0, 0}, bv = {0, 0, 0, 0};
    if (rotates) {
        const bf16* x = row + (size_t)h0 * head_dim + 8 * c;
        av = *reinterpret_cast<const u32x4*>(x);
        bv = *reinterpret_cast<const u32x4*>(x + half);
    }

    extern __shared__ float angles[];  // [half] sines, [half] cosines, then the tile of values [G][head_dim + pad]
    __shared__ int run_found;
    // is this token part of a run?  (lead: the run's first token; the same for all of the workgroup)
    const int lead = n - (G > 0 ? off % G : 0);
    const bool may_run = G > 0 && slot >= 0 && lead >= 0 && lead + G <= n_tokens;
    if (tid < 64) {  // (the first wave)
        bool follows = true;
        if (may_run && tid < G) follows = slots[lead + tid] == slot - off % (G > 0 ? G : 1) + tid;
        const bool all_follow = __ballot(follows) == __ballot(true);
        if (tid == 0) run_found = may_run && all_follow;
    }
    if (inv_freq) {
        const float pos = (float)positions[n];
        for (int i = tid; i < half; i += blockDim.x) {
            const float2 angle = rotary_angle(pos, inv_freq[i]);
            angles[i] = angle.x;
            angles[half + i] = angle.y;
        }
    }
    __syncthreads();
    const bool in_run = run_found != 0;

    // the values of the run's first head for this workgroup, asked for before the rotation
    constexpr int GG = G > 0 ? G : 1;
    const int pieces = head_dim / 8;  // 16-byte pieces of a head
    const int my_head = n - lead;      // this workgroup takes the run's KV heads my_head, my_head + G, ...
    const bf16* v_lead = qkv + (size_t)lead * row_width + (size_t)(n_heads + n_kv_heads) * head_dim;
    u32x4 v_first = {0, 0, 0, 0};
    if (in_run && my_head < n_kv_heads && tid < GG * pieces)
        v_first = *reinterpret_cast<const u32x4*>(v_lead + (size_t)(tid / pieces) * row_width + (size_t)my_head * head_dim +
                                                  8 * (tid % pieces));

    if (rotates) {
        float sn[8], cs[8];
        if (inv_freq) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sn[e] = angles[8 * c + e];
                cs[e] = angles[half + 8 * c + e];
            }
        }
        for (int h = h0; h < rot_heads; h += h_step) {
            u32x4 a_next = {0, 0, 0, 0}, b_next = {0, 0, 0, 0};
            if (h + h_step < rot_heads) {
                const bf16* x_next = row + (size_t)(h + h_step) * head_dim + 8 * c;
                a_next = *reinterpret_cast<const u32x4*>(x_next);
                b_next = *reinterpret_cast<const u32x4*>(x_next + half);
            }
            const bool is_key = h >= n_heads;
            if (!(is_key && k_pool != nullptr && slot < 0)) {  // (else: a key with nowhere to go)
                u32x4 ra = av, rb = bv;
                if (inv_freq) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float lo_a[2], lo_b[2];
#pragma unroll
                        for (int u = 0; u < 2; ++u) {
                            const float a = bf16_bits_to_f32((uint16_t)(u ? av[j] >> 16 : av[j] & 0xffffu));
                            const float b = bf16_bits_to_f32((uint16_t)(u ? bv[j] >> 16 : bv[j] & 0xffffu));
                            const float2 r = rotate_pair(a, b, cs[2 * j + u], sn[2 * j + u]);
                            lo_a[u] = r.x;
                            lo_b[u] = r.y;
                        }
                        ra[j] = pack_bf16x2(lo_a[0], lo_a[1]);
                        rb[j] = pack_bf16x2(lo_b[0], lo_b[1]);
                    }
                }
                bf16* dst = row + (size_t)h * head_dim + 8 * c;
                if (is_key && k_pool != nullptr)
                    dst = k_pool + (((size_t)page * n_kv_heads + (h - n_heads)) * block_size + off) * head_dim + 8 * c;
                *reinterpret_cast<u32x4*>(dst) = ra;
                *reinterpret_cast<u32x4*>(dst + half) = rb;
            }
            av = a_next;
            bv = b_next;
        }
    }

    if constexpr (G > 0) if (in_run) {
        uint16_t* tile = reinterpret_cast<uint16_t*>(angles + head_dim);
        const int pitch = head_dim + ROPE_TILE_PAD;
        constexpr int PARTS = G / 8;  // 16-byte pieces of a dimension's G tokens
        for (int kvh = my_head; kvh < n_kv_heads; kvh += GG) {  // (the same number of turns for the whole workgroup)
            for (int t = tid; t < GG * pieces; t += blockDim.x) {
                const int j = t / pieces, piece = t % pieces;
                const u32x4 vv = (kvh == my_head && t == tid)
                                     ? v_first
                                     : *reinterpret_cast<const u32x4*>(v_lead + (size_t)j * row_width +
                                                                       (size_t)kvh * head_dim + 8 * piece);
                *reinterpret_cast<u32x4*>(&tile[j * pitch + 8 * piece]) = vv;
            }
            __syncthreads();
            bf16* head = v_pool + ((size_t)page * n_kv_heads + kvh) * head_dim * block_size + (off - off % GG);
            for (int t = tid; t < head_dim * PARTS; t += blockDim.x) {
                const int d = t / PARTS, part = t % PARTS;
                u32x4 w;
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    w[m] = (uint32_t)tile[(8 * part + 2 * m) * pitch + d] |
                           ((uint32_t)tile[(8 * part + 2 * m + 1) * pitch + d] << 16);
                *reinterpret_cast<u32x4*>(head + (size_t)d * block_size + 8 * part) = w;
            }
            __syncthreads();
        }
        return;
    }
    if (slot >= 0) {
        const bf16* v = row + (size_t)(n_heads + n_kv_heads) * head_dim;
        for (int t = tid; t < n_kv_heads * head_dim / 8; t += blockDim.x) {
            const u32x4 vv = *reinterpret_cast<const u32x4*>(v + 8 * t);
            const int kvh = (8 * t) / head_dim, d = (8 * t) % head_dim;
            bf16* dst = v_pool + (((size_t)page * n_kv_heads + kvh) * head_dim + d) * block_size + off;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                dst[(size_t)e * block_size].bits = (uint16_t)(e & 1 ? vv[e / 2] >> 16 : vv[e / 2] & 0xffffu);
        }
    }
}

// ------------------------------------------------------------------ SiLU(gate) * up
// gate_up row = [gate (inter) | up (inter)]; out = T(T(silu(gate)) * up), the reference's
// rounding points (src/llmserve/model/llama.py:120).
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gate_up, int inter, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t n = idx / inter;
    const int i = (int)(idx % inter);
    const T* row = gate_up + n * 2 * (size_t)inter;
    const float g = to_f32(row[i]);
    const float u = to_f32(row[inter + i]);
    const float s = round_to<T>(g / (1.f + expf(-g)));
    out[idx] = from_f32<T>(s * u);
}

// bfloat16 rows of inter % 8 == 0: 8 elements per thread, 16-byte loads and stores.
__global__ void silu_mul_bf16_vec_kernel(bf16* __restrict__ out, const bf16* __restrict__ gate_up, int inter,
                                         size_t total_chunks) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total_chunks) return;
    const int cpr = inter / 8;  // chunks per row
    const size_t n = idx / cpr;
    const int c = (int)(idx % cpr);
    const uint4* row = reinterpret_cast<const uint4*>(gate_up + n * 2 * (size_t)inter);
    const uint4 gv = row[c], uv = row[cpr + c];
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float r2[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float g = bf16_bits_to_f32((uint16_t)(h ? gw[j] >> 16 : gw[j] & 0xffffu));
            const float u = bf16_bits_to_f32((uint16_t)(h ? uw[j] >> 16 : uw[j] & 0xffffu));
            r2[h] = round_to<bf16>(g / (1.f + expf(-g))) * u;
        }
        ow[j] = pack_bf16x2(r2[0], r2[1]);
    }
    reinterpret_cast<uint4*>(out)[idx] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// ------------------------------------------------------------------ scattered int32 writes
// dst[index[i]] = value[i] for index[i] >= 0: how a step's new pages reach the block tables that
// stay on the device.
__global__ void scatter_i32_kernel(int* __restrict__ dst, const int* __restrict__ index,
                                   const int* __restrict__ value, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && index[i] >= 0) dst[index[i]] = value[i];
}

// ------------------------------------------------------------------ launchers
#define DISPATCH_DTYPE(dtype, ...)                 \
    if ((dtype) == 0) {                            \
        typedef float T;                           \
        __VA_ARGS__                                \
    } else if ((dtype) == 1) {                     \
        typedef bf16 T;                            \
        __VA_ARGS__                                \
    } else {                                       \
        LLMS_REQUIRE(false, "dtype must be 0 (float32) or 1 (bfloat16)"); \
    }

__global__ void rotary_angles_kernel(float2* out, const int* positions, const float* inv_freq, int total, int half) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) out[i] = rotary_angle((float)positions[i / half], inv_freq[i % half]);
}

extern "C" {

int llms_embed_gather(int dtype, void* out, const void* table, const int* ids, int n_tokens, int hidden,
                      int vocab, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && hidden > 0 && vocab > 0, "embed_gather: sizes must be positive");
    DISPATCH_DTYPE(dtype, embed_gather_kernel<T><<<n_tokens, 256, 0, stream>>>((T*)out, (const T*)table, ids,
                                                                                hidden, vocab);)
    LLMS_LAUNCH_CHECK();
}

// parts (nullable, instead of delta): n_parts arrays of 32-bit partial sums, part_stride elements apart, each laid
// out like x; the delta is their sum, rounded to the dtype of x.
int llms_rmsnorm(int dtype, void* out, const void* x, const void* delta, void* resid_out, const void* weight,
                 const int* rows, float eps, int n_rows, int hidden, const float* parts, int n_parts,
                 size_t part_stride, hipStream_t stream) {
    LLMS_REQUIRE(n_rows > 0 && hidden > 0, "rmsnorm: sizes must be positive");
    LLMS_REQUIRE(!(rows && resid_out), "rmsnorm: a row gather cannot also write the residual back");
    LLMS_REQUIRE(!(parts && delta) && (!parts || n_parts > 0), "rmsnorm: delta or its partial sums, not both");
    if (dtype == 1 && hidden % 8 == 0 && hidden <= 8 * RV_CHUNKS * 256 && ((uintptr_t)x % 16) == 0 &&
        ((uintptr_t)out % 16) == 0 && ((uintptr_t)weight % 16) == 0 && (!delta || ((uintptr_t)delta % 16) == 0) &&
        (!parts || (((uintptr_t)parts % 16) == 0 && part_stride % 4 == 0)) &&
        (!resid_out || ((uintptr_t)resid_out % 16) == 0)) {
        const int chunks = hidden / 8;
        const int threads = chunks <= 64 ? 64 : chunks <= 128 ? 128 : 256;
        rmsnorm_bf16_vec_kernel<<<n_rows, threads, 0, stream>>>((bf16*)out, (const bf16*)x, (const bf16*)delta,
                                                                (bf16*)resid_out, (const bf16*)weight, rows, eps,
                                                                hidden, parts, n_parts, part_stride);
        LLMS_LAUNCH_CHECK();
    }
    const int threads = hidden >= 2048 ? 512 : 256;
    DISPATCH_DTYPE(dtype, rmsnorm_kernel<T><<<n_rows, threads, 0, stream>>>(
                              (T*)out, (const T*)x, (const T*)delta, (T*)resid_out, (const T*)weight, rows,
                              eps, hidden, parts, n_parts, part_stride);)
    LLMS_LAUNCH_CHECK();
}

int llms_rope_store(int dtype, void* qkv, const float* inv_freq, const int* positions, const int* slots,
                    void* k_pool, void* v_pool, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                    int block_size, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv_heads > 0, "rope_store: sizes must be positive");
    LLMS_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "rope_store: head_dim must be even");
    LLMS_REQUIRE(block_size > 0, "rope_store: block_size must be positive");
    LLMS_REQUIRE(slots == nullptr || (k_pool && v_pool), "rope_store: slots given without pools");
    if (dtype == 1 && head_dim % 16 == 0 && head_dim <= 4096 && ((uintptr_t)qkv % 16) == 0 &&
        (k_pool == nullptr || ((uintptr_t)k_pool % 16) == 0)) {
        const unsigned grid = (unsigned)((n_tokens + 127) / 128 * 128);
        // runs of tokens whose values go through LDS: as long as the page size allows, and the tile fits
        const bool runs = slots && ((uintptr_t)v_pool % 16) == 0 && head_dim <= 1024;
        const int run = !runs ? 0 : block_size % 16 == 0 ? 16 : block_size % 8 == 0 ? 8 : 0;
        const size_t lds = head_dim * sizeof(float) + (size_t)run * (head_dim + ROPE_TILE_PAD) * sizeof(uint16_t);
#define LLMS_ROPE_LAUNCH(G)                                                                                       \
    rope_store_bf16_vec_kernel<G><<<grid, 256, lds, stream>>>((bf16*)qkv, inv_freq, positions, slots, (bf16*)k_pool, \
                                                              (bf16*)v_pool, n_tokens, n_heads, n_kv_heads, head_dim, \
                                                              block_size)
        if (run == 16) LLMS_ROPE_LAUNCH(16);
        else if (run == 8) LLMS_ROPE_LAUNCH(8);
        else LLMS_ROPE_LAUNCH(0);
#undef LLMS_ROPE_LAUNCH
        LLMS_LAUNCH_CHECK();
    }
    DISPATCH_DTYPE(dtype, rope_store_kernel<T><<<n_tokens, 256, 0, stream>>>(
                              (T*)qkv, inv_freq, positions, slots, (T*)k_pool, (T*)v_pool, n_heads,
                              n_kv_heads, head_dim, block_size);)
    LLMS_LAUNCH_CHECK();
}

// out[m][i] = (sine, cosine) of positions[m] * inv_freq[i]: the angles of a step's tokens, once for all layers.
int llms_rotary_angles(float* out, const int* positions, const float* inv_freq, int n_tokens, int half,
                       hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && half > 0 && (long long)n_tokens * half < (1ll << 30), "rotary_angles: sizes out of range");
    const int total = n_tokens * half;
    rotary_angles_kernel<<<(total + 255) / 256, 256, 0, stream>>>(reinterpret_cast<float2*>(out), positions, inv_freq,
                                                                  total, half);
    LLMS_LAUNCH_CHECK();
}

int llms_scatter_i32(int* dst, const int* index, const int* value, int n, hipStream_t stream) {
    LLMS_REQUIRE(n > 0 && dst && index && value, "scatter_i32: bad arguments");
    scatter_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, index, value, n);
    LLMS_LAUNCH_CHECK();
}

int llms_silu_mul(int dtype, void* out, const void* gate_up, int n_rows, int inter, hipStream_t stream) {
    LLMS_REQUIRE(n_rows > 0 && inter > 0, "silu_mul: sizes must be positive");
    const size_t total = (size_t)n_rows * inter;
    if (dtype == 1 && inter % 8 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)gate_up % 16) == 0) {
        const size_t chunks = total / 8;
        silu_mul_bf16_vec_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, stream>>>((bf16*)out, (const bf16*)gate_up,
                                                                                         inter, chunks);
        LLMS_LAUNCH_CHECK();
    }
    const unsigned blocks = (unsigned)((total + 255) / 256);
    DISPATCH_DTYPE(dtype, silu_mul_kernel<T><<<blocks, 256, 0, stream>>>((T*)out, (const T*)gate_up, inter,
                                                                          total);)
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
