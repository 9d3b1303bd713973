// Causal attention of new tokens over the paged key/value cache, one wave per
// (token, query head), 32-bit arithmetic throughout.  It serves prompts, portions of
// prompts and single decoded tokens alike: a token at position p reads the keys
// max(0, p - window + 1) .. p of its own request through that request's block table
// (its own key was stored before this kernel runs).  Any head_dim up to 256, any
// block size, any number of heads and groups.  float and bfloat16 storage.
//
// Formula (src/llmserve/model/llama.py:94-106, src/llmserve/kvcache/paged.py:99-110):
//   query head h reads KV head h / (n_heads / n_kv_heads); s_j = (q . k_j) / sqrt(D);
//   a = softmax_j(s) over the visible keys; o = sum_j a_j v_j.
#include "common.h"

#define ATT_MAX_D 256
#define ATT_WAVES 4

template <typename T>
__global__ __launch_bounds__(ATT_WAVES* LLMS_WAVE) void attention_wave_kernel(
    T* __restrict__ out, int out_stride, const T* __restrict__ q, int q_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int* __restrict__ block_tables, const int* __restrict__ table_rows,
    int max_blocks, const int* __restrict__ token_seq, const int* __restrict__ positions, int n_heads, int n_kv_heads,
    int head_dim, int block_size, int window, float scale) {
    __shared__ float qs[ATT_WAVES][ATT_MAX_D];
    const int n = blockIdx.x;
    const int wave = threadIdx.x / LLMS_WAVE, lane = threadIdx.x % LLMS_WAVE;
    const int h = blockIdx.y * ATT_WAVES + wave;
    const bool active = h < n_heads;
    if (active) {
        const T* qrow = q + (size_t)n * q_stride + (size_t)h * head_dim;
        for (int d = lane; d < head_dim; d += LLMS_WAVE) qs[wave][d] = to_f32(qrow[d]) * scale;
    }
    __syncthreads();
    if (!active) return;

    const int p = positions[n];
    const int seq = token_seq[n];
    const int* table = block_tables + (size_t)(table_rows ? table_rows[seq] : seq) * max_blocks;
    const int kvh = h / (n_heads / n_kv_heads);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;

    float acc[ATT_MAX_D / LLMS_WAVE] = {};
    float m = -INFINITY, l = 0.f;
    for (int j0 = lo; j0 <= p; j0 += LLMS_WAVE) {
        const int j = j0 + lane;
        float s = -INFINITY;
        if (j <= p) {
            const int page = table[j / block_size], off = j % block_size;
            const T* kr = k_pool + (((size_t)page * n_kv_heads + kvh) * block_size + off) * head_dim;
            float dot = 0.f;
            for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[wave][d], to_f32(kr[d]), dot);
            s = dot;
        }
        const float m_new = fmaxf(m, wave_max(s));  // finite: key j0 is always visible
        const float pj = (j <= p) ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);  // 0 on the first tile (m = -inf)
        l = l * corr + wave_sum(pj);
#pragma unroll
        for (int i = 0; i < ATT_MAX_D / LLMS_WAVE; ++i) acc[i] *= corr;
        const int count = min(LLMS_WAVE, p - j0 + 1);
        for (int jj = 0; jj < count; ++jj) {
            const float pv = __shfl(pj, jj, LLMS_WAVE);
            const int key = j0 + jj;
            const int page = table[key / block_size], off = key % block_size;
            const T* vbase = v_pool + ((size_t)page * n_kv_heads + kvh) * head_dim * block_size + off;
#pragma unroll
            for (int i = 0; i < ATT_MAX_D / LLMS_WAVE; ++i) {
                const int d = lane + i * LLMS_WAVE;
                if (d < head_dim) acc[i] = fmaf(pv, to_f32(vbase[(size_t)d * block_size]), acc[i]);
            }
        }
        m = m_new;
    }
    T* orow = out + (size_t)n * out_stride + (size_t)h * head_dim;
    const float inv_l = 1.f / l;
#pragma unroll
    for (int i = 0; i < ATT_MAX_D / LLMS_WAVE; ++i) {
        const int d = lane + i * LLMS_WAVE;
        if (d < head_dim) orow[d] = from_f32<T>(acc[i] * inv_l);
    }
}

extern "C" {

int llms_attention_wave(int dtype, void* out, int out_stride, const void* q, int q_stride, const void* k_pool,
                        const void* v_pool, const int* block_tables, const int* table_rows, int max_blocks,
                        const int* token_seq,
                        const int* positions, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                        int block_size, int window, float scale, hipStream_t stream) {
    LLMS_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv_heads > 0, "attention: sizes must be positive");
    LLMS_REQUIRE(n_heads % n_kv_heads == 0, "attention: n_heads must be a multiple of n_kv_heads");
    LLMS_REQUIRE(head_dim > 0 && head_dim <= ATT_MAX_D, "attention: head_dim must be in 1..256");
    LLMS_REQUIRE(block_size > 0 && max_blocks > 0, "attention: block_size and max_blocks must be positive");
    LLMS_REQUIRE(window >= 0, "attention: window must be >= 0 (0 = all keys)");
    dim3 grid(n_tokens, (n_heads + ATT_WAVES - 1) / ATT_WAVES);
    LLMS_REQUIRE(grid.y <= 65535, "attention: too many heads");
    if (dtype == 0) {
        attention_wave_kernel<float><<<grid, ATT_WAVES * LLMS_WAVE, 0, stream>>>(
            (float*)out, out_stride, (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool,
            block_tables, table_rows, max_blocks, token_seq, positions, n_heads, n_kv_heads, head_dim, block_size, window,
            scale);
    } else if (dtype == 1) {
        attention_wave_kernel<bf16><<<grid, ATT_WAVES * LLMS_WAVE, 0, stream>>>(
            (bf16*)out, out_stride, (const bf16*)q, q_stride, (const bf16*)k_pool, (const bf16*)v_pool,
            block_tables, table_rows, max_blocks, token_seq, positions, n_heads, n_kv_heads, head_dim, block_size, window,
            scale);
    } else {
        LLMS_REQUIRE(false, "attention: dtype must be 0 (float32) or 1 (bfloat16)");
    }
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
