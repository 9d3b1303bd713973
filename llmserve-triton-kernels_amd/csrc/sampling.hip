// Token choice from 32-bit logits, one workgroup per row, nothing read back but the ids.
//
// greedy (temperature <= 0): argmax, the lowest index wins ties
//   (src/llmserve/sampling/sampler.py:20-21).
// otherwise (src/llmserve/sampling/sampler.py:23-38): z = logits / T;
//   top-k keeps z >= k-th largest (ties survive); top-p drops a token when the probability
//   mass of the tokens above it exceeds top_p (the largest is always kept); the token is
//   the first index, in vocabulary order, whose cumulative probability exceeds u * total,
//   u in [0,1) supplied by the caller.  (The reference draws with torch.multinomial; its
//   promise is reproducibility under a seed, which a caller-supplied u keeps.)
// Every reduction has an order fixed by the block size, so a row's result does not depend
// on the other rows of the batch.
#include "common.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);  // ascending as unsigned
}

__device__ __forceinline__ uint32_t block_sum_u32(uint32_t v, uint32_t* lds) {
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
#pragma unroll
    for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LLMS_WAVE);
    __syncthreads();
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    uint32_t t = 0;
    for (int i = 0; i < SAMPLE_THREADS / LLMS_WAVE; ++i) t += lds[i];
    return t;
}

// argmax over a row; returns the same (value, index) to every thread.
__device__ __forceinline__ int block_argmax(const float* __restrict__ row, int vocab, float* fl, int* il,
                                            float* max_out) {
    float best = -INFINITY;
    int besti = 0x7fffffff;
    // eight loads of a thread are in flight together (one after the other, each would wait for memory)
    for (int base = threadIdx.x; base < vocab; base += 8 * SAMPLE_THREADS) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = row[min(base + j * SAMPLE_THREADS, vocab - 1)];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = base + j * SAMPLE_THREADS;
            if (i < vocab && (v[j] > best || (v[j] == best && i < besti))) {
                best = v[j];
                besti = i;
            }
        }
    }
#pragma unroll
    for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, LLMS_WAVE);
        const int oi = __shfl_xor(besti, o, LLMS_WAVE);
        if (ov > best || (ov == best && oi < besti)) {
            best = ov;
            besti = oi;
        }
    }
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    __syncthreads();
    if (lane == 0) {
        fl[wave] = best;
        il[wave] = besti;
    }
    __syncthreads();
    best = fl[0];
    besti = il[0];
    for (int i = 1; i < SAMPLE_THREADS / LLMS_WAVE; ++i) {
        if (fl[i] > best || (fl[i] == best && il[i] < besti)) {
            best = fl[i];
            besti = il[i];
        }
    }
    if (besti == 0x7fffffff) besti = 0;  // a row of NaN or -inf
    *max_out = best;
    return besti;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    int* __restrict__ out, const float* __restrict__ logits, int ld, int vocab,
    const float* __restrict__ temperature, const int* __restrict__ top_k, const float* __restrict__ top_p,
    const float* __restrict__ uniform) {
    __shared__ float fl[SAMPLE_THREADS / LLMS_WAVE];
    __shared__ int il[SAMPLE_THREADS / LLMS_WAVE];
    __shared__ uint32_t ul[SAMPLE_THREADS / LLMS_WAVE];
    __shared__ int found;
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * ld;
    float zmax_raw;
    const int amax = block_argmax(row, vocab, fl, il, &zmax_raw);
    const float T = temperature ? temperature[r] : 0.f;
    if (!(T > 0.f)) {
        if (threadIdx.x == 0) out[r] = amax;
        return;
    }
    const float inv_t = 1.f / T;
    const float zmax = zmax_raw * inv_t;
    // threshold in key order: a token survives iff order_key(z) >= thr
    uint32_t thr = 0;
    const int k = top_k ? top_k[r] : 0;
    if (k > 0 && k < vocab) {
        uint32_t t = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = t | (1u << bit);
            uint32_t c = 0;
            for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) c += order_key(row[i] * inv_t) >= cand;
            if (block_sum_u32(c, ul) >= (uint32_t)k) t = cand;
        }
        thr = t;  // key of the k-th largest
    }
    const float p = top_p ? top_p[r] : 1.f;
    if (p < 1.f) {
        float e = 0.f;
        for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
            const float z = row[i] * inv_t;
            if (order_key(z) >= thr) e += expf(z - zmax);
        }
        const float limit = p * block_sum(e, fl);
        // largest t whose mass strictly above it still exceeds the limit; survivors are > t
        uint32_t t = 0;
        bool any = false;
        for (int bit = 31; bit >= -1; --bit) {
            const uint32_t cand = bit >= 0 ? (t | (1u << bit)) : 0u;
            if (bit < 0 && any) break;
            float above = 0.f;
            for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
                const float z = row[i] * inv_t;
                const uint32_t key = order_key(z);
                if (key >= thr && key > cand) above += expf(z - zmax);
            }
            if (block_sum(above, fl) > limit) {
                t = cand;
                any = true;
            }
        }
        if (any && t + 1u > thr) thr = t + 1u;
    }
    // total mass of the survivors, then the first index whose running sum passes u * total
    float e = 0.f;
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
        const float z = row[i] * inv_t;
        if (order_key(z) >= thr) e += expf(z - zmax);
    }
    const float target = uniform[r] * block_sum(e, fl);
    if (threadIdx.x == 0) found = 0x7fffffff;
    __syncthreads();
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    float running = 0.f;
    int last_kept = -1;
    for (int base = 0; base < vocab; base += SAMPLE_THREADS) {
        const int i = base + threadIdx.x;
        float v = 0.f;
        bool kept = false;
        if (i < vocab) {
            const float z = row[i] * inv_t;
            kept = order_key(z) >= thr;
            if (kept) v = expf(z - zmax);
        }
        float scan = v;  // inclusive scan inside the wave
#pragma unroll
        for (int o = 1; o < LLMS_WAVE; o <<= 1) {
            const float t = __shfl_up(scan, o, LLMS_WAVE);
            if (lane >= o) scan += t;
        }
        __syncthreads();
        if (lane == LLMS_WAVE - 1) fl[wave] = scan;
        __syncthreads();
        float before = running;
        for (int w = 0; w < wave; ++w) before += fl[w];
        float tile_total = 0.f;
        for (int w = 0; w < SAMPLE_THREADS / LLMS_WAVE; ++w) tile_total += fl[w];
        if (kept) {
            last_kept = i;
            if (before + scan > target) atomicMin(&found, i);
        }
        running += tile_total;
        __syncthreads();
        if (found != 0x7fffffff) break;
    }
    if (found == 0x7fffffff) {
        // rounding left the running sum at or below the target: take the last surviving index
        int lk = last_kept;
#pragma unroll
        for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) lk = max(lk, __shfl_xor(lk, o, LLMS_WAVE));
        __syncthreads();
        if (lane == 0) il[wave] = lk;
        __syncthreads();
        lk = il[0];
        for (int w = 1; w < SAMPLE_THREADS / LLMS_WAVE; ++w) lk = max(lk, il[w]);
        if (threadIdx.x == 0) out[r] = lk >= 0 ? lk : amax;
    } else if (threadIdx.x == 0) {
        out[r] = found;
    }
}

extern "C" {

// temperature, top_k, top_p may be null (greedy / off / off); uniform is needed when any
// temperature is positive.
int llms_sample_rows(int* out, const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                     const int* top_k, const float* top_p, const float* uniform, hipStream_t stream) {
    LLMS_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "sample_rows: bad sizes");
    LLMS_REQUIRE(temperature == nullptr || uniform != nullptr, "sample_rows: temperature needs uniform numbers");
    sample_rows_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(out, logits, ld, vocab, temperature, top_k, top_p,
                                                              uniform);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
