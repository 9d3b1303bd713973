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

// argmax over a row; returns the same (value, index) to every thread.  `value(j)` is the thread's j-th logit (element
// threadIdx.x + j * SAMPLE_THREADS of the row), for j < nj.
template <typename F>
__device__ __forceinline__ int block_argmax(F value, int nj, int vocab, float* fl, int* il, float* max_out) {
    float best = -INFINITY;
    int besti = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < nj; ++j) {
        const int i = threadIdx.x + j * SAMPLE_THREADS;
        const float v = value(j);
        if (i < vocab && (v > best || (v == best && i < besti))) {
            best = v;
            besti = i;
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

// VPT > 0: the row (vocab <= VPT * SAMPLE_THREADS) is read once and kept in registers, VPT logits per thread, for
// the up to 70 passes that follow (a pass over memory waits for every load in turn).  VPT = 0: any vocabulary, every
// pass reads the row again.
template <int VPT>
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
    const int nj = VPT > 0 ? VPT : (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    float held[VPT > 0 ? VPT : 1];
    if (VPT > 0) {
#pragma unroll
        for (int j = 0; j < VPT; ++j) held[j] = row[min((int)threadIdx.x + j * SAMPLE_THREADS, vocab - 1)];
    }
    // the thread's j-th logit (callers check that its index is below vocab)
    auto raw = [&](int j) -> float {
        if (VPT > 0) return held[j];
        return row[min((int)threadIdx.x + j * SAMPLE_THREADS, vocab - 1)];
    };
    float zmax_raw;
    const int amax = block_argmax(raw, nj, vocab, fl, il, &zmax_raw);
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
#pragma unroll
            for (int j = 0; j < nj; ++j)
                if ((int)threadIdx.x + j * SAMPLE_THREADS < vocab) c += order_key(raw(j) * inv_t) >= cand;
            if (block_sum_u32(c, ul) >= (uint32_t)k) t = cand;
        }
        thr = t;  // key of the k-th largest
    }
    const float p = top_p ? top_p[r] : 1.f;
    if (p < 1.f) {
        float e = 0.f;
#pragma unroll
        for (int j = 0; j < nj; ++j) {
            const float z = raw(j) * inv_t;
            if ((int)threadIdx.x + j * SAMPLE_THREADS < vocab && order_key(z) >= thr) e += expf(z - zmax);
        }
        const float limit = p * block_sum(e, fl);
        // largest t whose mass strictly above it still exceeds the limit; survivors are > t
        uint32_t t = 0;
        bool any = false;
        for (int bit = 31; bit >= -1; --bit) {
            const uint32_t cand = bit >= 0 ? (t | (1u << bit)) : 0u;
            if (bit < 0 && any) break;
            float above = 0.f;
#pragma unroll
            for (int j = 0; j < nj; ++j) {
                const float z = raw(j) * inv_t;
                const uint32_t key = order_key(z);
                if ((int)threadIdx.x + j * SAMPLE_THREADS < vocab && key >= thr && key > cand) above += expf(z - zmax);
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
#pragma unroll
    for (int j = 0; j < nj; ++j) {
        const float z = raw(j) * inv_t;
        if ((int)threadIdx.x + j * SAMPLE_THREADS < vocab && order_key(z) >= thr) e += expf(z - zmax);
    }
    const float target = uniform[r] * block_sum(e, fl);
    if (threadIdx.x == 0) found = 0x7fffffff;
    __syncthreads();
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    constexpr int NWAVES = SAMPLE_THREADS / LLMS_WAVE;
    int last_kept = -1;
    // the thread's weight in tile j (the SAMPLE_THREADS consecutive tokens from j * SAMPLE_THREADS on), 0 if dropped
    auto weight = [&](int j, bool& kept) -> float {
        const float z = raw(j) * inv_t;
        kept = j * SAMPLE_THREADS + (int)threadIdx.x < vocab && order_key(z) >= thr;
        return kept ? expf(z - zmax) : 0.f;
    };
    auto wave_scan = [&](float v) -> float {  // inclusive, in lane order
#pragma unroll
        for (int o = 1; o < LLMS_WAVE; o <<= 1) {
            const float t = __shfl_up(v, o, LLMS_WAVE);
            if (lane >= o) v += t;
        }
        return v;
    };
    if (VPT > 0) {
        // every wave's sum of every tile at once, then each thread walks the tiles' sums to the tile where the
        // running sum passes the target, and only that tile is scanned: 3 barriers instead of 3 per tile
        __shared__ float wave_total[VPT > 0 ? VPT : 1][NWAVES];
#pragma unroll
        for (int j = 0; j < nj; ++j) {
            bool kept;
            const float s = wave_scan(weight(j, kept));
            if (kept) last_kept = j * SAMPLE_THREADS + threadIdx.x;
            if (lane == LLMS_WAVE - 1) wave_total[j][wave] = s;
        }
        __syncthreads();
        float running = 0.f;
#pragma unroll
        for (int j = 0; j < nj; ++j) {
            float before = running, end = running;  // sums up to this wave, up to the tile's end: the same additions
            for (int w = 0; w < NWAVES; ++w) {
                if (w == wave) before = end;
                end += wave_total[j][w];
            }
            if (end > target) {  // (the same for every thread)
                bool kept;
                const float s = wave_scan(weight(j, kept));
                if (kept && before + s > target) atomicMin(&found, j * SAMPLE_THREADS + (int)threadIdx.x);
                break;
            }
            running = end;
        }
        __syncthreads();
    } else {
        float running = 0.f;
        for (int j = 0; j < nj; ++j) {
            bool kept;
            const float scan = wave_scan(weight(j, kept));
            __syncthreads();
            if (lane == LLMS_WAVE - 1) fl[wave] = scan;
            __syncthreads();
            float before = running;
            for (int w = 0; w < wave; ++w) before += fl[w];
            float tile_total = 0.f;
            for (int w = 0; w < NWAVES; ++w) tile_total += fl[w];
            if (kept) {
                last_kept = j * SAMPLE_THREADS + threadIdx.x;
                if (before + scan > target) atomicMin(&found, j * SAMPLE_THREADS + (int)threadIdx.x);
            }
            running += tile_total;
            __syncthreads();
            if (found != 0x7fffffff) break;
        }
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
    if (vocab <= 32 * SAMPLE_THREADS)  // (64 logits per thread would not fit the registers of 1,024 threads)
        sample_rows_kernel<32><<<n_rows, SAMPLE_THREADS, 0, stream>>>(out, logits, ld, vocab, temperature, top_k, top_p, uniform);
    else
        sample_rows_kernel<0><<<n_rows, SAMPLE_THREADS, 0, stream>>>(out, logits, ld, vocab, temperature, top_k, top_p, uniform);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
