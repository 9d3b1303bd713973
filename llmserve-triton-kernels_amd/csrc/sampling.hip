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
// Every reduction has an order fixed by the block size, or adds integers (counts, and masses in fixed point), so a
// row's result does not depend on the other rows of the batch nor on the order in which threads arrive.
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

// Selection by digits.  The histogram holds, for the keys whose decided upper bits equal the prefix, the count (W =
// uint32_t) or the mass in fixed point (W = unsigned long long) of those whose next 8 bits are d; `base` is the
// count (mass) of the keys above the prefix.  pick_digit finds the largest digit D with base + sum(hist[D..255]) >
// bound and hands D and base + sum(hist[D+1..255]) to every thread.  Sums of integers: the order of the atomic
// additions that filled the histogram does not matter.
// The histogram is 16 KB whatever W is: every digit has 64 bytes of copies (16 counts or 8 masses), and a thread adds
// to copy threadIdx.x % copies.  The upper digits of a row's keys are nearly all alike (sign and exponent of numbers
// of one size) and additions to one address of LDS are served one after the other; with the copies of a digit side
// by side they also fall into different banks.
#define HIST_BYTES 16384
typedef unsigned long long u64;

template <typename W>
__device__ __forceinline__ void hist_add(u64* hist, uint32_t digit, W v) {
    constexpr int COPIES = 64 / sizeof(W);
    atomicAdd(reinterpret_cast<W*>(hist) + digit * COPIES + threadIdx.x % COPIES, v);
}

__device__ __forceinline__ u64 shfl_xor_u64(u64 v, int o) {
    const unsigned lo = __shfl_xor((unsigned)v, o, LLMS_WAVE), hi = __shfl_xor((unsigned)(v >> 32), o, LLMS_WAVE);
    return ((u64)hi << 32) | lo;
}

__device__ __forceinline__ u64 shfl_down_u64(u64 v, int o) {
    const unsigned lo = __shfl_down((unsigned)v, o, LLMS_WAVE), hi = __shfl_down((unsigned)(v >> 32), o, LLMS_WAVE);
    return ((u64)hi << 32) | lo;
}

// Every thread takes the 16 bytes of the histogram at 16 * threadIdx.x (a quarter of digit threadIdx.x / 4's
// copies), leaves zeros there for the next pass, and four neighbours add up to the digit's sum; wave 0 then scans the
// 256 sums from the top.  fraction >= 0: the bound is fraction * (base + the whole histogram), returned in *bound.
template <typename W>
__device__ __forceinline__ void pick_digit(u64* hist, u64* digit_sum /* [256] */, u64 base, u64* bound, float fraction,
                                           u64* sel /* [3] */, int* digit, u64* above) {
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    __syncthreads();  // the histogram is complete
    {
        uint4* mine = reinterpret_cast<uint4*>(hist) + threadIdx.x;
        const uint4 w = *mine;
        *mine = make_uint4(0u, 0u, 0u, 0u);
        u64 sum = sizeof(W) == 4 ? (u64)w.x + w.y + w.z + w.w : (((u64)w.y << 32) | w.x) + (((u64)w.w << 32) | w.z);
        sum += shfl_xor_u64(sum, 1);
        sum += shfl_xor_u64(sum, 2);
        if (threadIdx.x % 4 == 0) digit_sum[threadIdx.x / 4] = sum;
    }
    __syncthreads();
    if (wave == 0) {
        u64 b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) b[i] = digit_sum[4 * lane + i];
        const u64 own = b[0] + b[1] + b[2] + b[3];
        u64 suffix = own;  // sum over this lane's and all higher lanes' bins
#pragma unroll
        for (int o = 1; o < LLMS_WAVE; o <<= 1) {
            const u64 t = shfl_down_u64(suffix, o);
            if (lane + o < LLMS_WAVE) suffix += t;
        }
        u64 limit = *bound;
        if (fraction >= 0.f) {
            const unsigned lo = __shfl((unsigned)suffix, 0, LLMS_WAVE), hi = __shfl((unsigned)(suffix >> 32), 0, LLMS_WAVE);
            limit = (u64)((double)fraction * (double)(base + (((u64)hi << 32) | lo)));
        }
        u64 s = base + suffix - own;  // everything above this lane's bins
        int best = -1;
        u64 best_above = 0;
#pragma unroll
        for (int i = 3; i >= 0; --i) {
            if (best < 0 && s + b[i] > limit) {
                best = 4 * lane + i;
                best_above = s;
            }
            s += b[i];
        }
        int top = best;
#pragma unroll
        for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) top = max(top, __shfl_xor(top, o, LLMS_WAVE));
        if (top >= 0 && best == top) {
            sel[0] = (u64)top;
            sel[1] = best_above;
        }
        if (top < 0 && lane == 0) {  // (cannot happen while base + the whole histogram exceeds the bound)
            sel[0] = 0;
            sel[1] = base + suffix - b[0];
        }
        if (lane == 0) sel[2] = limit;
    }
    __syncthreads();
    *digit = (int)sel[0];
    *above = sel[1];
    *bound = sel[2];
}

// argmax over a row; returns the same (value, index) to every thread.  `value(j)` is the thread's j-th logit and
// `index(j)` its place in the row, for j < nj.
template <int UNROLL, typename F, typename G>
__device__ __forceinline__ int block_argmax(F value, G index, int nj, int vocab, float* fl, int* il, float* max_out) {
    float best = -INFINITY;
    int besti = 0x7fffffff;
#pragma unroll UNROLL
    for (int j = 0; j < nj; ++j) {
        const int i = index(j);
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

#define LDS_ROW_MAX 32768  // logits of a row that is kept in LDS
#define SURVIVORS_MAX 1024

// IN_LDS (vocab <= LDS_ROW_MAX): the row is read once and kept in LDS for the dozen passes that follow; a pass over
// memory waits for every load in turn, and a row kept in registers forces every pass to be unrolled over all its
// elements, which leaves no registers for the passes' own values.  Thread t owns the `per` consecutive logits from
// t * per on, at held[t * stride + j] with an odd stride, so that the lanes of a wave read different banks; the final
// walk along the cumulative sum is then one scan over the threads' sums.  Otherwise any vocabulary: thread t owns
// the logits t, t + SAMPLE_THREADS, ... and every pass reads them from memory.
template <bool IN_LDS>
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    int* __restrict__ out, const float* __restrict__ logits, int ld, int vocab,
    const float* __restrict__ temperature, const int* __restrict__ top_k, const float* __restrict__ top_p,
    const float* __restrict__ uniform) {
    constexpr int NWAVES = SAMPLE_THREADS / LLMS_WAVE;
    __shared__ float fl[NWAVES];
    __shared__ int il[NWAVES];
    __shared__ int found;
    __shared__ int n_survivors;
    __shared__ u64 sel[3];
    __shared__ u64 digit_sum[256];
    __shared__ __align__(16) u64 hist[HIST_BYTES / 8];
    __shared__ float held[IN_LDS ? LDS_ROW_MAX + SAMPLE_THREADS : 1];
    __shared__ uint32_t survivor_key[IN_LDS ? SURVIVORS_MAX : 1], survivor_mass[IN_LDS ? SURVIVORS_MAX : 1];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int lane = tid % LLMS_WAVE, wave = tid / LLMS_WAVE;
    const float* row = logits + (size_t)r * ld;
    // (all of the row's options at once: each is a trip to memory)
    const float T = temperature ? temperature[r] : 0.f;
    const int k = top_k ? top_k[r] : 0;
    const float p = top_p ? top_p[r] : 1.f;
    const float u = T > 0.f ? uniform[r] : 0.f;
    const int per = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int stride = per | 1;
    float* mine = held + (IN_LDS ? tid * stride : 0);
    if (!(T > 0.f)) {  // greedy: one pass, straight from memory
        auto index = [&](int j) -> int { return tid + j * SAMPLE_THREADS; };
        float top;
        int amax;
        if (IN_LDS) {  // (all of a thread's loads in flight together)
            float v[LDS_ROW_MAX / SAMPLE_THREADS];
#pragma unroll
            for (int j = 0; j < LDS_ROW_MAX / SAMPLE_THREADS; ++j) v[j] = row[min(index(j), vocab - 1)];
            auto value = [&](int j) -> float { return v[j]; };
            amax = block_argmax<LDS_ROW_MAX / SAMPLE_THREADS>(value, index, LDS_ROW_MAX / SAMPLE_THREADS, vocab, fl, il, &top);
        } else {
            auto value = [&](int j) -> float { return row[min(index(j), vocab - 1)]; };
            amax = block_argmax<8>(value, index, per, vocab, fl, il, &top);
        }
        if (tid == 0) out[r] = amax;
        return;
    }
    if (IN_LDS) {
        // coalesced reads; logit i goes to its owner i / per, place i % per (kept up by additions)
        int owner = tid / per, place = tid % per;
        const int owner_step = SAMPLE_THREADS / per, place_step = SAMPLE_THREADS % per;
#pragma unroll 8
        for (int j = 0; j < per; ++j) {
            const int i = tid + j * SAMPLE_THREADS;
            held[owner * stride + place] = i < vocab ? row[i] : -INFINITY;
            owner += owner_step;
            place += place_step;
            if (place >= per) {
                place -= per;
                ++owner;
            }
        }
    }
    reinterpret_cast<uint4*>(hist)[tid] = make_uint4(0u, 0u, 0u, 0u);
    if (tid == 0) {
        found = 0;
        n_survivors = 0;
    }
    __syncthreads();
    auto index = [&](int j) -> int { return IN_LDS ? tid * per + j : tid + j * SAMPLE_THREADS; };
    auto in_row = [&](int j) -> bool { return index(j) < vocab; };
    auto raw = [&](int j) -> float { return IN_LDS ? mine[j] : row[min(index(j), vocab - 1)]; };
    float zmax_raw;
    const int amax = block_argmax<8>(raw, index, per, vocab, fl, il, &zmax_raw);
    const float inv_t = 1.f / T;
    const float zmax = zmax_raw * inv_t;
    if (IN_LDS) {
#pragma unroll 8
        for (int j = 0; j < per; ++j)
            if (in_row(j)) mine[j] *= inv_t;  // (from here on the row holds z)
    }
    auto z_of = [&](int j) -> float { return IN_LDS ? mine[j] : raw(j) * inv_t; };
    auto key_of = [&](int j) -> uint32_t { return order_key(z_of(j)); };
    // exp(z - zmax) by the hardware's 2^x (a multiply and one instruction; the library's exponential is fifteen, and
    // every pass below pays them for each of its elements)
    auto weight_of = [&](int j) -> float {
        return in_row(j) ? __builtin_amdgcn_exp2f((z_of(j) - zmax) * 1.44269504088896341f) : 0.f;
    };
    // threshold in key order: a token survives iff order_key(z) >= thr.  Both filters find their threshold by
    // digits of 8 bits, four passes each over a 256-bin histogram in LDS (a bit at a time it was 32 and 33 passes
    // with a sum over the workgroup in each).
    uint32_t thr = 0;
    if (k > 0 && k < vocab) {
        uint32_t prefix = 0;
        u64 above = 0, bound = (u64)k - 1;  // at least k keys at or above the threshold
        for (int shift = 24; shift >= 0; shift -= 8) {
            const uint32_t decided = shift == 24 ? 0u : ~0u << (shift + 8);
#pragma unroll 4
            for (int j = 0; j < per; ++j) {
                const uint32_t key = key_of(j);
                if (in_row(j) && (key & decided) == prefix) hist_add<uint32_t>(hist, (key >> shift) & 255u, 1u);
            }
            int digit;
            pick_digit<uint32_t>(hist, digit_sum, above, &bound, -1.f, sel, &digit, &above);
            prefix |= (uint32_t)digit << shift;
        }
        thr = prefix;  // key of the k-th largest
    }
    if (p < 1.f) {
        // masses in fixed point (2^-31 of the largest weight), so that their sums do not depend on an order
        auto mass_of = [&](int j) -> uint32_t { return (uint32_t)(weight_of(j) * 2147483648.f); };
        // what top-k left, when that is little, is gathered first: a thread then has one key for each pass, not `per`
        bool gathered = false;
        if (IN_LDS && thr != 0) {
#pragma unroll 4
            for (int j = 0; j < per; ++j) {
                const uint32_t key = key_of(j);
                if (in_row(j) && key >= thr) {
                    const int at = atomicAdd(&n_survivors, 1);
                    if (at < SURVIVORS_MAX) {
                        survivor_key[at] = key;
                        survivor_mass[at] = mass_of(j);
                    }
                }
            }
            __syncthreads();
            gathered = n_survivors <= SURVIVORS_MAX;
        }
        // the largest t with mass{key >= t} > limit = p * mass{all}: the survivors are the keys >= t (the mass above
        // each of them does not exceed the limit; the largest key always survives)
        uint32_t prefix = 0;
        u64 above = 0, limit = 0;
        for (int shift = 24; shift >= 0; shift -= 8) {
            const uint32_t decided = shift == 24 ? 0u : ~0u << (shift + 8);
            if (gathered) {
                if (tid < n_survivors) {
                    const uint32_t key = survivor_key[tid], mass = survivor_mass[tid];
                    if (mass && (key & decided) == prefix) hist_add<u64>(hist, (key >> shift) & 255u, (u64)mass);
                }
            } else {
#pragma unroll 4
                for (int j = 0; j < per; ++j) {
                    const uint32_t key = key_of(j);
                    if (key >= thr && (key & decided) == prefix) {
                        const uint32_t mass = mass_of(j);
                        if (mass) hist_add<u64>(hist, (key >> shift) & 255u, (u64)mass);
                    }
                }
            }
            int digit;
            pick_digit<u64>(hist, digit_sum, above, &limit, shift == 24 ? p : -1.f, sel, &digit, &above);
            prefix |= (uint32_t)digit << shift;
        }
        if (prefix > thr) thr = prefix;
    }
    // the first index, in the row's order, whose running sum of surviving weights passes u * (their sum)
    auto weight = [&](int j, bool& kept) -> float {
        kept = in_row(j) && key_of(j) >= thr;
        return kept ? weight_of(j) : 0.f;
    };
    auto wave_scan = [&](float v) -> float {  // inclusive, in lane order
#pragma unroll
        for (int o = 1; o < LLMS_WAVE; o <<= 1) {
            const float t = __shfl_up(v, o, LLMS_WAVE);
            if (lane >= o) v += t;
        }
        return v;
    };
    int last_kept = -1;
    bool missed;
    if (IN_LDS) {
        // a thread's logits are consecutive: its sum, a scan over the threads, and the one thread whose stretch
        // of the running sum holds the target walks its own logits.  A stretch's ends are the same expression in
        // the thread and in its neighbour, so the stretches leave no gap.
        float own = 0.f;
#pragma unroll 4
        for (int j = 0; j < per; ++j) {
            bool kept;
            own += weight(j, kept);
            if (kept) last_kept = index(j);
        }
        const float inclusive = wave_scan(own);
        float before_in_wave = __shfl_up(inclusive, 1, LLMS_WAVE);
        if (lane == 0) before_in_wave = 0.f;
        __syncthreads();  // (a slow thread may still be reading the argmax's fl)
        if (lane == LLMS_WAVE - 1) fl[wave] = inclusive;
        __syncthreads();
        float total = 0.f, wave_begin = 0.f;
        for (int w = 0; w < NWAVES; ++w) {
            if (w == wave) wave_begin = total;
            total += fl[w];
        }
        const float target = u * total;
        const float lower = lane == 0 ? wave_begin : wave_begin + before_in_wave, upper = wave_begin + inclusive;
        if (lower <= target && target < upper) {  // (one thread at most)
            float running = lower;
            int choice = last_kept;  // (if rounding keeps the walk below the target)
            for (int j = 0; j < per; ++j) {
                bool kept;
                running += weight(j, kept);
                if (kept && running > target) {
                    choice = index(j);
                    break;
                }
            }
            out[r] = choice;
            found = 1;
        }
        __syncthreads();
        missed = found == 0;
    } else {
        float e = 0.f;
#pragma unroll 4
        for (int j = 0; j < per; ++j) {
            bool kept;
            e += weight(j, kept);
        }
        const float target = u * block_sum(e, fl);
        if (tid == 0) found = 0x7fffffff;
        __syncthreads();
        float running = 0.f;
        for (int j = 0; j < per; ++j) {
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
                last_kept = index(j);
                if (before + scan > target) atomicMin(&found, index(j));
            }
            running += tile_total;
            __syncthreads();
            if (found != 0x7fffffff) break;
        }
        missed = found == 0x7fffffff;
        if (!missed && tid == 0) out[r] = found;
    }
    if (missed) {
        // rounding left the running sum at or below the target: take the last surviving index
        int lk = last_kept;
#pragma unroll
        for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) lk = max(lk, __shfl_xor(lk, o, LLMS_WAVE));
        __syncthreads();
        if (lane == 0) il[wave] = lk;
        __syncthreads();
        lk = il[0];
        for (int w = 1; w < NWAVES; ++w) lk = max(lk, il[w]);
        if (tid == 0) out[r] = lk >= 0 ? lk : amax;
    }
}

extern "C" {

// temperature, top_k, top_p may be null (greedy / off / off); uniform is needed when any
// temperature is positive.
int llms_sample_rows(int* out, const float* logits, int ld, int n_rows, int vocab, const float* temperature,
                     const int* top_k, const float* top_p, const float* uniform, hipStream_t stream) {
    LLMS_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "sample_rows: bad sizes");
    LLMS_REQUIRE(temperature == nullptr || uniform != nullptr, "sample_rows: temperature needs uniform numbers");
    if (vocab <= LDS_ROW_MAX)
        sample_rows_kernel<true><<<n_rows, SAMPLE_THREADS, 0, stream>>>(out, logits, ld, vocab, temperature, top_k, top_p, uniform);
    else
        sample_rows_kernel<false><<<n_rows, SAMPLE_THREADS, 0, stream>>>(out, logits, ld, vocab, temperature, top_k, top_p, uniform);
    LLMS_LAUNCH_CHECK();
}

}  // extern "C"
