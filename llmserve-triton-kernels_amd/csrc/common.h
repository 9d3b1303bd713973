// Shared helpers of the gfx950 kernels: element types, conversions, wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define LLMS_WAVE 64

// Error codes returned by the extern "C" launchers (0 = launched).
#define LLMS_OK 0
#define LLMS_ERR_ARG 1     // an argument the kernel cannot take (message printed to stderr)
#define LLMS_ERR_LAUNCH 2  // the HIP runtime refused the launch

#define LLMS_REQUIRE(cond, msg)                                        \
    do {                                                               \
        if (!(cond)) {                                                 \
            fprintf(stderr, "llmserve kernel argument error: %s\n", msg); \
            return LLMS_ERR_ARG;                                       \
        }                                                              \
    } while (0)

#define LLMS_LAUNCH_CHECK()                                            \
    do {                                                               \
        hipError_t e_ = hipGetLastError();                             \
        if (e_ != hipSuccess) {                                        \
            fprintf(stderr, "llmserve kernel launch failed: %s\n", hipGetErrorString(e_)); \
            return LLMS_ERR_LAUNCH;                                    \
        }                                                              \
        return LLMS_OK;                                                \
    } while (0)

#define LLMS_HIP_CHECK(call)                                           \
    do {                                                               \
        hipError_t e_ = (call);                                        \
        if (e_ != hipSuccess) {                                        \
            fprintf(stderr, "llmserve kernel set-up failed: %s\n", hipGetErrorString(e_)); \
            return LLMS_ERR_LAUNCH;                                    \
        }                                                              \
    } while (0)

// bfloat16 is carried as its 16 raw bits.
struct bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// Round to nearest even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

// Two floats rounded to bfloat16 and packed, `lo` in the low half: one instruction.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    const bf16x2_t v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return bf16_bits_to_f32(v.bits); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16 from_f32<bf16>(float v) {
    bf16 r;
    r.bits = f32_to_bf16_bits(v);
    return r;
}

// Value of v after one rounding to T (what a store followed by a load would give).
template <typename T>
__device__ __forceinline__ float round_to(float v) { return to_f32(from_f32<T>(v)); }

// Sine and cosine of position * frequency, and (a, b) turned by that angle, with the same bits in every kernel
// that rotates (the rotation kernel, and the products that rotate in their epilogue): a result that falls next to a
// rounding boundary of bfloat16 would otherwise differ between kernels that must agree.  The sine and cosine are
// never inlined (inlined, the compiler specialises and schedules them differently from kernel to kernel; the result
// comes back by value, since an address of a caller's variable would put it in private memory); the rotation is
// inlined, which keeps a call's register saves out of the epilogues, with every product and sum rounded on its own
// (no contraction to multiply-adds, which the compiler would otherwise choose by context).
__device__ __noinline__ float2 rotary_angle(float position, float frequency) {  // (sine, cosine)
#pragma clang fp contract(off)
    float sine, cosine;
    sincosf(position * frequency, &sine, &cosine);
    return make_float2(sine, cosine);
}
__device__ __forceinline__ float2 rotate_pair(float a, float b, float cs, float sn) {
#pragma clang fp contract(off)
    const float ac = a * cs, bs = b * sn, bc = b * cs, as = a * sn;
    return make_float2(ac - bs, bc + as);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LLMS_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = LLMS_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, LLMS_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads, same value returned to every thread.  The order
// of additions depends only on the block size, never on the data or the grid.
__device__ __forceinline__ float block_sum(float v, float* lds /* >= 16 floats */) {
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    const int nwaves = (blockDim.x + LLMS_WAVE - 1) / LLMS_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    // (all 16 places are read at once and those of waves that do not exist left out: a loop up to nwaves would
    // wait for LDS once per wave)
    float part[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) part[i] = lds[i];
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) t += i < nwaves ? part[i] : 0.f;
    return t;
}

__device__ __forceinline__ float block_max(float v, float* lds) {
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    const int nwaves = (blockDim.x + LLMS_WAVE - 1) / LLMS_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float part[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) part[i] = lds[i];
    float t = part[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) t = fmaxf(t, i < nwaves ? part[i] : part[0]);
    return t;
}
