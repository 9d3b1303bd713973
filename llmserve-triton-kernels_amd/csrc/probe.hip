// Measurements that decide how a decode step is laid out, not part of any step: what a kernel boundary costs in a
// captured chain of dependent launches, and what a barrier over the whole grid costs inside one kernel (an atomic
// counter and a bounded spin), with and without the release/acquire fences that make one workgroup's stores visible
// to workgroups on other XCDs.  Every spin has a limit, so a mistake gives a count of failures, never a hang.
#include "common.h"

__global__ void probe_tiny_kernel(float* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = p[i] * 1.0001f + 1.f;
}

// `rounds` barriers in a row; before each a workgroup writes a value, after it reads the value of a workgroup far
// away.  The counter only grows: barrier r is passed when it has reached (r + 1) * gridDim.x.
template <bool FENCE>
__global__ __launch_bounds__(256) void probe_barrier_kernel(unsigned* counter, float* data, int rounds, unsigned* fails,
                                                            float* sink) {
    const unsigned G = gridDim.x;
    float acc = 0.f;
    for (int r = 0; r < rounds; ++r) {
        data[(size_t)blockIdx.x * 256 + threadIdx.x] = (float)(r + 1) + acc * 1e-9f;
        if (FENCE) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        __syncthreads();
        if (threadIdx.x == 0) {
            __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned target = (unsigned)(r + 1) * G;
            int spins = 0;
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                if (++spins > (1 << 18)) {  // give up: the failure is counted and the kernel goes on to its end
                    atomicAdd(fails, 1u);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
        if (FENCE) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const unsigned far = (blockIdx.x + G / 2 + 1) % G;
        const float v = data[(size_t)far * 256 + threadIdx.x];
        if (FENCE && v < (float)(r + 1) - 0.5f) atomicAdd(fails + 1, 1u);  // a stale value
        acc += v;
    }
    if (acc == 12345.678f) sink[0] = acc;
}

#define PROBE_CHECK(call)                                                                          \
    do {                                                                                           \
        hipError_t e_ = (call);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            fprintf(stderr, "llmserve probe: %s failed: %s\n", #call, hipGetErrorString(e_));      \
            return LLMS_ERR_LAUNCH;                                                                \
        }                                                                                          \
    } while (0)

extern "C" {

// results[0..2]: microseconds per kernel in a captured chain of 200 dependent tiny kernels of 8, 256 and 1,024
// workgroups.  results[3 + i]: microseconds per grid barrier without fences for grids of 64, 256, 512, 1,024
// workgroups; results[7 + i]: with fences, for 64, 256, 512 (-1: the grid does not fit the chip at once, so it is not
// run).  results[10]: spin limits hit, results[11]: stale reads seen (both must be 0).  `scratch`: 1,024 * 256 floats
// and 64 further bytes of device memory, which the caller provides (and may hold anything); the caller has
// synchronized the device, the probe runs on a stream of its own.
int llms_probe_sync(float* results, void* scratch) {
    hipStream_t stream;  // a stream of its own: the default stream cannot be captured
    PROBE_CHECK(hipStreamCreate(&stream));
    float* buf = static_cast<float*>(scratch);
    unsigned* counter = reinterpret_cast<unsigned*>(buf + 1024 * 256);
    unsigned* fails = counter + 4;
    float* sink = reinterpret_cast<float*>(counter + 8);
    hipEvent_t a, b;
    PROBE_CHECK(hipEventCreate(&a));
    PROBE_CHECK(hipEventCreate(&b));
    float ms = 0.f;
    const int chain_grids[3] = {8, 256, 1024};
    for (int i = 0; i < 3; ++i) {
        hipGraph_t graph;
        hipGraphExec_t exec;
        PROBE_CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        for (int k = 0; k < 200; ++k) probe_tiny_kernel<<<chain_grids[i], 256, 0, stream>>>(buf, chain_grids[i] * 256);
        PROBE_CHECK(hipStreamEndCapture(stream, &graph));
        PROBE_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        PROBE_CHECK(hipGraphLaunch(exec, stream));
        PROBE_CHECK(hipStreamSynchronize(stream));
        PROBE_CHECK(hipEventRecord(a, stream));
        for (int k = 0; k < 5; ++k) PROBE_CHECK(hipGraphLaunch(exec, stream));
        PROBE_CHECK(hipEventRecord(b, stream));
        PROBE_CHECK(hipStreamSynchronize(stream));
        PROBE_CHECK(hipEventElapsedTime(&ms, a, b));
        results[i] = ms * 1e3f / 1000.f;
        PROBE_CHECK(hipGraphExecDestroy(exec));
        PROBE_CHECK(hipGraphDestroy(graph));
    }
    int device = 0, cus = 0;
    PROBE_CHECK(hipGetDevice(&device));
    PROBE_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    unsigned total_fails[2] = {0, 0};
    const int grids[4] = {64, 256, 512, 1024};
    for (int fence = 0; fence < 2; ++fence) {
        for (int i = 0; i < (fence ? 3 : 4); ++i) {
            int per_cu = 0;
            if (fence) PROBE_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, probe_barrier_kernel<true>, 256, 0));
            else PROBE_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, probe_barrier_kernel<false>, 256, 0));
            float& out = results[3 + 4 * fence + i];
            if (grids[i] > per_cu * cus) {  // workgroups that are not resident together would wait for each other for ever
                out = -1.f;
                continue;
            }
            float t[2];
            for (int k = 0; k < 2; ++k) {
                const int rounds = k == 0 ? 10 : 110;
                PROBE_CHECK(hipMemsetAsync(counter, 0, 64, stream));
                PROBE_CHECK(hipEventRecord(a, stream));
                if (fence) probe_barrier_kernel<true><<<grids[i], 256, 0, stream>>>(counter, buf, rounds, fails, sink);
                else probe_barrier_kernel<false><<<grids[i], 256, 0, stream>>>(counter, buf, rounds, fails, sink);
                PROBE_CHECK(hipEventRecord(b, stream));
                PROBE_CHECK(hipStreamSynchronize(stream));
                PROBE_CHECK(hipEventElapsedTime(&t[k], a, b));
                unsigned f[2];
                PROBE_CHECK(hipMemcpy(f, fails, sizeof(f), hipMemcpyDeviceToHost));
                total_fails[0] += f[0];
                total_fails[1] += f[1];
            }
            out = (t[1] - t[0]) * 1e3f / 100.f;
        }
    }
    results[10] = (float)total_fails[0];
    results[11] = (float)total_fails[1];
    PROBE_CHECK(hipEventDestroy(a));
    PROBE_CHECK(hipEventDestroy(b));
    PROBE_CHECK(hipStreamDestroy(stream));
    return LLMS_OK;
}

}  // extern "C"
