// Measurements that decide how a decode step is laid out, not part of any step: what a kernel boundary costs in a
// captured chain of dependent launches, and what a barrier over the whole grid costs inside one kernel (an atomic
// counter and a bounded spin), with and without the release/acquire fences that make one workgroup's stores visible
// to workgroups on other XCDs.  Every spin has a limit, so a mistake gives a count of failures, never a hang.
// What it costs workgroups to hand data to one another inside a kernel without waiting for each other (the last
// to arrive does the common work).  And what memory gives a kernel that only reads: a long stream, and a stream as short as one weight matrix of a
// decode step, which is the floor for any product that must read that matrix in a launch of its own.
#include "common.h"

#include <algorithm>

typedef __attribute__((ext_vector_type(4))) unsigned int probe_u32x4;

// Reads a matrix of `rows` rows of 4,096 bytes (a bfloat16 weight with K = 2,048) and keeps nothing.  A wave takes
// tiles of 16 rows, as the product kernels do.  PATTERN 0: an instruction covers 1 KB of one row; 1: 64 bytes of each
// of the 16 rows (the matrix instruction's operand layout read straight from memory); 2: 256 bytes of 4 rows.
template <int PATTERN>
__global__ __launch_bounds__(256) void probe_read_kernel(const char* __restrict__ buf, int rows, unsigned* sink) {
    constexpr int ROW = 4096;
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    probe_u32x4 acc = {0, 0, 0, 0};
    const int tiles = rows / 16, waves = gridDim.x * 4;
    for (int t = blockIdx.x * 4 + wave; t < tiles; t += waves) {
        const char* base = buf + (size_t)t * 16 * ROW;
#pragma unroll 16
        for (int i = 0; i < 16 * ROW / 1024; ++i) {
            size_t off;
            if (PATTERN == 0) off = (size_t)i * 1024 + lane * 16;
            else if (PATTERN == 1) off = (size_t)(lane % 16) * ROW + i * 64 + (lane / 16) * 16;
            else off = (size_t)((i / 16) * 4 + lane / 16) * ROW + (i % 16) * 256 + (lane % 16) * 16;
            acc ^= __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4*>(base + off));
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = acc.x;  // (keeps the loads; practically never true)
}

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

// Reads `bytes` (a multiple of 4 KB) and keeps nothing: a wave takes pieces of 4 KB, four loads in flight.
__global__ __launch_bounds__(256) void probe_read_flat_kernel(const char* __restrict__ buf, size_t bytes, unsigned* sink) {
    const int lane = threadIdx.x % LLMS_WAVE, wave = threadIdx.x / LLMS_WAVE;
    probe_u32x4 acc = {0, 0, 0, 0};
    const size_t pieces = bytes / 4096, waves = (size_t)gridDim.x * 4;
    for (size_t p = (size_t)blockIdx.x * 4 + wave; p < pieces; p += waves) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            acc ^= __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4*>(buf + p * 4096 + i * 1024 + lane * 16));
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = acc.x;
}

// What it costs workgroups to hand data to one another inside a kernel, the way the decode attention adds its
// shares up: groups of S workgroups; each writes 512 floats, is counted at its group's counter, and the last to be
// counted reads the 512 floats of every member and checks them (a stale value is counted), then sets the counter
// back to zero.  MODE 0: the stores alone.  MODE 1: stores and loads are relaxed atomic accesses at agent scope
// (written through, read past the L2 of the reader's XCD), ordered by a wait for the stores, no fence.  MODE 2:
// plain stores and loads with __threadfence() on both sides, the textbook way.  Nobody waits for anybody.
template <int MODE>
__global__ __launch_bounds__(256) void probe_handover_kernel(float* data, unsigned* counters, unsigned* stale, int S, int round,
                                                             float* out) {
    __shared__ unsigned last;
    const int wg = blockIdx.x, group = wg / S;
    float* mine = data + (size_t)wg * 512;
    const float v = (float)(round * 1000 + wg);
    for (int i = threadIdx.x; i < 512; i += 256) {
        if (MODE == 2) mine[i] = v + i;
        else __hip_atomic_store(mine + i, v + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (MODE == 0) return;
    if (MODE == 2) __threadfence();
    else __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned before = __hip_atomic_fetch_add(counters + group, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = before + 1 == (unsigned)S;
        if (last) __hip_atomic_store(counters + group, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last) return;
    if (MODE == 2) __threadfence();
    float got[8][2];  // (all loads asked for before the first is looked at; S <= 8)
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const float* theirs = data + (size_t)(group * S + min(s, S - 1)) * 512;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            got[s][j] = MODE == 2 ? theirs[threadIdx.x + 256 * j]
                                  : __hip_atomic_load(theirs + threadIdx.x + 256 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float acc = 0.f;
    unsigned bad = 0;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const float want = (float)(round * 1000 + group * S + min(s, S - 1));
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (got[s][j] != want + (float)(threadIdx.x + 256 * j)) ++bad;
            acc += got[s][j];
        }
    }
    if (bad) atomicAdd(stale, bad);
    out[(size_t)group * 256 + threadIdx.x] = acc;
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

// results[3 * i + m]: microseconds per launch of probe_handover_kernel<m> (m = 0 stores only, 1 atomic accesses
// without a fence, 2 fences) in a captured chain of 100 launches, for the i-th of the cases (workgroups, group
// size) = (64, 2), (64, 8), (256, 4), (1024, 4); results[12]: stale values seen by any of them (must be 0).
// `scratch`: 1,024 * 768 floats and 8,192 further bytes of device memory.  The caller has synchronized the device.
int llms_probe_handover(float* results, void* scratch) {
    hipStream_t stream;
    PROBE_CHECK(hipStreamCreate(&stream));
    float* data = static_cast<float*>(scratch);
    float* out = data + 1024 * 512;
    unsigned* counters = reinterpret_cast<unsigned*>(data + 1024 * 768);
    unsigned* stale = counters + 1024;
    PROBE_CHECK(hipMemsetAsync(counters, 0, 8192, stream));
    hipEvent_t a, b;
    PROBE_CHECK(hipEventCreate(&a));
    PROBE_CHECK(hipEventCreate(&b));
    const int cases[4][2] = {{64, 2}, {64, 8}, {256, 4}, {1024, 4}};
    float ms = 0.f;
    for (int i = 0; i < 4; ++i) {
        for (int mode = 0; mode < 3; ++mode) {
            const int grid = cases[i][0], S = cases[i][1];
            hipGraph_t graph;
            hipGraphExec_t exec;
            PROBE_CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
            for (int r = 0; r < 100; ++r) {
                if (mode == 0) probe_handover_kernel<0><<<grid, 256, 0, stream>>>(data, counters, stale, S, r + 1, out);
                else if (mode == 1) probe_handover_kernel<1><<<grid, 256, 0, stream>>>(data, counters, stale, S, r + 1, out);
                else probe_handover_kernel<2><<<grid, 256, 0, stream>>>(data, counters, stale, S, r + 1, out);
            }
            PROBE_CHECK(hipStreamEndCapture(stream, &graph));
            PROBE_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
            PROBE_CHECK(hipGraphLaunch(exec, stream));
            PROBE_CHECK(hipStreamSynchronize(stream));
            PROBE_CHECK(hipEventRecord(a, stream));
            for (int k = 0; k < 5; ++k) PROBE_CHECK(hipGraphLaunch(exec, stream));
            PROBE_CHECK(hipEventRecord(b, stream));
            PROBE_CHECK(hipStreamSynchronize(stream));
            PROBE_CHECK(hipEventElapsedTime(&ms, a, b));
            results[3 * i + mode] = ms * 1e3f / 500.f;
            PROBE_CHECK(hipGraphExecDestroy(exec));
            PROBE_CHECK(hipGraphDestroy(graph));
        }
    }
    unsigned seen = 0;
    PROBE_CHECK(hipMemcpy(&seen, stale, sizeof(seen), hipMemcpyDeviceToHost));
    results[12] = (float)seen;
    PROBE_CHECK(hipEventDestroy(a));
    PROBE_CHECK(hipEventDestroy(b));
    PROBE_CHECK(hipStreamDestroy(stream));
    return LLMS_OK;
}

// results[0..2]: GB/s of a kernel that reads all of `buf` once (`bytes` >= 1 GiB, so that nothing comes from the
// 256 MB memory-side cache), for the three patterns of probe_read_kernel.  results[3 + i]: microseconds per launch in
// a captured chain of 16 launches that each read the next piece of piece_bytes[i] bytes (probe_read_flat_kernel, a
// wave for every 4 KB up to 2,048 workgroups), i < n_pieces <= 8: what a kernel that must read that much costs at the
// least.  `sink`: 4 bytes of
// device memory.  The caller has synchronized the device; the probe runs on a stream of its own.
int llms_probe_stream(float* results, const void* buf, size_t bytes, const size_t* piece_bytes, int n_pieces, void* sink) {
    constexpr size_t TILE = 16 * 4096;
    LLMS_REQUIRE(buf != nullptr && bytes >= ((size_t)1 << 30) && n_pieces >= 0 && n_pieces <= 8, "probe_stream: bad arguments");
    for (int i = 0; i < n_pieces; ++i)
        LLMS_REQUIRE(piece_bytes[i] >= TILE && piece_bytes[i] * 16 <= bytes, "probe_stream: 16 pieces must fit the buffer");
    hipStream_t stream;
    PROBE_CHECK(hipStreamCreate(&stream));
    hipEvent_t a, b;
    PROBE_CHECK(hipEventCreate(&a));
    PROBE_CHECK(hipEventCreate(&b));
    const char* base = static_cast<const char*>(buf);
    unsigned* out = static_cast<unsigned*>(sink);
    float ms = 0.f;
    const int rows = (int)(bytes / TILE) * 16;
    for (int p = 0; p < 3; ++p) {
        for (int k = 0; k < 3; ++k) {  // (the last of three is timed)
            PROBE_CHECK(hipEventRecord(a, stream));
            if (p == 0) probe_read_kernel<0><<<2048, 256, 0, stream>>>(base, rows, out);
            else if (p == 1) probe_read_kernel<1><<<2048, 256, 0, stream>>>(base, rows, out);
            else probe_read_kernel<2><<<2048, 256, 0, stream>>>(base, rows, out);
            PROBE_CHECK(hipEventRecord(b, stream));
            PROBE_CHECK(hipStreamSynchronize(stream));
        }
        PROBE_CHECK(hipEventElapsedTime(&ms, a, b));
        results[p] = (float)((double)rows * 4096 / (ms * 1e-3) / 1e9);
    }
    for (int i = 0; i < n_pieces; ++i) {
        const size_t piece = piece_bytes[i] / 4096 * 4096;
        const int grid = (int)std::min<size_t>(2048, (piece / 4096 + 3) / 4);
        hipGraph_t graph;
        hipGraphExec_t exec;
        PROBE_CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        for (int k = 0; k < 16; ++k)
            probe_read_flat_kernel<<<grid, 256, 0, stream>>>(base + (size_t)k * piece, piece, out);
        PROBE_CHECK(hipStreamEndCapture(stream, &graph));
        PROBE_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        PROBE_CHECK(hipGraphLaunch(exec, stream));
        PROBE_CHECK(hipStreamSynchronize(stream));
        PROBE_CHECK(hipEventRecord(a, stream));
        for (int k = 0; k < 5; ++k) PROBE_CHECK(hipGraphLaunch(exec, stream));
        PROBE_CHECK(hipEventRecord(b, stream));
        PROBE_CHECK(hipStreamSynchronize(stream));
        PROBE_CHECK(hipEventElapsedTime(&ms, a, b));
        results[3 + i] = ms * 1e3f / 80.f;
        PROBE_CHECK(hipGraphExecDestroy(exec));
        PROBE_CHECK(hipGraphDestroy(graph));
    }
    PROBE_CHECK(hipEventDestroy(a));
    PROBE_CHECK(hipEventDestroy(b));
    PROBE_CHECK(hipStreamDestroy(stream));
    return LLMS_OK;
}

}  // extern "C"
