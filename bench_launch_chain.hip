// Latency probes behind the decode step's "launch chain" figures: what a boundary between two dependent launches
// costs, whether replaying the chain from a HIP graph changes it, what a grid-wide barrier among co-resident
// workgroups would cost instead, and what warm weights buy a small GEMV-sized read.  Stand-alone (no library):
//   hipcc --offload-arch=gfx950 -O2 -Xclang -target-feature -Xclang -packed-fp32-ops -o bench_launch_chain bench_launch_chain.hip && ./bench_launch_chain
// Every kernel here ends by itself: the barrier's wait is a bounded spin that sets a flag and leaves.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <vector>

#define CK(x)                                                          \
    do {                                                               \
        hipError_t e_ = (x);                                           \
        if (e_ != hipSuccess) {                                        \
            printf("%s: %s\n", #x, hipGetErrorString(e_));             \
            return 1;                                                  \
        }                                                              \
    } while (0)

namespace {

constexpr uint32_t kSpinMax = 1u << 20;

__global__ void tiny_kernel(float *p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = p[i] * 1.0001f + 1.0f;
}

// mode 0: barrier only.  mode 1: each workgroup writes 64 floats before the barrier and reads all G * 64 after it
// (what a persistent decode step would have to do at every former launch boundary).
__global__ __launch_bounds__(256) void grid_barrier_kernel(uint32_t *counter, uint32_t *timeout_flag, float *buf0, float *buf1,
                                                           float *out, uint32_t n_iter, int mode) {
    const uint32_t G = gridDim.x, tid = threadIdx.x, wg = blockIdx.x;
    float acc = 0.0f;
    bool dead = false;
    for (uint32_t it = 0; it < n_iter && !dead; it++) {
        float *buf = (it & 1) ? buf1 : buf0;
        if (mode == 1 && tid < 64) buf[wg * 64 + tid] = float(it + wg) + acc * 1e-30f;
        __syncthreads();
        if (tid == 0) {
            __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t want = (it + 1) * G;
            uint32_t spins = 0;
            while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < want) {
                if (++spins > kSpinMax) {
                    *timeout_flag = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __syncthreads();
        if (*reinterpret_cast<volatile uint32_t *>(timeout_flag)) dead = true;
        if (mode == 1) {
            __atomic_thread_fence(__ATOMIC_ACQUIRE);
            float s = 0.0f;
            for (uint32_t i = tid; i < G * 64; i += 256) s += __builtin_nontemporal_load(buf + i);
            acc += s;
        }
    }
    if (tid == 0) out[wg] = acc;
}

// a read of `bytes` bytes spread over the launch, 16 bytes a lane: the memory side of a small GEMV
__global__ __launch_bounds__(256) void read_kernel(const uint4 *src, size_t n16, uint32_t *sink) {
    uint32_t s = 0;
    for (size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x; i < n16; i += size_t(gridDim.x) * blockDim.x) {
        const uint4 v = src[i];
        s ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (s == 0x12345678u) *sink = s;
}

}  // namespace

int main() {
    hipStream_t st;
    CK(hipStreamCreate(&st));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    float ms = 0.0f;

    // ---- 1. a chain of dependent tiny kernels, launched one by one and replayed from a HIP graph
    {
        float *p;
        CK(hipMalloc(&p, 1 << 20));
        CK(hipMemset(p, 0, 1 << 20));
        const int N = 144, REP = 200;  // 144 launches: one token-step of the decode loop
        for (int g : {1, 16, 256}) {
            for (int i = 0; i < N; i++) hipLaunchKernelGGL(tiny_kernel, dim3(g), dim3(256), 0, st, p, 65536);
            CK(hipStreamSynchronize(st));
            CK(hipEventRecord(e0, st));
            for (int r = 0; r < REP; r++)
                for (int i = 0; i < N; i++) hipLaunchKernelGGL(tiny_kernel, dim3(g), dim3(256), 0, st, p, 65536);
            CK(hipEventRecord(e1, st));
            CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf("chain of %d dependent kernels, %3d workgroups each: stream launches %.2f us per kernel", N, g, ms * 1e3 / (N * REP));
            hipGraph_t graph;
            hipGraphExec_t exec;
            CK(hipStreamBeginCapture(st, hipStreamCaptureModeGlobal));
            for (int i = 0; i < N; i++) hipLaunchKernelGGL(tiny_kernel, dim3(g), dim3(256), 0, st, p, 65536);
            CK(hipStreamEndCapture(st, &graph));
            CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
            for (int r = 0; r < 3; r++) CK(hipGraphLaunch(exec, st));
            CK(hipStreamSynchronize(st));
            CK(hipEventRecord(e0, st));
            for (int r = 0; r < REP; r++) CK(hipGraphLaunch(exec, st));
            CK(hipEventRecord(e1, st));
            CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf(", graph replay %.2f us per kernel\n", ms * 1e3 / (N * REP));
            CK(hipGraphExecDestroy(exec));
            CK(hipGraphDestroy(graph));
        }
        CK(hipFree(p));
    }

    // ---- 1b. the same chain with kernels that do a small GEMV's worth of reading (3 MB each, 64 buffers in turn)
    {
        const size_t bytes = 3u << 20, n16 = bytes / 16;
        const int N = 144, REP = 100;
        uint4 *pool;
        uint32_t *sink;
        CK(hipMalloc(&pool, bytes * 64));
        CK(hipMemset(pool, 1, bytes * 64));
        CK(hipMalloc(&sink, 4));
        for (int wgs : {64, 256, 1024}) {
            auto enqueue = [&]() { for (int i = 0; i < N; i++) hipLaunchKernelGGL(read_kernel, dim3(wgs), dim3(256), 0, st, pool + size_t(i % 64) * n16, n16, sink); };
            enqueue(); CK(hipStreamSynchronize(st));
            CK(hipEventRecord(e0, st)); for (int r = 0; r < REP; r++) enqueue(); CK(hipEventRecord(e1, st)); CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf("chain of %d 3 MB reads, %4d workgroups each: stream launches %.2f us per kernel", N, wgs, ms * 1e3 / (N * REP));
            hipGraph_t graph; hipGraphExec_t exec;
            CK(hipStreamBeginCapture(st, hipStreamCaptureModeGlobal)); enqueue(); CK(hipStreamEndCapture(st, &graph));
            CK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
            for (int r = 0; r < 3; r++) CK(hipGraphLaunch(exec, st));
            CK(hipStreamSynchronize(st));
            CK(hipEventRecord(e0, st)); for (int r = 0; r < REP; r++) CK(hipGraphLaunch(exec, st)); CK(hipEventRecord(e1, st)); CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf(", graph replay %.2f us per kernel\n", ms * 1e3 / (N * REP));
            CK(hipGraphExecDestroy(exec)); CK(hipGraphDestroy(graph));
        }
        CK(hipFree(pool)); CK(hipFree(sink));
    }

    // ---- 2. a grid-wide barrier among co-resident workgroups (at most one per compute unit)
    {
        uint32_t *counter, *flag;
        float *b0, *b1, *out;
        CK(hipMalloc(&counter, 4));
        CK(hipMalloc(&flag, 4));
        CK(hipMalloc(&b0, 256 * 64 * 4));
        CK(hipMalloc(&b1, 256 * 64 * 4));
        CK(hipMalloc(&out, 256 * 4));
        const uint32_t n_iter = 2000;
        for (int mode = 0; mode < 2; mode++)
            for (uint32_t G : {32u, 64u, 128u, 256u}) {
                float best = 1e9f;
                for (int rep = 0; rep < 3; rep++) {
                    CK(hipMemset(counter, 0, 4));
                    CK(hipMemset(flag, 0, 4));
                    CK(hipDeviceSynchronize());
                    CK(hipEventRecord(e0, 0));
                    hipLaunchKernelGGL(grid_barrier_kernel, dim3(G), dim3(256), 0, 0, counter, flag, b0, b1, out, n_iter, mode);
                    CK(hipEventRecord(e1, 0));
                    CK(hipEventSynchronize(e1));
                    CK(hipEventElapsedTime(&ms, e0, e1));
                    if (ms < best) best = ms;
                    uint32_t f;
                    CK(hipMemcpy(&f, flag, 4, hipMemcpyDeviceToHost));
                    if (f) {
                        printf("grid barrier, %u workgroups: spin limit reached\n", G);
                        return 2;
                    }
                }
                std::vector<float> h(G);
                CK(hipMemcpy(h.data(), out, G * 4, hipMemcpyDeviceToHost));
                double want = 0;  // thread 0 of workgroup 0 sums the first float of workgroups 0, 4, 8, ... every iteration
                for (uint32_t it = 0; it < n_iter; it++)
                    for (uint32_t w = 0; w < G; w += 4) want += double(it + w);
                printf("grid barrier%s, %3u workgroups: %.2f us per barrier", mode ? " + 16 KB exchanged" : "", G, best * 1000.0f / n_iter);
                if (mode == 1) printf("  (data %s)", std::fabs(h[0] - want) / want < 1e-4 ? "ok" : "WRONG");
                printf("\n");
            }
        CK(hipFree(counter));
        CK(hipFree(flag));
        CK(hipFree(b0));
        CK(hipFree(b1));
        CK(hipFree(out));
    }

    // ---- 3. warm against cold weights: the same 3 MB read again and again, or 64 different ones in turn
    {
        const size_t bytes = 3u << 20, n16 = bytes / 16;
        const int n_buf = 64, REP = 2000;
        uint4 *pool;
        uint32_t *sink;
        CK(hipMalloc(&pool, bytes * n_buf));
        CK(hipMemset(pool, 1, bytes * n_buf));
        CK(hipMalloc(&sink, 4));
        for (int cold = 0; cold < 2; cold++) {
            for (int i = 0; i < 64; i++) hipLaunchKernelGGL(read_kernel, dim3(256), dim3(256), 0, st, pool, n16, sink);
            CK(hipStreamSynchronize(st));
            CK(hipEventRecord(e0, st));
            for (int i = 0; i < REP; i++)
                hipLaunchKernelGGL(read_kernel, dim3(256), dim3(256), 0, st, pool + (cold ? size_t(i % n_buf) * n16 : 0), n16, sink);
            CK(hipEventRecord(e1, st));
            CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf("3 MB read per launch, 256 workgroups, %s: %.2f us per launch\n",
                   cold ? "64 buffers in turn (192 MB: past the L2, inside the 256 MB last-level cache)" : "the same buffer every time", ms * 1e3 / REP);
        }
        CK(hipFree(pool));
        CK(hipFree(sink));
    }
    return 0;
}
