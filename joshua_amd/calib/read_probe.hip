// What one launch can do at best with a weight matrix of the benchmark's size: a plain read of `bytes` (default
// 33030144, Q4_K 14336 x 4096) with 128-bit loads and nothing else, timed with HIP events over 400 launches
//   * cold: 24 copies of the buffer rotated, so every launch reads from HBM (what bench.py's timed loop does),
//   * resident: one copy read again and again (served by the 256 MB Infinity Cache; bench.py's cache_resident leg),
//   * cold + stores: the same read with one dword stored per wave, about as many stores as the GEMV has rows,
// each with 4, 8 and 16 loads in flight per thread, and an empty launch for the fixed cost.  The GEMV's own time is to
// be read against these, not against 8 TB/s: the cold figure is the floor of any single dependent launch that has
// to read the matrix once.
//     hipcc --offload-arch=gfx950 -O3 -o read_probe read_probe.hip && ./read_probe [bytes]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CHECK(x)                                                              \
    do {                                                                      \
        hipError_t e_ = (x);                                                  \
        if (e_ != hipSuccess) {                                               \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));      \
            return 1;                                                         \
        }                                                                     \
    } while (0)

template <int U, bool STORE>
__global__ __launch_bounds__(256) void read_u4(const uint4 *__restrict__ p, size_t nvec, unsigned *__restrict__ out) {
    const size_t base = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const size_t i = base + (size_t)u * 256;
        v[u] = i < nvec ? p[i] : uint4{0, 0, 0, 0};
    }
    unsigned a = 0;
#pragma unroll
    for (int u = 0; u < U; u++) a ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (STORE) {
        if ((threadIdx.x & 63) == 0) out[blockIdx.x * 4 + (threadIdx.x >> 6)] = a;
    } else if (a == 0x12345678u) {  // practically never: keeps the loads alive
        out[blockIdx.x] = a;
    }
}

__global__ void empty_kernel() {}

template <int U, bool STORE>
static float time_us(const std::vector<uint4 *> &bufs, size_t nvec, unsigned *out, int iters) {
    const int grid = (int)((nvec + 256 * U - 1) / (256 * U));
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    for (int i = 0; i < 20; i++) hipLaunchKernelGGL((read_u4<U, STORE>), dim3(grid), dim3(256), 0, 0, bufs[i % bufs.size()], nvec, out);
    hipDeviceSynchronize();
    hipEventRecord(e0);
    for (int i = 0; i < iters; i++)
        hipLaunchKernelGGL((read_u4<U, STORE>), dim3(grid), dim3(256), 0, 0, bufs[i % bufs.size()], nvec, out);
    hipEventRecord(e1);
    hipEventSynchronize(e1);
    float ms = 0.0f;
    hipEventElapsedTime(&ms, e0, e1);
    return ms / iters * 1000.0f;
}

int main(int argc, char **argv) {
    const size_t bytes = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 33030144;
    const size_t nvec = bytes / 16;
    std::vector<uint4 *> bufs(24);
    for (auto &b : bufs) {
        CHECK(hipMalloc((void **)&b, bytes));
        CHECK(hipMemset(b, 1, bytes));
    }
    unsigned *out = nullptr;
    CHECK(hipMalloc((void **)&out, 4 << 20));
    const std::vector<uint4 *> one(1, bufs[0]);
    const int iters = 400;
    std::printf("%zu bytes a launch, %d launches a figure\n", bytes, iters);
    std::printf("%-28s %10s %10s\n", "", "us/launch", "GB/s");
#define ROW(NAME, U, STORE, BUFS)                                                    \
    do {                                                                             \
        const float t = time_us<U, STORE>(BUFS, nvec, out, iters);                   \
        std::printf("%-28s %10.2f %10.0f\n", NAME, t, (double)bytes / t / 1e3);      \
    } while (0)
    ROW("cold, 4 loads a thread", 4, false, bufs);
    ROW("cold, 8 loads a thread", 8, false, bufs);
    ROW("cold, 16 loads a thread", 16, false, bufs);
    ROW("resident, 4 loads a thread", 4, false, one);
    ROW("resident, 8 loads a thread", 8, false, one);
    ROW("cold + stores, 4 loads", 4, true, bufs);
    ROW("cold + stores, 8 loads", 8, true, bufs);
    ROW("resident + stores, 4 loads", 4, true, one);
#undef ROW
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    hipEventRecord(e0);
    for (int i = 0; i < 1000; i++) hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, 0);
    hipEventRecord(e1);
    hipEventSynchronize(e1);
    float ms = 0.0f;
    hipEventElapsedTime(&ms, e0, e1);
    std::printf("%-28s %10.2f\n", "empty launch", ms);
    return 0;
}
