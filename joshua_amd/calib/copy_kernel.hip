// Calibration for the HBM traffic counters: a plain 16-byte-per-thread copy of a known size,
// eight times over distinct cold regions.  Running it under
//     rocprofv3 --pmc FETCH_SIZE   (and again with --pmc WRITE_SIZE)
// gives what each counter reads per dispatch for exactly `bytes` read and `bytes` written; the ratio
// scales the same counters collected for the library's kernels.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

__global__ void copy_u4(const uint4 *__restrict__ a, uint4 *__restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) b[i] = a[i];
}

#define CHECK(x)                                                              \
    do {                                                                      \
        hipError_t e_ = (x);                                                  \
        if (e_ != hipSuccess) {                                               \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));      \
            return 1;                                                         \
        }                                                                     \
    } while (0)

int main(int argc, char **argv) {
    const size_t bytes = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 33030144;  // Q4_K 14336 x 4096
    const size_t n = bytes / 16;
    uint4 *a = nullptr, *b = nullptr;
    CHECK(hipMalloc((void **)&a, n * 16 * 8));
    CHECK(hipMalloc((void **)&b, n * 16 * 8));
    CHECK(hipMemset(a, 1, n * 16 * 8));
    CHECK(hipDeviceSynchronize());
    for (int i = 0; i < 8; i++)
        hipLaunchKernelGGL(copy_u4, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0, a + i * n, b + i * n, n);
    CHECK(hipDeviceSynchronize());
    std::printf("copied %zu bytes, 8 dispatches\n", n * 16);
    return 0;
}
