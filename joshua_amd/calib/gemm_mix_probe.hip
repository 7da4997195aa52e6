// Microbenchmark: the int8 GEMM's instruction mix a super-block iteration (MFMAs, LDS operand reads, vector instructions,
// one barrier), with 16x16x64 and with 32x32x32 MFMAs.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef int i4 __attribute__((ext_vector_type(4)));
typedef int i16 __attribute__((ext_vector_type(16)));
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)

template <int VPS>  // vector instructions a step
__device__ __forceinline__ void valu(float (&f)[8], float m) {
#pragma unroll
    for (int i = 0; i < VPS; i++) f[i & 7] = fmaf(f[i & 7], m, 1.0f);
}

// MODE 0: 56 steps of 2 LDS reads + 4 MFMA 16x16x64 + VPS vector instructions; 1: 28 steps of 2 LDS reads + 4 MFMA 32x32x32 + 2 VPS
template <int MODE, int VPS, bool LDS_READS>
__global__ __launch_bounds__(512) void k(int iters, int *out, float *fout) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 16384; i += 512) ((int *)lds)[i] = i * 2654435761u;
    __syncthreads();
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = (float)(lane + i);
    const float m = 0.999f;
    i4 a0 = i4{lane, lane + 1, lane + 2, lane + 3}, a1 = i4{lane * 3, 1, 2, 3};
    int sum = 0;
    if (MODE == 0) {
        i4 acc[12];
#pragma unroll
        for (int i = 0; i < 12; i++) acc[i] = i4{0, 0, 0, 0};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int s = 0; s < 56; s++) {
                i4 bh = a1, bl = a0;
                if (LDS_READS) {
                    bh = *(const i4 *)(lds + ((s * 2048 + lane * 16) & 65535));
                    bl = *(const i4 *)(lds + ((s * 2048 + 1024 + lane * 16) & 65535));
                }
                const int c = (s % 4) * 3;
                acc[c + 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, bl, acc[c + 1], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, bh, acc[c], 0, 0, 0);
                acc[c + 2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, bl, acc[c + 2], 0, 0, 0);
                acc[c + 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, bh, acc[c + 1], 0, 0, 0);
                valu<VPS>(f, m);
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < 12; i++) sum += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    } else {
        i16 acc[6];
#pragma unroll
        for (int i = 0; i < 6; i++)
#pragma unroll
            for (int j = 0; j < 16; j++) acc[i][j] = 0;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int s = 0; s < 28; s++) {
                i4 bh = a1, bl = a0;
                if (LDS_READS) {
                    bh = *(const i4 *)(lds + ((s * 2048 + lane * 16) & 65535));
                    bl = *(const i4 *)(lds + ((s * 2048 + 1024 + lane * 16) & 65535));
                }
                const int c = (s % 2) * 3;
                acc[c + 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bl, acc[c + 1], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bh, acc[c], 0, 0, 0);
                acc[c + 2] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bl, acc[c + 2], 0, 0, 0);
                acc[c + 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bh, acc[c + 1], 0, 0, 0);
                valu<2 * VPS>(f, m);
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < 6; i++)
#pragma unroll
            for (int j = 0; j < 16; j++) sum += acc[i][j];
    }
    float fs = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) fs += f[i];
    out[blockIdx.x * 512 + threadIdx.x] = sum;
    fout[blockIdx.x * 512 + threadIdx.x] = fs;
}

template <int MODE, int VPS, bool L>
float run(int iters, int *out, float *fout) {
    auto kern = k<MODE, VPS, L>;
    CK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 120 * 1024));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 120 * 1024, 0, 4, out, fout);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 120 * 1024, 0, iters, out, fout);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    return ms * 1e6f / iters;  // ns an iteration
}

int main() {
    int *out; float *fout;
    CK(hipMalloc(&out, 256 * 512 * 4)); CK(hipMalloc(&fout, 256 * 512 * 4));
    const int iters = 400;
    printf("ns a super-block iteration (8 waves a workgroup, one workgroup a compute unit; the kernel: 12150 clocks = 6.7 us at 1.82 GHz)\n");
    printf("16x16x64, 11 vector a step, LDS reads:    %8.0f\n", run<0, 11, true>(iters, out, fout));
    printf("16x16x64, 11 vector a step, no LDS reads: %8.0f\n", run<0, 11, false>(iters, out, fout));
    printf("16x16x64,  0 vector a step, LDS reads:    %8.0f\n", run<0, 0, true>(iters, out, fout));
    printf("16x16x64,  0 vector, no LDS reads:        %8.0f\n", run<0, 0, false>(iters, out, fout));
    printf("32x32x32, 22 vector a step, LDS reads:    %8.0f\n", run<1, 11, true>(iters, out, fout));
    printf("32x32x32, 22 vector a step, no LDS reads: %8.0f\n", run<1, 11, false>(iters, out, fout));
    printf("32x32x32,  0 vector a step, LDS reads:    %8.0f\n", run<1, 0, true>(iters, out, fout));
    printf("32x32x32,  0 vector, no LDS reads:        %8.0f\n", run<1, 0, false>(iters, out, fout));
    return 0;
}
