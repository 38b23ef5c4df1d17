// Measurement aid: what does the matrix pipe deliver on this part when nothing else runs?
// 256 workgroups x 8 wavefronts (two per SIMD, as in the 256 x 128 GEMM tile), each issuing v_mfma_f32_32x32x16_f16
// back to back on operands held in registers: no LDS, no loads.  Run once with all-zero operands and once with random
// fp16 operands: the part is power-managed and its clock under MFMA load depends on how many operand bits toggle, so
// the practical ceiling for real data is well below the nominal 2.5 PFLOP/s.  The shader clock is read with
// s_memtime against the 100 MHz wall clock (s_memrealtime).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1);} } while (0)

__global__ __launch_bounds__(512) void mfma_kernel(const half8_t* ops, float* out, unsigned long long* clocks, int iters) {
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { a[i] = ops[(threadIdx.x * 8 + i) & 4095]; b[i] = ops[(threadIdx.x * 8 + 4 + i) & 4095]; }
    float16_t acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    const unsigned long long c0 = __builtin_amdgcn_s_memtime(), w0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(i + u) & 3], b[i], acc[i], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_amdgcn_s_memtime(), w1 = __builtin_amdgcn_s_memrealtime();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0) { clocks[2 * blockIdx.x] = c1 - c0; clocks[2 * blockIdx.x + 1] = w1 - w0; }
}

int main() {
    const int iters = 20000, wgs = 256;
    half8_t* ops; float* out; unsigned long long* clocks;
    CK(hipMalloc(&ops, 4096 * sizeof(half8_t))); CK(hipMalloc(&out, wgs * 512 * 4)); CK(hipMalloc(&clocks, wgs * 16));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const char* names[] = {"all-zero operands", "random fp16 operands"};
    for (int v = 0; v < 2; ++v) {
        _Float16* h = (_Float16*)malloc(4096 * 16);
        srand(1);
        for (int i = 0; i < 4096 * 8; ++i) h[i] = v ? (_Float16)((rand() % 2001 - 1000) / 500.0f) : (_Float16)0.f;
        CK(hipMemcpy(ops, h, 4096 * 16, hipMemcpyHostToDevice));
        free(h);
        for (int r = 0; r < 3; ++r) hipLaunchKernelGGL(mfma_kernel, dim3(wgs), dim3(512), 0, 0, ops, out, clocks, iters);
        CK(hipDeviceSynchronize());
        CK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL(mfma_kernel, dim3(wgs), dim3(512), 0, 0, ops, out, clocks, iters);
        CK(hipEventRecord(e1, 0));
        CK(hipDeviceSynchronize());
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        unsigned long long hc[2]; CK(hipMemcpy(hc, clocks, 16, hipMemcpyDeviceToHost));
        const double flop = (double)wgs * 8 * iters * 16 * (2.0 * 32 * 32 * 16);
        printf("%-22s %8.3f ms  %7.1f TFLOP/s  (%.3f of 2500)  shader clock %.2f GHz\n", names[v], ms, flop / ms / 1e9,
               flop / ms / 1e9 / 2500.0, (double)hc[0] / ((double)hc[1] * 10.0));
    }
    return 0;
}
