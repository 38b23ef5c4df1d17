#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
// Measurement aid: what does the LDS traffic of ONE reduction step of the 256 x 128 GEMM workgroup cost by itself?
// Per step the workgroup (8 wavefronts) stores the activation tile and the dequantized weight slab (six 16-byte
// stores per thread = 48 KB) and every wavefront fetches sixteen 16-byte operand fragments (131 KB in all), in the
// kernel's own address patterns.  The 128 MFMAs of a step keep the matrix pipes busy for 1024 clocks; if the LDS
// traffic alone takes longer, the LDS pipe and not the matrix pipe bounds the kernel.  Clocks are s_memtime ticks.
// Also: LDS b128 write / read rates for the address patterns of a [rows][64 halves] fp16 tile.
// MODE 0: lane-contiguous (reference); 1: row stride 144 B (8 halves of padding), 8 lanes per row;
// 2: row stride 128 B with 16-byte units XOR-swizzled by (row >> 1) & 7.
template <int MODE>
__device__ __forceinline__ int waddr(int t, int pass) {       // byte address of thread t's 16-byte store
    const int row = (t >> 3) + 64 * pass, u = t & 7;
    if (MODE == 0) return (t + 512 * pass) * 16;
    if (MODE == 1) return row * 144 + u * 16;
    return row * 128 + ((u ^ ((row >> 1) & 7)) * 16);
}
template <int MODE>
__device__ __forceinline__ int raddr(int lane, int wrow0, int ks) {   // fragment read: row lane&31, k offset (lane>>5)*8 + 16*ks halves
    const int row = wrow0 + (lane & 31), u = (lane >> 5) + 2 * ks;
    if (MODE == 0) return ((lane + 64 * ks) * 16) + wrow0 * 16;
    if (MODE == 1) return row * 144 + u * 16;
    return row * 128 + ((u ^ ((row >> 1) & 7)) * 16);
}
template <int MODE, bool WRITE>
__global__ __launch_bounds__(512) void k(uint64_t* out, int iters) {
    __shared__ __attribute__((aligned(16))) unsigned char buf[256 * 144];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    for (int i = t; i < 256 * 144 / 4; i += 512) reinterpret_cast<uint32_t*>(buf)[i] = i;
    __syncthreads();
    uint4_t v = {(uint32_t)t, 1, 2, 3};
    uint32_t acc = 0;
    const uint64_t t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
        if (WRITE) {
#pragma unroll
            for (int p = 0; p < 4; ++p) { *reinterpret_cast<uint4_t*>(buf + waddr<MODE>(t, p)) = v; v.x += 1; }
        } else {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const uint4_t r = *reinterpret_cast<const uint4_t*>(buf + raddr<MODE>(lane, (wave >> 1) * 64 + 32 * i, ks));
                    acc ^= r.x ^ r.y ^ r.z ^ r.w;
                }
        }
        asm volatile("" ::: "memory");
    }
    __syncthreads();
    const uint64_t t1 = __builtin_amdgcn_s_memtime();
    if (acc == 0x12345u || reinterpret_cast<uint32_t*>(buf)[t] == 0x54321u) out[1000] = 1;
    if (t == 0) out[blockIdx.x] = t1 - t0;
}
template <int MODE, int NWR, int NRD>
__global__ __launch_bounds__(512) void kmix(uint64_t* out, int iters) {
    __shared__ __attribute__((aligned(16))) unsigned char buf[256 * 144 + 128 * 144];
    __shared__ __attribute__((aligned(16))) unsigned char wbuf[256 * 144 + 128 * 144];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    for (int i = t; i < (256 + 128) * 144 / 4; i += 512) reinterpret_cast<uint32_t*>(buf)[i] = i;
    __syncthreads();
    uint4_t v = {(uint32_t)t, 1, 2, 3};
    uint32_t acc = 0;
    const uint64_t t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int p = 0; p < NWR; ++p) { *reinterpret_cast<uint4_t*>(wbuf + waddr<MODE>(t, p)) = v; v.x += 1; }
#pragma unroll
        for (int ks = 0; ks < NRD / 4; ++ks)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4_t r = *reinterpret_cast<const uint4_t*>(buf + raddr<MODE>(lane, (i < 2 ? (wave >> 1) * 64 + 32 * i : 256 + (wave & 1) * 64 + 32 * (i - 2)), ks));
                acc ^= r.x ^ r.y ^ r.z ^ r.w;
            }
        asm volatile("" ::: "memory");
    }
    __syncthreads();
    const uint64_t t1 = __builtin_amdgcn_s_memtime();
    if (acc == 0x12345u || reinterpret_cast<uint32_t*>(wbuf)[t] == 0x54321u) out[1000] = 1;
    if (t == 0) out[blockIdx.x] = t1 - t0;
}
template <int MODE>
__global__ __launch_bounds__(512) void kmix2(uint64_t* out, int iters) {
    __shared__ __attribute__((aligned(16))) unsigned char buf[256 * 144 + 128 * 144];
    __shared__ __attribute__((aligned(16))) unsigned char wbuf[256 * 144 + 128 * 144];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    for (int i = t; i < (256 + 128) * 144 / 4; i += 512) reinterpret_cast<uint32_t*>(buf)[i] = i;
    __syncthreads();
    uint4_t v = {(uint32_t)t, 1, 2, 3};
    uint32_t acc = 0;
    const uint64_t t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
        int p = 0;
        uint4_t rr[16];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int q = ks * 4 + i;
                rr[q] = *reinterpret_cast<const uint4_t*>(buf + raddr<MODE>(lane, (i < 2 ? (wave >> 1) * 64 + 32 * i : 256 + (wave & 1) * 64 + 32 * (i - 2)), ks));
                if (q == 0 || q == 2 || q == 5 || q == 8 || q == 10 || q == 13) {
                    *reinterpret_cast<uint4_t*>(wbuf + waddr<MODE>(t, p)) = v; v.x += 1; ++p;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
        for (int q = 0; q < 16; ++q) acc ^= rr[q].x ^ rr[q].y ^ rr[q].z ^ rr[q].w;
        asm volatile("" ::: "memory");
    }
    __syncthreads();
    const uint64_t t1 = __builtin_amdgcn_s_memtime();
    if (acc == 0x12345u || reinterpret_cast<uint32_t*>(wbuf)[t] == 0x54321u) out[1000] = 1;
    if (t == 0) out[blockIdx.x] = t1 - t0;
}
template <typename K> void runc(const char* name, K kern) {
    uint64_t* d; (void)hipMalloc(&d, 2048 * 8); (void)hipMemset(d, 0, 2048 * 8);
    const int iters = 4000;
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 0, 0, d, iters);
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 0, 0, d, iters);
    (void)hipDeviceSynchronize();
    uint64_t h[8]; (void)hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost);
    printf("%s: %.0f clocks per iteration\n", name, (double)h[0] / iters);
    (void)hipFree(d);
}
template <typename K> void run(const char* name, K kern, double bytes_per_iter) {
    uint64_t* d; (void)hipMalloc(&d, 2048 * 8); (void)hipMemset(d, 0, 2048 * 8);
    const int iters = 4000;
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 0, 0, d, iters);
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 0, 0, d, iters);
    (void)hipDeviceSynchronize();
    uint64_t h[8]; (void)hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost);
    printf("%s: %.1f bytes/clk/CU\n", name, bytes_per_iter * iters / (double)h[0]);
    (void)hipFree(d);
}
int main() {
    run("write contiguous     ", k<0, true>, 512 * 4 * 16.0);
    run("write stride 144     ", k<1, true>, 512 * 4 * 16.0);
    run("write swizzled 128   ", k<2, true>, 512 * 4 * 16.0);
    run("read  contiguous     ", k<0, false>, 512 * 8 * 16.0);
    run("read  stride 144     ", k<1, false>, 512 * 8 * 16.0);
    run("read  swizzled 128   ", k<2, false>, 512 * 8 * 16.0);
    runc("6 stores only (48 KB)            ", kmix<1, 6, 0>);
    runc("16 fragment reads only (131 KB)  ", kmix<1, 0, 16>);
    runc("6 stores + 16 reads (GEMM step)  ", kmix<1, 6, 16>);
    runc("same, stores spread among reads  ", kmix2<1>);
    return 0;
}
