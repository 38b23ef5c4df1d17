// Measurement aid: how long does one launch need just to READ the packed weights of a layer?
// The streaming GEMV cannot be faster than a kernel that only pulls the same bytes, so this is the floor its
// roofline fraction is judged against.  Same harness as the benchmark's headline step: 96 launches over 96 distinct
// weight buffers (nothing is cache-resident), captured once as a HIP graph and replayed; time from HIP events on the
// launch stream.  Patterns: `contiguous` (every wavefront reads 4 KB in a row), `gemv` (the GEMV's own addresses:
// 64-column strips, a lane reads 16 bytes of 4 adjacent columns, consecutive steps 4 packed rows apart), and an empty
// kernel for the fixed cost of a launch.
//   usage: read_floor [K] [N]     (defaults 4096 11008)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include "../q4_common.hpp"
using namespace q4;
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1);} } while (0)

template <int NSTEP, bool GEMV_PATTERN, bool STREAM>
__global__ __launch_bounds__(512) void read_kernel(const uint32_t* w, int K8, int N, uint32_t* sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const rsrc_t rw = make_rsrc(w, (unsigned)((size_t)K8 * N * 4));
    uint4_t v[NSTEP];
    if (!GEMV_PATTERN) {
        const size_t gw = (size_t)blockIdx.x * nw + wave;
        const int off = (int)(gw * NSTEP * 1024 + lane * 16);
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) v[t] = STREAM ? buf_load128_stream(rw, off, t * 1024) : buf_load128(rw, off, t * 1024);
    } else {
        const int kk = lane >> 4, c = lane & 15;
        const int r0 = (blockIdx.y * nw + wave) * 4 * NSTEP;
        const int off = ((r0 + kk) * N + blockIdx.x * 64 + 4 * c) * 4;
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) v[t] = STREAM ? buf_load128_stream(rw, off, 16 * t * N) : buf_load128(rw, off, 16 * t * N);
    }
    uint32_t x = 0;
#pragma unroll
    for (int t = 0; t < NSTEP; ++t) x ^= v[t].x ^ v[t].y ^ v[t].z ^ v[t].w;
    if (x == 0x12345677u) sink[threadIdx.x] = x;          // never true for the fill pattern: keeps the loads alive
}

__global__ void empty_kernel(uint32_t* sink) { if (sink == nullptr) sink[0] = 1; }

int main(int argc, char** argv) {
    const int K = argc > 1 ? atoi(argv[1]) : 4096, N = argc > 2 ? atoi(argv[2]) : 11008;
    if (K % 1024 || N % 64) { printf("K must be a multiple of 1024, N of 64\n"); return 1; }
    const int NL = 96, reps = 20, K8 = K / 8;
    const size_t bytes = (size_t)K8 * N * 4;
    std::vector<uint32_t*> ws(NL);
    for (int i = 0; i < NL; ++i) { CK(hipMalloc(&ws[i], bytes)); CK(hipMemset(ws[i], 0x5a, bytes)); }
    uint32_t* sink; CK(hipMalloc(&sink, 4096 * 4));
    hipStream_t s; CK(hipStreamCreate(&s));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const char* names[] = {"empty kernel", "contiguous, plain loads", "contiguous, streaming loads", "gemv pattern, plain loads",
                           "gemv pattern, streaming loads"};
    printf("layer K=%d N=%d: %.3f MB of packed weights per launch, %d distinct buffers, graph of %d launches x %d replays\n",
           K, N, bytes / 1e6, NL, NL, reps);
    for (int pass = 0; pass < 2; ++pass)
        for (int v = 0; v < 5; ++v) {
            hipGraph_t g; hipGraphExec_t ge;
            CK(hipStreamBeginCapture(s, hipStreamCaptureModeGlobal));
            for (int i = 0; i < NL; ++i) {
                const dim3 block(512), gc((unsigned)(bytes / (1024 * 4 * 8))), gg(N / 64, K8 / (4 * 4 * 8));
                switch (v) {
                    case 0: hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, s, sink); break;
                    case 1: hipLaunchKernelGGL((read_kernel<4, false, false>), gc, block, 0, s, ws[i], K8, N, sink); break;
                    case 2: hipLaunchKernelGGL((read_kernel<4, false, true>), gc, block, 0, s, ws[i], K8, N, sink); break;
                    case 3: hipLaunchKernelGGL((read_kernel<4, true, false>), gg, block, 0, s, ws[i], K8, N, sink); break;
                    default: hipLaunchKernelGGL((read_kernel<4, true, true>), gg, block, 0, s, ws[i], K8, N, sink); break;
                }
            }
            CK(hipStreamEndCapture(s, &g));
            CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
            for (int r = 0; r < 3; ++r) CK(hipGraphLaunch(ge, s));
            CK(hipStreamSynchronize(s));
            CK(hipEventRecord(e0, s));
            for (int r = 0; r < reps; ++r) CK(hipGraphLaunch(ge, s));
            CK(hipEventRecord(e1, s));
            CK(hipStreamSynchronize(s));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1));
            const double us = ms * 1e3 / (reps * NL);
            if (pass == 1) {
                if (v == 0) printf("%-32s %7.3f us per launch\n", names[v], us);
                else printf("%-32s %7.3f us per launch  %6.0f GB/s  %.3f of 8000 GB/s\n", names[v], us, bytes / us / 1e3, bytes / us / 1e3 / 8000.0);
            }
            CK(hipGraphExecDestroy(ge)); CK(hipGraphDestroy(g));
        }
    return 0;
}
