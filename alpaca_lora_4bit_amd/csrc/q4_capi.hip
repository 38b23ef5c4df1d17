// C ABI of libq4gptq (declared in include/q4_gptq.h): argument validation + kernel launches.
// No torch types, no allocation, no synchronisation.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include "q4_gptq.h"

extern "C" {
int q4_launch_dequant(const int32_t*, const int32_t*, const void*, const int32_t*, int, void*, int, int, hipStream_t);
int q4_launch_permute_rows(const int32_t*, const int32_t*, int32_t*, int, int, hipStream_t);
int q4_launch_permute_cols(const void*, const int32_t*, void*, int, int, hipStream_t);
int q4_launch_gemv(const void*, const int32_t*, const int32_t*, const void*, const int32_t*, const int32_t*, int, void*,
                   int, int, int, int, int, void*, hipStream_t);
struct q4_drop_args { uint32_t seed_lo, seed_hi, thr15; float scale; };     // q4::DropArgs of q4_common.hpp
int q4_launch_gemm(int, const void*, const int32_t*, const int32_t*, const void*, const int32_t*, int, const void*,
                   const void*, const void*, int, int, int, float, int, void*, int, int, int, int, const q4_drop_args*,
                   void*, size_t, hipStream_t);
int q4_launch_dropout_keep(uint8_t*, int, int, const q4_drop_args*, hipStream_t);
size_t q4_gemm_plan_workspace(int, int, int, int);
int q4_gemv_sorted_applicable(int, int);
int q4_launch_gemv_v1(const void*, const int32_t*, const void*, const void*, void*, int, int, int, int, void*, hipStream_t);
int q4_launch_lora_down(const void*, const void*, int, int, int, void*, int, int, int, const q4_drop_args*, hipStream_t);
int q4_launch_lora_grad(const void*, const void*, float*, int, int, float, int, int, int, const q4_drop_args*, void*,
                        hipStream_t);
int q4_launch_lora_grad_pair(const void*, const void*, float*, int, int, int, const void*, const void*, float*, int, int, int,
                             float, int, int, const q4_drop_args*, void*, hipStream_t);
size_t q4_lora_grad_workspace(int, int, int);
int q4_launch_gemv_group(int, const void* const*, const int32_t* const*, const int32_t* const*, const void* const*,
                         void* const*, const int*, int, int, int, int, int, void*, hipStream_t);
size_t q4_noalloc_scratch_bytes(void);
void* q4_noalloc_scratch_ptr(int*);
int q4_launch_zero_words(void*, size_t, hipStream_t);
int q4_gemm_group_applicable(int, int, int, int, const int*);
size_t q4_gemm_group_plan_workspace(int, int, int, int, const int*);
int q4_launch_gemm_group(int, int, const void* const*, const int32_t* const*, const int32_t* const*, const void* const*, int,
                         const void* const*, const void* const*, const void* const*, const int*, const int*, const int*,
                         const float*, const int*, void* const*, int, int, const int*, const q4_drop_args* const*, void*, size_t,
                         hipStream_t);
int q4_mlp_applicable(int, int, int, int);
size_t q4_mlp_plan_workspace(int, int, int);
size_t q4_mlp_status_offset(int, int, int);
int q4_launch_mlp(const void*, const int32_t* const*, const int32_t* const*, const void* const*, int, void*, void*, void*, int, int,
                  int, void*, int, hipStream_t);
int q4_stream_fwd_applicable(int, int, int, int, int);
int q4_stream_dx_applicable(int, int, int, int, int);
int q4_skinny_applicable(int, int, int, int, int);
int q4_skinny_dx_applicable(int, int, int, int, int);
}

namespace {
inline bool misaligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

// Public dropout descriptor -> kernel arguments.  Returns false for p outside [0, 1).
bool make_drop(const q4_dropout_t* d, q4_drop_args* out, const q4_drop_args** ptr) {
    *ptr = nullptr;
    if (!d) return true;
    if (!(d->p >= 0.0f) || !(d->p < 1.0f)) return false;
    uint32_t thr = (uint32_t)(d->p * 32768.0f + 0.5f);
    if (thr > 32767u) thr = 32767u;
    out->seed_lo = d->seed_lo; out->seed_hi = d->seed_hi; out->thr15 = thr;
    out->scale = 32768.0f / (float)(32768u - thr);
    if (thr != 0) *ptr = out;
    return true;
}

int check_layer(const void* qweight, const void* qzeros, const void* scales, const void* g_idx,
                int groupsize, int K, int N, int G) {
    if (!qweight || !qzeros || !scales) return Q4_ERR_NULL_POINTER;
    if (K < 64 || N < 64 || G < 1 || (K % 32) != 0 || (N % 64) != 0) return Q4_ERR_BAD_SHAPE;
    if (!g_idx) {
        if (groupsize < 32 || (groupsize % 32) != 0) return Q4_ERR_BAD_SHAPE;
        if ((long)G * groupsize < K) return Q4_ERR_BAD_SHAPE;
    }
    if (misaligned(qweight) || misaligned(qzeros) || misaligned(scales) || (g_idx && misaligned(g_idx)))
        return Q4_ERR_MISALIGNED;
    return Q4_OK;
}
}  // namespace

extern "C" int q4_abi_version(void) { return 14; }

extern "C" const char* q4_error_string(int code) {
    switch (code) {
        case Q4_OK: return "ok";
        case Q4_ERR_NULL_POINTER: return "a required pointer is NULL";
        case Q4_ERR_BAD_SHAPE: return "shape outside the supported range (see q4_gptq.h)";
        case Q4_ERR_WORKSPACE: return "workspace missing or too small";
        case Q4_ERR_LAUNCH: return "kernel launch failed";
        case Q4_ERR_MISALIGNED: return "pointer not 16-byte aligned";
        case Q4_ERR_TOO_LARGE: return "problem larger than the library's built-in scratch (see q4_gemv_noalloc_max_outputs)";
        case Q4_ERR_RUNTIME: return "a HIP runtime call failed (see hipGetLastError)";
        default: return "unknown error";
    }
}

extern "C" int q4_dequant_f16(const int32_t* qweight, const int32_t* qzeros, const void* scales,
                              const int32_t* g_idx, int groupsize, void* out, int K, int N, int G, void* stream) {
    int rc = check_layer(qweight, qzeros, scales, g_idx, groupsize, K, N, G);
    if (rc != Q4_OK) return rc;
    if (!out) return Q4_ERR_NULL_POINTER;
    if (misaligned(out)) return Q4_ERR_MISALIGNED;
    if (!g_idx && groupsize % 8 != 0) return Q4_ERR_BAD_SHAPE;
    return q4_launch_dequant(qweight, qzeros, scales, g_idx, groupsize, out, K, N, (hipStream_t)stream);
}

extern "C" int q4_launch_dequant_f32(const int32_t*, const int32_t*, const float*, const int32_t*, int, float*, int, int, hipStream_t);

extern "C" int q4_dequant_f32(const int32_t* qweight, const int32_t* qzeros, const float* scales,
                              const int32_t* g_idx, int groupsize, float* out, int K, int N, int G, void* stream) {
    int rc = check_layer(qweight, qzeros, scales, g_idx, groupsize, K, N, G);
    if (rc != Q4_OK) return rc;
    if (!out) return Q4_ERR_NULL_POINTER;
    if (misaligned(out)) return Q4_ERR_MISALIGNED;
    if (!g_idx && groupsize % 8 != 0) return Q4_ERR_BAD_SHAPE;
    return q4_launch_dequant_f32(qweight, qzeros, scales, g_idx, groupsize, out, K, N, (hipStream_t)stream);
}

extern "C" {
int q4_launch_dequant_v1(const int32_t*, const void*, const void*, void*, int, int, hipStream_t);
int q4_launch_dequant2(const int32_t*, const int32_t*, const void*, const int32_t*, int, void*, int, int, hipStream_t);
}

extern "C" int q4_dequant_v1_f16(const int32_t* qweight, const void* scales, const void* zeros, void* out,
                                 int K, int N, void* stream) {
    if (!qweight || !scales || !zeros || !out) return Q4_ERR_NULL_POINTER;
    if (K < 8 || N < 64 || (K % 8) != 0 || (N % 64) != 0) return Q4_ERR_BAD_SHAPE;
    if (misaligned(qweight) || misaligned(scales) || misaligned(zeros) || misaligned(out)) return Q4_ERR_MISALIGNED;
    return q4_launch_dequant_v1(qweight, scales, zeros, out, K, N, (hipStream_t)stream);
}

extern "C" int q4_dequant2_f16(const int32_t* qweight, const int32_t* qzeros, const void* scales,
                               const int32_t* g_idx, int groupsize, void* out, int K, int N, int G, void* stream) {
    if (!qweight || !qzeros || !scales || !out) return Q4_ERR_NULL_POINTER;
    if (K < 16 || N < 64 || (K % 16) != 0 || (N % 64) != 0 || G < 1) return Q4_ERR_BAD_SHAPE;
    if (!g_idx && (groupsize < 16 || (groupsize % 16) != 0 || (long long)G * groupsize < K)) return Q4_ERR_BAD_SHAPE;
    if (misaligned(qweight) || misaligned(scales) || misaligned(out) || (reinterpret_cast<uintptr_t>(qzeros) & 3u))
        return Q4_ERR_MISALIGNED;
    return q4_launch_dequant2(qweight, qzeros, scales, g_idx, groupsize, out, K, N, (hipStream_t)stream);
}

extern "C" int q4_permute_rows(const int32_t* qweight, const int32_t* perm, int32_t* out, int K, int N, void* stream) {
    if (!qweight || !perm || !out) return Q4_ERR_NULL_POINTER;
    if (K < 8 || N < 1 || (K % 8) != 0) return Q4_ERR_BAD_SHAPE;
    if (qweight == out) return Q4_ERR_BAD_SHAPE;                      // not in place
    if ((reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(perm) | reinterpret_cast<uintptr_t>(out)) & 3u)
        return Q4_ERR_MISALIGNED;
    return q4_launch_permute_rows(qweight, perm, out, K, N, (hipStream_t)stream);
}

extern "C" int q4_permute_cols_f16(const void* in, const int32_t* idx, void* out, int M, int K, void* stream) {
    if (!in || !idx || !out) return Q4_ERR_NULL_POINTER;
    if (M < 1 || K < 8 || (K % 8) != 0 || K > 32768) return Q4_ERR_BAD_SHAPE;        // one row fits 64 KB of LDS
    if (in == out) return Q4_ERR_BAD_SHAPE;                                          // not in place
    if (misaligned(in) || misaligned(out) || misaligned(idx)) return Q4_ERR_MISALIGNED;
    return q4_launch_permute_cols(in, idx, out, M, K, (hipStream_t)stream);
}

static int gemv_check(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                      const int32_t* g_idx, int groupsize, const void* y, int M, int max_rows, int K, int N, int G) {
    int rc = check_layer(qweight, qzeros, scales, g_idx, groupsize, K, N, G);
    if (rc != Q4_OK) return rc;
    if (!x || !y) return Q4_ERR_NULL_POINTER;
    if (M < 1 || M > max_rows || K > 32 * 255 * 8 * 16) return Q4_ERR_BAD_SHAPE;
    if ((long long)(K / 8) * N * 4 >= 0x70000000ll) return Q4_ERR_BAD_SHAPE;      /* 32-bit buffer offsets */
    if (misaligned(x) || misaligned(y)) return Q4_ERR_MISALIGNED;
    return Q4_OK;
}

static int gemv_common(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                       const int32_t* g_idx, const int32_t* perm, int groupsize, void* y, int accumulate,
                       int M, int max_rows, int K, int N, int G, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = gemv_check(x, qweight, qzeros, scales, g_idx, groupsize, y, M, max_rows, K, N, G);
    if (rc != Q4_OK) return rc;
    if (!workspace || workspace_bytes < q4_gemv_workspace_bytes(M, K, N)) return Q4_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    return q4_launch_gemv(x, qweight, qzeros, scales, g_idx, perm, groupsize, y, accumulate, M, K, N, G, workspace,
                          (hipStream_t)stream);
}

extern "C" int q4_gemv_f16(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                           const int32_t* g_idx, int groupsize, void* y, int accumulate,
                           int M, int K, int N, int G, void* workspace, size_t workspace_bytes, void* stream) {
    return gemv_common(x, qweight, qzeros, scales, g_idx, nullptr, groupsize, y, accumulate, M, 16, K, N, G, workspace,
                       workspace_bytes, stream);
}

extern "C" size_t q4_gemv_grouped_workspace_bytes(int M, int total_N) {
    if (M < 1 || total_N < 1) return 0;
    return (size_t)M * (size_t)total_N * 8;
}

extern "C" int q4_gemv_grouped_f16(const q4_gemv_layer_t* layers, int n_layers, int groupsize, int accumulate,
                                   int M, int K, void* workspace, size_t workspace_bytes, void* stream) {
    if (!layers) return Q4_ERR_NULL_POINTER;
    if (n_layers < 1 || n_layers > Q4_GEMV_MAX_GROUP) return Q4_ERR_BAD_SHAPE;
    if (groupsize < 32 || (groupsize % 32) != 0 || K < 64) return Q4_ERR_BAD_SHAPE;
    const int G = (K + groupsize - 1) / groupsize;
    const void* x[Q4_GEMV_MAX_GROUP]; const int32_t* qw[Q4_GEMV_MAX_GROUP]; const int32_t* qz[Q4_GEMV_MAX_GROUP];
    const void* sc[Q4_GEMV_MAX_GROUP]; void* y[Q4_GEMV_MAX_GROUP]; int N[Q4_GEMV_MAX_GROUP];
    long long total_n = 0;
    for (int i = 0; i < n_layers; ++i) {
        const q4_gemv_layer_t& l = layers[i];
        int rc = gemv_check(l.x, l.qweight, l.qzeros, l.scales, nullptr, groupsize, l.y, M, 16, K, l.N, G);
        if (rc != Q4_OK) return rc;
        x[i] = l.x; qw[i] = l.qweight; qz[i] = l.qzeros; sc[i] = l.scales; y[i] = l.y; N[i] = l.N;
        total_n += l.N;
    }
    if (total_n > 0x7fffffff / 64) return Q4_ERR_BAD_SHAPE;
    if (!workspace || workspace_bytes < q4_gemv_grouped_workspace_bytes(M, (int)total_n)) return Q4_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    return q4_launch_gemv_group(n_layers, x, qw, qz, sc, y, N, groupsize, accumulate, M, K, G, workspace,
                                (hipStream_t)stream);
}

extern "C" size_t q4_mlp_decode_workspace_bytes(int M, int H, int I) {
    if (M < 1 || M > 16 || H < 128 || I < 128) return 0;
    return q4_mlp_plan_workspace(M, H, I);
}

extern "C" size_t q4_mlp_decode_status_offset(int M, int H, int I) {
    if (M < 1 || M > 16 || H < 128 || I < 128) return 0;
    return q4_mlp_status_offset(M, H, I);
}

extern "C" int q4_mlp_decode_f16(const void* x, const q4_layer_t* gate, const q4_layer_t* up, const q4_layer_t* down,
                                 int groupsize, void* gate_out, void* up_out, void* y, int M, int H, int I,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !y || !gate || !up || !down) return Q4_ERR_NULL_POINTER;
    if (M < 1 || M > 16 || H < 128 || I < 128) return Q4_ERR_BAD_SHAPE;
    const q4_layer_t* ls[3] = {gate, up, down};
    const int32_t* qw[3]; const int32_t* qz[3]; const void* sc[3];
    for (int i = 0; i < 3; ++i) {
        const int K = i < 2 ? H : I, N = i < 2 ? I : H;
        const int rc = check_layer(ls[i]->qweight, ls[i]->qzeros, ls[i]->scales, nullptr, groupsize, K, N,
                                   groupsize > 0 ? (K + groupsize - 1) / groupsize : 0);
        if (rc != Q4_OK) return rc;
        if ((unsigned long long)(K / 8) * (unsigned long long)N * 4ull >= (1ull << 32)) return Q4_ERR_BAD_SHAPE;
        qw[i] = ls[i]->qweight; qz[i] = ls[i]->qzeros; sc[i] = ls[i]->scales;
    }
    if (!q4_mlp_applicable(M, H, I, groupsize)) return Q4_ERR_BAD_SHAPE;
    if (misaligned(x) || misaligned(y) || (gate_out && misaligned(gate_out)) || (up_out && misaligned(up_out)))
        return Q4_ERR_MISALIGNED;
    if (!workspace || workspace_bytes < q4_mlp_plan_workspace(M, H, I)) return Q4_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    return q4_launch_mlp(x, qw, qz, sc, groupsize, gate_out, up_out, y, M, H, I, workspace, 0, (hipStream_t)stream);
}

extern "C" size_t q4_gemv_noalloc_max_outputs(void) { return q4_noalloc_scratch_bytes() / 8; }

extern "C" int q4_gemv_noalloc_f16(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                   const int32_t* g_idx, int groupsize, void* y, int accumulate,
                                   int M, int K, int N, int G, void* stream) {
    // every check of the allocating entry point first, so that a rejected call enqueues nothing
    int rc = gemv_check(x, qweight, qzeros, scales, g_idx, groupsize, y, M, 16, K, N, G);
    if (rc != Q4_OK) return rc;
    const size_t words = (size_t)M * (size_t)N;
    if (words > q4_gemv_noalloc_max_outputs()) return Q4_ERR_TOO_LARGE;
    // the array belongs to the CURRENT device: the output must live there too
    hipPointerAttribute_t attr;
    int dev = -1;
    if (hipPointerGetAttributes(&attr, y) != hipSuccess || hipGetDevice(&dev) != hipSuccess || attr.device != dev) {
        (void)hipGetLastError();
        return Q4_ERR_RUNTIME;
    }
    int herr = 0;
    void* scratch = q4_noalloc_scratch_ptr(&herr);
    if (!scratch) return Q4_ERR_RUNTIME;
    // the array keeps whatever the previous call on this device left (zeros, unless that call was cut short)
    rc = q4_launch_zero_words(scratch, words, (hipStream_t)stream);
    if (rc != Q4_OK) return rc;
    return gemv_common(x, qweight, qzeros, scales, g_idx, nullptr, groupsize, y, accumulate, M, 16, K, N, G, scratch,
                       words * 8, stream);
}

extern "C" int q4_gemv_sorted_f16(const void* x, const int32_t* qweight_sorted, const int32_t* qzeros, const void* scales,
                                  const int32_t* perm, int groupsize, void* y, int accumulate,
                                  int M, int K, int N, int G, void* workspace, size_t workspace_bytes, void* stream) {
    if (!perm) return Q4_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(perm) & 3u) return Q4_ERR_MISALIGNED;
    if (M >= 1 && !q4_gemv_sorted_applicable(M, K)) return Q4_ERR_BAD_SHAPE;
    return gemv_common(x, qweight_sorted, qzeros, scales, nullptr, perm, groupsize, y, accumulate, M, 4, K, N, G, workspace,
                       workspace_bytes, stream);
}

extern "C" int q4_gemv_v1_f16(const void* x, const int32_t* qweight, const void* scales, const void* zeros, void* y,
                              int accumulate, int M, int K, int N, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x || !qweight || !scales || !zeros || !y) return Q4_ERR_NULL_POINTER;
    if (M < 1 || M > 16 || K < 64 || N < 64 || (K % 32) != 0 || (N % 64) != 0 || K > 32 * 255 * 8 * 16) return Q4_ERR_BAD_SHAPE;
    if ((long long)(K / 8) * N * 4 >= 0x70000000ll) return Q4_ERR_BAD_SHAPE;      /* 32-bit buffer offsets */
    if (misaligned(x) || misaligned(qweight) || misaligned(y) || (reinterpret_cast<uintptr_t>(scales) & 7u) ||
        (reinterpret_cast<uintptr_t>(zeros) & 7u))
        return Q4_ERR_MISALIGNED;
    if (!workspace || workspace_bytes < q4_gemv_workspace_bytes(M, K, N)) return Q4_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    return q4_launch_gemv_v1(x, qweight, scales, zeros, y, accumulate, M, K, N, workspace, (hipStream_t)stream);
}

static int gemm_common(int fwd, const void* act, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                       const int32_t* g_idx, int groupsize, const void* bias, const void* la, const void* lb,
                       int lb_sr, int lb_sc, int lb_is_f32, float lb_scale, int R,
                       void* out, int M, int K, int N, int G, const q4_dropout_t* drop,
                       void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_layer(qweight, qzeros, scales, g_idx, groupsize, K, N, G);
    if (rc != Q4_OK) return rc;
    q4_drop_args da;
    const q4_drop_args* dp;
    if (!make_drop(drop, &da, &dp)) return Q4_ERR_BAD_SHAPE;
    if (!act || !out) return Q4_ERR_NULL_POINTER;
    if (M < 1 || (K % 128) != 0 || (N % 128) != 0) return Q4_ERR_BAD_SHAPE;
    if (!g_idx && (groupsize % 64) != 0) return Q4_ERR_BAD_SHAPE;
    // the kernels address the packed weights through 32-bit buffer offsets
    if ((unsigned long long)(K / 8) * (unsigned long long)N * 4ull >= (1ull << 32)) return Q4_ERR_BAD_SHAPE;
    if ((unsigned long long)(K > N ? K : N) * 512ull >= (1ull << 32)) return Q4_ERR_BAD_SHAPE;
    if ((la != nullptr) != (lb != nullptr)) return Q4_ERR_NULL_POINTER;
    if (la && (R < 8 || R > 64 || (R % 8) != 0)) return Q4_ERR_BAD_SHAPE;
    if (misaligned(act) || misaligned(out) || (la && misaligned(la))) return Q4_ERR_MISALIGNED;
    if (lb && (reinterpret_cast<uintptr_t>(lb) & (lb_is_f32 ? 3u : 1u))) return Q4_ERR_MISALIGNED;
    if (lb && (lb_sr < 1 || lb_sc < 1)) return Q4_ERR_BAD_SHAPE;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    return q4_launch_gemm(fwd, act, qweight, qzeros, scales, g_idx, groupsize, bias, la, lb, lb_sr, lb_sc, lb_is_f32,
                          lb_scale, R, out, M, K, N, G, dp, workspace, workspace ? workspace_bytes : 0, (hipStream_t)stream);
}

extern "C" int q4_gemm_fwd_f16(const void* x, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                               const int32_t* g_idx, int groupsize, const void* bias,
                               const void* xa, const void* lora_b, int ldb_r, int ldb_n, int lora_is_f32,
                               float lora_scale, int R, void* y, int M, int K, int N, int G,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return gemm_common(1, x, qweight, qzeros, scales, g_idx, groupsize, bias, xa, lora_b, ldb_r, ldb_n, lora_is_f32,
                       lora_scale, R, y, M, K, N, G, nullptr, workspace, workspace_bytes, stream);
}

extern "C" int q4_gemm_bwd_dx_f16(const void* dy, const int32_t* qweight, const int32_t* qzeros, const void* scales,
                                  const int32_t* g_idx, int groupsize,
                                  const void* dyb, const void* lora_a, int lda_r, int lda_k, int lora_is_f32,
                                  float lora_scale, int R, void* dx, int M, int K, int N, int G,
                                  const q4_dropout_t* drop, void* workspace, size_t workspace_bytes, void* stream) {
    return gemm_common(0, dy, qweight, qzeros, scales, g_idx, groupsize, nullptr, dyb, lora_a, lda_r, lda_k, lora_is_f32,
                       lora_scale, R, dx, M, K, N, G, drop, workspace, workspace_bytes, stream);
}

extern "C" size_t q4_gemm_workspace_bytes(int fwd, int M, int K, int N) {
    if (M < 1 || K < 128 || N < 128) return 0;
    return q4_gemm_plan_workspace(fwd, M, K, N);
}

// The same tests, in the same order, as q4_launch_gemm applies to a product without adapter term.
extern "C" int q4_gemm_route(int fwd, int M, int K, int N, int groupsize, int has_g_idx) {
    if (M < 1 || K < 128 || N < 128 || (K % 128) != 0 || (N % 128) != 0) return Q4_ERR_BAD_SHAPE;
    if (!has_g_idx && (groupsize < 1 || (groupsize % 64) != 0)) return Q4_ERR_BAD_SHAPE;
    if (fwd) {
        if (q4_stream_fwd_applicable(M, K, N, groupsize, has_g_idx)) return Q4_ROUTE_STREAM;
        if (q4_skinny_applicable(M, K, N, groupsize, has_g_idx)) return Q4_ROUTE_SKINNY;
    } else {
        if (q4_stream_dx_applicable(M, K, N, groupsize, has_g_idx)) return Q4_ROUTE_STREAM;
        if (q4_skinny_dx_applicable(M, K, N, groupsize, has_g_idx)) return Q4_ROUTE_SKINNY;
    }
    return Q4_ROUTE_TILED;
}

extern "C" int q4_gemm_grouped_applicable(int fwd, int n_layers, int M, int K, const int* N) {
    if (!N || n_layers < 2 || n_layers > 4 || M < 1 || K < 128 || (K % 128) != 0) return 0;
    for (int i = 0; i < n_layers; ++i)
        if (N[i] < 128 || (N[i] % 128) != 0) return 0;
    return q4_gemm_group_applicable(fwd, n_layers, M, K, N) ? 1 : 0;
}

extern "C" size_t q4_gemm_grouped_workspace_bytes(int fwd, int n_layers, int M, int K, const int* N) {
    if (!N || n_layers < 2 || n_layers > 4 || M < 1 || K < 128) return 0;
    return q4_gemm_group_plan_workspace(fwd, n_layers, M, K, N);
}

static int gemm_grouped_common(int fwd, const q4_gemm_layer_t* layers, int n, int groupsize, void* dx, int M, int K,
                               void* workspace, size_t workspace_bytes, void* stream) {
    if (!layers) return Q4_ERR_NULL_POINTER;
    if (n < 2 || n > 4 || M < 1 || (K % 128) != 0 || groupsize < 64 || (groupsize % 64) != 0) return Q4_ERR_BAD_SHAPE;
    if (!fwd && !dx) return Q4_ERR_NULL_POINTER;
    if (!fwd && misaligned(dx)) return Q4_ERR_MISALIGNED;
    const void* act[4]; const int32_t* qw[4]; const int32_t* qz[4]; const void* sc[4]; const void* bias[4];
    const void* la[4]; const void* lb[4]; int sr[4], scs[4], f32[4], R[4], N[4]; float lsc[4]; void* out[4];
    q4_drop_args da[4]; const q4_drop_args* dp[4];
    for (int i = 0; i < n; ++i) {
        const q4_gemm_layer_t& l = layers[i];
        const int rc = check_layer(l.qweight, l.qzeros, l.scales, nullptr, groupsize, K, l.N, (K + groupsize - 1) / groupsize);
        if (rc != Q4_OK) return rc;
        if ((l.N % 128) != 0) return Q4_ERR_BAD_SHAPE;
        if ((unsigned long long)(K / 8) * (unsigned long long)l.N * 4ull >= (1ull << 32)) return Q4_ERR_BAD_SHAPE;
        if ((unsigned long long)(K > l.N ? K : l.N) * 512ull >= (1ull << 32)) return Q4_ERR_BAD_SHAPE;
        if (!l.act || (fwd && !l.out)) return Q4_ERR_NULL_POINTER;
        if (fwd && l.act != layers[0].act) return Q4_ERR_BAD_SHAPE;            // the forward shares one x
        if ((l.la != nullptr) != (l.lb != nullptr)) return Q4_ERR_NULL_POINTER;
        if (l.la && (l.R < 8 || l.R > 64 || (l.R % 8) != 0 || l.lb_r < 1 || l.lb_c < 1)) return Q4_ERR_BAD_SHAPE;
        if (misaligned(l.act) || (fwd && misaligned(l.out)) || (l.la && misaligned(l.la))) return Q4_ERR_MISALIGNED;
        if (l.lb && (reinterpret_cast<uintptr_t>(l.lb) & (l.lb_is_f32 ? 3u : 1u))) return Q4_ERR_MISALIGNED;
        if (!make_drop(fwd ? nullptr : l.drop, &da[i], &dp[i])) return Q4_ERR_BAD_SHAPE;
        act[i] = l.act; qw[i] = l.qweight; qz[i] = l.qzeros; sc[i] = l.scales; bias[i] = l.bias; la[i] = l.la; lb[i] = l.lb;
        sr[i] = l.lb_r; scs[i] = l.lb_c; f32[i] = l.lb_is_f32; lsc[i] = l.lb_scale; R[i] = l.la ? l.R : 0;
        out[i] = fwd ? l.out : dx; N[i] = l.N;
    }
    if (!q4_gemm_group_applicable(fwd, n, M, K, N)) return Q4_ERR_BAD_SHAPE;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    if (q4_gemm_group_plan_workspace(fwd, n, M, K, N) > (workspace ? workspace_bytes : 0)) return Q4_ERR_WORKSPACE;
    return q4_launch_gemm_group(fwd, n, act, qw, qz, sc, groupsize, bias, la, lb, sr, scs, f32, lsc, R, out, M, K, N, dp,
                                workspace, workspace ? workspace_bytes : 0, (hipStream_t)stream);
}

extern "C" int q4_gemm_grouped_fwd_f16(const q4_gemm_layer_t* layers, int n_layers, int groupsize, int M, int K, void* stream) {
    return gemm_grouped_common(1, layers, n_layers, groupsize, nullptr, M, K, nullptr, 0, stream);
}

extern "C" int q4_gemm_grouped_bwd_dx_f16(const q4_gemm_layer_t* layers, int n_layers, int groupsize, void* dx, int M, int K,
                                          void* workspace, size_t workspace_bytes, void* stream) {
    return gemm_grouped_common(0, layers, n_layers, groupsize, dx, M, K, workspace, workspace_bytes, stream);
}

extern "C" int q4_lora_down_f16(const void* in, const void* w, int w_sr, int w_sc, int w_is_f32, void* out,
                                int M, int C, int R, const q4_dropout_t* drop, void* stream) {
    if (!in || !w || !out) return Q4_ERR_NULL_POINTER;
    q4_drop_args da;
    const q4_drop_args* dp;
    if (!make_drop(drop, &da, &dp)) return Q4_ERR_BAD_SHAPE;
    if (M < 1 || C < 32 || (C % 32) != 0 || R < 1 || R > 64 || w_sr < 1 || w_sc < 1) return Q4_ERR_BAD_SHAPE;
    /* 32-bit buffer offsets: the 16-row block of `in` and the span of the adapter matrix */
    if ((long long)C * 32 >= 0x70000000ll) return Q4_ERR_BAD_SHAPE;
    if (((long long)(R - 1) * w_sr + (long long)(C - 1) * w_sc + 1) * (w_is_f32 ? 4 : 2) >= 0x70000000ll) return Q4_ERR_BAD_SHAPE;
    if (misaligned(in) || (reinterpret_cast<uintptr_t>(out) & 1u) || (reinterpret_cast<uintptr_t>(w) & (w_is_f32 ? 3u : 1u)))
        return Q4_ERR_MISALIGNED;
    return q4_launch_lora_down(in, w, w_sr, w_sc, w_is_f32, out, M, C, R, dp, (hipStream_t)stream);
}

extern "C" size_t q4_lora_grad_workspace_bytes(int M, int C, int R) {
    if (M < 1 || C < 8 || R < 2 || R > 32 || (R & 1)) return 0;
    return q4_lora_grad_workspace(M, C, R);
}

extern "C" int q4_lora_grad_f32(const void* p, const void* in, float* out, int o_sr, int o_sc, float alpha,
                                int M, int C, int R, const q4_dropout_t* drop,
                                void* workspace, size_t workspace_bytes, void* stream) {
    if (!p || !in || !out) return Q4_ERR_NULL_POINTER;
    q4_drop_args da;
    const q4_drop_args* dp;
    if (!make_drop(drop, &da, &dp)) return Q4_ERR_BAD_SHAPE;
    if (M < 1 || C < 8 || (C % 8) != 0 || R < 2 || R > 32 || (R & 1) || o_sr < 1 || o_sc < 1) return Q4_ERR_BAD_SHAPE;
    if ((long long)M * C * 2 >= 0x70000000ll || C > (1 << 20)) return Q4_ERR_BAD_SHAPE;     /* 32-bit buffer offsets */
    if (misaligned(p) || misaligned(in) || (reinterpret_cast<uintptr_t>(out) & 3u)) return Q4_ERR_MISALIGNED;
    const size_t need = q4_lora_grad_workspace(M, C, R);
    if (need > 0) {
        if (!workspace || workspace_bytes < need) return Q4_ERR_WORKSPACE;
        if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    }
    return q4_launch_lora_grad(p, in, out, o_sr, o_sc, alpha, M, C, R, dp, workspace, (hipStream_t)stream);
}

extern "C" int q4_lora_grad_pair_f32(const void* p1, const void* in1, float* out1, int o1_sr, int o1_sc, int C1,
                                     const void* p2, const void* in2, float* out2, int o2_sr, int o2_sc, int C2,
                                     float alpha, int M, int R, const q4_dropout_t* drop1,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    if (!p1 || !in1 || !out1 || !p2 || !in2 || !out2) return Q4_ERR_NULL_POINTER;
    q4_drop_args da;
    const q4_drop_args* dp;
    if (!make_drop(drop1, &da, &dp)) return Q4_ERR_BAD_SHAPE;
    if (M < 1 || R < 2 || R > 32 || (R & 1)) return Q4_ERR_BAD_SHAPE;
    const int Cs[2] = {C1, C2};
    const int strides[4] = {o1_sr, o1_sc, o2_sr, o2_sc};
    for (int i = 0; i < 2; ++i) {
        if (Cs[i] < 8 || (Cs[i] % 8) != 0 || Cs[i] > (1 << 20) || strides[2 * i] < 1 || strides[2 * i + 1] < 1) return Q4_ERR_BAD_SHAPE;
        if ((long long)M * Cs[i] * 2 >= 0x70000000ll) return Q4_ERR_BAD_SHAPE;               /* 32-bit buffer offsets */
    }
    if (misaligned(p1) || misaligned(in1) || misaligned(p2) || misaligned(in2) ||
        (reinterpret_cast<uintptr_t>(out1) & 3u) || (reinterpret_cast<uintptr_t>(out2) & 3u))
        return Q4_ERR_MISALIGNED;
    const size_t need = q4_lora_grad_workspace(M, C1, R) + q4_lora_grad_workspace(M, C2, R);
    if (need > 0) {
        if (!workspace || workspace_bytes < need) return Q4_ERR_WORKSPACE;
        if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return Q4_ERR_MISALIGNED;
    }
    return q4_launch_lora_grad_pair(p1, in1, out1, o1_sr, o1_sc, C1, p2, in2, out2, o2_sr, o2_sc, C2, alpha, M, R,
                                    dp, workspace, (hipStream_t)stream);
}

extern "C" float q4_dropout_scale(float p) {
    q4_dropout_t d = {0u, 0u, p};
    q4_drop_args da = {0u, 0u, 0u, 1.0f};
    const q4_drop_args* dp;
    if (!make_drop(&d, &da, &dp)) return 0.0f;
    return dp ? da.scale : 1.0f;
}

extern "C" int q4_dropout_keep_u8(uint8_t* keep, int M, int C, const q4_dropout_t* drop, void* stream) {
    if (!keep || !drop) return Q4_ERR_NULL_POINTER;
    if (M < 1 || C < 2 || (C % 2) != 0) return Q4_ERR_BAD_SHAPE;
    q4_drop_args da;
    const q4_drop_args* dp;
    if (!make_drop(drop, &da, &dp)) return Q4_ERR_BAD_SHAPE;
    if (!dp) { da.seed_lo = drop->seed_lo; da.seed_hi = drop->seed_hi; da.thr15 = 0; da.scale = 1.0f; }
    return q4_launch_dropout_keep(keep, M, C, &da, (hipStream_t)stream);
}
