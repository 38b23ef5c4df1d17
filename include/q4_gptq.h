/* C ABI of libq4gptq: 4-bit GPTQ dequantize / multiply kernels for AMD MI355X (gfx950).
 *
 * Plain pointers and sizes only.  Every pointer is DEVICE memory on the current HIP device
 * unless said otherwise; `stream` is a hipStream_t passed as void* (NULL = the null stream).
 * All calls are asynchronous on `stream`, keep no reference to any argument after the
 * kernels they enqueue have run, and return Q4_OK or a negative Q4_ERR_* code (never throw,
 * never abort).  Tensors are dense row-major in the GPTQ "v2" layout:
 *
 *   qweight int32  [K/8, N]   eight 4-bit codes per word along K (code of row k in bits 4*(k%8)..)
 *   qzeros  int32  [G, N/8]   eight 4-bit zero codes per word along N; the zero point is code+1
 *   scales  fp16   [G, N]
 *   g_idx   int32  [K]        group of row k (act-order); NULL means k / groupsize
 *   W[k,n] = rn16( rn16(s*q) - rn16(s*(z+1)) ),  s = scales[g,n], g = g_idx[k]
 *
 * Shape limits common to all entry points: K % 32 == 0, N % 64 == 0, K,N >= 64, G >= 1,
 * 0 <= g_idx[k] < G (not checked on the device side of the hot loops: validate on the host).
 *
 * The reference is johnsmith0031/alpaca_lora_4bit; paths below are relative to its
 * src/alpaca_lora_4bit/.
 */
#ifndef Q4_GPTQ_H
#define Q4_GPTQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The library is built with -fvisibility=hidden: the functions declared here are its whole exported set. */
#define Q4_API __attribute__((visibility("default")))

#define Q4_OK 0
#define Q4_ERR_NULL_POINTER (-1)   /* a required pointer is NULL */
#define Q4_ERR_BAD_SHAPE (-2)      /* a size violates the limits above / of the entry point */
#define Q4_ERR_WORKSPACE (-3)      /* workspace missing or smaller than *_workspace_bytes() */
#define Q4_ERR_LAUNCH (-4)         /* hipLaunch reported an error (see hipGetLastError) */
#define Q4_ERR_MISALIGNED (-5)     /* a pointer is not 16-byte aligned */
#define Q4_ERR_TOO_LARGE (-6)      /* larger than the library's built-in scratch (allocation-free entry point) */
#define Q4_ERR_RUNTIME (-7)        /* a HIP runtime call other than a launch failed */

/* Library ABI version (bumped when a signature changes). */
Q4_API int q4_abi_version(void);

/* Static string for a return code. */
Q4_API const char *q4_error_string(int code);

/* Dense dequantization: out fp16 [K, N] = W.
 * Replaces quant_cuda.vecquant4recons_v2(mat, res, scales, zeros, g_idx)
 * (quant_cuda/quant_cuda.cpp:137-148, kernel quant_cuda/quant_cuda_kernel.cu:1127-1183).
 * Bit-exact with that kernel's fp16 instantiation. */
Q4_API int q4_dequant_f16(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                   const int32_t *g_idx, int groupsize, void *out,
                   int K, int N, int G, void *stream);

/* Dense dequantization in float: scales fp32 [G, N], out fp32 [K, N].
 * Replaces the float instantiation of the same operator (AT_DISPATCH on scales.type(),
 * quant_cuda/quant_cuda_kernel.cu:1173-1181; reached from matmul_utils_4bit.py:121-122 when a
 * model's scales were converted to float).  zero = rn32(s * (z + 1)), W = fma(s, q, -zero): the
 * product and the difference round once together, as in the reference's build (nvcc contracts
 * a * b - c by default and setup.py sets no flag); rounding them separately moves a value by at
 * most one unit in the last place.  Same shape rules as q4_dequant_f16. */
Q4_API int q4_dequant_f32(const int32_t *qweight, const int32_t *qzeros, const float *scales,
                   const int32_t *g_idx, int groupsize, float *out,
                   int K, int N, int G, void *stream);

/* Dense dequantization of the older "v1" layout: one fp16 scale and one fp16 zero per column
 * (scales, zeros: [N]),  W[k,n] = rn16( rn16(s[n]*q) - zero[n] ).
 * Replaces quant_cuda.vecquant4recons_v1 (quant_cuda/quant_cuda.cpp:131-135, kernel quant_cuda_kernel.cu:1076-1097). */
Q4_API int q4_dequant_v1_f16(const int32_t *qweight, const void *scales, const void *zeros, void *out,
                      int K, int N, void *stream);

/* Dense dequantization of 2-bit v2 layers: qweight int32 [K/16, N] (sixteen codes per word along K),
 * qzeros int32 [G, N/16], scales fp16 [G, N], W = rn16( rn16(s*q) - rn16(s*(z+1)) ).  K % 16 == 0.
 * Replaces quant_cuda.vecquant2recons_v2 (quant_cuda/quant_cuda.cpp:150-161, kernel quant_cuda_kernel.cu:1185-1211). */
Q4_API int q4_dequant2_f16(const int32_t *qweight, const int32_t *qzeros, const void *scales,
                    const int32_t *g_idx, int groupsize, void *out, int K, int N, int G, void *stream);

/* Row permutation of packed weights: out int32 [K/8, N] holds in row p the 4-bit codes of row perm[p]
 * of qweight (perm int32 [K], a permutation of 0..K-1, not checked).  No counterpart in the reference:
 * it is the one-time repack that lets an act-order layer (rows assigned to groups through g_idx,
 * autograd_4bit.py:185, quant_cuda_kernel.cu:1143) run through the sequential-group kernels -- sort
 * the rows by group, gather x through the same permutation.  Not in place. */
Q4_API int q4_permute_rows(const int32_t *qweight, const int32_t *perm, int32_t *out, int K, int N, void *stream);

/* Column gather of activations: out fp16 [M, K], out[m, p] = in[m, idx[p]] (idx int32 [K], values in 0..K-1; out of
 * range values are clamped).  The run-time companion of q4_permute_rows: gather x through the row sort before a
 * product with the sorted weights (idx = perm), gather grad_input back after it (idx = inverse permutation).  No
 * counterpart in the reference (its kernels read g_idx per row instead).  K % 8 == 0, K <= 32768; in, out and idx
 * 16-byte aligned; not in place. */
Q4_API int q4_permute_cols_f16(const void *in, const int32_t *idx, void *out, int M, int K, void *stream);

/* Decode GEMV / skinny GEMM, 1 <= M <= 16:  y fp16 [M, N] = x fp16 [M, K] @ W  (fp32 accumulate).
 * If accumulate != 0 the product is added to the existing contents of y.
 * Replaces quant_cuda.vecquant4matmul / vecquant4matmul_faster / vecquant4matmul_old_faster
 * (quant_cuda/quant_cuda.cpp:55-61, 93-113; kernels quant_cuda_kernel.cu:443-536, 874-1073)
 * as dispatched by matmul_utils_4bit.py:59-95.  g_idx == NULL selects sequential groups of
 * `groupsize` rows (the old_faster convention, quant_cuda_kernel.cu:1024); otherwise rows are
 * gathered through g_idx (the vecquant4matmul convention, :513-520).
 * `workspace` must hold q4_gemv_workspace_bytes(M, K, N) = 8*M*N bytes, 256-byte aligned, and must be
 * ZERO before its first use; every call leaves it zeroed again (it carries the fixed-point split-K
 * sums).  Calls sharing one workspace must be ordered on one stream.  K <= 1 044 480. */
Q4_API size_t q4_gemv_workspace_bytes(int M, int K, int N);
Q4_API int q4_gemv_f16(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                const int32_t *g_idx, int groupsize, void *y, int accumulate,
                int M, int K, int N, int G,
                void *workspace, size_t workspace_bytes, void *stream);

/* Several layers in ONE launch: y_i fp16 [M, N_i] = x_i fp16 [M, K] @ W_i for 1 <= n_layers <= Q4_GEMV_MAX_GROUP layers
 * that share M, K and the group size (sequential groups only: g_idx[k] == k / groupsize), each read in place from
 * its own tensors -- q_proj | k_proj | v_proj or gate_proj | up_proj of a decoder block with x_i all the same
 * pointer.  The reference gets the same effect by concatenating the packed tensors of the projections along N
 * (model_attn_mlp_patch.py:88-100, 180-190) and calling vecquant4matmul once; here the checkpoint tensors stay as
 * they are.  `layers` is an array in HOST memory (copied into the kernel arguments; not referenced after the call
 * returns).  Per layer the limits of q4_gemv_f16 apply; K <= 1 044 480.  `workspace`: q4_gemv_grouped_workspace_bytes(M,
 * N_0 + .. + N_{n-1}) = 8 * M * sum(N_i) bytes, 256-byte aligned, zero before its first use, left zero by every call
 * (a workspace kept for q4_gemv_f16 can be shared: same convention). */
#define Q4_GEMV_MAX_GROUP 4
typedef struct q4_gemv_layer {
    const void *x;             /* fp16 [M, K] */
    const int32_t *qweight;    /* int32 [K/8, N] */
    const int32_t *qzeros;     /* int32 [G, N/8], G = ceil(K / groupsize) */
    const void *scales;        /* fp16 [G, N] */
    void *y;                   /* fp16 [M, N] */
    int N;
} q4_gemv_layer_t;
Q4_API size_t q4_gemv_grouped_workspace_bytes(int M, int total_N);
Q4_API int q4_gemv_grouped_f16(const q4_gemv_layer_t *layers, int n_layers, int groupsize, int accumulate,
                        int M, int K, void *workspace, size_t workspace_bytes, void *stream);

/* Decode step of a gated MLP block in ONE launch:
 *   y fp16 [M, H] = down( silu(gate(x)) * up(x) ),   x fp16 [M, H], 1 <= M <= 16,
 * gate and up: 4-bit layers H -> I, down: I -> H, sequential groups (g_idx NULL), no bias.  Replaces the three
 * products and two elementwise kernels of QuantLlamaMLP.forward (model_attn_mlp_patch.py:224-228: gate_up_proj,
 * act_fn(gate) * up, down_proj) for the rows a decode step has; the intermediate is rounded to fp16 where those
 * modules round it (gate, up, silu(gate), the product).  The workgroups of the down projection run in the same grid
 * as those of gate and up, request their packed weights at once and then wait, on the device, for the part of the
 * intermediate they need: the weight stream never pauses between the products and one launch gap disappears.
 * gate_out / up_out (fp16 [M, I]) receive the two projections when not NULL.
 * Shapes: groupsize % 128 == 0, H % 128 == 0, I % 128 == 0 (otherwise Q4_ERR_BAD_SHAPE: use three q4_gemv_f16 calls).
 * `workspace`: q4_mlp_decode_workspace_bytes(M, H, I) bytes, 256-byte aligned, all zero before its first use; every
 * call leaves it ready for the next call OF THE SAME (M, H, I) on the same stream (it holds accumulators that end at
 * zero, the hand-over words and a ticket that numbers the launches); clear it before using it for another shape.
 * Calls that share a workspace must not overlap.  The waits inside the kernel are bounded: a wavefront that gives up
 * sets the 32-bit word at workspace + q4_mlp_decode_status_offset(M, H, I) to 1 (the output is then invalid); it is
 * never set when workgroups start in index order, which is how the hardware dispatches them. */
typedef struct {
    const int32_t *qweight;   /* [K/8, N] */
    const int32_t *qzeros;    /* [G, N/8] */
    const void *scales;       /* fp16 [G, N] */
} q4_layer_t;
Q4_API size_t q4_mlp_decode_workspace_bytes(int M, int H, int I);
Q4_API size_t q4_mlp_decode_status_offset(int M, int H, int I);
Q4_API int q4_mlp_decode_f16(const void *x, const q4_layer_t *gate, const q4_layer_t *up, const q4_layer_t *down,
                             int groupsize, void *gate_out, void *up_out, void *y, int M, int H, int I,
                             void *workspace, size_t workspace_bytes, void *stream);

/* q4_gemv_f16 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same product, same arguments
 * minus the workspace: the split-K accumulators live in a device array inside the library (4 MiB per device that
 * runs the library, held until the process ends), so the call needs M * N <= q4_gemv_noalloc_max_outputs()
 * = 524 288 (e.g. 16 rows x 32 768 columns) and returns Q4_ERR_TOO_LARGE beyond that.  It calls no hipMalloc /
 * hipFree and no allocating library routine; it enqueues a small fill kernel that zeroes the accumulators and
 * then the same kernels as q4_gemv_f16, and gives bit-identical results.  All calls on one device share the
 * one array: calls that overlap on a device (two streams, two threads) race -- order them on one stream.
 * The array is that of the CURRENT device: y must live on it (Q4_ERR_RUNTIME otherwise).  The first call on a device
 * looks the array's address up (hipGetSymbolAddress) and must therefore come before stream capture begins; every
 * later call may be captured into a HIP graph and replayed. */
Q4_API size_t q4_gemv_noalloc_max_outputs(void);
Q4_API int q4_gemv_noalloc_f16(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                        const int32_t *g_idx, int groupsize, void *y, int accumulate,
                        int M, int K, int N, int G, void *stream);

/* The same product for an act-order layer whose packed rows were sorted by group with q4_permute_rows.
 * Limits: 1 <= M <= 4, K >= 1024 and M * (2*K + 4096) <= 65536 bytes, i.e. the activation rows fit in LDS
 * (K <= 30720 at M=1, K <= 6144 at M=4).  `qweight_sorted` is the sorted copy, `perm` [K] int32 the
 * permutation it was made with (perm[p] = original index of sorted row p, every value in [0, K): the kernel
 * does not range-check it), `groupsize` = K / G.  x is the ORIGINAL activation matrix: the kernel gathers
 * x[:, perm[p]] itself, through LDS, while its weight loads are in flight, which replaces the separate gather
 * the caller would otherwise run before q4_gemv_f16.  The values are those of the reference's act-order
 * product (quant_cuda_kernel.cu:443-536 with per-row g_idx).  Workspace as for q4_gemv_f16. */
Q4_API int q4_gemv_sorted_f16(const void *x, const int32_t *qweight_sorted, const int32_t *qzeros, const void *scales,
                       const int32_t *perm, int groupsize, void *y, int accumulate,
                       int M, int K, int N, int G,
                       void *workspace, size_t workspace_bytes, void *stream);

/* The same product for the v1 layout (one fp16 scale and one fp16 zero value per column, W = s*q - zero):
 *   y fp16 [M, N] = x fp16 [M, K] @ W,  1 <= M <= 16.
 * Replaces quant_cuda.vecquant4matmul_v1_faster (quant_cuda/quant_cuda.cpp:163-175; kernel
 * quant_cuda_kernel.cu:1244-1302, launcher :1304-1335) as called from matmul_utils_4bit.py:36-56.
 * `scales`, `zeros` fp16 [N], 8-byte aligned.  Workspace as for q4_gemv_f16. */
Q4_API int q4_gemv_v1_f16(const void *x, const int32_t *qweight, const void *scales, const void *zeros, void *y,
                   int accumulate, int M, int K, int N,
                   void *workspace, size_t workspace_bytes, void *stream);

/* Dropout on the adapter input (the reference applies nn.Dropout to x in front of lora_A, models.py:63-66, default
 * p = 0.05, arg_parser.py:48).  The mask is never stored: element (m, c) of the [M, C] adapter input is dropped iff
 * a 15-bit draw that is a pure function of (seed_lo, seed_hi, m, c) is below round(p * 32768); what survives is
 * multiplied by q4_dropout_scale(p) = 32768 / (32768 - round(p * 32768)).  Every entry point below that takes a
 * `const q4_dropout_t *drop` (HOST pointer, read during the call; NULL or p == 0: no dropout) regenerates the same
 * mask from the same descriptor, so forward and backward agree as long as the caller passes the same seed.
 *   draw(m, c): w = ((m * 0x9E3779B1 + seed_lo) ^ ((c >> 1) * 0x85EBCA6B + seed_hi));  w ^= w >> 16;  w *= 0x7FEB352D;
 *               w ^= w >> 15;  w *= 0x846CA68B;  w ^= w >> 16   (32-bit unsigned);   draw = (w >> 16 * (c & 1)) & 0x7FFF.
 * 0 <= p < 1.  q4_dropout_keep_u8 writes the mask itself (1 = kept) for callers that want to see it; C even. */
typedef struct q4_dropout {
    uint32_t seed_lo, seed_hi;
    float p;
} q4_dropout_t;
Q4_API float q4_dropout_scale(float p);
Q4_API int q4_dropout_keep_u8(uint8_t *keep, int M, int C, const q4_dropout_t *drop, void *stream);

/* Forward GEMM, any M >= 1:
 *   y fp16 [M, N] = x fp16 [M, K] @ W  (+ bias fp16 [N])  (+ lora_scale * xa fp16 [M, R] @ Bm [R, N])
 * with fp32 accumulation on MFMA; W tiles are dequantized in LDS and never written to HBM.
 * Replaces vecquant4recons_v2 + torch.matmul(x, buffer) (matmul_utils_4bit.py:114-124),
 * the bias add (autograd_4bit.py:206-207) and, when xa/lora_b are given, the adapter term
 * result += lora_B(lora_A(x)) * scaling (models.py:58-66) where xa = x @ A^T.
 * The adapter matrix is addressed as Bm[r, n] = lora_b[r*ldb_r + n*ldb_n], fp16 or (lora_is_f32 != 0)
 * fp32, so lora_B.weight [N, R] (ldb_r = 1, ldb_n = R) is passed in place: no cast, no transpose.
 * bias, xa, lora_b may be NULL; R is 0 or a multiple of 8, at most 64.
 * Both GEMM entry points need K % 128 == 0, N % 128 == 0, K*N < 2^33, and with g_idx == NULL also
 * groupsize % 64 == 0 and every |scale| < 64 (the sequential-group dequant forms s*q with a fused
 * multiply-add on 1024+q; pass g_idx to lift the restriction on the scales).
 * `workspace` (optional, may be NULL; 256-byte aligned, contents irrelevant): with few output tiles (small M),
 * and for the tiles of a last round that would fill at most half of the CUs, the reduction is split over
 * several workgroups per tile that leave fp32 partial tiles in it, added in a fixed order by a second kernel.
 * q4_gemm_workspace_bytes(fwd, M, K, N) is the size that allows the preferred split (0 when none is wanted); a
 * smaller workspace means fewer splits, none means no split.  Products without adapter term on sequential groups
 * of a multiple of 128 rows take weight-streaming kernels where those are faster: 17..64 rows (grad-input: 17..48)
 * with partial rows in the workspace, and some hundred rows of an output that one round of workgroups covers as a
 * single launch without workspace.  Every route returns the same values for the same inputs on every call. */
Q4_API size_t q4_gemm_workspace_bytes(int fwd, int M, int K, int N);

/* Which kernel family the two GEMM entry points run for a product WITHOUT adapter term, given a workspace of
 * q4_gemm_workspace_bytes(): Q4_ROUTE_TILED (dequantize-into-LDS MFMA tiles), Q4_ROUTE_SKINNY (17..64 rows, partial rows
 * in the workspace), Q4_ROUTE_STREAM (some hundred rows, one launch without workspace), or a negative Q4_ERR_* code for
 * a shape neither entry point takes.  A planning query for callers and tests; it launches nothing.  No counterpart in
 * the reference, whose only route is recons + torch.matmul (matmul_utils_4bit.py:114-127). */
#define Q4_ROUTE_TILED 0
#define Q4_ROUTE_SKINNY 1
#define Q4_ROUTE_STREAM 2
Q4_API int q4_gemm_route(int fwd, int M, int K, int N, int groupsize, int has_g_idx);
Q4_API int q4_gemm_fwd_f16(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                    const int32_t *g_idx, int groupsize, const void *bias,
                    const void *xa, const void *lora_b, int ldb_r, int ldb_n, int lora_is_f32, float lora_scale,
                    int R, void *y, int M, int K, int N, int G,
                    void *workspace, size_t workspace_bytes, void *stream);

/* Backward GEMM (grad of the input):
 *   dx fp16 [M, K] = dy fp16 [M, N] @ W^T  (+ lora_scale * dyb fp16 [M, R] @ Am [R, K])
 * Replaces vecquant4recons_v2 + torch.matmul(grad_output, buffer.T)
 * (matmul_utils_4bit.py:114-126 with transpose=True, called from autograd_4bit.py:53) and the
 * adapter's contribution to grad_input, with dyb = dy @ B and Am[r, k] = lora_a[r*lda_r + k*lda_k]
 * (lora_A.weight [R, K]: lda_r = K, lda_k = 1).
 * With `drop` the adapter term of dx[m, k] is kept (and scaled) only where the dropout mask keeps x[m, k]: the
 * gradient of lora_B(lora_A(dropout(x))) with respect to x. */
Q4_API int q4_gemm_bwd_dx_f16(const void *dy, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                       const int32_t *g_idx, int groupsize,
                       const void *dyb, const void *lora_a, int lda_r, int lda_k, int lora_is_f32, float lora_scale,
                       int R, void *dx, int M, int K, int N, int G, const q4_dropout_t *drop,
                       void *workspace, size_t workspace_bytes, void *stream);

/* The two GEMMs for 2..4 layers that share M, K and the group size (q|k|v, gate|up of a decoder block), each on its
 * own tensors, in ONE launch.  Sequential groups only (no g_idx), every |scale| < 64, M > 128; otherwise, and for
 * shapes with too few tiles to fill the GPU, Q4_ERR_BAD_SHAPE: use the per-layer entry points.
 *   q4_gemm_grouped_fwd_f16:     y_i [M, N_i] = x @ W_i (+ bias_i) (+ lb_scale_i * la_i @ Lb_i), la_i = xa_i [M, R_i];
 *                                act of every layer = x.  No workspace.
 *   q4_gemm_grouped_bwd_dx_f16:  dx [M, K] = sum_i ( dy_i @ W_i^T + mask_i * lb_scale_i * la_i @ Lb_i ), act = dy_i
 *                                [M, N_i], la_i = dyb_i [M, R_i], Lb_i = lora_A_i [R_i, K], mask_i the dropout mask of
 *                                drop_i (NULL: none).  The layers are the shares of one split reduction: fp32 partial
 *                                tiles in `workspace` (q4_gemm_grouped_workspace_bytes), added in a fixed order.
 * They replace the per-projection recons + torch.matmul calls (matmul_utils_4bit.py:114-127) that the reference fuses
 * by concatenating the packed tensors (model_attn_mlp_patch.py:88-100, 180-190), and for the grad-input also the
 * additions with which autograd sums the per-projection results.  Lb_i[r, c] = lb[r*lb_r + c*lb_c], fp16 or fp32. */
typedef struct {
    const void *act;
    const int32_t *qweight, *qzeros;
    const void *scales;
    const void *bias;             /* forward only; fp16 [N] or NULL */
    const void *la, *lb;          /* both NULL: no adapter term */
    int lb_r, lb_c, lb_is_f32;
    float lb_scale;
    int R;                        /* 0 or a multiple of 8, at most 64 */
    void *out;                    /* forward: y_i; grad-input: unused */
    int N;
    const q4_dropout_t *drop;     /* grad-input only */
} q4_gemm_layer_t;
/* 1 when the two entry points below take this shape (enough tiles for one launch), 0 otherwise. */
Q4_API int q4_gemm_grouped_applicable(int fwd, int n_layers, int M, int K, const int *N);
Q4_API size_t q4_gemm_grouped_workspace_bytes(int fwd, int n_layers, int M, int K, const int *N);
Q4_API int q4_gemm_grouped_fwd_f16(const q4_gemm_layer_t *layers, int n_layers, int groupsize, int M, int K, void *stream);
Q4_API int q4_gemm_grouped_bwd_dx_f16(const q4_gemm_layer_t *layers, int n_layers, int groupsize, void *dx, int M, int K,
                                      void *workspace, size_t workspace_bytes, void *stream);

/* Rank-R down projection of the adapter:  out fp16 [M, R] = in fp16 [M, C] @ Wm^T,
 * Wm[j, c] = w[j*w_sr + c*w_sc] (fp16, or fp32 when w_is_f32 != 0).  xa = x @ A^T (w = lora_A.weight,
 * w_sr = K, w_sc = 1) and dyb = dy @ B (w = lora_B.weight, w_sr = 1, w_sc = R): the two products that
 * lora_A(x) and the backward of lora_B perform in the reference (models.py:66).  C % 32 == 0, 1 <= R <= 64.
 * With `drop`: out = dropout(in) @ Wm^T, i.e. lora_A(dropout(x)). */
Q4_API int q4_lora_down_f16(const void *in, const void *w, int w_sr, int w_sc, int w_is_f32, void *out,
                     int M, int C, int R, const q4_dropout_t *drop, void *stream);

/* Gradient of an adapter matrix:  out fp32 [j*o_sr + c*o_sc] = alpha * sum_m p[m, j] * in[m, c]
 * with p fp16 [M, R] and in fp16 [M, C]:  dA = scaling * dyb^T @ x (out = [R, K], o_sr = K, o_sc = 1) and
 * dB = scaling * dy^T @ xa (out = lora_B.weight.grad [N, R], o_sr = 1, o_sc = R) -- what torch autograd
 * computes for the two adapter Linears of models.py:66.  R even, 2 <= R <= 32; C % 8 == 0.
 * `workspace`: q4_lora_grad_workspace_bytes(M, C, R) bytes (0 for small M: then it may be NULL), 256-byte
 * aligned, contents irrelevant before and after the call: it carries fp32 partial sums of row blocks,
 * which a second kernel adds in a fixed order (bit-reproducible).  With `drop`, `in` is replaced by dropout(in)
 * (dA of lora_A(dropout(x))). */
Q4_API size_t q4_lora_grad_workspace_bytes(int M, int C, int R);
Q4_API int q4_lora_grad_f32(const void *p, const void *in, float *out, int o_sr, int o_sc, float alpha,
                     int M, int C, int R, const q4_dropout_t *drop,
                     void *workspace, size_t workspace_bytes, void *stream);

/* Both adapter gradients of a layer in one launch (plus one for the two reductions): problem 1 and problem 2 as
 * for q4_lora_grad_f32, sharing M, R and alpha -- dA from (dyb, x, C1 = K) and dB from (xa, dy, C2 = N) in the
 * backward of models.py:66.  `workspace`: q4_lora_grad_workspace_bytes(M, C1, R) +
 * q4_lora_grad_workspace_bytes(M, C2, R) bytes, 256-byte aligned, contents irrelevant.  `drop1` applies to in1 only
 * (x in dA; xa in dB already carries the mask). */
Q4_API int q4_lora_grad_pair_f32(const void *p1, const void *in1, float *out1, int o1_sr, int o1_sc, int C1,
                          const void *p2, const void *in2, float *out2, int o2_sr, int o2_sc, int C2,
                          float alpha, int M, int R, const q4_dropout_t *drop1,
                          void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* Q4_GPTQ_H */
