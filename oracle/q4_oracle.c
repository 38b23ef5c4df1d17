/* CPU oracle for the 4-bit GPTQ dequant-matmul path, plain C.
 *
 * TEST INFRASTRUCTURE ONLY: linked or loaded by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py, never by the product library.
 *
 * Second, independent restatement of the reference arithmetic (the first is q4_oracle.py):
 * no numpy, and its own software fp16 rounding, so a mistake in either shows up as a
 * disagreement between them.  Reference lines are relative to the reference checkout,
 * src/alpaca_lora_4bit/quant_cuda/quant_cuda_kernel.cu unless another file is named.
 */
#include <stdint.h>
#include <string.h>
#include <stddef.h>

/* ---- IEEE binary16 <-> binary32, round to nearest even, subnormals kept ------------- */
float q4o_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                       /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t q4o_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u)                           /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0u));
    if (absx >= 0x477FF000u)                           /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;     /* 24-bit significand */
    int shift;                                         /* bits dropped from man */
    uint32_t hexp;
    if (e >= -14) { shift = 13; hexp = (uint32_t)(e + 15); }
    else {
        shift = 13 + (-14 - e); hexp = 0;
        if (shift > 25) return sign;                   /* below half the least subnormal */
    }
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    /* kept holds the implicit bit for normals (0x400); adding lets a carry bump the exponent */
    uint32_t out = (hexp ? ((hexp - 1) << 10) : 0u) + kept;
    return (uint16_t)(sign | out);
}

static inline uint16_t mul16(uint16_t a, uint16_t b) {
    return q4o_f32_to_f16(q4o_f16_to_f32(a) * q4o_f16_to_f32(b));   /* product exact in f32 */
}
static inline uint16_t sub16(uint16_t a, uint16_t b) {
    /* difference in double is exact for any two finite halves; one rounding to f16 via f32
       would be a double rounding, so round the double directly through a 2-step that is
       exact here: halves span 2^-24..2^15, the exact difference needs <= 40 bits < 53. */
    double d = (double)q4o_f16_to_f32(a) - (double)q4o_f16_to_f32(b);
    float f = (float)d;                                /* may round: 24 >= 2*11+2 keeps it innocuous */
    return q4o_f32_to_f16(f);
}

/* One element of VecQuant4ReconsV2Kernel<Half> (:1146-1151):
 *   zero = scale * Half(z + 1);  result = scale * Half(q) - zero;   three roundings. */
uint16_t q4o_dequant_scalar(uint16_t scale, int q, int z) {
    uint16_t zero = mul16(scale, q4o_f32_to_f16((float)(z + 1)));
    uint16_t prod = mul16(scale, q4o_f32_to_f16((float)q));
    return sub16(prod, zero);
}

/* Dense dequant, :1127-1153.  qweight [K/8, N], qzeros [G, N/8], scales [G, N] (fp16 bits),
 * g_idx [K], out [K, N] (fp16 bits), row-major, res[n_rows*width + n_cols] (:1152). */
void q4o_dequant_v2(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                    const int32_t *g_idx, uint16_t *out, int K, int N, int G) {
    (void)G;
    int zero_width = N / 8;
    for (int k = 0; k < K; k++) {
        int g = g_idx[k];                                              /* :1143 */
        int shift = (k % 8) * 4;                                       /* :1149 */
        const int32_t *wrow = qweight + (size_t)(k / 8) * N;           /* :1148 */
        for (int n = 0; n < N; n++) {
            uint32_t zw = (uint32_t)qzeros[(size_t)g * zero_width + n / 8];
            int z = (int)((zw >> ((n % 8) * 4)) & 0xFu);               /* :1144-1147 */
            int q = (int)(((uint32_t)wrow[n] >> shift) & 0xFu);        /* :1150-1151 */
            out[(size_t)k * N + n] = q4o_dequant_scalar(scales[(size_t)g * N + n], q, z);
        }
    }
}

/* y[M,N] = x[M,K] @ W[K,N], fp16 inputs, fp32 accumulation: the torch.matmul(x, buffer) of
 * matmul_utils_4bit.py:124 (cuBLAS accumulates fp16 GEMMs in fp32). */
void q4o_matmul(const uint16_t *x, const uint16_t *W, float *y, int M, int K, int N) {
    for (int m = 0; m < M; m++) {
        float *yr = y + (size_t)m * N;
        for (int n = 0; n < N; n++) yr[n] = 0.0f;
        for (int k = 0; k < K; k++) {
            float xv = q4o_f16_to_f32(x[(size_t)m * K + k]);
            const uint16_t *wr = W + (size_t)k * N;
            for (int n = 0; n < N; n++) yr[n] += xv * q4o_f16_to_f32(wr[n]);
        }
    }
}

/* dx[M,K] = dy[M,N] @ W[K,N]^T: torch.matmul(x, buffer.T), matmul_utils_4bit.py:126. */
void q4o_matmul_t(const uint16_t *dy, const uint16_t *W, float *dx, int M, int K, int N) {
    for (int m = 0; m < M; m++)
        for (int k = 0; k < K; k++) {
            const uint16_t *wr = W + (size_t)k * N;
            const uint16_t *dr = dy + (size_t)m * N;
            float acc = 0.0f;
            for (int n = 0; n < N; n++) acc += q4o_f16_to_f32(dr[n]) * q4o_f16_to_f32(wr[n]);
            dx[(size_t)m * K + k] = acc;
        }
}

/* Exhaustive helper: for `ns` scale bit patterns, all 16x16 (q, z) pairs.
 * out[(i*16 + q)*16 + z]. */
void q4o_dequant_table(const uint16_t *scale_bits, int ns, uint16_t *out) {
    for (int i = 0; i < ns; i++)
        for (int q = 0; q < 16; q++)
            for (int z = 0; z < 16; z++)
                out[((size_t)i * 16 + q) * 16 + z] = q4o_dequant_scalar(scale_bits[i], q, z);
}
