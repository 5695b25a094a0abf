/*
 * rt_oracle.c -- CPU oracle for the GGUF quantized-inference hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the CPU baseline that is timed beside them.  Nothing in
 * the shipped library links, imports or calls it.
 *
 * What it restates (paths relative to the reference checkout):
 *   - dequantize-then-dense-matmul shape of the reference CPU path:
 *       example-cli/src/model/formats/tensor_loader.rs:41-67   (decode whole tensor to floats)
 *       src/nn/linear.rs:150-182                               (y = x . W^T, W stored [out,in])
 *       src/tensor/ops/matrix.rs:42-157                        (naive loops, sequential k-sum)
 *   - RMSNorm        src/nn/normalization.rs:652-701  (eps inside the sqrt, gamma * (x / rms))
 *   - SwiGLU         src/nn/activation.rs:378-419     (a * (b * 1/(1+exp(-b))))
 *   - attention      example-cli/src/model/architectures/attention.rs:233-338
 *                    (scores * 1/sqrt(d_k), max-subtracted softmax per row, weights . V)
 *   - block order    example-cli/src/model/architectures/gpt.rs:43-55,192-215
 *                    (x + attn(norm1 x), then x + ffn(norm2 x), final norm, vocab projection)
 *   - greedy pick    example-cli/src/model/sampling.rs:28-35 (temperature 0 / top_k 1 = argmax)
 *   - LE scalar decode  tensor_loader.rs:144-211, IEEE binary16 via the `half` crate :255-269
 *
 * What the reference does NOT hold and this file therefore owns (parity with
 * the reference is unpinned for these; they are pinned by closed forms,
 * exhaustive packer round trips and an independent NumPy decoder in tests/):
 *   - the Q8_0 / Q8_1 / Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q2_K / Q3_K / Q4_K / Q5_K / Q6_K block decoders.  The reference only fixes
 *     type ids and block byte sizes (example-cli/src/model/formats/gguf.rs:78-144)
 *     and decodes every quantized type with a placeholder
 *     (tensor_loader.rs:125-141,213-218).  The layouts below are the public
 *     ggml block definitions.
 *   - RoPE (absent from the reference) and the causal fp16 KV cache
 *     (example-cli/src/model/transformer.rs:221-270 is an unused shell).
 *
 * All arithmetic is IEEE f32 evaluated in the order written; build with
 * -ffp-contract=off so no FMA contraction changes a bit.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_Q4_0 = 2, ORC_Q4_1 = 3, ORC_Q5_0 = 6, ORC_Q5_1 = 7, ORC_Q8_0 = 8, ORC_Q8_1 = 9, ORC_Q2_K = 10, ORC_Q3_K = 11, ORC_Q4_K = 12, ORC_Q5_K = 13, ORC_Q6_K = 14 };

/* ------------------------------------------------------------------ fp16 */

/* IEEE binary16 -> binary32, exact (same mapping as half::f16::to_f32). */
ORC_API float orc_h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
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

/* binary32 -> binary16, round to nearest even (same as half::f16::from_f32). */
ORC_API uint16_t orc_f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 255) return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0));
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exp / inf: correct */
    return (uint16_t)(sign | half);
}

static inline uint16_t rd_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* ------------------------------------------------------- block geometry */

ORC_API int orc_block_elems(int type) {
    switch (type) {
    case ORC_Q8_0: case ORC_Q8_1: case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: return 32;
    case ORC_Q2_K: case ORC_Q3_K: case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: return 256;
    case ORC_F32: case ORC_F16: return 1;
    default: return 0;
    }
}

/* Byte sizes as in gguf.rs:125-144. */
ORC_API int orc_block_bytes(int type) {
    switch (type) {
    case ORC_Q8_0: return 34;
    case ORC_Q8_1: return 36;
    case ORC_Q4_0: return 18;
    case ORC_Q4_1: return 20;
    case ORC_Q5_0: return 22;
    case ORC_Q5_1: return 24;
    case ORC_Q2_K: return 84;   /* the public ggml block; the table at gguf.rs:137 lists 82 */
    case ORC_Q3_K: return 110;
    case ORC_Q4_K: return 144;
    case ORC_Q5_K: return 176;
    case ORC_Q6_K: return 210;
    case ORC_F32: return 4;
    case ORC_F16: return 2;
    default: return 0;
    }
}

/* ---------------------------------------------------------- block decode */

/* Q8_0: { f16 d; i8 qs[32] }   y[i] = d * qs[i] */
static void deq_q8_0(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b));
    const int8_t *qs = (const int8_t *)(b + 2);
    for (int i = 0; i < 32; i++) y[i] = d * (float)qs[i];
}

/* Q8_1: { f16 d; f16 s; i8 qs[32] }   y[i] = d * qs[i]; s = d * sum(qs) is carried for integer dot products and is not
 * part of any value (type id 9 of example-cli/src/model/formats/gguf.rs:89, 36 bytes at :136) */
static void deq_q8_1(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b));
    const int8_t *qs = (const int8_t *)(b + 4);
    for (int i = 0; i < 32; i++) y[i] = d * (float)qs[i];
}

/* Q4_0: { f16 d; u8 qs[16] }   low nibbles are elements 0..15, high nibbles 16..31 */
static void deq_q4_0(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b));
    const uint8_t *qs = b + 2;
    for (int j = 0; j < 16; j++) {
        y[j] = (float)((int)(qs[j] & 0x0F) - 8) * d;
        y[j + 16] = (float)((int)(qs[j] >> 4) - 8) * d;
    }
}

/* Q4_1: { f16 d; f16 m; u8 qs[16] }   y = q * d + m, nibble order as Q4_0 */
static void deq_q4_1(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b)), m = orc_h2f(rd_u16(b + 2));
    const uint8_t *qs = b + 4;
    for (int j = 0; j < 16; j++) {
        y[j] = (float)(qs[j] & 0x0F) * d + m;
        y[j + 16] = (float)(qs[j] >> 4) * d + m;
    }
}

/* Q5_0: { f16 d; u8 qh[4]; u8 qs[16] }   qh read as a little-endian u32: bit j is the fifth bit of element j */
static void deq_q5_0(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b));
    uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
    const uint8_t *qs = b + 6;
    for (int j = 0; j < 16; j++) {
        int x0 = (int)((qs[j] & 0x0F) | (((qh >> j) << 4) & 0x10)) - 16;
        int x1 = (int)((qs[j] >> 4) | ((qh >> (j + 12)) & 0x10)) - 16;
        y[j] = (float)x0 * d;
        y[j + 16] = (float)x1 * d;
    }
}

/* Q5_1: { f16 d; f16 m; u8 qh[4]; u8 qs[16] }   y = q5 * d + m */
static void deq_q5_1(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b)), m = orc_h2f(rd_u16(b + 2));
    uint32_t qh = (uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24);
    const uint8_t *qs = b + 8;
    for (int j = 0; j < 16; j++) {
        int x0 = (int)((qs[j] & 0x0F) | (((qh >> j) << 4) & 0x10));
        int x1 = (int)((qs[j] >> 4) | ((qh >> (j + 12)) & 0x10));
        y[j] = (float)x0 * d + m;
        y[j + 16] = (float)x1 * d + m;
    }
}

/* Q2_K: { u8 scales[16]; u8 qs[64]; f16 d; f16 dmin } (84 B, type id 10, gguf.rs:88): per 16 elements a scale byte whose
 * low nibble scales d and whose high nibble scales dmin; values are 2-bit fields of qs. */
static void deq_q2_k(const uint8_t *b, float *y) {
    const uint8_t *sc = b, *q = b + 16;
    float d = orc_h2f(rd_u16(b + 80)), mn = orc_h2f(rd_u16(b + 82));
    int is = 0;
    for (int n = 0; n < 256; n += 128) {
        int shift = 0;
        for (int j = 0; j < 4; j++) {
            uint8_t s = sc[is++];
            float dl = d * (float)(s & 0xF), ml = mn * (float)(s >> 4);
            for (int l = 0; l < 16; l++) *y++ = dl * (float)((q[l] >> shift) & 3) - ml;
            s = sc[is++];
            dl = d * (float)(s & 0xF); ml = mn * (float)(s >> 4);
            for (int l = 0; l < 16; l++) *y++ = dl * (float)((q[l + 16] >> shift) & 3) - ml;
            shift += 2;
        }
        q += 32;
    }
}

/* Q3_K: { u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d } (110 B, type id 11, gguf.rs:89,138).
 * Sixteen 6-bit scales (stored + 32), one per 16 elements: the low four bits of scale k sit in a nibble of
 * scales[0..7], the high two in a 2-bit field of scales[8..11], gathered here with the word shuffle of the
 * public ggml definition.  Element values are a 2-bit field of qs minus 4 unless its hmask bit is set. */
static void deq_q3_k(const uint8_t *b, float *y) {
    const uint32_t kmask1 = 0x03030303u, kmask2 = 0x0f0f0f0fu;
    const uint8_t *hm = b, *q = b + 32;
    float d_all = orc_h2f(rd_u16(b + 108));
    uint32_t aux[4];
    memcpy(aux, b + 96, 12);
    uint32_t tmp = aux[2];
    aux[2] = ((aux[0] >> 4) & kmask2) | (((tmp >> 4) & kmask1) << 4);
    aux[3] = ((aux[1] >> 4) & kmask2) | (((tmp >> 6) & kmask1) << 4);
    aux[0] = (aux[0] & kmask2) | (((tmp >> 0) & kmask1) << 4);
    aux[1] = (aux[1] & kmask2) | (((tmp >> 2) & kmask1) << 4);
    int8_t scales[16];
    memcpy(scales, aux, 16);
    int is = 0;
    uint8_t m = 1;
    for (int n = 0; n < 256; n += 128) {
        int shift = 0;
        for (int j = 0; j < 4; j++) {
            float dl = d_all * (float)(scales[is++] - 32);
            for (int l = 0; l < 16; l++) *y++ = dl * (float)((int)((q[l] >> shift) & 3) - ((hm[l] & m) ? 0 : 4));
            dl = d_all * (float)(scales[is++] - 32);
            for (int l = 0; l < 16; l++) *y++ = dl * (float)((int)((q[l + 16] >> shift) & 3) - ((hm[l + 16] & m) ? 0 : 4));
            shift += 2;
            m <<= 1;
        }
        q += 32;
    }
}

/* 6-bit scale / min of sub-block j from the 12 packed bytes of a Q4_K super-block. */
static inline void q4k_scale_min(int j, const uint8_t *s, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        *m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* Q4_K: { f16 d; f16 dmin; u8 scales[12]; u8 qs[128] } */
static void deq_q4_k(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b));
    float dmin = orc_h2f(rd_u16(b + 2));
    const uint8_t *scales = b + 4;
    const uint8_t *q = b + 16;
    for (int g = 0; g < 4; g++) {
        uint8_t sc, m;
        q4k_scale_min(2 * g, scales, &sc, &m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        q4k_scale_min(2 * g + 1, scales, &sc, &m);
        float d2 = d * (float)sc, m2 = dmin * (float)m;
        for (int l = 0; l < 32; l++) y[64 * g + l] = d1 * (float)(q[l] & 0x0F) - m1;
        for (int l = 0; l < 32; l++) y[64 * g + 32 + l] = d2 * (float)(q[l] >> 4) - m2;
        q += 32;
    }
}

/*
 * Q5_K: { f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128] } (176 B, type id 13, gguf.rs:91,137): Q4_K with a
 * fifth bit per element; sub-block j takes bit j of qh[l].  Build-owned like the other block decoders
 * (the public ggml definition); the reference holds nothing that pins it: parity unpinned.
 */
static void deq_q5_k(const uint8_t *b, float *y) {
    float d = orc_h2f(rd_u16(b));
    float dmin = orc_h2f(rd_u16(b + 2));
    const uint8_t *scales = b + 4;
    const uint8_t *qh = b + 16;
    const uint8_t *q = b + 48;
    for (int g = 0; g < 4; g++) {
        uint8_t sc, m;
        q4k_scale_min(2 * g, scales, &sc, &m);
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        q4k_scale_min(2 * g + 1, scales, &sc, &m);
        float d2 = d * (float)sc, m2 = dmin * (float)m;
        int u1 = 1 << (2 * g), u2 = 2 << (2 * g);
        for (int l = 0; l < 32; l++) y[64 * g + l] = d1 * (float)((q[l] & 0x0F) + ((qh[l] & u1) ? 16 : 0)) - m1;
        for (int l = 0; l < 32; l++) y[64 * g + 32 + l] = d2 * (float)((q[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
        q += 32;
    }
}

/* Q6_K: { u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d } */
static void deq_q6_k(const uint8_t *b, float *y) {
    const uint8_t *ql = b;
    const uint8_t *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    float d = orc_h2f(rd_u16(b + 208));
    for (int h = 0; h < 2; h++) {
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0x0F) | (((qh[l] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            y[l] = d * (float)sc[is + 0] * (float)q1;
            y[l + 32] = d * (float)sc[is + 2] * (float)q2;
            y[l + 64] = d * (float)sc[is + 4] * (float)q3;
            y[l + 96] = d * (float)sc[is + 6] * (float)q4;
        }
        y += 128; ql += 64; qh += 32; sc += 8;
    }
}

static void deq_row(int type, const uint8_t *row, size_t n_cols, float *y) {
    switch (type) {
    case ORC_Q8_0: for (size_t b = 0; b < n_cols / 32; b++) deq_q8_0(row + 34 * b, y + 32 * b); break;
    case ORC_Q8_1: for (size_t b = 0; b < n_cols / 32; b++) deq_q8_1(row + 36 * b, y + 32 * b); break;
    case ORC_Q4_0: for (size_t b = 0; b < n_cols / 32; b++) deq_q4_0(row + 18 * b, y + 32 * b); break;
    case ORC_Q4_1: for (size_t b = 0; b < n_cols / 32; b++) deq_q4_1(row + 20 * b, y + 32 * b); break;
    case ORC_Q5_0: for (size_t b = 0; b < n_cols / 32; b++) deq_q5_0(row + 22 * b, y + 32 * b); break;
    case ORC_Q5_1: for (size_t b = 0; b < n_cols / 32; b++) deq_q5_1(row + 24 * b, y + 32 * b); break;
    case ORC_Q2_K: for (size_t b = 0; b < n_cols / 256; b++) deq_q2_k(row + 84 * b, y + 256 * b); break;
    case ORC_Q3_K: for (size_t b = 0; b < n_cols / 256; b++) deq_q3_k(row + 110 * b, y + 256 * b); break;
    case ORC_Q4_K: for (size_t b = 0; b < n_cols / 256; b++) deq_q4_k(row + 144 * b, y + 256 * b); break;
    case ORC_Q5_K: for (size_t b = 0; b < n_cols / 256; b++) deq_q5_k(row + 176 * b, y + 256 * b); break;
    case ORC_Q6_K: for (size_t b = 0; b < n_cols / 256; b++) deq_q6_k(row + 210 * b, y + 256 * b); break;
    case ORC_F32: memcpy(y, row, n_cols * 4); break;
    case ORC_F16: for (size_t i = 0; i < n_cols; i++) y[i] = orc_h2f(rd_u16(row + 2 * i)); break;
    }
}

ORC_API size_t orc_row_bytes(int type, size_t n_cols) {
    int be = orc_block_elems(type);
    if (be == 0 || n_cols % (size_t)be) return 0;
    return n_cols / (size_t)be * (size_t)orc_block_bytes(type);
}

/* Whole tensor to dense f32 (tensor_loader.rs:41-67 with real block decode).  Returns 0, or -1 on a bad type / shape. */
ORC_API int orc_dequant_nt(int type, const void *raw, size_t n_rows, size_t n_cols, float *out, int nthreads) {
    size_t rb = orc_row_bytes(type, n_cols);
    if (rb == 0) return -1;
    const uint8_t *p = (const uint8_t *)raw;
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)n_rows; r++) deq_row(type, p + rb * (size_t)r, n_cols, out + n_cols * (size_t)r);
    return 0;
}

ORC_API int orc_dequant(int type, const void *raw, size_t n_rows, size_t n_cols, float *out) {
    return orc_dequant_nt(type, raw, n_rows, n_cols, out, 0);
}

/* ------------------------------------------------------ dense x . W^T */

/*
 * y[m,n] = sum_k x[m,k] * w[n,k], one sequential f32 chain per output element
 * (matrix.rs:63-81 after linear.rs:170 has transposed W).  Threads split rows
 * of W; every output is still one sequential k-sum, so the thread count does
 * not change a bit of the result.
 */
ORC_API void orc_matmul_xwt(const float *x, const float *w, float *y, size_t M, size_t N, size_t K, int nthreads) {
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel for schedule(static)
    for (long n = 0; n < (long)N; n++) {
        const float *wr = w + K * (size_t)n;
        for (size_t m = 0; m < M; m++) {
            const float *xr = x + K * m;
            float sum = 0.0f;
            for (size_t k = 0; k < K; k++) sum = sum + xr[k] * wr[k];
            y[m * N + (size_t)n] = sum;
        }
    }
}

/*
 * Per-tensor affine int8 matmul: QuantizedOps::qmatmul (src/quantization/operations.rs:195-260), the routine
 * OptimizedOps::qmatmul ends in on every device (hardware/mod.rs:25-46 -> hardware/cpu.rs:281-288).
 * a[m,k], b[k,n] row-major; sum = sum_l (a - za)(b - zb) in 64-bit; the result is re-quantized with the
 * output scale sa*sb and zero point 0:  q = round(((float)sum * scale) / scale), clamped to int8
 * (Rust's `as i32` maps NaN to 0 and saturates; f32::round rounds halves away from zero, as roundf does).
 * Returns the output scale.
 */
ORC_API float orc_qmatmul_i8(const int8_t *a, float sa, int za, const int8_t *b, float sb, int zb, size_t m, size_t n, size_t k,
                             int8_t *out) {
    const float scale = sa * sb;
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            long long sum = 0;
            for (size_t l = 0; l < k; l++) sum += (long long)((int)a[i * k + l] - za) * (long long)((int)b[l * n + j] - zb);
            volatile float fp = (float)sum * scale;      /* two roundings, as written in the reference */
            float q = roundf(fp / scale);
            int v;
            if (q != q) v = 0;
            else if (q >= 2147483648.0f) v = 2147483647;
            else if (q <= -2147483648.0f) v = -2147483647 - 1;
            else v = (int)q;
            out[i * n + j] = (int8_t)(v > 127 ? 127 : (v < -128 ? -128 : v));
        }
    return scale;
}

/*
 * Same numbers as orc_dequant + orc_matmul_xwt without materialising W: each
 * row is decoded into a scratch line and consumed at once.  Four rows are
 * interleaved so four independent chains hide the add latency; each chain is
 * still the sequential k-sum.
 */
ORC_API int orc_qgemv(int type, const void *raw, size_t N, size_t K, const float *x, size_t M, float *y, int nthreads) {
    size_t rb = orc_row_bytes(type, K);
    if (rb == 0) return -1;
    const uint8_t *p = (const uint8_t *)raw;
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel
    {
        float *buf = (float *)malloc(4 * K * sizeof(float));
#pragma omp for schedule(static)
        for (long n4 = 0; n4 < (long)((N + 3) / 4); n4++) {
            size_t n0 = (size_t)n4 * 4;
            size_t cnt = N - n0 < 4 ? N - n0 : 4;
            for (size_t j = 0; j < cnt; j++) deq_row(type, p + rb * (n0 + j), K, buf + K * j);
            for (size_t j = cnt; j < 4; j++) memset(buf + K * j, 0, K * sizeof(float));
            const float *w0 = buf, *w1 = buf + K, *w2 = buf + 2 * K, *w3 = buf + 3 * K;
            for (size_t m = 0; m < M; m++) {
                const float *xr = x + K * m;
                float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
                for (size_t k = 0; k < K; k++) {
                    float xv = xr[k];
                    s0 = s0 + xv * w0[k];
                    s1 = s1 + xv * w1[k];
                    s2 = s2 + xv * w2[k];
                    s3 = s3 + xv * w3[k];
                }
                float s[4] = { s0, s1, s2, s3 };
                for (size_t j = 0; j < cnt; j++) y[m * N + n0 + j] = s[j];
            }
        }
        free(buf);
    }
    return 0;
}

/* acc[m] = sum_k xt[k][m] * wr[k]; the m loop is the vector loop, k stays sequential. */
__attribute__((target_clones("avx2", "default")))
static void gemm_row(const float *wr, const float *xt, float *acc, size_t K, size_t M) {
    for (size_t m = 0; m < M; m++) acc[m] = 0.0f;
    for (size_t k = 0; k < K; k++) {
        float wv = wr[k];
        const float *xr = xt + k * M;
        for (size_t m = 0; m < M; m++) acc[m] = acc[m] + xr[m] * wv;
    }
}

/*
 * Batched form for many tokens: X is transposed to [K][M] so the m loop is the
 * vector loop; each (m,n) output is still one sequential k-sum in f32.
 */
ORC_API int orc_qgemm(int type, const void *raw, size_t N, size_t K, const float *x, size_t M, float *y, int nthreads) {
    size_t rb = orc_row_bytes(type, K);
    if (rb == 0) return -1;
    if (M < 4) return orc_qgemv(type, raw, N, K, x, M, y, nthreads);
    const uint8_t *p = (const uint8_t *)raw;
    float *xt = (float *)malloc(K * M * sizeof(float));
    for (size_t m = 0; m < M; m++)
        for (size_t k = 0; k < K; k++) xt[k * M + m] = x[m * K + k];
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel
    {
        float *wr = (float *)malloc(K * sizeof(float));
        float *acc = (float *)malloc(M * sizeof(float));
#pragma omp for schedule(static)
        for (long n = 0; n < (long)N; n++) {
            deq_row(type, p + rb * (size_t)n, K, wr);
            gemm_row(wr, xt, acc, K, M);
            for (size_t m = 0; m < M; m++) y[m * N + (size_t)n] = acc[m];
        }
        free(wr);
        free(acc);
    }
    free(xt);
    return 0;
}

/* f64 accumulation of the same products: the tight yardstick the tolerance tests use. */
ORC_API int orc_qgemv_f64(int type, const void *raw, size_t N, size_t K, const float *x, size_t M, double *y,
                          double *wnorm, int nthreads) {
    size_t rb = orc_row_bytes(type, K);
    if (rb == 0) return -1;
    const uint8_t *p = (const uint8_t *)raw;
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
#pragma omp parallel
    {
        float *wr = (float *)malloc(K * sizeof(float));
#pragma omp for schedule(static)
        for (long n = 0; n < (long)N; n++) {
            deq_row(type, p + rb * (size_t)n, K, wr);
            if (wnorm) {
                double s = 0.0;
                for (size_t k = 0; k < K; k++) s += (double)wr[k] * (double)wr[k];
                wnorm[n] = sqrt(s);
            }
            for (size_t m = 0; m < M; m++) {
                double s = 0.0;
                const float *xr = x + K * m;
                for (size_t k = 0; k < K; k++) s += (double)xr[k] * (double)wr[k];
                y[m * N + (size_t)n] = s;
            }
        }
        free(wr);
    }
    return 0;
}

/* ------------------------------------------------------------ decode ops */

/* normalization.rs:682-696: ms = fold(acc + x^2) / n ; rms = sqrt(ms + eps) ; y = gamma * (x / rms) */
ORC_API void orc_rmsnorm(const float *x, const float *gamma, size_t n, float eps, size_t M, float *y) {
    for (size_t m = 0; m < M; m++) {
        const float *xr = x + n * m;
        float acc = 0.0f;
        for (size_t i = 0; i < n; i++) acc = acc + xr[i] * xr[i];
        float ms = acc / (float)n;
        float rms = sqrtf(ms + eps);
        for (size_t i = 0; i < n; i++) y[n * m + i] = gamma[i] * (xr[i] / rms);
    }
}

/* activation.rs:404-414 with a = up, b = gate:  out = up * (gate * (1 / (1 + exp(-gate)))) */
ORC_API void orc_swiglu(const float *gate, const float *up, size_t n, float *out) {
    for (size_t i = 0; i < n; i++) {
        float b = gate[i];
        float sw = b * (1.0f / (1.0f + expf(-b)));
        out[i] = up[i] * sw;
    }
}

/* inv_freq[i] = theta^(-2i/head_dim), evaluated in double and rounded once to f32. */
ORC_API void orc_rope_inv_freq(int head_dim, float theta, float *inv_freq) {
    for (int i = 0; i < head_dim / 2; i++)
        inv_freq[i] = (float)pow((double)theta, -2.0 * (double)i / (double)head_dim);
}

/* Interleaved-pair rotary embedding in place: pair i of every head turns by pos * inv_freq[i]. */
ORC_API void orc_rope(float *x, int n_heads, int head_dim, int pos, const float *inv_freq) {
    for (int h = 0; h < n_heads; h++) {
        float *v = x + (size_t)h * head_dim;
        for (int i = 0; i < head_dim / 2; i++) {
            float ang = (float)pos * inv_freq[i];
            float c = cosf(ang), s = sinf(ang);
            float a = v[2 * i], b = v[2 * i + 1];
            v[2 * i] = a * c - b * s;
            v[2 * i + 1] = a * s + b * c;
        }
    }
}

/* Cache row for position pos: round f32 -> f16 (RNE). Layout [pos][head][dim]. */
ORC_API void orc_kv_append(uint16_t *cache, const float *v, size_t pos, size_t row_elems) {
    for (size_t i = 0; i < row_elems; i++) cache[pos * row_elems + i] = orc_f2h(v[i]);
}

/*
 * One query against positions 0..n_pos-1 of an fp16 cache laid out
 * [pos][kv head][dim] (attention.rs:233-338 restricted to one query row, which
 * makes the attention causal by construction).  Grouped-query form: query head h
 * reads key / value head h / (n_heads / n_kv_heads); the reference has one head
 * count, which is n_kv_heads == n_heads here.
 */
ORC_API void orc_attn_decode_gqa(const float *q, const uint16_t *kc, const uint16_t *vc, int n_pos, int n_heads, int n_kv_heads,
                                 int head_dim, float *out) {
    float scale = 1.0f / sqrtf((float)head_dim);
    size_t row = (size_t)n_kv_heads * head_dim;
    int group = n_heads / n_kv_heads;
#pragma omp parallel for schedule(static)
    for (int h = 0; h < n_heads; h++) {
        float *sc = (float *)malloc((size_t)n_pos * sizeof(float));
        const float *qh = q + (size_t)h * head_dim;
        size_t kvo = (size_t)(h / group) * head_dim;
        float mx = -INFINITY;
        for (int j = 0; j < n_pos; j++) {
            const uint16_t *kr = kc + (size_t)j * row + kvo;
            float s = 0.0f;
            for (int d = 0; d < head_dim; d++) s = s + qh[d] * orc_h2f(kr[d]);
            s = s * scale;
            sc[j] = s;
            if (s > mx) mx = s;
        }
        float sum = 0.0f;
        for (int j = 0; j < n_pos; j++) { sc[j] = expf(sc[j] - mx); sum = sum + sc[j]; }
        for (int j = 0; j < n_pos; j++) sc[j] = sc[j] / sum;
        for (int d = 0; d < head_dim; d++) {
            float v = 0.0f;
            for (int j = 0; j < n_pos; j++) v = v + sc[j] * orc_h2f(vc[(size_t)j * row + kvo + d]);
            out[(size_t)h * head_dim + d] = v;
        }
        free(sc);
    }
}

ORC_API void orc_attn_decode(const float *q, const uint16_t *kc, const uint16_t *vc, int n_pos, int n_heads,
                             int head_dim, float *out) {
    orc_attn_decode_gqa(q, kc, vc, n_pos, n_heads, n_heads, head_dim, out);
}

/* Greedy pick; ties go to the lowest index. */
ORC_API int orc_argmax(const float *v, size_t n) {
    size_t best = 0;
    for (size_t i = 1; i < n; i++) if (v[i] > v[best]) best = i;
    return (int)best;
}

ORC_API void orc_add(float *x, const float *y, size_t n) { for (size_t i = 0; i < n; i++) x[i] = x[i] + y[i]; }

/* ------------------------------------------------------------ llama loop */

typedef struct {
    int type;
    const void *raw; /* borrowed */
    size_t n_rows, n_cols;
} orc_tensor;

typedef struct {
    int n_layers, hidden, n_heads, n_kv_heads, head_dim, ffn, vocab, max_pos;
    float eps, theta;
    orc_tensor tok_embd, output;
    const float *out_norm;
    orc_tensor *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;
    const float **attn_norm, **ffn_norm;
    uint16_t *kcache, *vcache; /* [layer][pos][hidden] */
    float *inv_freq;
    int nthreads;
} orc_llama;

ORC_API orc_llama *orc_llama_create(int n_layers, int hidden, int n_heads, int ffn, int vocab, int max_pos, float eps,
                                    float theta, int nthreads) {
    orc_llama *m = (orc_llama *)calloc(1, sizeof(orc_llama));
    m->n_layers = n_layers; m->hidden = hidden; m->n_heads = n_heads; m->n_kv_heads = n_heads; m->head_dim = hidden / n_heads;
    m->ffn = ffn; m->vocab = vocab; m->max_pos = max_pos; m->eps = eps; m->theta = theta; m->nthreads = nthreads;
    size_t L = (size_t)n_layers;
    m->wq = calloc(L, sizeof(orc_tensor)); m->wk = calloc(L, sizeof(orc_tensor)); m->wv = calloc(L, sizeof(orc_tensor));
    m->wo = calloc(L, sizeof(orc_tensor)); m->wgate = calloc(L, sizeof(orc_tensor)); m->wup = calloc(L, sizeof(orc_tensor));
    m->wdown = calloc(L, sizeof(orc_tensor));
    m->attn_norm = calloc(L, sizeof(float *)); m->ffn_norm = calloc(L, sizeof(float *));
    m->kcache = calloc(L * (size_t)max_pos * (size_t)hidden, 2);
    m->vcache = calloc(L * (size_t)max_pos * (size_t)hidden, 2);
    m->inv_freq = malloc(sizeof(float) * (size_t)(m->head_dim / 2));
    orc_rope_inv_freq(m->head_dim, theta, m->inv_freq);
    return m;
}

/* Grouped-query attention: n_kv_heads key / value heads (wk, wv have n_kv_heads * head_dim rows).  Before the first forward. */
ORC_API int orc_llama_set_kv_heads(orc_llama *m, int n_kv_heads) {
    if (n_kv_heads <= 0 || m->n_heads % n_kv_heads != 0) return -1;
    m->n_kv_heads = n_kv_heads;
    return 0;
}

ORC_API void orc_llama_destroy(orc_llama *m) {
    if (!m) return;
    free(m->wq); free(m->wk); free(m->wv); free(m->wo); free(m->wgate); free(m->wup); free(m->wdown);
    free(m->attn_norm); free(m->ffn_norm); free(m->kcache); free(m->vcache); free(m->inv_freq); free(m);
}

/* slot: 0 tok_embd, 1 output, 2 out_norm(f32), per layer: 10 q, 11 k, 12 v, 13 o, 14 gate, 15 up, 16 down, 17 attn_norm, 18 ffn_norm */
ORC_API int orc_llama_set_tensor(orc_llama *m, int slot, int layer, int type, const void *raw, size_t n_rows, size_t n_cols) {
    orc_tensor t = { type, raw, n_rows, n_cols };
    if (slot >= 10 && (layer < 0 || layer >= m->n_layers)) return -1;
    switch (slot) {
    case 0: m->tok_embd = t; break;
    case 1: m->output = t; break;
    case 2: m->out_norm = (const float *)raw; break;
    case 10: m->wq[layer] = t; break;
    case 11: m->wk[layer] = t; break;
    case 12: m->wv[layer] = t; break;
    case 13: m->wo[layer] = t; break;
    case 14: m->wgate[layer] = t; break;
    case 15: m->wup[layer] = t; break;
    case 16: m->wdown[layer] = t; break;
    case 17: m->attn_norm[layer] = (const float *)raw; break;
    case 18: m->ffn_norm[layer] = (const float *)raw; break;
    default: return -1;
    }
    return 0;
}

static void lin(const orc_llama *m, const orc_tensor *t, const float *x, size_t M, float *y) {
    orc_qgemm(t->type, t->raw, t->n_rows, t->n_cols, x, M, y, m->nthreads);
}

/*
 * Feed n_tok tokens at positions pos0.. (teacher forced), write logits of every
 * fed token to logits[n_tok][vocab] (or only the last one when last_only).
 * Per token the order is the pre-norm residual block of gpt.rs:43-55 with
 * RMSNorm / RoPE / SwiGLU substituted and a causal fp16 cache.
 */
ORC_API int orc_llama_forward(orc_llama *m, const int *tokens, int n_tok, int pos0, float *logits, int last_only) {
    size_t H = (size_t)m->hidden, F = (size_t)m->ffn, T = (size_t)n_tok;
    if (pos0 < 0 || pos0 + n_tok > m->max_pos) return -1;
    float *x = malloc(T * H * 4), *h = malloc(T * H * 4), *q = malloc(T * H * 4), *k = malloc(T * H * 4);
    float *v = malloc(T * H * 4), *a = malloc(T * H * 4), *o = malloc(T * H * 4);
    float *g = malloc(T * F * 4), *u = malloc(T * F * 4);
    size_t erb = orc_row_bytes(m->tok_embd.type, H);
    for (size_t t = 0; t < T; t++) {
        if (tokens[t] < 0 || tokens[t] >= m->vocab) return -2;
        deq_row(m->tok_embd.type, (const uint8_t *)m->tok_embd.raw + erb * (size_t)tokens[t], H, x + H * t);
    }
    const size_t KD = (size_t)m->n_kv_heads * (size_t)m->head_dim;       /* width of k, v and of a cache row */
    for (int l = 0; l < m->n_layers; l++) {
        uint16_t *kc = m->kcache + (size_t)l * (size_t)m->max_pos * H;
        uint16_t *vc = m->vcache + (size_t)l * (size_t)m->max_pos * H;
        orc_rmsnorm(x, m->attn_norm[l], H, m->eps, T, h);
        lin(m, &m->wq[l], h, T, q); lin(m, &m->wk[l], h, T, k); lin(m, &m->wv[l], h, T, v);
        for (size_t t = 0; t < T; t++) {
            int pos = pos0 + (int)t;
            orc_rope(q + H * t, m->n_heads, m->head_dim, pos, m->inv_freq);
            orc_rope(k + KD * t, m->n_kv_heads, m->head_dim, pos, m->inv_freq);
            orc_kv_append(kc, k + KD * t, (size_t)pos, KD);
            orc_kv_append(vc, v + KD * t, (size_t)pos, KD);
        }
        for (size_t t = 0; t < T; t++)
            orc_attn_decode_gqa(q + H * t, kc, vc, pos0 + (int)t + 1, m->n_heads, m->n_kv_heads, m->head_dim, a + H * t);
        lin(m, &m->wo[l], a, T, o);
        orc_add(x, o, T * H);
        orc_rmsnorm(x, m->ffn_norm[l], H, m->eps, T, h);
        lin(m, &m->wgate[l], h, T, g); lin(m, &m->wup[l], h, T, u);
        orc_swiglu(g, u, T * F, g);
        lin(m, &m->wdown[l], g, T, o);
        orc_add(x, o, T * H);
    }
    orc_rmsnorm(x, m->out_norm, H, m->eps, T, h);
    if (last_only) lin(m, &m->output, h + H * (T - 1), 1, logits);
    else lin(m, &m->output, h, T, logits);
    free(x); free(h); free(q); free(k); free(v); free(a); free(o); free(g); free(u);
    return 0;
}

/* Hardware threads OpenMP would use by default (not affected by earlier nthreads arguments). */
ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_num_procs();
#else
    return 1;
#endif
}
