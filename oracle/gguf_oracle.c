/* CPU oracle for the quantized-matmul hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference operators so
 * that the HIP kernels can be checked against it.  Nothing that ships may link,
 * import or call it: only the test-suite, the smoke check and the CPU-baseline
 * leg of the benchmark do.
 *
 * What each function follows (paths relative to the reference checkout):
 *   block layouts            csrc/vendor/llama_cpp/common.cuh:78-127
 *   scalar dequantizer       csrc/ck/gguf_decode.cuh:13-31,54-149
 *   IQ2_S codebook           csrc/vendor/llama_cpp/iq2_s_grid.cuh:7-264
 *   q8_1 activation blocks   csrc/mmq_core.cuh:151-209
 *   forward scale algebra    csrc/vendor/llama_cpp/mmq-load-targets.cuh and
 *                            mmq-vec-dot-targets.cuh (Q4_K/Q5_K: :184-195 and
 *                            :46-61; Q3_K: :42-93 and :162-190; IQ2_S: :463-509;
 *                            Q6_K: :378-441 and :298-327)
 *   grad-input definition    csrc/ck/mmq_backward.cuh:496-1004 (dX = dY * bf16(W),
 *                            fp32 accumulate, one bf16 rounding)
 *
 * Pinning status (the checks live in tests/test_oracle.py):
 *   dequantizer   - pinned: hand-built known-answer blocks per type, single-bit
 *                   walks over every field, an independent numpy decoder written
 *                   from the ggml row-dequantizer definition, the codebook
 *                   checksum and its first/last entries.
 *   q8_1          - pinned: invariants (|q|<=127, max|q|=127, |x-d*q|<=d/2,
 *                   zero block), half-away-from-zero ties, brute force.
 *   mmq_forward   - pinned: equals dequantized-weight x dequantized-activation
 *                   matmul computed independently in numpy float64.
 *   mmq_forward_half_scales (Q4_K/Q5_K with the four per-block scale values
 *                   rounded to fp16 where the reference stores them as half2:
 *                   csrc/vendor/llama_cpp/mmq-load-targets.cuh:190-195,
 *                   csrc/mmq_core.cuh:202-203, used at
 *                   mmq-vec-dot-targets.cuh:47-60) - pinned: the rounding helper
 *                   equals numpy's float16 conversion on every finite half
 *                   neighbourhood tested (ties, subnormals, overflow), and the
 *                   function equals a numpy float64 restatement with float16 casts.
 *   linear/grad   - pinned: equal numpy float64 matmuls on the dequantized rows;
 *                   one-hot cotangent reproduces dequantized rows bit for bit.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "iq2s_codebook_packed.h"

#define QK_K 256

enum {
    TGO_Q3_K = 11,
    TGO_Q4_K = 12,
    TGO_Q5_K = 13,
    TGO_Q6_K = 14,
    TGO_IQ2_S = 22,
};

/* ---- scalar conversions ------------------------------------------------- */

static float half_bits_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t expo = (h >> 10) & 0x1fu;
    const uint32_t mant = h & 0x3ffu;
    uint32_t bits;
    if (expo == 0) {
        if (mant == 0) {
            bits = sign;
        } else {
            /* subnormal half: value = mant * 2^-24, exactly representable */
            float value = (float)mant * (1.0f / 16777216.0f);
            memcpy(&bits, &value, 4);
            bits |= sign;
        }
    } else if (expo == 31) {
        bits = sign | 0x7f800000u | (mant << 13);
    } else {
        bits = sign | ((expo + 112u) << 23) | (mant << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* float -> nearest half (ties to even), as bits: overflow to infinity, gradual underflow. */
static uint16_t float_to_half_bits(float f) {
    uint32_t bits;
    memcpy(&bits, &f, 4);
    const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    const uint32_t magnitude = bits & 0x7fffffffu;
    if (magnitude >= 0x7f800000u) {                       /* infinity or NaN */
        return (uint16_t)(sign | 0x7c00u | (magnitude > 0x7f800000u ? 0x200u : 0u));
    }
    if (magnitude >= 0x477ff000u) {                       /* rounds to 65520 or more: infinity */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (magnitude < 0x38800000u) {                        /* below 2^-14: subnormal half, unit 2^-24 */
        float absolute;
        memcpy(&absolute, &magnitude, 4);
        /* (adding 0.5 * 2^23 units and reading the integer is exact round-to-nearest-even here) */
        const volatile float shifted = absolute * 16777216.0f + 8388608.0f;
        const float integer = shifted - 8388608.0f;
        return (uint16_t)(sign | (uint16_t)integer);
    }
    uint32_t rounded = magnitude + 0x0fffu + ((magnitude >> 13) & 1u);   /* nearest even on 13 dropped bits */
    return (uint16_t)(sign | (uint16_t)((rounded - 0x38000000u) >> 13));
}

static float round_to_half(float f) {
    return half_bits_to_float(float_to_half_bits(f));
}

void tgo_oracle_round_to_half(const float * in, int64_t count, float * out) {
    for (int64_t i = 0; i < count; ++i) {
        out[i] = round_to_half(in[i]);
    }
}

static float bf16_bits_to_float(uint16_t b) {
    const uint32_t bits = (uint32_t)b << 16;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* round-to-nearest-even, the rounding of __float2bfloat16 */
static uint16_t float_to_bf16_bits(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((bits >> 16) | 0x0040u);
    }
    const uint32_t lsb = (bits >> 16) & 1u;
    bits += 0x7fffu + lsb;
    return (uint16_t)(bits >> 16);
}

static uint16_t load_u16(const uint8_t * p) {
    return (uint16_t)(p[0] | ((uint16_t)p[1] << 8));
}

/* ---- layouts (common.cuh:78-127) ---------------------------------------- */

int tgo_oracle_block_bytes(int qtype) {
    switch (qtype) {
        case TGO_Q3_K: return 110;  /* hmask[32] qs[64] scales[12] d        */
        case TGO_Q4_K: return 144;  /* d dmin scales[12] qs[128]            */
        case TGO_Q5_K: return 176;  /* d dmin scales[12] qh[32] qs[128]     */
        case TGO_Q6_K: return 210;  /* ql[128] qh[64] scales[16] d          */
        case TGO_IQ2_S: return 82;  /* d qs[64] qh[8] scales[8]             */
        default: return 0;
    }
}

void tgo_oracle_iq2s_grid(uint64_t * out) {
    static const uint64_t magnitude[3] = {0x08, 0x19, 0x2b};
    for (int i = 0; i < TGO_IQ2S_GRID_ENTRIES; ++i) {
        uint64_t word = 0;
        for (int e = 0; e < 8; ++e) {
            const int digit = (tgo_oracle_iq2s_packed[i] >> (2 * e)) & 3;
            word |= magnitude[digit] << (8 * e);
        }
        out[i] = word;
    }
}

/* 6-bit scale / min of the K-quants (gguf_decode.cuh:13-31) */
static int k_scale(const uint8_t * scales, int group) {
    if (group < 4) {
        return scales[group] & 0x3f;
    }
    const int j = group - 4;
    return (scales[8 + j] & 0x0f) | ((scales[j] >> 2) & 0x30);
}

static int k_min(const uint8_t * scales, int group) {
    if (group < 4) {
        return scales[4 + group] & 0x3f;
    }
    const int j = group - 4;
    return (scales[8 + j] >> 4) | ((scales[4 + j] >> 2) & 0x30);
}

/* Integer fields of one weight, shared by the dequantizer and the forward
 * algebra: value = scale_a * (float)quant - scale_b, see decode_value. */
typedef struct {
    int quant;      /* signed integer quant                                  */
    int sub_scale;  /* integer sub-block scale (Q3_K/Q6_K: signed, IQ2_S: s) */
    int sub_min;    /* integer sub-block min (Q4_K/Q5_K), else 0             */
} weight_fields;

static weight_fields fields_q3_k(const uint8_t * b, int i) {
    const uint8_t * hmask = b;
    const uint8_t * qs = b + 32;
    const uint8_t * scales = b + 96;
    const int sg = i >> 4;
    const int low = sg < 8 ? scales[sg] : scales[sg - 8] >> 4;
    const int high = scales[8 + (sg & 3)] >> (2 * (sg >> 2));
    weight_fields f;
    f.sub_scale = ((low & 0x0f) | ((high & 0x03) << 4)) - 32;
    const int rem = i & 127;
    const int lo2 = (qs[(i >> 7) * 32 + (rem & 31)] >> (2 * (rem >> 5))) & 3;
    const int hb = ((hmask[i & 31] >> (i >> 5)) & 1) ^ 1;
    f.quant = lo2 - (hb << 2);
    f.sub_min = 0;
    return f;
}

static weight_fields fields_q4_k(const uint8_t * b, int i) {
    const uint8_t * scales = b + 4;
    const uint8_t * qs = b + 16;
    const int g = i >> 5;
    weight_fields f;
    f.quant = (qs[(g >> 1) * 32 + (i & 31)] >> (4 * (g & 1))) & 0x0f;
    f.sub_scale = k_scale(scales, g);
    f.sub_min = k_min(scales, g);
    return f;
}

static weight_fields fields_q5_k(const uint8_t * b, int i) {
    const uint8_t * scales = b + 4;
    const uint8_t * qh = b + 16;
    const uint8_t * qs = b + 48;
    const int g = i >> 5;
    const int lo = (qs[(g >> 1) * 32 + (i & 31)] >> (4 * (g & 1))) & 0x0f;
    const int hi = (qh[i & 31] >> g) & 1;
    weight_fields f;
    f.quant = lo | (hi << 4);
    f.sub_scale = k_scale(scales, g);
    f.sub_min = k_min(scales, g);
    return f;
}

static weight_fields fields_q6_k(const uint8_t * b, int i) {
    const uint8_t * ql = b;
    const uint8_t * qh = b + 128;
    const int8_t * scales = (const int8_t *)(b + 192);
    const int c = i >> 7;
    const int r = i & 127;
    const int lo = (ql[c * 64 + (r & 63)] >> (4 * (r >> 6))) & 0x0f;
    const int hi = (qh[c * 32 + (i & 31)] >> (2 * ((r >> 5) & 3))) & 3;
    weight_fields f;
    f.quant = (lo | (hi << 4)) - 32;
    f.sub_scale = scales[i >> 4];
    f.sub_min = 0;
    return f;
}

static weight_fields fields_iq2_s(const uint8_t * b, int i) {
    const uint8_t * qs = b + 2;
    const uint8_t * qh = b + 66;
    const uint8_t * scales = b + 74;
    const int gg = i >> 3;
    const int e = i & 7;
    const int hi = (qh[gg >> 2] >> (2 * (gg & 3))) & 3;
    const int idx = qs[gg] | (hi << 8);
    const int digit = (tgo_oracle_iq2s_packed[idx] >> (2 * e)) & 3;
    const int magnitude = digit == 0 ? 8 : (digit == 1 ? 25 : 43);
    const int negative = (qs[32 + gg] >> e) & 1;
    const int sg = i >> 4;
    weight_fields f;
    f.quant = negative ? -magnitude : magnitude;
    f.sub_scale = (scales[sg >> 1] >> (4 * (sg & 1))) & 0x0f;
    f.sub_min = 0;
    return f;
}

static weight_fields fields_of(int qtype, const uint8_t * block, int i) {
    switch (qtype) {
        case TGO_Q3_K: return fields_q3_k(block, i);
        case TGO_Q4_K: return fields_q4_k(block, i);
        case TGO_Q5_K: return fields_q5_k(block, i);
        case TGO_Q6_K: return fields_q6_k(block, i);
        default: return fields_iq2_s(block, i);
    }
}

/* super-block scales: d, and dmin where the type has one */
static void block_scales(int qtype, const uint8_t * block, float * d, float * dmin) {
    *dmin = 0.0f;
    switch (qtype) {
        case TGO_Q3_K: *d = half_bits_to_float(load_u16(block + 108)); break;
        case TGO_Q4_K:
        case TGO_Q5_K:
            *d = half_bits_to_float(load_u16(block));
            *dmin = half_bits_to_float(load_u16(block + 2));
            break;
        case TGO_Q6_K: *d = half_bits_to_float(load_u16(block + 208)); break;
        default: *d = half_bits_to_float(load_u16(block)); break;
    }
}

/* decode_gguf_value<type> (gguf_decode.cuh:54-149); fp32 operation order kept */
static float decode_value(int qtype, const uint8_t * block, int i) {
    float d, dmin;
    block_scales(qtype, block, &d, &dmin);
    const weight_fields f = fields_of(qtype, block, i);
    if (qtype == TGO_Q4_K || qtype == TGO_Q5_K) {
        const volatile float scaled = d * (float)f.sub_scale;
        const volatile float minimum = dmin * (float)f.sub_min;
        const volatile float product = scaled * (float)f.quant;
        return product - minimum;
    }
    if (qtype == TGO_IQ2_S) {
        const volatile float scaled = d * (0.5f + (float)f.sub_scale);
        const volatile float db = scaled * 0.25f;
        return db * (float)f.quant;
    }
    const volatile float scaled = d * (float)f.sub_scale;
    return scaled * (float)f.quant;
}

float tgo_oracle_decode_value(int qtype, const uint8_t * packed_row, int block_index, int value_index) {
    const int bytes = tgo_oracle_block_bytes(qtype);
    return decode_value(qtype, packed_row + (int64_t)block_index * bytes, value_index);
}

void tgo_oracle_dequant_f32(int qtype, const uint8_t * packed, int64_t rows, int64_t k, float * out) {
    const int bytes = tgo_oracle_block_bytes(qtype);
    const int64_t blocks = k / QK_K;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < blocks; ++b) {
            const uint8_t * block = packed + (r * blocks + b) * bytes;
            for (int i = 0; i < QK_K; ++i) {
                out[r * k + b * QK_K + i] = decode_value(qtype, block, i);
            }
        }
    }
}

void tgo_oracle_dequant_bf16(int qtype, const uint8_t * packed, int64_t rows, int64_t k, uint16_t * out) {
    const int bytes = tgo_oracle_block_bytes(qtype);
    const int64_t blocks = k / QK_K;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < blocks; ++b) {
            const uint8_t * block = packed + (r * blocks + b) * bytes;
            for (int i = 0; i < QK_K; ++i) {
                out[r * k + b * QK_K + i] = float_to_bf16_bits(decode_value(qtype, block, i));
            }
        }
    }
}

void tgo_oracle_f32_to_bf16(const float * in, int64_t count, uint16_t * out) {
    for (int64_t i = 0; i < count; ++i) {
        out[i] = float_to_bf16_bits(in[i]);
    }
}

/* ---- q8_1 activation quantizer (mmq_core.cuh:151-209) -------------------- */
/* Per 32 values: amax; d = amax/127 (0 for a zero block); q = roundf(x*(127/amax));
 * sum = fp32 sum of the unquantized values in the reference's order: four values
 * per lane added left to right, then an xor butterfly over eight lanes with
 * offsets 4, 2, 1.  The reference stores (d, sum) as fp16 for Q4_K/Q5_K; the
 * oracle returns the fp32 values and leaves that last rounding to the caller. */
void tgo_oracle_quantize_q8_1(const uint16_t * x, int64_t rows, int64_t k,
                              int8_t * q, float * d_out, float * sum_out) {
    const int64_t blocks = k / 32;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < blocks; ++b) {
            const uint16_t * src = x + r * k + b * 32;
            float v[32];
            float amax = 0.0f;
            for (int i = 0; i < 32; ++i) {
                v[i] = bf16_bits_to_float(src[i]);
                amax = fmaxf(amax, fabsf(v[i]));
            }
            float lane[8];
            for (int t = 0; t < 8; ++t) {
                volatile float s = v[4 * t] + v[4 * t + 1];
                s = s + v[4 * t + 2];
                s = s + v[4 * t + 3];
                lane[t] = s;
            }
            const volatile float a0 = lane[0] + lane[4];
            const volatile float a1 = lane[1] + lane[5];
            const volatile float a2 = lane[2] + lane[6];
            const volatile float a3 = lane[3] + lane[7];
            const volatile float b0 = a0 + a2;
            const volatile float b1 = a1 + a3;
            const float total = b0 + b1;

            const float d = amax == 0.0f ? 0.0f : amax / 127.0f;
            const float d_inv = amax == 0.0f ? 0.0f : 127.0f / amax;
            for (int i = 0; i < 32; ++i) {
                const volatile float scaled = v[i] * d_inv;
                q[r * k + b * 32 + i] = (int8_t)roundf(scaled);
            }
            d_out[r * blocks + b] = d;
            sum_out[r * blocks + b] = total;
        }
    }
}

/* ---- forward: quantized-activation algebra ------------------------------ */
/* y[r,n] = sum over 32-value activation blocks of
 *   Q4_K/Q5_K : (d*sc)*dx*sum(q*qx) - (dmin*m)*sx
 *   Q3_K/Q6_K : per 16 values  (d*sc)*dx*sum(q*qx)
 *   IQ2_S     : per 16 values  ((d*(0.5+s))*0.25)*dx*sum(q*qx)
 * with every scale an fp32 number and the accumulation in float64, so the
 * result is the exact value of the algebra up to float64 rounding. */
void tgo_oracle_mmq_forward(int qtype, const uint16_t * x, const uint8_t * w,
                            int64_t rows, int64_t n, int64_t k, float * y) {
    const int bytes = tgo_oracle_block_bytes(qtype);
    const int64_t blocks = k / QK_K;
    int8_t * qx = (int8_t *)malloc((size_t)(rows * k));
    float * dx = (float *)malloc(sizeof(float) * (size_t)(rows * (k / 32)));
    float * sx = (float *)malloc(sizeof(float) * (size_t)(rows * (k / 32)));
    tgo_oracle_quantize_q8_1(x, rows, k, qx, dx, sx);

#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < n; ++col) {
        int * quant = (int *)malloc(sizeof(int) * (size_t)k);
        float * scale16 = (float *)malloc(sizeof(float) * (size_t)(k / 16));
        float * min32 = (float *)malloc(sizeof(float) * (size_t)(k / 32));
        for (int64_t b = 0; b < blocks; ++b) {
            const uint8_t * block = w + (col * blocks + b) * bytes;
            float d, dmin;
            block_scales(qtype, block, &d, &dmin);
            for (int i = 0; i < QK_K; ++i) {
                const weight_fields f = fields_of(qtype, block, i);
                quant[b * QK_K + i] = f.quant;
                if ((i & 15) == 0) {
                    float s;
                    if (qtype == TGO_IQ2_S) {
                        const volatile float t = d * (0.5f + (float)f.sub_scale);
                        s = t * 0.25f;
                    } else {
                        s = d * (float)f.sub_scale;
                    }
                    scale16[(b * QK_K + i) >> 4] = s;
                }
                if ((i & 31) == 0) {
                    min32[(b * QK_K + i) >> 5] = dmin * (float)f.sub_min;
                }
            }
        }
        for (int64_t r = 0; r < rows; ++r) {
            double acc = 0.0;
            for (int64_t g = 0; g < k / 16; ++g) {
                long dot = 0;
                for (int i = 0; i < 16; ++i) {
                    dot += (long)quant[g * 16 + i] * (long)qx[r * k + g * 16 + i];
                }
                acc += (double)scale16[g] * (double)dx[r * (k / 32) + (g >> 1)] * (double)dot;
                if ((g & 1) == 0) {
                    acc -= (double)min32[g >> 1] * (double)sx[r * (k / 32) + (g >> 1)];
                }
            }
            y[r * n + col] = (float)acc;
        }
        free(quant);
        free(scale16);
        free(min32);
    }
    free(qx);
    free(dx);
    free(sx);
}

/* The same algebra for Q4_K / Q5_K with the reference's fp16 storage of the per-block scale values:
 * weights   (d*sc, -dmin*m) as half2, the product formed in half arithmetic
 *           (csrc/vendor/llama_cpp/mmq-load-targets.cuh:190-195: dm * make_half2(sc, m));
 * activation (d, sum) as half2 (csrc/mmq_core.cuh:202-203);
 * result    sum += dmA.x*dsB.x*dot + dmA.y*dsB.y (mmq-vec-dot-targets.cuh:47-60).
 * Accumulated in float64: what is modelled is the four roundings to fp16, not the reference's fp32
 * summation order. */
void tgo_oracle_mmq_forward_half_scales(int qtype, const uint16_t * x, const uint8_t * w,
                                        int64_t rows, int64_t n, int64_t k, float * y) {
    if (qtype != TGO_Q4_K && qtype != TGO_Q5_K) {
        tgo_oracle_mmq_forward(qtype, x, w, rows, n, k, y);   /* the other formats keep fp32 scales in the reference */
        return;
    }
    const int bytes = tgo_oracle_block_bytes(qtype);
    const int64_t blocks = k / QK_K;
    const int64_t groups = k / 32;
    int8_t * qx = (int8_t *)malloc((size_t)(rows * k));
    float * dx = (float *)malloc(sizeof(float) * (size_t)(rows * groups));
    float * sx = (float *)malloc(sizeof(float) * (size_t)(rows * groups));
    tgo_oracle_quantize_q8_1(x, rows, k, qx, dx, sx);
    for (int64_t i = 0; i < rows * groups; ++i) {
        dx[i] = round_to_half(dx[i]);
        sx[i] = round_to_half(sx[i]);
    }
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < n; ++col) {
        int * quant = (int *)malloc(sizeof(int) * (size_t)k);
        float * scale32 = (float *)malloc(sizeof(float) * (size_t)groups);
        float * min32 = (float *)malloc(sizeof(float) * (size_t)groups);
        for (int64_t b = 0; b < blocks; ++b) {
            const uint8_t * block = w + (col * blocks + b) * bytes;
            float d, dmin;
            block_scales(qtype, block, &d, &dmin);
            for (int i = 0; i < QK_K; ++i) {
                const weight_fields f = fields_of(qtype, block, i);
                quant[b * QK_K + i] = f.quant;
                if ((i & 31) == 0) {
                    /* (a product of two halves is exact in fp32, so rounding it is the half multiply) */
                    scale32[(b * QK_K + i) >> 5] = round_to_half(d * (float)f.sub_scale);
                    min32[(b * QK_K + i) >> 5] = round_to_half(-dmin * (float)f.sub_min);
                }
            }
        }
        for (int64_t r = 0; r < rows; ++r) {
            double acc = 0.0;
            for (int64_t g = 0; g < groups; ++g) {
                long dot = 0;
                for (int i = 0; i < 32; ++i) {
                    dot += (long)quant[g * 32 + i] * (long)qx[r * k + g * 32 + i];
                }
                acc += (double)scale32[g] * (double)dx[r * groups + g] * (double)dot;
                acc += (double)min32[g] * (double)sx[r * groups + g];
            }
            y[r * n + col] = (float)acc;
        }
        free(quant);
        free(scale32);
        free(min32);
    }
    free(qx);
    free(dx);
    free(sx);
}

/* ---- forward / backward against bf16-dequantized weights ---------------- */
/* y = x * bf16(W)^T with float64 accumulation: the "dequantize then matmul"
 * path the forward tolerance is measured against. */
void tgo_oracle_linear_forward(int qtype, const uint16_t * x, const uint8_t * w,
                               int64_t rows, int64_t n, int64_t k, float * y) {
    uint16_t * wb = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(n * k));
    tgo_oracle_dequant_bf16(qtype, w, n, k, wb);
#pragma omp parallel for schedule(static)
    for (int64_t col = 0; col < n; ++col) {
        for (int64_t r = 0; r < rows; ++r) {
            double acc = 0.0;
            for (int64_t i = 0; i < k; ++i) {
                acc += (double)bf16_bits_to_float(x[r * k + i]) *
                       (double)bf16_bits_to_float(wb[col * k + i]);
            }
            y[r * n + col] = (float)acc;
        }
    }
    free(wb);
}

/* dX = dY * bf16(W), float64 accumulation (exact value of the definition). */
void tgo_oracle_grad_input(int qtype, const uint16_t * dy, const uint8_t * w,
                           int64_t rows, int64_t n, int64_t k, float * dx) {
    uint16_t * wb = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(n * k));
    tgo_oracle_dequant_bf16(qtype, w, n, k, wb);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        double * acc = (double *)calloc((size_t)k, sizeof(double));
        for (int64_t col = 0; col < n; ++col) {
            const double g = (double)bf16_bits_to_float(dy[r * n + col]);
            if (g == 0.0) {
                continue;
            }
            for (int64_t i = 0; i < k; ++i) {
                acc[i] += g * (double)bf16_bits_to_float(wb[col * k + i]);
            }
        }
        for (int64_t i = 0; i < k; ++i) {
            dx[r * k + i] = (float)acc[i];
        }
        free(acc);
    }
    free(wb);
}
