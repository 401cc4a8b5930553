/*
 * espresso_oracle.c — CPU restatement of the reference's quantized-decode path.
 * TEST INFRASTRUCTURE ONLY; see espresso_oracle.h for the rules and the
 * pinning status of each function.  Build: make -C oracle  (gcc, -ffp-contract=off).
 */
#include "espresso_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ fp16 */

/* IEEE binary32 -> binary16, round-to-nearest-even, subnormals kept, overflow
 * to infinity, NaN kept quiet.  Swift `Float16(x)`
 * (RealModelInferenceEngine.swift:6720-6722, WeightBlob.swift:60). */
uint16_t orc_f32_to_f16(float value) {
    uint32_t f;
    memcpy(&f, &value, 4);
    uint32_t sign = (f >> 16) & 0x8000u;
    uint32_t absf = f & 0x7FFFFFFFu;
    if (absf >= 0x7F800000u) { /* inf / nan */
        if (absf > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((absf >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absf >= 0x477FF000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absf < 0x33000001u) { /* <= 2^-25 rounds to zero (tie at 2^-25 goes to even = 0) */
        return (uint16_t)sign;
    }
    int32_t exp = (int32_t)(absf >> 23) - 127;
    uint32_t mant = (absf & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t half;
    int shift;
    if (exp < -14) {
        /* subnormal half: value = mant * 2^(exp-23); unit = 2^-24 */
        shift = (-14 - exp) + 13;
        half = 0;
    } else {
        shift = 13;
        half = (uint32_t)(exp + 15) << 10;
    }
    uint32_t kept = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (exp >= -14) kept &= 0x3FFu; /* drop the implicit bit for normals */
    uint32_t out = half + kept;
    if (rem > halfway || (rem == halfway && (out & 1u))) out += 1u; /* carries into exponent correctly */
    return (uint16_t)(sign | out);
}

/* binary16 -> binary32, exact (BlobWeightLoader.swift:52). */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t mant = h & 0x3FFu;
    uint32_t f;
    if (exp == 0) {
        if (mant == 0) {
            f = sign;
        } else {
            int e = -1;
            do { mant <<= 1; e++; } while ((mant & 0x400u) == 0);
            f = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        f = sign | 0x7F800000u | (mant << 13);
    } else {
        f = sign | ((exp + 112u) << 23) | (mant << 13);
    }
    float out;
    memcpy(&out, &f, 4);
    return out;
}

void orc_round_f16_vector(float *values, size_t count) {
    for (size_t i = 0; i < count; i++) values[i] = orc_f16_to_f32(orc_f32_to_f16(values[i]));
}

static uint16_t load_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }
static void store_u16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)(v & 0xFF); p[1] = (uint8_t)(v >> 8); }

/* ------------------------------------------------------ GGUF block codecs */

/* ggml dequantize_row_q8_0: block = { fp16 d; int8 qs[32] }, w = d * q. */
void orc_dequant_q8_0(const uint8_t *blocks, size_t elements, float *out) {
    size_t nb = elements / ORC_QK;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = blocks + b * ORC_Q8_0_BLOCK_BYTES;
        float d = orc_f16_to_f32(load_u16(blk));
        const int8_t *qs = (const int8_t *)(blk + 2);
        for (int j = 0; j < ORC_QK; j++) out[b * ORC_QK + j] = (float)qs[j] * d;
    }
}

/* ggml dequantize_row_q4_0: block = { fp16 d; uint8 qs[16] };
 * w[j] = ((qs[j] & 0xF) - 8) * d, w[j+16] = ((qs[j] >> 4) - 8) * d. */
void orc_dequant_q4_0(const uint8_t *blocks, size_t elements, float *out) {
    size_t nb = elements / ORC_QK;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = blocks + b * ORC_Q4_0_BLOCK_BYTES;
        float d = orc_f16_to_f32(load_u16(blk));
        const uint8_t *qs = blk + 2;
        for (int j = 0; j < ORC_QK / 2; j++) {
            int x0 = (qs[j] & 0x0F) - 8;
            int x1 = (qs[j] >> 4) - 8;
            out[b * ORC_QK + j] = (float)x0 * d;
            out[b * ORC_QK + j + ORC_QK / 2] = (float)x1 * d;
        }
    }
}

/* ggml get_scale_min_k4 */
void orc_q4_k_scale_min(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ggml dequantize_row_q4_K: block = { fp16 d; fp16 dmin; uint8 scales[12]; uint8 qs[128] }.
 * w = (d*sc)*nibble - (dmin*m); both products are rounded to fp32 before the
 * multiply/subtract (two roundings, no fused multiply-add). */
void orc_dequant_q4_k(const uint8_t *blocks, size_t elements, float *out) {
    size_t nb = elements / ORC_QK_K;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = blocks + b * ORC_Q4_K_BLOCK_BYTES;
        float d = orc_f16_to_f32(load_u16(blk));
        float dmin = orc_f16_to_f32(load_u16(blk + 2));
        const uint8_t *scales = blk + 4;
        const uint8_t *q = blk + 16;
        float *y = out + b * ORC_QK_K;
        int is = 0;
        for (int j = 0; j < ORC_QK_K; j += 64) {
            uint8_t sc, m;
            orc_q4_k_scale_min(is + 0, scales, &sc, &m);
            volatile float d1 = d * (float)sc;
            volatile float m1 = dmin * (float)m;
            orc_q4_k_scale_min(is + 1, scales, &sc, &m);
            volatile float d2 = d * (float)sc;
            volatile float m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) {
                volatile float p = d1 * (float)(q[l] & 0xF);
                *y++ = p - m1;
            }
            for (int l = 0; l < 32; l++) {
                volatile float p = d2 * (float)(q[l] >> 4);
                *y++ = p - m2;
            }
            q += 32;
            is += 2;
        }
    }
}

/* ggml quantize_row_q8_0_ref: d = amax/127 (fp32), stored as fp16; q = roundf(x * (1/d)). */
void orc_quantize_q8_0(const float *x, size_t elements, uint8_t *blocks) {
    size_t nb = elements / ORC_QK;
    for (size_t b = 0; b < nb; b++) {
        float amax = 0.0f;
        for (int j = 0; j < ORC_QK; j++) {
            float v = fabsf(x[b * ORC_QK + j]);
            if (v > amax) amax = v;
        }
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        uint8_t *blk = blocks + b * ORC_Q8_0_BLOCK_BYTES;
        store_u16(blk, orc_f32_to_f16(d));
        for (int j = 0; j < ORC_QK; j++) {
            float x0 = x[b * ORC_QK + j] * id;
            blk[2 + j] = (uint8_t)(int8_t)roundf(x0);
        }
    }
}

/* ggml quantize_row_q4_0_ref: d = (value of largest |x|) / -8. */
void orc_quantize_q4_0(const float *x, size_t elements, uint8_t *blocks) {
    size_t nb = elements / ORC_QK;
    for (size_t b = 0; b < nb; b++) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < ORC_QK; j++) {
            float v = x[b * ORC_QK + j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        float d = max / -8.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        uint8_t *blk = blocks + b * ORC_Q4_0_BLOCK_BYTES;
        store_u16(blk, orc_f32_to_f16(d));
        for (int j = 0; j < ORC_QK / 2; j++) {
            float x0 = x[b * ORC_QK + j] * id;
            float x1 = x[b * ORC_QK + ORC_QK / 2 + j] * id;
            int q0 = (int)(int8_t)(x0 + 8.5f);
            int q1 = (int)(int8_t)(x1 + 8.5f);
            if (q0 > 15) q0 = 15;
            if (q1 > 15) q1 = 15;
            blk[2 + j] = (uint8_t)(q0 | (q1 << 4));
        }
    }
}

static int nearest_int(float v) { return (int)lrintf(v); }

/* A valid Q4_K packer with the structure of ggml's quantize_row_q4_K_ref but
 * a plain min/max fit per sub-block instead of its iterative search.  Parity is
 * judged on what the packed bytes dequantize to, not on the packer. */
void orc_quantize_q4_k(const float *x, size_t elements, uint8_t *blocks) {
    size_t nb = elements / ORC_QK_K;
    for (size_t b = 0; b < nb; b++) {
        const float *xb = x + b * ORC_QK_K;
        uint8_t *blk = blocks + b * ORC_Q4_K_BLOCK_BYTES;
        float scales[8], mins[8];
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) {
            float lo = xb[32 * j], hi = xb[32 * j];
            for (int l = 1; l < 32; l++) {
                float v = xb[32 * j + l];
                if (v < lo) lo = v;
                if (v > hi) hi = v;
            }
            if (lo > 0.0f) lo = 0.0f;
            scales[j] = (hi - lo) / 15.0f;
            mins[j] = -lo;
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        uint8_t ls[8], lm[8];
        uint8_t *sc12 = blk + 4;
        memset(sc12, 0, 12);
        for (int j = 0; j < 8; j++) {
            int a = nearest_int(inv_scale * scales[j]);
            int m = nearest_int(inv_min * mins[j]);
            if (a > 63) a = 63;
            if (m > 63) m = 63;
            ls[j] = (uint8_t)a;
            lm[j] = (uint8_t)m;
            if (j < 4) {
                sc12[j] = ls[j];
                sc12[j + 4] = lm[j];
            } else {
                sc12[j + 4] = (uint8_t)((ls[j] & 0xF) | ((lm[j] & 0xF) << 4));
                sc12[j - 4] |= (uint8_t)((ls[j] >> 4) << 6);
                sc12[j] |= (uint8_t)((lm[j] >> 4) << 6);
            }
        }
        uint16_t d16 = orc_f32_to_f16(max_scale / 63.0f);
        uint16_t dmin16 = orc_f32_to_f16(max_min / 63.0f);
        store_u16(blk, d16);
        store_u16(blk + 2, dmin16);
        float d = orc_f16_to_f32(d16), dmin = orc_f16_to_f32(dmin16);
        uint8_t L[ORC_QK_K];
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            orc_q4_k_scale_min(j, sc12, &sc, &m);
            float dd = d * (float)sc;
            float dm = dmin * (float)m;
            for (int l = 0; l < 32; l++) {
                int q = 0;
                if (dd != 0.0f) {
                    q = nearest_int((xb[32 * j + l] + dm) / dd);
                    if (q < 0) q = 0;
                    if (q > 15) q = 15;
                }
                L[32 * j + l] = (uint8_t)q;
            }
        }
        uint8_t *qs = blk + 16;
        for (int j = 0; j < ORC_QK_K; j += 64) {
            for (int l = 0; l < 32; l++) qs[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
            qs += 32;
        }
    }
}

size_t orc_format_bytes(int format, size_t elements) {
    switch (format) {
    case ORC_FMT_F32: return elements * 4;
    case ORC_FMT_F16: return elements * 2;
    case ORC_FMT_Q8_0: return elements / ORC_QK * ORC_Q8_0_BLOCK_BYTES;
    case ORC_FMT_Q4_0: return elements / ORC_QK * ORC_Q4_0_BLOCK_BYTES;
    case ORC_FMT_Q4_K: return elements / ORC_QK_K * ORC_Q4_K_BLOCK_BYTES;
    default: return 0;
    }
}

int orc_dequantize(int format, const uint8_t *blocks, size_t elements, float *out) {
    switch (format) {
    case ORC_FMT_F32: memcpy(out, blocks, elements * 4); return 0;
    case ORC_FMT_F16:
        for (size_t i = 0; i < elements; i++) out[i] = orc_f16_to_f32(load_u16(blocks + 2 * i));
        return 0;
    case ORC_FMT_Q8_0: orc_dequant_q8_0(blocks, elements, out); return 0;
    case ORC_FMT_Q4_0: orc_dequant_q4_0(blocks, elements, out); return 0;
    case ORC_FMT_Q4_K: orc_dequant_q4_k(blocks, elements, out); return 0;
    default: return -1;
    }
}

int orc_quantize(int format, const float *x, size_t elements, uint8_t *blocks) {
    switch (format) {
    case ORC_FMT_F32: memcpy(blocks, x, elements * 4); return 0;
    case ORC_FMT_F16:
        for (size_t i = 0; i < elements; i++) store_u16(blocks + 2 * i, orc_f32_to_f16(x[i]));
        return 0;
    case ORC_FMT_Q8_0: orc_quantize_q8_0(x, elements, blocks); return 0;
    case ORC_FMT_Q4_0: orc_quantize_q4_0(x, elements, blocks); return 0;
    case ORC_FMT_Q4_K: orc_quantize_q4_k(x, elements, blocks); return 0;
    default: return -1;
    }
}

/* ----------------------------------------------------------- math helpers */

/* Worker threads for orc_matvec (1 = the single-threaded loop of the reference).  Timing and long walks only:
 * results are bit-identical for every count. */
static int g_threads = 1;
void orc_set_threads(int threads) { g_threads = threads < 1 ? 1 : threads; }
int orc_get_threads(void) { return g_threads; }

/* Dot product in a fixed order: eight interleaved partial sums (element i goes
 * to lane i mod 8, ascending), combined pairwise.  The reference calls
 * Accelerate (vDSP_mmul / vDSP_dotpr / vDSP_svesq), whose order is not
 * published; this order is this restatement's definition. */
static float dot8(const float *a, const float *b, int n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int i = 0;
    for (; i + 8 <= n; i += 8) {
        for (int j = 0; j < 8; j++) acc[j] += a[i + j] * b[i + j];
    }
    for (int j = 0; i < n; i++, j++) acc[j] += a[i] * b[i];
    return ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
}

/* RealModelInferenceEngine.swift:6724-6743 — sumSq, inv = 1/sqrtf(sumSq/n + eps),
 * (x * inv) then * weight. */
void orc_rmsnorm(const float *x, const float *weight, float eps, int n, float *out) {
    float sum_sq = dot8(x, x, n);
    float inv = 1.0f / sqrtf(sum_sq / (float)n + eps);
    for (int i = 0; i < n; i++) {
        float scaled = x[i] * inv;
        out[i] = scaled * weight[i];
    }
}

/* RealModelInferenceEngine.swift:6648-6672 (twin: CPUOps/RMSNorm.swift:183-201). */
void orc_per_head_rmsnorm(float *values, const float *weights, int heads, int head_dim, float eps) {
    for (int h = 0; h < heads; h++) {
        float *v = values + (size_t)h * head_dim;
        float sum_sq = 0.0f;
        for (int l = 0; l < head_dim; l++) sum_sq += v[l] * v[l];
        float inv = 1.0f / sqrtf(sum_sq / (float)head_dim + eps);
        for (int l = 0; l < head_dim; l++) {
            float scale = inv * weights[l];
            v[l] *= scale;
        }
    }
}

/* RealModelInferenceEngine.swift:6674-6718 — y = W x, W row-major [rows, cols]. */
void orc_matvec(const float *matrix, int rows, int cols, const float *x, float *y) {
    /* Rows are independent and each row's sum keeps its order, so the result does not depend on the thread count. */
    int threads = g_threads;
    if (threads > 1 && (size_t)rows * (size_t)cols >= ((size_t)1 << 18)) {
#pragma omp parallel for num_threads(threads) schedule(static)
        for (int r = 0; r < rows; r++) y[r] = dot8(matrix + (size_t)r * cols, x, cols);
        return;
    }
    for (int r = 0; r < rows; r++) y[r] = dot8(matrix + (size_t)r * cols, x, cols);
}

/* RealModelInferenceEngine.swift:6745-6772 (twin: CPUOps/RoPE.swift:56-110). */
void orc_rope_half_split(float *values, int heads, int head_dim, int position, float theta) {
    int half = head_dim / 2;
    for (int h = 0; h < heads; h++) {
        float *v = values + (size_t)h * head_dim;
        for (int p = 0; p < half; p++) {
            float frequency = 1.0f / powf(theta, (float)(2 * p) / (float)head_dim);
            float angle = (float)position * frequency;
            float c = cosf(angle), s = sinf(angle);
            float v0 = v[p], v1 = v[p + half];
            float a = v0 * c, b = v1 * s;
            float e = v0 * s, f = v1 * c;
            v[p] = a - b;
            v[p + half] = e + f;
        }
    }
}

/* RealModelInferenceEngine.swift:6774-6823 — caches are channel-major
 * [kvDim, cacheStride]; sequential sums exactly as the reference's loops. */
void orc_attention_decode(const float *q, const float *k_cache, const float *v_cache, int heads,
                          int kv_heads, int head_dim, int visible, int cache_stride, float *context) {
    int per_kv = heads / (kv_heads > 0 ? kv_heads : 1);
    if (per_kv < 1) per_kv = 1;
    float scale = 1.0f / sqrtf((float)head_dim);
    float *scores = (float *)malloc(sizeof(float) * (size_t)visible);
    for (int h = 0; h < heads; h++) {
        int kvh = h / per_kv;
        if (kvh > kv_heads - 1) kvh = kv_heads - 1;
        const float *qh = q + (size_t)h * head_dim;
        size_t kv_base = (size_t)kvh * head_dim;
        for (int t = 0; t < visible; t++) {
            float dot = 0.0f;
            for (int d = 0; d < head_dim; d++) dot += qh[d] * k_cache[(kv_base + d) * cache_stride + t];
            scores[t] = dot * scale;
        }
        float max_score = scores[0];
        for (int t = 1; t < visible; t++) if (scores[t] > max_score) max_score = scores[t];
        float denom = 0.0f;
        for (int t = 0; t < visible; t++) {
            scores[t] = expf(scores[t] - max_score);
            denom += scores[t];
        }
        float inv_denom = denom > 0.0f ? 1.0f / denom : 0.0f;
        for (int d = 0; d < head_dim; d++) {
            float accum = 0.0f;
            for (int t = 0; t < visible; t++) {
                float w = scores[t] * inv_denom;
                accum += w * v_cache[(kv_base + d) * cache_stride + t];
            }
            context[(size_t)h * head_dim + d] = accum;
        }
    }
    free(scores);
}

/* RealModelInferenceEngine.swift:6825-6827 — the tanh form. */
float orc_silu_tanh(float value) {
    float half = 0.5f * value;
    return half * (1.0f + tanhf(half));
}

int orc_naive_argmax(const float *values, int count) {
    int best = 0;
    for (int i = 1; i < count; i++) if (values[i] > values[best]) best = i;
    return best;
}

/* RealModelInferenceEngine.swift:8182-8275 (public twin: Espresso/PartitionedArgmax.swift:17-123).
 * Blocks of block_size rows; a block is skipped when maxRowNorm*|x| < best;
 * first max inside a block, strict > across blocks: lowest index wins ties. */
int orc_partitioned_argmax(const float *classifier, const float *input, int vocab, int dim,
                           int block_size, int *blocks_pruned) {
    int num_blocks = (vocab + block_size - 1) / block_size;
    float *block_max = (float *)calloc((size_t)num_blocks, sizeof(float));
    for (int b = 0; b < num_blocks; b++) {
        int start = b * block_size, end = start + block_size > vocab ? vocab : start + block_size;
        float bm = 0.0f;
        for (int r = start; r < end; r++) {
            const float *row = classifier + (size_t)r * dim;
            float norm = sqrtf(dot8(row, row, dim));
            if (norm > bm) bm = norm;
        }
        block_max[b] = bm;
    }
    float input_norm = sqrtf(dot8(input, input, dim));
    float *scratch = (float *)malloc(sizeof(float) * (size_t)block_size);
    int best_index = 0, pruned = 0;
    float best_value = -INFINITY;
    for (int b = 0; b < num_blocks; b++) {
        int start = b * block_size, end = start + block_size > vocab ? vocab : start + block_size;
        int count = end - start;
        if (b > 0 && best_value > -INFINITY) {
            float upper = block_max[b] * input_norm;
            if (upper < best_value) { pruned++; continue; }
        }
        orc_matvec(classifier + (size_t)start * dim, count, dim, input, scratch);
        int bi = orc_naive_argmax(scratch, count);
        if (scratch[bi] > best_value) { best_value = scratch[bi]; best_index = start + bi; }
    }
    if (blocks_pruned) *blocks_pruned = pruned;
    free(scratch);
    free(block_max);
    return best_index;
}

/* --------------------------------------------------------------- BLOBFILE */

size_t orc_blob_bytes(size_t elements) { return 128 + elements * 2; }

/* WeightBlob.swift:6-38 */
void orc_blob_build(const float *weights, size_t elements, uint8_t *out) {
    memset(out, 0, 128);
    out[0] = 1;
    out[4] = 2;
    out[64] = 0xEF; out[65] = 0xBE; out[66] = 0xAD; out[67] = 0xDE;
    out[68] = 1;
    uint32_t payload = (uint32_t)(elements * 2);
    for (int i = 0; i < 4; i++) out[72 + i] = (uint8_t)(payload >> (8 * i));
    out[80] = 128;
    for (size_t i = 0; i < elements; i++) store_u16(out + 128 + 2 * i, orc_f32_to_f16(weights[i]));
}

/* BlobWeightLoader.swift:25-90 */
long orc_blob_parse(const uint8_t *data, size_t bytes, float *out, size_t out_capacity) {
    if (bytes < 128) return -1;
    uint32_t magic = 0, size = 0, offset = 0;
    for (int i = 0; i < 4; i++) {
        magic |= (uint32_t)data[64 + i] << (8 * i);
        size |= (uint32_t)data[72 + i] << (8 * i);
        offset |= (uint32_t)data[80 + i] << (8 * i);
    }
    if (magic != 0xDEADBEEFu) return -2;
    if (offset != 128) return -3;
    if (size % 2 != 0) return -5;
    if (bytes < 128 + (size_t)size) return -4;
    size_t count = size / 2;
    if (out) {
        if (count > out_capacity) count = out_capacity;
        for (size_t i = 0; i < count; i++) out[i] = orc_f16_to_f32(load_u16(data + 128 + 2 * i));
    }
    return (long)(size / 2);
}

/* ---------------------------------------------------------------- runtime */

typedef struct {
    float *rms_att, *wq, *wk, *wv, *wo, *rms_ffn, *w1, *w2, *w3, *q_norm, *k_norm;
} orc_layer;

struct orc_llama_runtime {
    orc_llama_config c;
    float *token_embedding, *final_norm, *lm_head;
    orc_layer *layers;
    float **k_cache, **v_cache; /* per layer [kvDim * maxSeq], channel-major (:604-611) */
    float *last_hidden;
    int visible;
    /* scratch */
    float *hidden, *normed, *q, *k, *v, *ctx, *proj, *gate, *up, *act, *down, *logits;
};

struct orc_llama_checkpoint {
    int visible, n_layer;
    size_t cache_count, d_model;
    float *last_hidden;
    float **k_cache, **v_cache;
};

static int attn_dim(const orc_llama_config *c) { return c->n_head * c->head_dim; }
static int kv_dim(const orc_llama_config *c) { return c->n_kv_head * c->head_dim; }

orc_llama_runtime *orc_llama_create(const orc_llama_config *config) {
    /* validateRuntimeConfig, RealModelInferenceEngine.swift:7615-7634 */
    if (config->n_layer <= 0 || config->n_head <= 0 || config->n_kv_head <= 0 || config->d_model <= 0 ||
        config->head_dim <= 0 || config->hidden_dim <= 0 || config->vocab <= 0 || config->max_seq <= 0 ||
        config->n_head % config->n_kv_head != 0 || config->head_dim % 2 != 0)
        return NULL;
    orc_llama_runtime *rt = (orc_llama_runtime *)calloc(1, sizeof(*rt));
    rt->c = *config;
    const orc_llama_config *c = &rt->c;
    rt->layers = (orc_layer *)calloc((size_t)c->n_layer, sizeof(orc_layer));
    rt->k_cache = (float **)calloc((size_t)c->n_layer, sizeof(float *));
    rt->v_cache = (float **)calloc((size_t)c->n_layer, sizeof(float *));
    size_t cache = (size_t)kv_dim(c) * c->max_seq;
    for (int l = 0; l < c->n_layer; l++) {
        rt->k_cache[l] = (float *)calloc(cache, sizeof(float));
        rt->v_cache[l] = (float *)calloc(cache, sizeof(float));
    }
    rt->last_hidden = (float *)calloc((size_t)c->d_model, sizeof(float));
    int widest = c->d_model;
    if (attn_dim(c) > widest) widest = attn_dim(c);
    rt->hidden = (float *)calloc((size_t)c->d_model, sizeof(float));
    rt->normed = (float *)calloc((size_t)c->d_model, sizeof(float));
    rt->q = (float *)calloc((size_t)attn_dim(c), sizeof(float));
    rt->k = (float *)calloc((size_t)kv_dim(c), sizeof(float));
    rt->v = (float *)calloc((size_t)kv_dim(c), sizeof(float));
    rt->ctx = (float *)calloc((size_t)attn_dim(c), sizeof(float));
    rt->proj = (float *)calloc((size_t)c->d_model, sizeof(float));
    rt->gate = (float *)calloc((size_t)c->hidden_dim, sizeof(float));
    rt->up = (float *)calloc((size_t)c->hidden_dim, sizeof(float));
    rt->act = (float *)calloc((size_t)c->hidden_dim, sizeof(float));
    rt->down = (float *)calloc((size_t)c->d_model, sizeof(float));
    rt->logits = (float *)calloc((size_t)c->vocab, sizeof(float));
    return rt;
}

static void free_layer(orc_layer *L) {
    free(L->rms_att); free(L->wq); free(L->wk); free(L->wv); free(L->wo); free(L->rms_ffn);
    free(L->w1); free(L->w2); free(L->w3); free(L->q_norm); free(L->k_norm);
}

void orc_llama_free(orc_llama_runtime *rt) {
    if (!rt) return;
    for (int l = 0; l < rt->c.n_layer; l++) {
        free_layer(&rt->layers[l]);
        free(rt->k_cache[l]);
        free(rt->v_cache[l]);
    }
    free(rt->layers); free(rt->k_cache); free(rt->v_cache);
    free(rt->token_embedding); free(rt->final_norm); free(rt->lm_head); free(rt->last_hidden);
    free(rt->hidden); free(rt->normed); free(rt->q); free(rt->k); free(rt->v); free(rt->ctx);
    free(rt->proj); free(rt->gate); free(rt->up); free(rt->act); free(rt->down); free(rt->logits);
    free(rt);
}

int orc_llama_set_weight(orc_llama_runtime *rt, int layer, int slot, const float *data, size_t count) {
    const orc_llama_config *c = &rt->c;
    float **dst = NULL;
    size_t expected = 0;
    size_t d = (size_t)c->d_model;
    switch (slot) {
    case ORC_W_TOKEN_EMBEDDING: dst = &rt->token_embedding; expected = (size_t)c->vocab * d; break;
    case ORC_W_FINAL_NORM: dst = &rt->final_norm; expected = d; break;
    case ORC_W_LM_HEAD: dst = &rt->lm_head; expected = (size_t)c->vocab * d; break;
    default:
        if (layer < 0 || layer >= c->n_layer) return -1;
        {
            orc_layer *L = &rt->layers[layer];
            switch (slot) {
            case ORC_W_RMS_ATT: dst = &L->rms_att; expected = d; break;
            case ORC_W_WQ: dst = &L->wq; expected = d * attn_dim(c); break;
            case ORC_W_WK: dst = &L->wk; expected = d * kv_dim(c); break;
            case ORC_W_WV: dst = &L->wv; expected = d * kv_dim(c); break;
            case ORC_W_WO: dst = &L->wo; expected = d * attn_dim(c); break;
            case ORC_W_RMS_FFN: dst = &L->rms_ffn; expected = d; break;
            case ORC_W_W1: dst = &L->w1; expected = d * c->hidden_dim; break;
            case ORC_W_W2: dst = &L->w2; expected = d * c->hidden_dim; break;
            case ORC_W_W3: dst = &L->w3; expected = d * c->hidden_dim; break;
            case ORC_W_Q_NORM: dst = &L->q_norm; expected = (size_t)c->head_dim; break;
            case ORC_W_K_NORM: dst = &L->k_norm; expected = (size_t)c->head_dim; break;
            default: return -1;
            }
        }
    }
    if (count != expected) return -2;
    free(*dst);
    *dst = (float *)malloc(sizeof(float) * count);
    memcpy(*dst, data, sizeof(float) * count);
    return 0;
}

/* Same as orc_llama_set_weight for a matrix given as GGUF blocks: dequantised straight into the runtime's own
 * buffer (no intermediate fp32 copy of an 8B-parameter model on the caller's side). */
int orc_llama_set_weight_blocks(orc_llama_runtime *rt, int layer, int slot, int format, const uint8_t *blocks, size_t count) {
    float *values = (float *)malloc(sizeof(float) * count);
    if (!values) return -4;
    if (orc_dequantize(format, blocks, count, values) != 0) { free(values); return -3; }
    /* hand the buffer over instead of copying it */
    const orc_llama_config *c = &rt->c;
    float **dst = NULL;
    size_t expected = 0;
    size_t d = (size_t)c->d_model;
    switch (slot) {
    case ORC_W_TOKEN_EMBEDDING: dst = &rt->token_embedding; expected = (size_t)c->vocab * d; break;
    case ORC_W_LM_HEAD: dst = &rt->lm_head; expected = (size_t)c->vocab * d; break;
    default:
        if (layer < 0 || layer >= c->n_layer) { free(values); return -1; }
        {
            orc_layer *L = &rt->layers[layer];
            switch (slot) {
            case ORC_W_WQ: dst = &L->wq; expected = d * attn_dim(c); break;
            case ORC_W_WK: dst = &L->wk; expected = d * kv_dim(c); break;
            case ORC_W_WV: dst = &L->wv; expected = d * kv_dim(c); break;
            case ORC_W_WO: dst = &L->wo; expected = d * attn_dim(c); break;
            case ORC_W_W1: dst = &L->w1; expected = d * c->hidden_dim; break;
            case ORC_W_W2: dst = &L->w2; expected = d * c->hidden_dim; break;
            case ORC_W_W3: dst = &L->w3; expected = d * c->hidden_dim; break;
            default: free(values); return -1;
            }
        }
    }
    if (count != expected) { free(values); return -2; }
    free(*dst);
    *dst = values;
    return 0;
}

/* Switches the activation mode of an existing runtime (weights stay): 0 = the reference's default, fp32 activations
 * into every matrix product; 1 = rounded to fp16 first, as the GPU kernels take them. */
void orc_llama_set_gemv_inputs_fp16(orc_llama_runtime *rt, int enabled) { rt->c.gemv_inputs_fp16 = enabled; }

/* :616-635 */
void orc_llama_reset(orc_llama_runtime *rt) {
    size_t cache = (size_t)kv_dim(&rt->c) * rt->c.max_seq;
    for (int l = 0; l < rt->c.n_layer; l++) {
        memset(rt->k_cache[l], 0, cache * sizeof(float));
        memset(rt->v_cache[l], 0, cache * sizeof(float));
    }
    memset(rt->last_hidden, 0, sizeof(float) * (size_t)rt->c.d_model);
    rt->visible = 0;
}

static void maybe_round(const orc_llama_config *c, float *v, int n) {
    if (c->round_intermediates_fp16) orc_round_f16_vector(v, (size_t)n);
}
/* gemv_inputs_fp16: 0 = the reference's default (fp32 activations into every matrix product); 1 = every product's input is
 * rounded to fp16 first; any other value is a mask of the inputs that are rounded (2 attention norm, 4 attention context,
 * 8 FFN norm, 16 SiLU(gate)*up, 32 final norm), for measuring what each rounding contributes. */
enum { IN_ATT_NORM = 2, IN_CONTEXT = 4, IN_FFN_NORM = 8, IN_ACT = 16, IN_FINAL_NORM = 32 };
static void gemv_input(const orc_llama_config *c, float *v, int n, int which) {
    if (c->gemv_inputs_fp16 == 1 || (c->gemv_inputs_fp16 & which)) orc_round_f16_vector(v, (size_t)n);
}

/* forwardToken, :686-823 (identical body at :6221-6347). */
static int forward_token(orc_llama_runtime *rt, uint32_t token, int position) {
    const orc_llama_config *c = &rt->c;
    if ((int64_t)token >= (int64_t)c->vocab) return -3;
    int d = c->d_model, ad = attn_dim(c), kd = kv_dim(c), S = c->max_seq;
    memcpy(rt->hidden, rt->token_embedding + (size_t)token * d, sizeof(float) * (size_t)d);
    for (int l = 0; l < c->n_layer; l++) {
        orc_layer *L = &rt->layers[l];
        orc_rmsnorm(rt->hidden, L->rms_att, c->norm_eps, d, rt->normed);
        gemv_input(c, rt->normed, d, IN_ATT_NORM);
        orc_matvec(L->wq, ad, d, rt->normed, rt->q); maybe_round(c, rt->q, ad);
        orc_matvec(L->wk, kd, d, rt->normed, rt->k); maybe_round(c, rt->k, kd);
        orc_matvec(L->wv, kd, d, rt->normed, rt->v); maybe_round(c, rt->v, kd);
        if (L->q_norm) orc_per_head_rmsnorm(rt->q, L->q_norm, c->n_head, c->head_dim, c->norm_eps);
        if (L->k_norm) orc_per_head_rmsnorm(rt->k, L->k_norm, c->n_kv_head, c->head_dim, c->norm_eps);
        orc_rope_half_split(rt->q, c->n_head, c->head_dim, position, c->rope_theta); maybe_round(c, rt->q, ad);
        orc_rope_half_split(rt->k, c->n_kv_head, c->head_dim, position, c->rope_theta); maybe_round(c, rt->k, kd);
        if (c->kv_fp16) { orc_round_f16_vector(rt->k, (size_t)kd); orc_round_f16_vector(rt->v, (size_t)kd); }
        for (int ch = 0; ch < kd; ch++) {
            rt->k_cache[l][(size_t)ch * S + position] = rt->k[ch];
            rt->v_cache[l][(size_t)ch * S + position] = rt->v[ch];
        }
        orc_attention_decode(rt->q, rt->k_cache[l], rt->v_cache[l], c->n_head, c->n_kv_head, c->head_dim,
                             position + 1, S, rt->ctx);
        gemv_input(c, rt->ctx, ad, IN_CONTEXT);
        orc_matvec(L->wo, d, ad, rt->ctx, rt->proj);
        for (int i = 0; i < d; i++) rt->proj[i] = rt->hidden[i] + rt->proj[i];
        maybe_round(c, rt->proj, d);
        orc_rmsnorm(rt->proj, L->rms_ffn, c->norm_eps, d, rt->normed);
        gemv_input(c, rt->normed, d, IN_FFN_NORM);
        orc_matvec(L->w1, c->hidden_dim, d, rt->normed, rt->gate);
        orc_matvec(L->w3, c->hidden_dim, d, rt->normed, rt->up);
        for (int i = 0; i < c->hidden_dim; i++) rt->act[i] = orc_silu_tanh(rt->gate[i]) * rt->up[i];
        gemv_input(c, rt->act, c->hidden_dim, IN_ACT);
        orc_matvec(L->w2, d, c->hidden_dim, rt->act, rt->down);
        for (int i = 0; i < d; i++) rt->hidden[i] = rt->proj[i] + rt->down[i];
        maybe_round(c, rt->hidden, d);
    }
    return 0;
}

/* :672-680 */
int orc_llama_advance(orc_llama_runtime *rt, uint32_t token) {
    if (rt->visible >= rt->c.max_seq) return -2;
    int rc = forward_token(rt, token, rt->visible);
    if (rc != 0) return rc;
    memcpy(rt->last_hidden, rt->hidden, sizeof(float) * (size_t)rt->c.d_model);
    maybe_round(&rt->c, rt->last_hidden, rt->c.d_model);
    rt->visible += 1;
    return 0;
}

/* :637-645 */
int orc_llama_prefill(orc_llama_runtime *rt, const uint32_t *tokens, int count) {
    if (count <= 0) return -1;
    orc_llama_reset(rt);
    for (int i = 0; i < count; i++) {
        int rc = orc_llama_advance(rt, tokens[i]);
        if (rc != 0) return rc;
    }
    return 0;
}

static void final_normed(orc_llama_runtime *rt) {
    orc_rmsnorm(rt->last_hidden, rt->final_norm, rt->c.norm_eps, rt->c.d_model, rt->normed);
    gemv_input(&rt->c, rt->normed, rt->c.d_model, IN_FINAL_NORM);
}

/* :663-670 + :825-849; classifierArgmaxBlockSize = 4000 */
uint32_t orc_llama_select_greedy(orc_llama_runtime *rt) {
    final_normed(rt);
    return (uint32_t)orc_partitioned_argmax(rt->lm_head, rt->normed, rt->c.vocab, rt->c.d_model, 4000, NULL);
}

void orc_llama_logits(orc_llama_runtime *rt, float *logits) {
    final_normed(rt);
    orc_matvec(rt->lm_head, rt->c.vocab, rt->c.d_model, rt->normed, logits);
}

float orc_llama_top2_margin(orc_llama_runtime *rt) {
    orc_llama_logits(rt, rt->logits);
    int best = orc_naive_argmax(rt->logits, rt->c.vocab);
    float second = -INFINITY;
    for (int i = 0; i < rt->c.vocab; i++)
        if (i != best && rt->logits[i] > second) second = rt->logits[i];
    return rt->logits[best] - second;
}

int orc_llama_visible(const orc_llama_runtime *rt) { return rt->visible; }
void orc_llama_set_visible(orc_llama_runtime *rt, int visible) { rt->visible = visible; }
const float *orc_llama_last_hidden(const orc_llama_runtime *rt) { return rt->last_hidden; }

orc_llama_checkpoint *orc_llama_capture(const orc_llama_runtime *rt) {
    orc_llama_checkpoint *ck = (orc_llama_checkpoint *)calloc(1, sizeof(*ck));
    ck->visible = rt->visible;
    ck->n_layer = rt->c.n_layer;
    ck->d_model = (size_t)rt->c.d_model;
    ck->cache_count = (size_t)kv_dim(&rt->c) * rt->c.max_seq;
    ck->last_hidden = (float *)malloc(sizeof(float) * ck->d_model);
    memcpy(ck->last_hidden, rt->last_hidden, sizeof(float) * ck->d_model);
    ck->k_cache = (float **)calloc((size_t)ck->n_layer, sizeof(float *));
    ck->v_cache = (float **)calloc((size_t)ck->n_layer, sizeof(float *));
    for (int l = 0; l < ck->n_layer; l++) {
        ck->k_cache[l] = (float *)malloc(sizeof(float) * ck->cache_count);
        ck->v_cache[l] = (float *)malloc(sizeof(float) * ck->cache_count);
        memcpy(ck->k_cache[l], rt->k_cache[l], sizeof(float) * ck->cache_count);
        memcpy(ck->v_cache[l], rt->v_cache[l], sizeof(float) * ck->cache_count);
    }
    return ck;
}

void orc_llama_rollback(orc_llama_runtime *rt, const orc_llama_checkpoint *ck) {
    rt->visible = ck->visible;
    memcpy(rt->last_hidden, ck->last_hidden, sizeof(float) * ck->d_model);
    for (int l = 0; l < ck->n_layer; l++) {
        memcpy(rt->k_cache[l], ck->k_cache[l], sizeof(float) * ck->cache_count);
        memcpy(rt->v_cache[l], ck->v_cache[l], sizeof(float) * ck->cache_count);
    }
}

void orc_llama_checkpoint_free(orc_llama_checkpoint *ck) {
    if (!ck) return;
    for (int l = 0; l < ck->n_layer; l++) { free(ck->k_cache[l]); free(ck->v_cache[l]); }
    free(ck->k_cache); free(ck->v_cache); free(ck->last_hidden); free(ck);
}

/* generateIncrementalExactCPULlama, :6349-6431 with temperature 0;
 * effectiveMaxTokens = min(maxTokens, maxSeq - promptLen) (:1425-1426). */
int orc_llama_generate(orc_llama_runtime *rt, const uint32_t *prompt, int prompt_count,
                       int max_tokens, uint32_t *out_tokens, float *out_min_margin) {
    if (prompt_count <= 0) return -1;
    if (prompt_count >= rt->c.max_seq) return -2;
    int eff = max_tokens;
    if (eff > rt->c.max_seq - prompt_count) eff = rt->c.max_seq - prompt_count;
    int rc = orc_llama_prefill(rt, prompt, prompt_count);
    if (rc != 0) return rc;
    int generated = 0, all = prompt_count;
    float min_margin = INFINITY;
    while (generated < eff) {
        uint32_t next = orc_llama_select_greedy(rt);
        if (out_min_margin) {
            float m = orc_llama_top2_margin(rt);
            if (m < min_margin) min_margin = m;
        }
        if (rt->c.eos_token >= 0 && next == (uint32_t)rt->c.eos_token) {
            out_tokens[generated++] = next;
            break;
        }
        out_tokens[generated++] = next;
        all++;
        if (generated >= eff || all >= rt->c.max_seq) break;
        rc = orc_llama_advance(rt, next); /* position = all - 1 = visible */
        if (rc != 0) return rc;
    }
    if (out_min_margin) *out_min_margin = min_margin;
    return generated;
}

/* generateIncrementalExactTwoTokenDraftLlama, :6014-6190. */
int orc_llama_generate_two_token(orc_llama_runtime *full, orc_llama_runtime *draft,
                                 const uint32_t *prompt, int prompt_count, int max_tokens,
                                 uint32_t *out_tokens, orc_two_token_stats *stats) {
    if (prompt_count <= 0) return -1;
    if (prompt_count >= full->c.max_seq) return -2;
    int eff = max_tokens;
    if (eff > full->c.max_seq - prompt_count) eff = full->c.max_seq - prompt_count;
    int rc;
    if ((rc = orc_llama_prefill(full, prompt, prompt_count)) != 0) return rc;
    if ((rc = orc_llama_prefill(draft, prompt, prompt_count)) != 0) return rc;
    int generated = 0, all = prompt_count, max_seq = full->c.max_seq, eos = full->c.eos_token;
    int passes = 0, committed_total = 0, accepted_total = 0;
    if (stats) memset(stats, 0, sizeof(*stats));
    if (eff <= 0) return 0;

    uint32_t first = orc_llama_select_greedy(full);
    if (eos >= 0 && first == (uint32_t)eos) { out_tokens[generated++] = first; return generated; }
    out_tokens[generated++] = first; all++;
    if (generated >= eff || all >= max_seq) return generated;
    if ((rc = orc_llama_advance(full, first)) != 0) return rc;
    if ((rc = orc_llama_advance(draft, first)) != 0) return rc;

    while (generated < eff && all < max_seq) {
        passes++;
        int remaining = eff - generated;
        if (max_seq - all < remaining) remaining = max_seq - all;
        orc_llama_checkpoint *ck = orc_llama_capture(draft);
        uint32_t p0 = orc_llama_select_greedy(draft);
        if ((rc = orc_llama_advance(draft, p0)) != 0) { orc_llama_checkpoint_free(ck); return rc; }
        uint32_t e0 = orc_llama_select_greedy(full);
        int accepted = 0, committed = 0;
        if (e0 == p0) accepted++; else orc_llama_rollback(draft, ck);
        orc_llama_checkpoint_free(ck);
        out_tokens[generated++] = e0; all++; committed++;
        if (eos >= 0 && e0 == (uint32_t)eos) { committed_total += committed; accepted_total += accepted; break; }
        if ((rc = orc_llama_advance(full, e0)) != 0) return rc;
        if (e0 != p0 && (rc = orc_llama_advance(draft, e0)) != 0) return rc;
        if (generated >= eff || all >= max_seq || remaining <= 1) {
            committed_total += committed; accepted_total += accepted;
            continue;
        }
        uint32_t p1 = orc_llama_select_greedy(draft);
        uint32_t e1 = orc_llama_select_greedy(full);
        if (e1 == p1) accepted++;
        out_tokens[generated++] = e1; all++; committed++;
        if (eos >= 0 && e1 == (uint32_t)eos) { committed_total += committed; accepted_total += accepted; break; }
        if ((rc = orc_llama_advance(full, e1)) != 0) return rc;
        if ((rc = orc_llama_advance(draft, e1)) != 0) return rc;
        committed_total += committed; accepted_total += accepted;
    }
    if (stats) { stats->passes = passes; stats->committed_total = committed_total; stats->accepted_total = accepted_total; }
    return generated;
}

/* ---- INT4 classifier (TensorBufferINT4.swift:53-135, INT4Classifier.swift:40-160) -------------------- */
static int int4_q(float v, float row_min, float scale) {
    int q = (int)roundf((v - row_min) / scale);
    return q < 0 ? 0 : (q > 15 ? 15 : q);
}

void orc_int4_quantize(const float *src, int rows, int cols, uint8_t *packed, float *scales, float *biases) {
    const int bpr = (cols + 1) / 2;
    memset(packed, 0, (size_t)rows * bpr);
    for (int r = 0; r < rows; r++) {
        const float *row = src + (size_t)r * cols;
        float row_min = row[0], row_max = row[0];
        for (int c = 1; c < cols; c++) {
            if (row[c] < row_min) row_min = row[c];
            if (row[c] > row_max) row_max = row[c];
        }
        const float range = row_max - row_min;
        const float scale = range < 1e-10f ? 1.0f : range / 15.0f;
        scales[r] = scale;
        biases[r] = row_min;
        uint8_t *out = packed + (size_t)r * bpr;
        int c = 0, b = 0;
        while (c + 1 < cols) {
            out[b++] = (uint8_t)((int4_q(row[c], row_min, scale) << 4) | int4_q(row[c + 1], row_min, scale));
            c += 2;
        }
        if (c < cols) out[b] = (uint8_t)(int4_q(row[c], row_min, scale) << 4);
    }
}

float orc_int4_input_sum(const float *input, int dim) {
    float s = 0.0f;
    for (int i = 0; i < dim; i++) s += input[i];
    return s;
}

static float int4_row_dot(const uint8_t *row, float scale, float bias, const float *input, float input_sum, int dim) {
    float dot = 0.0f;
    const int pairs = dim / 2;
    for (int i = 0; i < pairs; i++) {
        const float hi = (float)((row[i] >> 4) & 0xF), lo = (float)(row[i] & 0xF);
        dot += hi * input[2 * i] + lo * input[2 * i + 1];
    }
    if (dim & 1) dot += (float)((row[pairs] >> 4) & 0xF) * input[dim - 1];
    return scale * dot + bias * input_sum;
}

void orc_int4_matvec(const uint8_t *packed, const float *scales, const float *biases, const float *input,
                     int vocab, int dim, float *out) {
    const int bpr = (dim + 1) / 2;
    const float sum = orc_int4_input_sum(input, dim);
    for (int r = 0; r < vocab; r++) out[r] = int4_row_dot(packed + (size_t)r * bpr, scales[r], biases[r], input, sum, dim);
}

int orc_int4_argmax(const uint8_t *packed, const float *scales, const float *biases, const float *input,
                    int vocab, int dim) {
    const int bpr = (dim + 1) / 2;
    const float sum = orc_int4_input_sum(input, dim);
    int best = 0;
    float best_value = -3.4028234663852886e38f;
    for (int r = 0; r < vocab; r++) {
        const float logit = int4_row_dot(packed + (size_t)r * bpr, scales[r], biases[r], input, sum, dim);
        if (logit > best_value) { best_value = logit; best = r; }
    }
    return best;
}

/* ---- temperature sampling (RealModelInferenceEngine.swift:8036-8068) ----------------------------------- */
static int first_max(const float *v, int n) {
    int best = 0;
    for (int i = 1; i < n; i++) if (v[best] < v[i]) best = i;
    return best;
}

int orc_sample_token(const float *logits, int count, float temperature, double unit) {
    if (count <= 0) return 0;
    if (temperature <= 0.0f) return first_max(logits, count);
    float max_logit = logits[0];
    for (int i = 1; i < count; i++) if (logits[i] > max_logit) max_logit = logits[i];
    double *scaled = (double *)malloc(sizeof(double) * (size_t)count);
    double total = 0.0;
    for (int i = 0; i < count; i++) {
        scaled[i] = exp((double)((logits[i] - max_logit) / temperature));
        total += scaled[i];
    }
    int out = count - 1;
    if (!isfinite(total) || total <= 0.0) {
        out = first_max(logits, count);
    } else {
        double threshold = unit * total;
        for (int i = 0; i < count; i++) {
            threshold -= scaled[i];
            if (threshold <= 0.0) { out = i; break; }
        }
    }
    free(scaled);
    return out;
}
