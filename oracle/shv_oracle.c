/*
 * shv_oracle.c — CPU restatement of the reference's Go/CPU token-loop arithmetic.
 * TEST INFRASTRUCTURE ONLY (see shv_oracle.h).  Build: -O2 -ffp-contract=off, no -ffast-math.
 */
#include "shv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t f32_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
static inline float bits_f32(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }

/* ------------------------------------------------------------------ fp16 --- */

/* safetensors/safetensors.go:425-466: round half to even, overflow to Inf, subnormals kept. */
uint16_t shv_ref_f32_to_f16(float f) {
    uint32_t b = f32_bits(f);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    int32_t exp = (int32_t)((b >> 23) & 0xff) - 127;
    uint32_t mant = b & 0x7fffff;

    if (((b >> 23) & 0xff) == 0xff) {
        if (mant != 0) return sign | 0x7e00;
        return sign | 0x7c00;
    }
    if (exp > 15) return sign | 0x7c00;
    if (exp >= -14) {
        uint16_t h = sign | (uint16_t)((exp + 15) << 10) | (uint16_t)(mant >> 13);
        if ((mant & 0x1000) != 0 && ((mant & 0x0fff) != 0 || (h & 1) != 0)) h++;
        return h;
    }
    if (exp >= -25) {
        unsigned shift = (unsigned)(-exp - 1);
        uint32_t full = mant | 0x800000;
        uint32_t m = full >> shift;
        uint32_t rem = full & ((1u << shift) - 1);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (m & 1) == 1)) m++;
        return sign | (uint16_t)m;
    }
    return sign;
}

/* safetensors/safetensors.go:472-496 */
float shv_ref_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t exp = (uint32_t)(h >> 10) & 0x1f;
    uint32_t mant = (uint32_t)(h & 0x3ff);
    if (exp == 0) {
        if (mant == 0) return bits_f32(sign);
        float f = (float)mant * (1.0f / 16777216.0f);
        return sign ? -f : f;
    }
    if (exp == 0x1f) {
        if (mant == 0) return bits_f32(sign | 0x7f800000);
        return bits_f32(sign | 0x7fc00000);
    }
    return bits_f32(sign | ((exp + 127 - 15) << 23) | (mant << 13));
}

/* llm/hc.go:318-360: x rounded to the nearest half, returned as a float32. */
float shv_ref_f16_round(float x) {
    uint32_t b = f32_bits(x);
    uint32_t sign = b & 0x80000000u;
    int32_t exp = (int32_t)((b >> 23) & 0xff) - 127;
    uint32_t man = b & 0x7fffff;
    const float sub14 = 1.0f / (float)(1 << 24);
    if (exp == 128) return x;
    if (exp > 15) return bits_f32(sign | 0x7f800000);
    if (exp < -25) return bits_f32(sign);
    if (exp < -14) {
        uint32_t shift = (uint32_t)(-exp - 14) + 13;
        uint32_t full = man | 0x800000;
        uint32_t q = full >> shift;
        uint32_t rem = full & ((1u << shift) - 1);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1) == 1)) q++;
        float v = (float)q * sub14;
        return sign ? -v : v;
    }
    {
        uint32_t q = man >> 13;
        uint32_t rem = man & 0x1fff;
        if (rem > 0x1000 || (rem == 0x1000 && (q & 1) == 1)) q++;
        uint32_t e = ((uint32_t)(exp + 127) << 23) + (q << 13);
        return bits_f32(sign | e);
    }
}

/* ------------------------------------------------------------ Q4_K decode --- */

/* gguf/dequant.go:238-243 (ggml get_scale_min_k4) */
void shv_ref_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
        return;
    }
    *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
    *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
}

static inline float f16_at(const uint8_t *b, int off) {
    return shv_ref_f16_to_f32((uint16_t)(b[off] | (b[off + 1] << 8)));
}

/* gguf/dequant.go:252-276: d1 = d*sc and m1 = dmin*m are formed first, then d1*q - m1. */
void shv_ref_dequant_q4k(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++) {
        const uint8_t *blk = data + b * SHV_Q4K_BYTES;
        float d = f16_at(blk, 0);
        float dmin = f16_at(blk, 2);
        const uint8_t *scales = blk + 4;
        const uint8_t *q = blk + 16;
        int is = 0;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc, m;
            shv_ref_scale_min_k4(is, scales, &sc, &m);
            float d1 = d * (float)sc, m1 = dmin * (float)m;
            shv_ref_scale_min_k4(is + 1, scales, &sc, &m);
            float d2 = d * (float)sc, m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) *dst++ = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) *dst++ = d2 * (float)(q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

/* ------------------------------------------- the other GGUF tensor types --- */
/* What a checkpoint of the UD-Q4_K_XL family mixes with Q4_K, and what the reference's loader
 * accepts (Dequantizable, gguf/dequant.go:103-110).  Each arm is pinned bit for bit by ggml's own
 * to_float output in gguf/testdata (gguf/dequant_test.go:40-92). */

static inline float bf16_at(const uint8_t *b, int off) {
    uint32_t u = ((uint32_t)b[off] | ((uint32_t)b[off + 1] << 8)) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t u32_at(const uint8_t *b, int off) {
    return (uint32_t)b[off] | ((uint32_t)b[off + 1] << 8) | ((uint32_t)b[off + 2] << 16) | ((uint32_t)b[off + 3] << 24);
}

/* gguf/dequant.go:44-46 */
static const int8_t kvalues_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* gguf/dequant.go:128-137: 32 int8 levels times one half scale */
static void dequant_q8_0(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 34) {
        float d = f16_at(data, 0);
        for (int j = 0; j < 32; j++) *dst++ = (float)(int8_t)data[2 + j] * d;
    }
}

/* gguf/dequant.go:146-161: level*d + m, low nibbles are elements 0..15, high nibbles 16..31 */
static void dequant_q4_1(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 20, dst += 32) {
        float d = f16_at(data, 0), m = f16_at(data, 2);
        for (int j = 0; j < 16; j++) {
            dst[j] = (float)(data[4 + j] & 0x0F) * d + m;
            dst[j + 16] = (float)(data[4 + j] >> 4) * d + m;
        }
    }
}

/* gguf/dequant.go:171-190: five-bit levels centred by 16; the fifth bit of element j is bit j of qh */
static void dequant_q5_0(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 22, dst += 32) {
        float d = f16_at(data, 0);
        uint32_t qh = u32_at(data, 2);
        for (int j = 0; j < 16; j++) {
            int x0 = (int)((data[6 + j] & 0x0F) | (((qh >> j) << 4) & 0x10)) - 16;
            int x1 = (int)((data[6 + j] >> 4) | ((qh >> (j + 12)) & 0x10)) - 16;
            dst[j] = (float)x0 * d;
            dst[j + 16] = (float)x1 * d;
        }
    }
}

/* gguf/dequant.go:197-217 */
static void dequant_q5_1(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 24, dst += 32) {
        float d = f16_at(data, 0), m = f16_at(data, 2);
        uint32_t qh = u32_at(data, 4);
        for (int j = 0; j < 16; j++) {
            uint8_t x0 = (uint8_t)((data[8 + j] & 0x0F) | (((qh >> j) << 4) & 0x10));
            uint8_t x1 = (uint8_t)((data[8 + j] >> 4) | ((qh >> (j + 12)) & 0x10));
            dst[j] = (float)x0 * d + m;
            dst[j + 16] = (float)x1 * d + m;
        }
    }
}

/* gguf/dequant.go:222-234: nibbles index the non-linear codebook */
static void dequant_iq4_nl(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 18, dst += 32) {
        float d = f16_at(data, 0);
        for (int j = 0; j < 16; j++) {
            dst[j] = d * (float)kvalues_iq4nl[data[2 + j] & 0xF];
            dst[j + 16] = d * (float)kvalues_iq4nl[data[2 + j] >> 4];
        }
    }
}

/* gguf/dequant.go:282-317: Q4_K with a 32-byte plane of fifth bits; one byte of qh serves the
 * same position of all eight sub-blocks, two bits per 64 elements */
static void dequant_q5_k(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 176) {
        float d = f16_at(data, 0), dmin = f16_at(data, 2);
        const uint8_t *scales = data + 4, *qh = data + 16, *ql = data + 48;
        int is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 256; j += 64) {
            uint8_t sc, m;
            shv_ref_scale_min_k4(is, scales, &sc, &m);
            float d1 = d * (float)sc, m1 = dmin * (float)m;
            shv_ref_scale_min_k4(is + 1, scales, &sc, &m);
            float d2 = d * (float)sc, m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) *dst++ = d1 * (float)((ql[l] & 0xF) + ((qh[l] & u1) ? 16 : 0)) - m1;
            for (int l = 0; l < 32; l++) *dst++ = d2 * (float)((ql[l] >> 4) + ((qh[l] & u2) ? 16 : 0)) - m2;
            ql += 32;
            is += 2;
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
}

/* gguf/dequant.go:331-356: six-bit levels centred by 32, sixteen signed int8 group scales, the
 * half super-scale last; d*scale is formed first, then times the level */
static void dequant_q6_k(const uint8_t *data, int64_t nb, float *dst) {
    for (int64_t b = 0; b < nb; b++, data += 210, dst += 256) {
        const uint8_t *ql = data, *qh = data + 128, *sc = data + 192;
        float d = f16_at(data, 208);
        for (int n = 0; n < 256; n += 128) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                uint8_t h = qh[n / 4 + l];
                int q1 = (int)((ql[n / 2 + l] & 0xF) | (((h >> 0) & 3) << 4)) - 32;
                int q2 = (int)((ql[n / 2 + l + 32] & 0xF) | (((h >> 2) & 3) << 4)) - 32;
                int q3 = (int)((ql[n / 2 + l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
                int q4 = (int)((ql[n / 2 + l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32;
                const uint8_t *g = sc + n / 16 + is;
                dst[n + l] = d * (float)(int8_t)g[0] * (float)q1;
                dst[n + l + 32] = d * (float)(int8_t)g[2] * (float)q2;
                dst[n + l + 64] = d * (float)(int8_t)g[4] * (float)q3;
                dst[n + l + 96] = d * (float)(int8_t)g[6] * (float)q4;
            }
        }
    }
}

/* Bytes of n elements of a ggml type, or -1 (TypeSize/BlockSize, gguf/gguf.go). */
int64_t shv_ref_type_bytes(int type, int64_t n) {
    switch (type) {
        case SHV_GGML_F32: return n * 4;
        case SHV_GGML_F16: case SHV_GGML_BF16: return n * 2;
        case SHV_GGML_Q8_0: return n % 32 ? -1 : n / 32 * 34;
        case SHV_GGML_Q4_1: return n % 32 ? -1 : n / 32 * 20;
        case SHV_GGML_Q5_0: return n % 32 ? -1 : n / 32 * 22;
        case SHV_GGML_Q5_1: return n % 32 ? -1 : n / 32 * 24;
        case SHV_GGML_IQ4_NL: return n % 32 ? -1 : n / 32 * 18;
        case SHV_GGML_Q4_K: return n % 256 ? -1 : n / 256 * 144;
        case SHV_GGML_Q5_K: return n % 256 ? -1 : n / 256 * 176;
        case SHV_GGML_Q6_K: return n % 256 ? -1 : n / 256 * 210;
    }
    return -1;
}

/* Dequantize (gguf/dequant.go:52-98): n elements of a type to float32; 0 on success, -1 for a
 * type the loader refuses or a count that is not whole blocks. */
int shv_ref_dequant(int type, const uint8_t *data, int64_t n, float *dst) {
    if (shv_ref_type_bytes(type, n) < 0) return -1;
    switch (type) {
        case SHV_GGML_F32: memcpy(dst, data, (size_t)n * 4); return 0;
        case SHV_GGML_F16: for (int64_t i = 0; i < n; i++) dst[i] = f16_at(data + 2 * i, 0); return 0;
        case SHV_GGML_BF16: for (int64_t i = 0; i < n; i++) dst[i] = bf16_at(data + 2 * i, 0); return 0;
        case SHV_GGML_Q8_0: dequant_q8_0(data, n / 32, dst); return 0;
        case SHV_GGML_Q4_1: dequant_q4_1(data, n / 32, dst); return 0;
        case SHV_GGML_Q5_0: dequant_q5_0(data, n / 32, dst); return 0;
        case SHV_GGML_Q5_1: dequant_q5_1(data, n / 32, dst); return 0;
        case SHV_GGML_IQ4_NL: dequant_iq4_nl(data, n / 32, dst); return 0;
        case SHV_GGML_Q4_K: shv_ref_dequant_q4k(data, n / 256, dst); return 0;
        case SHV_GGML_Q5_K: dequant_q5_k(data, n / 256, dst); return 0;
        case SHV_GGML_Q6_K: dequant_q6_k(data, n / 256, dst); return 0;
    }
    return -1;
}

/* --------------------------------------------------------- Q4_K quantiser --- */

/* llm/sim.go:1172-1180: ggml nearest_int is round-half-to-even. */
static inline float nearest_int(float v) { return (float)rint((double)v); }
/* llm/sim.go:1182-1187 */
static inline float sqrt32(float v) { return v <= 0 ? 0.0f : (float)sqrt((double)v); }
static inline float abs32(float v) { return v < 0 ? -v : v; }
/* llm/sim.go:1155-1163 */
static inline int clamp63(float v) { return v < 0 ? 0 : (v > 63 ? 63 : (int)v); }

static inline uint8_t clamp_level(float f, int nmax) {
    float l = nearest_int(f);
    if (l < 0) l = 0;
    if (l > (float)nmax) l = (float)nmax;
    return (uint8_t)l;
}

/* llm/sim.go:982-1060 (ggml make_qkx2_quants).  Returns scale, *the_min = -min.
 * Every accumulator is float32, as ggml's and the reference's are. */
float shv_ref_make_qkx_quants(const float *x, int n, int nmax, const float *w, uint8_t *lv,
                              uint8_t *laux, float rmin, float rdelta, int nstep, float *the_min) {
    float min = x[0], max = x[0];
    float sumW = w[0], sumX = w[0] * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        sumW += w[i];
        sumX += w[i] * x[i];
    }
    if (min > 0) min = 0;
    if (max <= min) {
        for (int i = 0; i < n; i++) lv[i] = 0;
        *the_min = -min;
        return 0;
    }
    float iscale = (float)nmax / (max - min);
    float scale = 1 / iscale;
    float bestErr = 0;
    for (int i = 0; i < n; i++) {
        lv[i] = clamp_level(iscale * (x[i] - min), nmax);
        float diff = scale * (float)lv[i] + min - x[i];
        bestErr += w[i] * diff * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
        float sumL = 0, sumL2 = 0, sumXL = 0;
        for (int i = 0; i < n; i++) {
            uint8_t l = clamp_level(iscale * (x[i] - min), nmax);
            laux[i] = l;
            float fl = (float)l;
            sumL += w[i] * fl;
            sumL2 += w[i] * fl * fl;
            sumXL += w[i] * fl * x[i];
        }
        float det = sumW * sumL2 - sumL * sumL;
        if (det <= 0) continue;
        float thisScale = (sumW * sumXL - sumX * sumL) / det;
        float thisMin = (sumL2 * sumX - sumL * sumXL) / det;
        if (thisMin > 0) {
            thisMin = 0;
            thisScale = sumXL / sumL2;
        }
        float err = 0;
        for (int i = 0; i < n; i++) {
            float diff = thisScale * (float)laux[i] + thisMin - x[i];
            err += w[i] * diff * diff;
        }
        if (err < bestErr) {
            memcpy(lv, laux, (size_t)n);
            bestErr = err;
            scale = thisScale;
            min = thisMin;
        }
    }
    *the_min = -min;
    return scale;
}

/* llm/quantk.go:211-226 */
static void pack_scale_min_k4(uint8_t *dst, const int *ls, const int *lm) {
    memset(dst, 0, 12);
    for (int j = 0; j < 8; j++) {
        uint8_t s = (uint8_t)ls[j], m = (uint8_t)lm[j];
        if (j < 4) {
            dst[j] = s;
            dst[j + 4] = m;
        } else {
            dst[j + 4] = (uint8_t)((s & 0xF) | ((m & 0xF) << 4));
            dst[j - 4] |= (uint8_t)((s >> 4) << 6);
            dst[j] |= (uint8_t)((m >> 4) << 6);
        }
    }
}

/* One super-block: asymEnc.Encode's uncalibrated arm (llm/quantk.go:115-179) followed by
 * packQ4KRecord + packKRow's nibble order (llm/quantk.go:306-320, llm/moebank.go:489-532). */
static void encode_q4k_block(const float *blk, uint8_t *rec) {
    enum { SUB = 8, GROUP = 32, NMAX = 15 };
    float scales[SUB], mins[SUB], w[GROUP];
    uint8_t lv[GROUP], laux[GROUP], Q[SUB * GROUP];
    int LS[SUB], LM[SUB];
    float maxScale = 0, maxMin = 0;
    for (int j = 0; j < SUB; j++) {
        const float *g = blk + j * GROUP;
        float sum2 = 0;
        for (int i = 0; i < GROUP; i++) sum2 += g[i] * g[i];
        float avx = sqrt32(sum2 / (float)GROUP);
        for (int i = 0; i < GROUP; i++) w[i] = avx + abs32(g[i]);
        scales[j] = shv_ref_make_qkx_quants(g, GROUP, NMAX, w, lv, laux, -1.0f, 0.1f, 20, &mins[j]);
        if (scales[j] > maxScale) maxScale = scales[j];
        if (mins[j] > maxMin) maxMin = mins[j];
    }
    float invScale = 0, invMin = 0;
    if (maxScale > 0) invScale = 63 / maxScale;
    if (maxMin > 0) invMin = 63 / maxMin;
    for (int j = 0; j < SUB; j++) {
        LS[j] = clamp63(nearest_int(invScale * scales[j]));
        LM[j] = clamp63(nearest_int(invMin * mins[j]));
    }
    float d = maxScale / 63, dmin = maxMin / 63;
    uint16_t D = shv_ref_f32_to_f16(d), DMin = shv_ref_f32_to_f16(dmin);
    float DF = shv_ref_f16_to_f32(D), DMinF = shv_ref_f16_to_f32(DMin);
    for (int j = 0; j < SUB; j++) {
        const float *g = blk + j * GROUP;
        uint8_t *q = Q + j * GROUP;
        float ds = DF * (float)LS[j], dm = DMinF * (float)LM[j];
        if (ds == 0) {
            memset(q, 0, GROUP);
            continue;
        }
        for (int i = 0; i < GROUP; i++) {
            float l = nearest_int((g[i] + dm) / ds);
            if (l < 0) l = 0;
            if (l > (float)NMAX) l = (float)NMAX;
            q[i] = (uint8_t)l;
        }
    }
    memset(rec, 0, SHV_Q4K_BYTES);
    rec[0] = (uint8_t)(D & 0xff);
    rec[1] = (uint8_t)(D >> 8);
    rec[2] = (uint8_t)(DMin & 0xff);
    rec[3] = (uint8_t)(DMin >> 8);
    pack_scale_min_k4(rec + 4, LS, LM);
    uint8_t *ql = rec + 16;
    for (int h = 0; h < 4; h++)
        for (int l = 0; l < 32; l++) {
            uint8_t lo = Q[h * 64 + l], hi = Q[h * 64 + 32 + l];
            ql[h * 32 + l] = (uint8_t)((lo & 0xF) | ((hi & 0xF) << 4));
        }
}

void shv_ref_quantize_q4k_row(const float *row, int64_t k, uint8_t *dst) {
    for (int64_t b = 0; b * SHV_Q4K_BLOCK < k; b++)
        encode_q4k_block(row + b * SHV_Q4K_BLOCK, dst + b * SHV_Q4K_BYTES);
}

void shv_ref_quantize_q4k(const float *w, int64_t rows, int64_t k, uint8_t *dst) {
    int64_t row_bytes = k / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) shv_ref_quantize_q4k_row(w + r * k, k, dst + r * row_bytes);
}

/* ----------------------------------------------------------- dense helpers --- */

/* llm/hc.go:255-264: one float32 accumulator per row, left to right. */
void shv_ref_matvec(float *y, const float *w, const float *x, int n, int k) {
    for (int r = 0; r < n; r++) {
        const float *row = w + (size_t)r * k;
        float s = 0;
        for (int i = 0; i < k; i++) s += row[i] * x[i];
        y[r] = s;
    }
}

static void gemv_q4k_range(float *y, const uint8_t *w, const float *x, int lo, int hi, int k,
                           float *rowbuf) {
    size_t row_bytes = (size_t)k / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    for (int r = lo; r < hi; r++) {
        shv_ref_dequant_q4k(w + (size_t)r * row_bytes, k / SHV_Q4K_BLOCK, rowbuf);
        float s = 0;
        for (int i = 0; i < k; i++) s += rowbuf[i] * x[i];
        y[r] = s;
    }
}

void shv_ref_gemv_q4k(float *y, const uint8_t *w, const float *x, int n, int k, int threads) {
    if (threads <= 1) {
        float *buf = (float *)malloc(sizeof(float) * (size_t)k);
        gemv_q4k_range(y, w, x, 0, n, k, buf);
        free(buf);
        return;
    }
    if (threads > n) threads = n;
    int chunk = (n + threads - 1) / threads; /* one contiguous chunk per worker, llm/hc.go:232-252 */
#pragma omp parallel for num_threads(threads) schedule(static, 1)
    for (int t = 0; t < threads; t++) {
        int lo = t * chunk, hi = lo + chunk;
        if (hi > n) hi = n;
        if (lo < hi) {
            float *buf = (float *)malloc(sizeof(float) * (size_t)k);
            gemv_q4k_range(y, w, x, lo, hi, k, buf);
            free(buf);
        }
    }
}

/* The same matvec over rows of any accepted tensor type: each row through Tensor.DequantizeRow
 * (gguf/dequant.go:119-124), then llm/hc.go:255-264.  type 0 stands for Q4_K here (no bank is
 * stored as float32).  Returns -1 for rows the type cannot hold. */
int shv_ref_gemv_any(float *y, int type, const uint8_t *w, const float *x, int n, int k, int threads) {
    if (type == 0) type = SHV_GGML_Q4_K;
    if (type == SHV_GGML_Q4_K && k % SHV_Q4K_BLOCK == 0) {
        shv_ref_gemv_q4k(y, w, x, n, k, threads);
        return 0;
    }
    int64_t row_bytes = shv_ref_type_bytes(type, k);
    if (row_bytes < 0) return -1;
    if (threads < 1) threads = 1;
    if (threads > n) threads = n;
    int chunk = (n + threads - 1) / threads;
#pragma omp parallel for num_threads(threads) schedule(static, 1)
    for (int t = 0; t < threads; t++) {
        int lo = t * chunk, hi = lo + chunk;
        if (hi > n) hi = n;
        if (lo >= hi) continue;
        float *buf = (float *)malloc(sizeof(float) * (size_t)k);
        for (int r = lo; r < hi; r++) {
            shv_ref_dequant(type, w + (size_t)r * (size_t)row_bytes, k, buf);
            float s = 0;
            for (int i = 0; i < k; i++) s += buf[i] * x[i];
            y[r] = s;
        }
        free(buf);
    }
    return 0;
}

/* llm/hc.go:266-268 */
float shv_ref_sigmoid(float x) { return (float)(1 / (1 + exp(-(double)x))); }
float shv_ref_silu(float x) { return x * shv_ref_sigmoid(x); }

/* llm/deltanet.go:450-455: the add inside the log is float32 on purpose. */
float shv_ref_softplus(float x) {
    if (x > 20) return x;
    return (float)log((double)(1 + (float)exp((double)x)));
}

/* llm/hc.go:176-190 with hc=1: sum of squares in float64. */
void shv_ref_rmsnorm(float *dst, const float *src, const float *gamma, int n, float eps) {
    double ss = 0;
    for (int i = 0; i < n; i++) ss += (double)src[i] * (double)src[i];
    float scale = (float)(1 / sqrt(ss / (double)n + (double)eps));
    for (int i = 0; i < n; i++) dst[i] = src[i] * scale * gamma[i];
}

/* llm/attn.go:510-522 */
void shv_ref_head_norm(float *x, const float *gamma, int dim, int n, float eps) {
    for (int r = 0; r < n; r++) {
        float *row = x + (size_t)r * dim;
        double ss = 0;
        for (int i = 0; i < dim; i++) ss += (double)row[i] * (double)row[i];
        float scale = (float)(1 / sqrt(ss / (double)dim + (double)eps));
        for (int i = 0; i < dim; i++) row[i] = row[i] * scale * gamma[i];
    }
}

/* llm/sample.go:359-367: first maximum; NaN never wins because the test is `>`. */
int32_t shv_ref_argmax(const float *logits, int64_t n) {
    int32_t best = 0;
    float bestV = -INFINITY;
    for (int64_t i = 0; i < n; i++)
        if (logits[i] > bestV) {
            best = (int32_t)i;
            bestV = logits[i];
        }
    return best;
}

/* -------------------------------------------------------------------- MoE --- */

/* llm/moe.go:426-443 */
void shv_ref_softmax(float *dst, const float *src, int n) {
    float max = -INFINITY;
    for (int i = 0; i < n; i++)
        if (src[i] > max) max = src[i];
    float sum = 0;
    for (int i = 0; i < n; i++) {
        float e = (float)exp((double)(src[i] - max));
        dst[i] = e;
        sum += e;
    }
    float inv = 1 / sum;
    for (int i = 0; i < n; i++) dst[i] *= inv;
}

/* Stable descending order of probs: an insertion into a sorted prefix keeps equal
 * probabilities in ascending index order, which is sort.SliceStable's result
 * (llm/moe.go:249-252).  Only the first `used` places are needed. */
static void stable_top(const float *probs, int n, int used, int32_t *top) {
    int cnt = 0;
    for (int e = 0; e < n; e++) {
        int pos = cnt;
        while (pos > 0 && probs[e] > probs[top[pos - 1]]) pos--;
        if (pos >= used) continue;
        int last = cnt < used ? cnt : used - 1;
        for (int i = last; i > pos; i--) top[i] = top[i - 1];
        top[pos] = e;
        if (cnt < used) cnt++;
    }
}

#define MOE_WEIGHTS_SUM_FLOOR 6.103515625e-5f /* llm/moe.go:278 */

/* llm/moe.go:219-274 */
void shv_ref_moe_route(const shv_ref_moe_cfg *c, const shv_ref_moe_w *w, const float *x, int n_tok,
                       float *logits, float *probs, int32_t *topk, float *weights_norm) {
    int nE = c->n_expert, used = c->n_used;
    for (int i = 0; i < n_tok; i++) {
        const float *xi = x + (size_t)i * c->n_embd;
        float *lg = logits + (size_t)i * nE;
        float *pr = probs + (size_t)i * nE;
        shv_ref_matvec(lg, w->router, xi, nE, c->n_embd);
        shv_ref_softmax(pr, lg, nE);
        int32_t *top = topk + (size_t)i * used;
        stable_top(pr, nE, used, top);
        float sum = 0;
        for (int k = 0; k < used; k++) sum += pr[top[k]];
        if (sum < MOE_WEIGHTS_SUM_FLOOR) sum = MOE_WEIGHTS_SUM_FLOOR;
        for (int k = 0; k < used; k++) weights_norm[(size_t)i * used + k] = pr[top[k]] / sum;
    }
}

/* llm/moe.go:289-409.  One (token, slot) pair at a time; the reference walks by expert only
 * to dequantise each bank once, which changes no value. */
void shv_ref_moe_block(const shv_ref_moe_cfg *c, const shv_ref_moe_w *w, const float *x, int n_tok,
                       float *out, float *logits, int32_t *topk, float *weights_norm,
                       float *swiglu, float *moe_out, float *sh_gate_sig, int threads) {
    int H = c->n_embd, nE = c->n_expert, used = c->n_used, ff = c->ffn_expert, ffs = c->ffn_shared;
    float *lg = logits ? logits : (float *)malloc(sizeof(float) * (size_t)n_tok * nE);
    float *pr = (float *)malloc(sizeof(float) * (size_t)n_tok * nE);
    int32_t *tk = topk ? topk : (int32_t *)malloc(sizeof(int32_t) * (size_t)n_tok * used);
    float *wn = weights_norm ? weights_norm : (float *)malloc(sizeof(float) * (size_t)n_tok * used);
    shv_ref_moe_route(c, w, x, n_tok, lg, pr, tk, wn);

    /* banks in the checkpoint's own types (llm/moe.go walks them through Dequantize whatever they are) */
    const int tg = w->types[0] ? w->types[0] : SHV_GGML_Q4_K, tu = w->types[1] ? w->types[1] : SHV_GGML_Q4_K;
    const int td = w->types[2] ? w->types[2] : SHV_GGML_Q4_K, tgs = w->types[3], tus = w->types[4], tds = w->types[5];
    size_t g_row = (size_t)shv_ref_type_bytes(tg, H), u_row = (size_t)shv_ref_type_bytes(tu, H);
    size_t dn_row = (size_t)shv_ref_type_bytes(td, ff);
    int big = ff > ffs ? ff : ffs;
    float *gate = (float *)malloc(sizeof(float) * big);
    float *up = (float *)malloc(sizeof(float) * big);
    float *sw = (float *)malloc(sizeof(float) * big);
    float *down = (float *)malloc(sizeof(float) * H);
    float *weighted = (float *)malloc(sizeof(float) * (size_t)used * H);

    for (int i = 0; i < n_tok; i++) {
        const float *xi = x + (size_t)i * H;
        float *o = out + (size_t)i * H;
        /* routed experts, llm/moe.go:289-359 */
        for (int k = 0; k < used; k++) {
            int e = tk[(size_t)i * used + k];
            shv_ref_gemv_any(gate, tg, w->gate_exps + (size_t)e * ff * g_row, xi, ff, H, threads);
            shv_ref_gemv_any(up, tu, w->up_exps + (size_t)e * ff * u_row, xi, ff, H, threads);
            for (int j = 0; j < ff; j++) sw[j] = shv_ref_silu(gate[j]) * up[j];
            if (swiglu) memcpy(swiglu + ((size_t)i * used + k) * ff, sw, sizeof(float) * ff);
            shv_ref_gemv_any(down, td, w->down_exps + (size_t)e * H * dn_row, sw, H, ff, threads);
            float wt = wn[(size_t)i * used + k];
            for (int j = 0; j < H; j++) weighted[(size_t)k * H + j] = down[j] * wt;
        }
        /* summed in slot order, llm/moe.go:347-357 */
        for (int j = 0; j < H; j++) o[j] = 0;
        for (int k = 0; k < used; k++)
            for (int j = 0; j < H; j++) o[j] += weighted[(size_t)k * H + j];
        if (moe_out) memcpy(moe_out + (size_t)i * H, o, sizeof(float) * H);
        /* shared expert, llm/moe.go:363-409 */
        shv_ref_gemv_any(gate, tgs, w->gate_sh, xi, ffs, H, threads);
        shv_ref_gemv_any(up, tus, w->up_sh, xi, ffs, H, threads);
        for (int j = 0; j < ffs; j++) sw[j] = shv_ref_silu(gate[j]) * up[j];
        shv_ref_gemv_any(down, tds, w->down_sh, sw, H, ffs, threads);
        float g = 0;
        for (int j = 0; j < H; j++) g += w->shared_gate[j] * xi[j];
        float s = shv_ref_sigmoid(g);
        if (sh_gate_sig) sh_gate_sig[i] = s;
        for (int j = 0; j < H; j++) o[j] = o[j] + down[j] * s;
    }
    free(weighted); free(down); free(sw); free(up); free(gate);
    if (!weights_norm) free(wn);
    if (!topk) free(tk);
    free(pr);
    if (!logits) free(lg);
}

/* --------------------------------------------------------------- DeltaNet --- */

/* llm/deltanet.go:423-443 */
static void l2_norm_heads(float *out, const float *x, int dim, int n, float eps, int mode_max) {
    for (int r = 0; r < n; r++) {
        const float *row = x + (size_t)r * dim;
        double ss = 0;
        for (int i = 0; i < dim; i++) ss += (double)row[i] * (double)row[i];
        float scale;
        if (mode_max) {
            double s = sqrt(ss);
            scale = (float)(1 / (s > (double)eps ? s : (double)eps));
        } else {
            scale = (float)(1 / sqrt(ss + (double)eps));
        }
        float *o = out + (size_t)r * dim;
        for (int i = 0; i < dim; i++) o[i] = row[i] * scale;
    }
}

/* llm/deltanet.go:365-403: state row j holds column j of S (s[j*d+i] = S[i][j]). */
void shv_ref_delta_rule(int d, int n_head_k, int n_head_v, int n_tok, const float *qnorm,
                        const float *knorm, const float *v, const float *gate,
                        const float *beta_sig, float *state_s, float *out, const int *k_of) {
    float scale = (float)(1 / sqrt((double)d));
    float *delta = (float *)malloc(sizeof(float) * d);
    for (int h = 0; h < n_head_v; h++) {
        int hk = k_of[h];
        float *s = state_s + (size_t)h * d * d;
        for (int i = 0; i < n_tok; i++) {
            const float *q = qnorm + ((size_t)i * n_head_k + hk) * d;
            const float *k = knorm + ((size_t)i * n_head_k + hk) * d;
            const float *vv = v + ((size_t)i * n_head_v + h) * d;
            float g = (float)exp((double)gate[(size_t)i * n_head_v + h]);
            float beta = beta_sig[(size_t)i * n_head_v + h];
            for (int j = 0; j < d * d; j++) s[j] *= g;
            for (int j = 0; j < d; j++) {
                const float *row = s + (size_t)j * d;
                float sum = 0;
                for (int x = 0; x < d; x++) sum += row[x] * k[x];
                delta[j] = (vv[j] - sum) * beta;
            }
            float *o = out + ((size_t)i * n_head_v + h) * d;
            for (int j = 0; j < d; j++) {
                float *row = s + (size_t)j * d;
                float dj = delta[j];
                float sum = 0;
                for (int x = 0; x < d; x++) {
                    row[x] += dj * k[x];
                    sum += row[x] * q[x];
                }
                o[j] = sum * scale;
            }
        }
    }
    free(delta);
}

/* llm/deltanet.go:212-352 */
void shv_ref_deltanet_layer(const shv_ref_dn_cfg *c, const shv_ref_dn_w *w, const float *xn,
                            int n_tok, float *state_conv, float *state_s, float *result,
                            float *qkv_mixed_t, float *qnorm_t, float *knorm_t, float *gate_t,
                            float *beta_sig_t, float *attn_out_t, float *final_t,
                            int head_map_divide, int threads) {
    int H = c->n_embd, d = c->head_dim, hk = c->n_head_k, hv = c->n_head_v, conv = c->conv;
    int qk = hk * d, vw = hv * d, cw = 2 * qk + vw, inner = vw, hist = conv - 1;
    size_t T = (size_t)n_tok;
    float *qkv = (float *)malloc(sizeof(float) * T * cw);
    float *z = (float *)malloc(sizeof(float) * T * inner);
    float *alpha = (float *)malloc(sizeof(float) * T * hv);
    float *beta = (float *)malloc(sizeof(float) * T * hv);
    float *gate = (float *)malloc(sizeof(float) * T * hv);
    float *bsig = (float *)malloc(sizeof(float) * T * hv);
    float *csilu = (float *)malloc(sizeof(float) * T * cw);
    float *Q = (float *)malloc(sizeof(float) * T * qk);
    float *K = (float *)malloc(sizeof(float) * T * qk);
    float *V = (float *)malloc(sizeof(float) * T * vw);
    float *QN = (float *)malloc(sizeof(float) * T * qk);
    float *KN = (float *)malloc(sizeof(float) * T * qk);
    float *O = (float *)malloc(sizeof(float) * T * vw);
    float *F = (float *)malloc(sizeof(float) * T * inner);

    /* the four projections, llm/deltanet.go:253-264 */
    for (int i = 0; i < n_tok; i++) {
        const float *x = xn + (size_t)i * H;
        shv_ref_gemv_q4k(qkv + (size_t)i * cw, w->qkv, x, cw, H, threads);
        shv_ref_gemv_q4k(z + (size_t)i * inner, w->z, x, inner, H, threads);
        shv_ref_gemv_q4k(alpha + (size_t)i * hv, w->alpha, x, hv, H, 1);
        shv_ref_gemv_q4k(beta + (size_t)i * hv, w->beta, x, hv, H, 1);
    }
    /* decay and write strength, llm/deltanet.go:266-271 */
    for (size_t i = 0; i < T * hv; i++) {
        int h = (int)(i % hv);
        float asp = shv_ref_softplus(alpha[i] + w->dt_bias[h]);
        gate[i] = asp * w->a[h];
        bsig[i] = shv_ref_sigmoid(beta[i]);
    }
    /* depthwise causal conv over history + batch, SiLU, split, llm/deltanet.go:276-300 */
    for (int i = 0; i < n_tok; i++) {
        for (int ch = 0; ch < cw; ch++) {
            const float *k = w->conv1d + (size_t)ch * conv;
            float s = 0;
            for (int j = 0; j < conv; j++) {
                int p = i + j - hist;
                float xv = p < 0 ? state_conv[(size_t)ch * hist + hist + p] : qkv[(size_t)p * cw + ch];
                s += xv * k[j];
            }
            csilu[(size_t)i * cw + ch] = shv_ref_silu(s);
        }
        memcpy(Q + (size_t)i * qk, csilu + (size_t)i * cw, sizeof(float) * qk);
        memcpy(K + (size_t)i * qk, csilu + (size_t)i * cw + qk, sizeof(float) * qk);
        memcpy(V + (size_t)i * vw, csilu + (size_t)i * cw + 2 * qk, sizeof(float) * vw);
    }
    /* new conv history, llm/deltanet.go:302-316 */
    {
        float *next = (float *)malloc(sizeof(float) * (size_t)cw * hist);
        for (int ch = 0; ch < cw; ch++)
            for (int p = 0; p < hist; p++) {
                int src = n_tok - hist + p;
                next[(size_t)ch * hist + p] = src < 0 ? state_conv[(size_t)ch * hist + hist + src]
                                                      : qkv[(size_t)src * cw + ch];
            }
        memcpy(state_conv, next, sizeof(float) * (size_t)cw * hist);
        free(next);
    }
    l2_norm_heads(QN, Q, d, hk * n_tok, c->eps, c->qk_norm_max);
    l2_norm_heads(KN, K, d, hk * n_tok, c->eps, c->qk_norm_max);

    int *k_of = (int *)malloc(sizeof(int) * hv);
    for (int h = 0; h < hv; h++) k_of[h] = head_map_divide ? h / (hv / hk) : h % hk; /* :412-418 */
    shv_ref_delta_rule(d, hk, hv, n_tok, QN, KN, V, gate, bsig, state_s, O, k_of);
    free(k_of);

    /* gated output norm, llm/deltanet.go:329-341 */
    for (size_t i = 0; i < T * hv; i++) {
        const float *x = O + i * d;
        double ss = 0;
        for (int j = 0; j < d; j++) ss += (double)x[j] * (double)x[j];
        float scale = (float)(1 / sqrt(ss / (double)d + (double)c->eps));
        for (int j = 0; j < d; j++)
            F[i * d + j] = x[j] * scale * w->norm[j] * shv_ref_sigmoid(z[i * d + j]);
    }
    for (int i = 0; i < n_tok; i++)
        shv_ref_gemv_q4k(result + (size_t)i * H, w->out, F + (size_t)i * inner, H, inner, threads);

    if (qkv_mixed_t) memcpy(qkv_mixed_t, qkv, sizeof(float) * T * cw);
    if (qnorm_t) memcpy(qnorm_t, QN, sizeof(float) * T * qk);
    if (knorm_t) memcpy(knorm_t, KN, sizeof(float) * T * qk);
    if (gate_t) memcpy(gate_t, gate, sizeof(float) * T * hv);
    if (beta_sig_t) memcpy(beta_sig_t, bsig, sizeof(float) * T * hv);
    if (attn_out_t) memcpy(attn_out_t, O, sizeof(float) * T * vw);
    if (final_t) memcpy(final_t, F, sizeof(float) * T * inner);
    free(F); free(O); free(KN); free(QN); free(V); free(K); free(Q); free(csilu);
    free(bsig); free(gate); free(beta); free(alpha); free(z); free(qkv);
}

/* -------------------------------------------------------------- attention --- */

/* llm/attn.go:544-586 on text positions (t = h = w = pos, fourth section 0). */
void shv_ref_rope(const shv_ref_attn_cfg *c, float *x, const int32_t *pos, int n_heads,
                  int head_dim, int n_tok) {
    int rot = c->rope_dims;
    if (rot > head_dim) rot = head_dim;
    int half = rot / 2;
    int sect = c->sections[0] + c->sections[1] + c->sections[2] + c->sections[3];
    if (sect == 0) sect = half;
    double scale = pow((double)c->rope_base, -2 / (double)rot);
    for (int t = 0; t < n_tok; t++) {
        double theta[4] = {(double)pos[t], (double)pos[t], (double)pos[t], 0};
        for (int i = 0; i < half; i++) {
            int sector = i % sect;
            double th;
            if (sector % 3 == 0 && sector < 3 * c->sections[0]) th = theta[0];
            else if (sector % 3 == 1 && sector < 3 * c->sections[1]) th = theta[1];
            else if (sector % 3 == 2 && sector < 3 * c->sections[2]) th = theta[2];
            else th = theta[3];
            float cs = (float)cos(th), sn = (float)sin(th);
            for (int h = 0; h < n_heads; h++) {
                float *row = x + ((size_t)t * n_heads + h) * head_dim;
                float x0 = row[i], x1 = row[i + half];
                row[i] = x0 * cs - x1 * sn;
                row[i + half] = x0 * sn + x1 * cs;
            }
            for (int j = 0; j < 4; j++) theta[j] *= scale;
        }
    }
}

/* llm/attn.go:135-219 (dense arm) + attention :444-496, generalised to a cache that already
 * holds `past` cells: the row at position p sees cells 0..p. */
/* allow: NULL (dense), or [n_tok][past + n_tok] bytes, the selection of llm/attn.go:423-443: a
 * cell it leaves out is unreadable however visible the causal mask says it is. */
static void attn_layer_core(const shv_ref_attn_cfg *c, const shv_ref_attn_w *w, const float *xn,
                            int n_tok, int past, uint16_t *kcache, uint16_t *vcache, float *out,
                            float *q_rot, float *pregate_t, const uint8_t *allow, int threads) {
    int H = c->n_embd, nh = c->n_head, nkv = c->n_head_kv, d = c->head_dim;
    int qw = nh * d * 2, gw = nh * d, kvw = nkv * d;
    size_t T = (size_t)n_tok;
    float *qfull = (float *)malloc(sizeof(float) * T * qw);
    float *Q = (float *)malloc(sizeof(float) * T * gw);
    float *G = (float *)malloc(sizeof(float) * T * gw);
    float *K = (float *)malloc(sizeof(float) * T * kvw);
    float *V = (float *)malloc(sizeof(float) * T * kvw);
    int32_t *pos = (int32_t *)malloc(sizeof(int32_t) * T);
    for (int i = 0; i < n_tok; i++) {
        const float *x = xn + (size_t)i * H;
        shv_ref_gemv_q4k(qfull + (size_t)i * qw, w->q, x, qw, H, threads);
        shv_ref_gemv_q4k(K + (size_t)i * kvw, w->k, x, kvw, H, threads);
        shv_ref_gemv_q4k(V + (size_t)i * kvw, w->v, x, kvw, H, threads);
        for (int h = 0; h < nh; h++) {
            const float *src = qfull + (size_t)i * qw + (size_t)h * 2 * d;
            memcpy(Q + ((size_t)i * nh + h) * d, src, sizeof(float) * d);
            memcpy(G + (size_t)i * gw + (size_t)h * d, src + d, sizeof(float) * d);
        }
        pos[i] = past + i;
    }
    shv_ref_head_norm(Q, w->q_norm, d, nh * n_tok, c->eps);
    shv_ref_head_norm(K, w->k_norm, d, nkv * n_tok, c->eps);
    shv_ref_rope(c, Q, pos, nh, d, n_tok);
    shv_ref_rope(c, K, pos, nkv, d, n_tok);
    /* into the fp16 cache, llm/attn.go:176-184 */
    for (size_t i = 0; i < T * kvw; i++) {
        kcache[(size_t)past * kvw + i] = shv_ref_f32_to_f16(K[i]);
        vcache[(size_t)past * kvw + i] = shv_ref_f32_to_f16(V[i]);
    }
    if (q_rot) memcpy(q_rot, Q, sizeof(float) * T * gw);

    /* attention, llm/attn.go:444-496 */
    int rep = nh / nkv;
    float scale = (float)(1 / sqrt((double)d));
    float *pre = (float *)calloc(T * gw, sizeof(float));
#pragma omp parallel for collapse(2) num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (int i = 0; i < n_tok; i++) {
        for (int h = 0; h < nh; h++) {
            int cells = past + i + 1;
            const uint8_t *al = allow ? allow + (size_t)i * (past + n_tok) : NULL;
            float *scores = (float *)malloc(sizeof(float) * cells);
            int kvh = h / rep;
            const float *qv = Q + ((size_t)i * nh + h) * d;
            int n = 0;
            for (int j = 0; j < cells; j++) {
                if (al && !al[j]) continue;
                const uint16_t *kv = kcache + ((size_t)j * nkv + kvh) * d;
                float s = 0;
                for (int x = 0; x < d; x++) s += qv[x] * shv_ref_f16_to_f32(kv[x]);
                scores[n++] = s * scale;
            }
            float max = scores[0];
            for (int j = 1; j < n; j++)
                if (scores[j] > max) max = scores[j];
            float sum = 0;
            for (int j = 0; j < n; j++) {
                scores[j] = (float)exp((double)(scores[j] - max));
                sum += scores[j];
            }
            float *dst = pre + ((size_t)i * nh + h) * d;
            n = 0;
            for (int j = 0; j < cells; j++) {
                if (al && !al[j]) continue;
                float wgt = scores[n++] / sum;
                const uint16_t *vv = vcache + ((size_t)j * nkv + kvh) * d;
                for (int x = 0; x < d; x++) dst[x] += wgt * shv_ref_f16_to_f32(vv[x]);
            }
            free(scores);
        }
    }
    if (pregate_t) memcpy(pregate_t, pre, sizeof(float) * T * gw);
    /* sigmoid gate and output projection, llm/attn.go:198-217 */
    for (size_t i = 0; i < T * gw; i++) pre[i] = pre[i] * shv_ref_sigmoid(G[i]);
    for (int i = 0; i < n_tok; i++)
        shv_ref_gemv_q4k(out + (size_t)i * H, w->o, pre + (size_t)i * gw, H, gw, threads);
    free(pre); free(pos); free(V); free(K); free(G); free(Q); free(qfull);
}

void shv_ref_attn_layer(const shv_ref_attn_cfg *c, const shv_ref_attn_w *w, const float *xn,
                        int n_tok, int past, uint16_t *kcache, uint16_t *vcache, float *out,
                        float *q_rot, float *pregate_t, int threads) {
    attn_layer_core(c, w, xn, n_tok, past, kcache, vcache, out, q_rot, pregate_t, NULL, threads);
}

/* ---------------------------------------------------- block-sparse indexer --- */

/* llm/attn.go:672-682 */
uint32_t shv_ref_f2ui(float v) {
    uint32_t y = f32_bits(v);
    if (y & 0x80000000u) return y ^ 0xFFFFFFFFu;
    return y | 0x80000000u;
}

/* llm/attn.go:637-670 */
uint32_t shv_ref_topk_threshold(const float *x, int len, int n) {
    uint32_t histo[256];
    uint32_t prefix = 0, desired = (uint32_t)n;
    for (int shift = 24; shift >= 0; shift -= 8) {
        memset(histo, 0, sizeof histo);
        uint32_t hi_mask = 0;
        if (shift + 8 < 32) hi_mask = 0xFFFFFFFFu << (unsigned)(shift + 8);
        uint32_t prefix_hi = prefix & hi_mask;
        for (int i = 0; i < len; i++) {
            uint32_t key = shv_ref_f2ui(x[i]);
            if ((key & hi_mask) == prefix_hi) histo[(key >> (unsigned)shift) & 255]++;
        }
        uint32_t acc = 0, b = 0;
        for (int bb = 255; bb >= 0; bb--) {
            uint32_t cnt = histo[bb];
            if (acc + cnt >= desired) { b = (uint32_t)bb; break; }
            acc += cnt;
        }
        prefix |= b << (unsigned)shift;
        desired -= acc;
    }
    return prefix;
}

/* llm/attn.go:615-632 */
int shv_ref_topk(const float *x, int len, int n, int32_t *sel) {
    uint32_t thr = shv_ref_topk_threshold(x, len, n);
    int m = 0;
    for (int i = 0; i < len; i++)
        if (shv_ref_f2ui(x[i]) > thr) sel[m++] = i;
    int above = m;
    for (int i = 0; i < len && m < n; i++)
        if (shv_ref_f2ui(x[i]) == thr) sel[m++] = i;
    return above;
}

/* llm/attn.go:231-421 at cell positions past..past+n_tok-1 of a sequence whose earlier raw keys
 * are in idxcache; fills allow [n_tok][past+n_tok] (llm/attn.go:423-443). */
static void qsa_indexer(const shv_ref_attn_cfg *c, const shv_ref_attn_w *w, const float *xn, int n_tok, int past,
                        uint16_t *idxcache, int n_kv, uint8_t *allow, int32_t *topk_t, int32_t *above_t, float *score_t,
                        int threads) {
    int H = c->n_embd, D = c->idx_dim, IH = c->idx_heads, R = c->ratio;
    int N = past + n_tok;                       /* occupied cells after this pass */
    int n_blocks = (n_kv + R - 1) / R;
    int n_bid = N / R;                          /* whole blocks only */
    /* the raw key, cached before the norm and the rotation, rounded to halves by the cache */
    float *raw = (float *)malloc(sizeof(float) * D);
    for (int i = 0; i < n_tok; i++) {
        shv_ref_matvec(raw, w->idx_k, xn + (size_t)i * H, D, H);
        for (int j = 0; j < D; j++) idxcache[(size_t)(past + i) * D + j] = shv_ref_f32_to_f16(raw[j]);
    }
    free(raw);
    /* pooled keys: a block that does not exist pools cell 0 `ratio` times (the zero fill) */
    float *pooled = (float *)calloc((size_t)n_blocks * D, sizeof(float));
    float inv = 1 / (float)R;
    for (int b = 0; b < n_blocks; b++) {
        float *dst = pooled + (size_t)b * D;
        for (int s_ = 0; s_ < R; s_++) {
            int cell = b < n_bid ? b * R + s_ : 0;
            for (int j = 0; j < D; j++) dst[j] += shv_ref_f16_to_f32(idxcache[(size_t)cell * D + j]);
        }
        for (int j = 0; j < D; j++) dst[j] *= inv;
    }
    shv_ref_head_norm(pooled, w->idx_k_norm, D, n_blocks, c->eps);
    int32_t *blk_pos = (int32_t *)calloc((size_t)n_blocks, sizeof(int32_t));
    for (int b = 0; b < n_bid && b < n_blocks; b++) blk_pos[b] = b * R;   /* a block's position is its first cell's */
    shv_ref_rope(c, pooled, blk_pos, 1, D, n_blocks);
    free(blk_pos);
    float *idxq = (float *)malloc(sizeof(float) * (size_t)n_tok * IH * D);
    int32_t *pos = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_tok);
    for (int i = 0; i < n_tok; i++) {
        shv_ref_matvec(idxq + (size_t)i * IH * D, w->idx_q, xn + (size_t)i * H, IH * D, H);
        pos[i] = past + i;
    }
    shv_ref_head_norm(idxq, w->idx_q_norm, D, IH * n_tok, c->eps);
    shv_ref_rope(c, idxq, pos, IH, D, n_tok);
    free(pos);
    /* rectified per-head dot products, summed */
    float *score = (float *)malloc(sizeof(float) * (size_t)n_tok * n_blocks);
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(static)
    for (int i = 0; i < n_tok; i++) {
        for (int b = 0; b < n_blocks; b++) {
            float s = 0;
            const float *k = pooled + (size_t)b * D;
            for (int h = 0; h < IH; h++) {
                const float *q = idxq + ((size_t)i * IH + h) * D;
                float d = 0;
                for (int j = 0; j < D; j++) d += q[j] * k[j];
                if (d > 0) s += d;
            }
            score[(size_t)i * n_blocks + b] = s;
        }
    }
    if (score_t) memcpy(score_t, score, sizeof(float) * (size_t)n_tok * n_blocks);
    /* bias, expansion to cells, causal mask, selection */
    int dead_bid = n_bid >= n_blocks ? n_blocks - 1 : n_bid;
    int width = c->top_k + R - 1;
    if (width > n_kv) width = n_kv;
    memset(allow, 0, (size_t)n_tok * N);
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(static)
    for (int i = 0; i < n_tok; i++) {
        int p = past + i;
        float *bias = (float *)malloc(sizeof(float) * n_blocks);
        float *cellv = (float *)malloc(sizeof(float) * n_kv);
        int32_t *sel = (int32_t *)malloc(sizeof(int32_t) * width);
        int tail_start = (p + 1) / R * R;
        for (int b = 0; b < n_blocks; b++) {
            if (b >= n_bid) bias[b] = -INFINITY;
            else if (b * R >= tail_start) bias[b] = 1e9f;
            else bias[b] = 0;
        }
        if (n_bid < n_blocks) bias[dead_bid] = 1e9f;
        for (int j = 0; j < n_kv; j++) {
            int blk = j < n_bid * R ? j / R : dead_bid;
            float v = score[(size_t)i * n_blocks + blk] + bias[blk];
            if (j > p || j >= N) v = -INFINITY;
            cellv[j] = v;
        }
        int ab = shv_ref_topk(cellv, n_kv, width, sel);
        if (topk_t) memcpy(topk_t + (size_t)i * width, sel, sizeof(int32_t) * width);
        if (above_t) above_t[i] = ab;
        for (int k = 0; k < width; k++)
            if (sel[k] < N) allow[(size_t)i * N + sel[k]] = 1;
        free(sel); free(cellv); free(bias);
    }
    free(score); free(idxq); free(pooled);
}

void shv_ref_attn_layer_qsa(const shv_ref_attn_cfg *c, const shv_ref_attn_w *w, const float *xn,
                            int n_tok, int past, uint16_t *kcache, uint16_t *vcache, uint16_t *idxcache,
                            int n_kv, float *out, float *q_rot, float *pregate_t, int32_t *topk_t,
                            int32_t *above_t, float *score_t, int threads) {
    if (c->ratio <= 0) {
        attn_layer_core(c, w, xn, n_tok, past, kcache, vcache, out, q_rot, pregate_t, NULL, threads);
        return;
    }
    uint8_t *allow = (uint8_t *)malloc((size_t)n_tok * (past + n_tok));
    qsa_indexer(c, w, xn, n_tok, past, idxcache, n_kv, allow, topk_t, above_t, score_t, threads);
    attn_layer_core(c, w, xn, n_tok, past, kcache, vcache, out, q_rot, pregate_t, allow, threads);
    free(allow);
}

/* ------------------------------------------------------------- token loop --- */

void shv_ref_model_extend_rows(const shv_ref_model_cfg *c, const shv_ref_model_w *w, shv_ref_model_state *st,
                               const int32_t *ids, int n_tok, float *logits_rows, float *hidden_rows, int threads) {
    int H = c->n_embd;
    size_t T = (size_t)n_tok;
    float *x = (float *)malloc(sizeof(float) * T * H);
    float *xn = (float *)malloc(sizeof(float) * T * H);
    float *y = (float *)malloc(sizeof(float) * T * H);
    for (int t = 0; t < n_tok; t++)
        for (int i = 0; i < H; i++) x[(size_t)t * H + i] = shv_ref_f16_to_f32(w->embd[(size_t)ids[t] * H + i]);
    for (int l = 0; l < c->n_layer; l++) {
        const shv_ref_layer_w *lw = &w->layers[l];
        for (int t = 0; t < n_tok; t++) shv_ref_rmsnorm(xn + (size_t)t * H, x + (size_t)t * H, lw->attn_norm, H, c->eps);
        if ((l + 1) % c->attn_every == 0)
            shv_ref_attn_layer_qsa(&c->attn, &lw->attn, xn, n_tok, st->past, st->kcache[l], st->vcache[l],
                                   (c->attn.ratio > 0 && st->idxcache) ? st->idxcache[l] : NULL, c->max_cells, y, NULL, NULL, NULL, NULL, NULL,
                                   threads);
        else
            shv_ref_deltanet_layer(&c->dn, &lw->dn, xn, n_tok, st->dn_conv[l], st->dn_s[l], y, NULL, NULL, NULL,
                                   NULL, NULL, NULL, NULL, 0, threads);
        for (size_t i = 0; i < T * H; i++) x[i] += y[i];
        for (int t = 0; t < n_tok; t++) shv_ref_rmsnorm(xn + (size_t)t * H, x + (size_t)t * H, lw->ffn_norm, H, c->eps);
        shv_ref_moe_block(&c->moe, &lw->moe, xn, n_tok, y, NULL, NULL, NULL, NULL, NULL, NULL, threads);
        for (size_t i = 0; i < T * H; i++) x[i] += y[i];
    }
    st->past += n_tok;
    if (hidden_rows) memcpy(hidden_rows, x, sizeof(float) * T * H);
    if (logits_rows) {
        for (int t = 0; t < n_tok; t++) {
            shv_ref_rmsnorm(xn, x + (size_t)t * H, w->out_norm, H, c->eps);
            shv_ref_gemv_q4k(logits_rows + (size_t)t * c->vocab, w->lm_head, xn, c->vocab, H, threads);
        }
    }
    free(y); free(xn); free(x);
}

void shv_ref_model_extend(const shv_ref_model_cfg *c, const shv_ref_model_w *w, shv_ref_model_state *st,
                          const int32_t *ids, int n_tok, float *logits, float *hidden, int threads) {
    int H = c->n_embd;
    float *rows = (float *)malloc(sizeof(float) * (size_t)n_tok * H);
    shv_ref_model_extend_rows(c, w, st, ids, n_tok, NULL, rows, threads);
    const float *last = rows + (size_t)(n_tok - 1) * H;
    if (hidden) memcpy(hidden, last, sizeof(float) * H);
    if (logits) {
        float *xn = (float *)malloc(sizeof(float) * H);
        shv_ref_rmsnorm(xn, last, w->out_norm, H, c->eps);
        shv_ref_gemv_q4k(logits, w->lm_head, xn, c->vocab, H, threads);
        free(xn);
    }
    free(rows);
}

/* llm/mtp.go:31-53 without hyper-connection streams; the block itself is the trunk's attention
 * layer and MoE (llm/mtp.go:47-49). */
void shv_ref_mtp_rows(const shv_ref_model_cfg *c, const shv_ref_model_w *w, const shv_ref_mtp_w *mw,
                      uint16_t *kcache, uint16_t *vcache, const float *hs, const int32_t *ids, int n_tok,
                      int pos, float *logits, float *res, int threads) {
    if (n_tok <= 0) return;
    int H = c->n_embd;
    size_t T = (size_t)n_tok;
    float *x = (float *)malloc(sizeof(float) * T * H);
    float *xn = (float *)malloc(sizeof(float) * T * H);
    float *y = (float *)malloc(sizeof(float) * T * H);
    float *cat = (float *)malloc(sizeof(float) * 2 * H);
    float *e = (float *)malloc(sizeof(float) * H);
    for (int t = 0; t < n_tok; t++) {
        for (int i = 0; i < H; i++) e[i] = shv_ref_f16_to_f32(w->embd[(size_t)ids[t] * H + i]);
        shv_ref_rmsnorm(cat, e, mw->enorm, H, c->eps);
        shv_ref_rmsnorm(cat + H, hs + (size_t)t * H, mw->hnorm, H, c->eps);
        shv_ref_gemv_q4k(x + (size_t)t * H, mw->eh_proj, cat, H, 2 * H, threads);
    }
    const shv_ref_layer_w *lw = &mw->layer;
    for (int t = 0; t < n_tok; t++) shv_ref_rmsnorm(xn + (size_t)t * H, x + (size_t)t * H, lw->attn_norm, H, c->eps);
    shv_ref_attn_cfg dense = c->attn;
    dense.ratio = 0;  /* the draft block is plain attention whatever the trunk's layers are */
    shv_ref_attn_layer(&dense, &lw->attn, xn, n_tok, pos, kcache, vcache, y, NULL, NULL, threads);
    for (size_t i = 0; i < T * H; i++) x[i] += y[i];
    for (int t = 0; t < n_tok; t++) shv_ref_rmsnorm(xn + (size_t)t * H, x + (size_t)t * H, lw->ffn_norm, H, c->eps);
    shv_ref_moe_block(&c->moe, &lw->moe, xn, n_tok, y, NULL, NULL, NULL, NULL, NULL, NULL, threads);
    for (size_t i = 0; i < T * H; i++) x[i] += y[i];
    if (res) memcpy(res, x, sizeof(float) * T * H);
    if (logits) {
        shv_ref_rmsnorm(xn, x + (T - 1) * H, mw->head_norm, H, c->eps);
        shv_ref_gemv_q4k(logits, w->lm_head, xn, c->vocab, H, threads);
    }
    free(e); free(cat); free(y); free(xn); free(x);
}
