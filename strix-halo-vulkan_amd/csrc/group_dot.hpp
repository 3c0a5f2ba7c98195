// Rows of any tensor type the reference's loader accepts, a 32-element group at a time: the
// weights formed exactly as the format's CPU arm forms them (gguf/dequant.go:128-356) and dotted
// with 32 activations.  Shared by the any-type GEMV and the any-type expert kernels.
#pragma once
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace shv_any {

using namespace shv;

__device__ __forceinline__ float half_at(const uint8_t *b) { return f16_bits_to_f32(static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8)); }
__device__ __forceinline__ uint32_t u32_at(const uint8_t *b) {
    return static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8) | (static_cast<uint32_t>(b[2]) << 16) | (static_cast<uint32_t>(b[3]) << 24);
}
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *q, uint32_t &sc, uint32_t &m) {
    if (j < 4) {
        sc = q[j] & 63u;
        m = q[j + 4] & 63u;
    } else {
        sc = (q[j + 4] & 0xFu) | ((q[j - 4] >> 6) << 4);
        m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}
static __device__ const int8_t kValuesIQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// Bytes of a row of k elements.
__host__ __device__ inline long long row_bytes(int type, int k) {
    switch (type) {
        case SHV_GGML_F32: return 4ll * k;
        case SHV_GGML_F16: case SHV_GGML_BF16: return 2ll * k;
        case SHV_GGML_Q8_0: return k / 32 * 34ll;
        case SHV_GGML_Q4_1: return k / 32 * 20ll;
        case SHV_GGML_Q5_0: return k / 32 * 22ll;
        case SHV_GGML_Q5_1: return k / 32 * 24ll;
        case SHV_GGML_IQ4_NL: return k / 32 * 18ll;
        case SHV_GGML_Q4_K: return k / 256 * 144ll;
        case SHV_GGML_Q5_K: return k / 256 * 176ll;
        case SHV_GGML_Q6_K: return k / 256 * 210ll;
    }
    return -1;
}

// The dot product of group g (32 elements) of a row with x[0..31].  Weights are formed as the
// format's dequantiser forms them; the sum over the group is sequential in element order.
template <int TYPE>
__device__ __forceinline__ float group_dot(const uint8_t *row, int g, const float *x) {
    float acc = 0.f;
    if constexpr (TYPE == SHV_GGML_F32) {
        for (int j = 0; j < 32; j++) acc = fmaf(__uint_as_float(u32_at(row + (g * 32 + j) * 4)), x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_F16) {
        for (int j = 0; j < 32; j++) acc = fmaf(half_at(row + (g * 32 + j) * 2), x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_BF16) {
        for (int j = 0; j < 32; j++) {
            const uint8_t *b = row + (g * 32 + j) * 2;
            acc = fmaf(__uint_as_float((static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8)) << 16), x[j], acc);
        }
    } else if constexpr (TYPE == SHV_GGML_Q8_0) {
        const uint8_t *b = row + g * 34;
        const float d = half_at(b);
        for (int j = 0; j < 32; j++) acc = fmaf(static_cast<float>(static_cast<int8_t>(b[2 + j])) * d, x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_Q4_1) {
        const uint8_t *b = row + g * 20;
        const float d = half_at(b), m = half_at(b + 2);
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(b[4 + j] & 0x0F) * d + m, x[j], acc);
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(b[4 + j] >> 4) * d + m, x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_Q5_0) {
        const uint8_t *b = row + g * 22;
        const float d = half_at(b);
        const uint32_t qh = u32_at(b + 2);
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(static_cast<int>((b[6 + j] & 0x0Fu) | (((qh >> j) << 4) & 0x10u)) - 16) * d, x[j], acc);
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(static_cast<int>((b[6 + j] >> 4) | ((qh >> (j + 12)) & 0x10u)) - 16) * d, x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_Q5_1) {
        const uint8_t *b = row + g * 24;
        const float d = half_at(b), m = half_at(b + 2);
        const uint32_t qh = u32_at(b + 4);
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>((b[8 + j] & 0x0Fu) | (((qh >> j) << 4) & 0x10u)) * d + m, x[j], acc);
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>((b[8 + j] >> 4) | ((qh >> (j + 12)) & 0x10u)) * d + m, x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_IQ4_NL) {
        const uint8_t *b = row + g * 18;
        const float d = half_at(b);
        for (int j = 0; j < 16; j++) acc = fmaf(d * static_cast<float>(kValuesIQ4NL[b[2 + j] & 0xF]), x[j], acc);
        for (int j = 0; j < 16; j++) acc = fmaf(d * static_cast<float>(kValuesIQ4NL[b[2 + j] >> 4]), x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_Q4_K || TYPE == SHV_GGML_Q5_K) {
        constexpr bool five = TYPE == SHV_GGML_Q5_K;
        const int sub = g & 7;
        const uint8_t *b = row + (g >> 3) * (five ? 176 : 144);
        uint32_t sc, m;
        scale_min_k4(sub, b + 4, sc, m);
        const float d1 = half_at(b) * static_cast<float>(sc), m1 = half_at(b + 2) * static_cast<float>(m);
        const uint8_t *ql = b + (five ? 48 : 16) + (sub >> 1) * 32, *qh = b + 16;
        const uint32_t bit = 1u << sub;
        for (int l = 0; l < 32; l++) {
            uint32_t v = (sub & 1) ? ql[l] >> 4 : ql[l] & 0xFu;
            if (five && (qh[l] & bit)) v += 16;
            acc = fmaf(d1 * static_cast<float>(v) - m1, x[l], acc);
        }
    } else if constexpr (TYPE == SHV_GGML_Q6_K) {
        const int sub = g & 7;
        const uint8_t *b = row + (g >> 3) * 210;
        const uint8_t *ql = b, *qh = b + 128, *scs = b + 192;
        const float d = half_at(b + 208);
        const int n0 = (sub >> 2) * 128, quarter = sub & 3;
        for (int l = 0; l < 32; l++) {
            const uint32_t h = qh[n0 / 4 + l];
            const uint32_t lo = ql[n0 / 2 + l + (quarter & 1) * 32];
            const uint32_t nib = quarter >= 2 ? lo >> 4 : lo & 0xFu;
            const int q = static_cast<int>(nib | (((h >> (2 * quarter)) & 3u) << 4)) - 32;
            const float s = static_cast<float>(static_cast<int8_t>(scs[n0 / 16 + l / 16 + 2 * quarter]));
            acc = fmaf(d * s * static_cast<float>(q), x[l], acc);
        }
    }
    return acc;
}

// The same with the type known only at run time (uniform over a wave).
__device__ __forceinline__ float group_dot_rt(int type, const uint8_t *row, int g, const float *x) {
    switch (type) {
        case SHV_GGML_F32: return group_dot<SHV_GGML_F32>(row, g, x);
        case SHV_GGML_F16: return group_dot<SHV_GGML_F16>(row, g, x);
        case SHV_GGML_BF16: return group_dot<SHV_GGML_BF16>(row, g, x);
        case SHV_GGML_Q8_0: return group_dot<SHV_GGML_Q8_0>(row, g, x);
        case SHV_GGML_Q4_1: return group_dot<SHV_GGML_Q4_1>(row, g, x);
        case SHV_GGML_Q5_0: return group_dot<SHV_GGML_Q5_0>(row, g, x);
        case SHV_GGML_Q5_1: return group_dot<SHV_GGML_Q5_1>(row, g, x);
        case SHV_GGML_IQ4_NL: return group_dot<SHV_GGML_IQ4_NL>(row, g, x);
        case SHV_GGML_Q4_K: return group_dot<SHV_GGML_Q4_K>(row, g, x);
        case SHV_GGML_Q5_K: return group_dot<SHV_GGML_Q5_K>(row, g, x);
        case SHV_GGML_Q6_K: return group_dot<SHV_GGML_Q6_K>(row, g, x);
    }
    return 0.f;
}

// Whether k elements make whole blocks of the type.
inline bool whole_rows(int type, int k) {
    const int blk = type == SHV_GGML_Q4_K || type == SHV_GGML_Q5_K || type == SHV_GGML_Q6_K ? 256 : 32;
    return k > 0 && k % blk == 0 && row_bytes(type, k) > 0;
}

}  // namespace shv_any
