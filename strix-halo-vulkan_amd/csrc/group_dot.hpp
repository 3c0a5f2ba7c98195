// Rows of any tensor type the reference's loader accepts, a 32-element group at a time: the
// weights formed exactly as the format's CPU arm forms them (gguf/dequant.go:128-356) and dotted
// with 32 activations.  Shared by the any-type GEMV and the any-type expert kernels.
#pragma once
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace shv_any {

using namespace shv;

// N bytes from an address aligned to A (2, 4 or 16), in registers: loads as wide as the alignment
// allows instead of a byte at a time.  Indices are compile-time once the loops are unrolled.
template <int N, int A>
struct Span {
    static_assert(A == 2 || A == 4 || A == 16, "alignment");
    static_assert(N % A == 0, "whole loads");
    uint32_t w[(N + 3) / 4];
    __device__ __forceinline__ void load(const uint8_t *p) {
        if constexpr (A == 16) {
#pragma unroll
            for (int i = 0; i < N / 16; i++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(p + 16 * i);
                w[4 * i] = v.x, w[4 * i + 1] = v.y, w[4 * i + 2] = v.z, w[4 * i + 3] = v.w;
            }
        } else if constexpr (A == 4) {
#pragma unroll
            for (int i = 0; i < N / 4; i++) w[i] = *reinterpret_cast<const uint32_t *>(p + 4 * i);
        } else {
#pragma unroll
            for (int i = 0; i < (N + 3) / 4; i++) w[i] = 0;
#pragma unroll
            for (int i = 0; i < N / 2; i++) w[i >> 1] |= static_cast<uint32_t>(*reinterpret_cast<const uint16_t *>(p + 2 * i)) << (16 * (i & 1));
        }
    }
    __device__ __forceinline__ uint32_t u8(int i) const { return (w[i >> 2] >> ((i & 3) * 8)) & 0xFFu; }
    __device__ __forceinline__ int i8(int i) const { return static_cast<int>(w[i >> 2] << (24 - (i & 3) * 8)) >> 24; }
    __device__ __forceinline__ uint32_t u16(int i) const { return u8(i) | (u8(i + 1) << 8); }       // little-endian, at byte i
    __device__ __forceinline__ uint32_t u32(int i) const { return u16(i) | (u16(i + 2) << 16); }
    __device__ __forceinline__ float half(int i) const { return f16_bits_to_f32(u16(i)); }
};

// ggml's get_scale_min_k4 (gguf/dequant.go:238-243) over the 12 packed bytes at `at` of a span
template <typename S>
__device__ __forceinline__ void scale_min_k4(int j, const S &q, int at, uint32_t &sc, uint32_t &m) {
    // j differs from lane to lane: the three bytes are picked by comparison, not by indexing registers
    const int lo = j & 3;
    uint32_t b0 = 0, b4 = 0, b8 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (i == lo) b0 = q.u8(at + i), b4 = q.u8(at + 4 + i), b8 = q.u8(at + 8 + i);
    }
    if (j < 4) {
        sc = b0 & 63u;
        m = b4 & 63u;
    } else {
        sc = (b8 & 0xFu) | ((b0 >> 6) << 4);
        m = (b8 >> 4) | ((b4 >> 6) << 4);
    }
}

// kvalues_iq4nl (gguf/dequant.go:222-226), four to a word
__device__ __forceinline__ int iq4nl_value(uint32_t n) {
    constexpr uint32_t t0 = 0xBFAD9881u, t1 = 0xF6EADDCFu, t2 = 0x26190D01u, t3 = 0x71594535u;  // -127 -104 -83 -65 | -49 -35 -22 -10 | 1 13 25 38 | 53 69 89 113
    const uint32_t wv = (n & 8u) ? ((n & 4u) ? t3 : t2) : ((n & 4u) ? t1 : t0);
    return static_cast<int>(wv << (24 - (n & 3u) * 8)) >> 24;
}

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
// row is 16-byte aligned (a tensor's base is, and every row length here keeps the alignment its
// loads assume); x is 16-byte aligned.
template <int TYPE>
__device__ __forceinline__ float group_dot(const uint8_t *row, int g, const float *xp) {
    float x[32];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 v = reinterpret_cast<const float4 *>(xp)[i];
        x[4 * i] = v.x, x[4 * i + 1] = v.y, x[4 * i + 2] = v.z, x[4 * i + 3] = v.w;
    }
    float acc = 0.f;
    if constexpr (TYPE == SHV_GGML_F32) {
        Span<128, 16> s;
        s.load(row + g * 128);
#pragma unroll
        for (int j = 0; j < 32; j++) acc = fmaf(__uint_as_float(s.w[j]), x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_F16) {
        Span<64, 16> s;
        s.load(row + g * 64);
#pragma unroll
        for (int j = 0; j < 32; j++) acc = fmaf(s.half(2 * j), x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_BF16) {
        Span<64, 16> s;
        s.load(row + g * 64);
#pragma unroll
        for (int j = 0; j < 32; j++) acc = fmaf(__uint_as_float(s.u16(2 * j) << 16), x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_Q8_0) {
        Span<34, 2> s;
        s.load(row + g * 34);
        const float d = s.half(0);
#pragma unroll
        for (int j = 0; j < 32; j++) acc = fmaf(static_cast<float>(s.i8(2 + j)) * d, x[j], acc);
    } else if constexpr (TYPE == SHV_GGML_Q4_1) {
        Span<20, 4> s;
        s.load(row + g * 20);
        const float d = s.half(0), m = s.half(2);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(s.u8(4 + j) & 0x0F) * d + m, x[j], acc);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(s.u8(4 + j) >> 4) * d + m, x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_Q5_0) {
        Span<22, 2> s;
        s.load(row + g * 22);
        const float d = s.half(0);
        const uint32_t qh = s.u32(2);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(static_cast<int>((s.u8(6 + j) & 0x0Fu) | (((qh >> j) << 4) & 0x10u)) - 16) * d, x[j], acc);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>(static_cast<int>((s.u8(6 + j) >> 4) | ((qh >> (j + 12)) & 0x10u)) - 16) * d, x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_Q5_1) {
        Span<24, 4> s;
        s.load(row + g * 24);
        const float d = s.half(0), m = s.half(2);
        const uint32_t qh = s.w[1];
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>((s.u8(8 + j) & 0x0Fu) | (((qh >> j) << 4) & 0x10u)) * d + m, x[j], acc);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(static_cast<float>((s.u8(8 + j) >> 4) | ((qh >> (j + 12)) & 0x10u)) * d + m, x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_IQ4_NL) {
        Span<18, 2> s;
        s.load(row + g * 18);
        const float d = s.half(0);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(d * static_cast<float>(iq4nl_value(s.u8(2 + j) & 0xFu)), x[j], acc);
#pragma unroll
        for (int j = 0; j < 16; j++) acc = fmaf(d * static_cast<float>(iq4nl_value(s.u8(2 + j) >> 4)), x[j + 16], acc);
    } else if constexpr (TYPE == SHV_GGML_Q4_K || TYPE == SHV_GGML_Q5_K) {
        constexpr bool five = TYPE == SHV_GGML_Q5_K;
        const int sub = g & 7;
        const uint8_t *b = row + (g >> 3) * (five ? 176 : 144);
        Span<16, 16> hd;  // d, dmin, the 12 packed scale bytes
        hd.load(b);
        uint32_t sc, m;
        scale_min_k4(sub, hd, 4, sc, m);
        const float d1 = hd.half(0) * static_cast<float>(sc), m1 = hd.half(2) * static_cast<float>(m);
        Span<32, 16> ql, qh;
        ql.load(b + (five ? 48 : 16) + (sub >> 1) * 32);
        if constexpr (five) qh.load(b + 16);
        const uint32_t bit = 1u << sub;
        const int shift = (sub & 1) * 4;
#pragma unroll
        for (int l = 0; l < 32; l++) {
            uint32_t v = (ql.u8(l) >> shift) & 0xFu;
            if constexpr (five) {
                if (qh.u8(l) & bit) v += 16;
            }
            acc = fmaf(d1 * static_cast<float>(v) - m1, x[l], acc);
        }
    } else if constexpr (TYPE == SHV_GGML_Q6_K) {
        const int sub = g & 7;
        const uint8_t *b = row + (g >> 3) * 210;
        const int n0 = (sub >> 2) * 128, quarter = sub & 3;
        Span<32, 2> ql, qh;
        ql.load(b + n0 / 2 + (quarter & 1) * 32);
        qh.load(b + 128 + n0 / 4);
        Span<2, 2> sc, dd;
        sc.load(b + 192 + n0 / 16 + 2 * quarter);
        dd.load(b + 208);
        const float d = dd.half(0);
        const float s0 = static_cast<float>(sc.i8(0)), s1 = static_cast<float>(sc.i8(1));
        const int nshift = quarter >= 2 ? 4 : 0, hshift = 2 * quarter;
#pragma unroll
        for (int l = 0; l < 32; l++) {
            const uint32_t nib = (ql.u8(l) >> nshift) & 0xFu;
            const int q = static_cast<int>(nib | (((qh.u8(l) >> hshift) & 3u) << 4)) - 32;
            acc = fmaf(d * (l < 16 ? s0 : s1) * static_cast<float>(q), x[l], acc);
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
