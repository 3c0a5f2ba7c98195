// y = W x for a weight matrix in any tensor type the reference's loader accepts: the CPU path's
// matvec over Tensor.DequantizeRow (llm/hc.go:255-264, gguf/dequant.go:119-124) for the tensors
// of a checkpoint that are not Q4_K (a UD-Q4_K_XL file keeps dense projections in Q8_0 and some
// banks in Q5_K / Q6_K).  HBM-bound like the Q4_K kernel, not yet tuned like it: a lane takes one
// 32-element group of a row, dequantises it exactly as the format's CPU arm does and multiplies
// it with its 32 activations from LDS; a wave owns a row at a time and adds the lanes up.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kRowsPerWave = 4;  // rows a wave has in flight

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
__device__ const int8_t kValuesIQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

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

// grid: ceil(n / (4 waves * kRowsPerWave)) blocks; x staged once per block in LDS
template <int TYPE>
__global__ __launch_bounds__(kBlock) void gemv_any_kernel(shv_gemv_args a) {
    extern __shared__ __align__(16) float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int c = tid; c < a.k; c += kBlock) xs[c] = a.x[c];
    __syncthreads();
    const long long rb = row_bytes(TYPE, a.k);
    const int groups = a.k / 32;
    const long long row0 = (static_cast<long long>(blockIdx.x) * 4 + wave) * kRowsPerWave;
#pragma unroll
    for (int r = 0; r < kRowsPerWave; r++) {
        const long long row = row0 + r;
        if (row >= a.n) break;
        const uint8_t *rp = static_cast<const uint8_t *>(a.w) + row * rb;
        float acc = 0.f;
        for (int g = lane; g < groups; g += 64) acc += group_dot<TYPE>(rp, g, xs + g * 32);
        acc = wave_sum_all(acc);
        if (lane == 0) a.y[row] = a.residual ? acc + a.residual[row] : acc;
    }
}

template <int TYPE>
int launch_type(shv_ctx *ctx, const shv_gemv_args &a) {
    const long long per_block = 4ll * kRowsPerWave;
    const long long blocks = (a.n + per_block - 1) / per_block;
    SHV_REQUIRE(blocks < (1ll << 31), "gemv: %d rows is too many for one launch", a.n);
    const size_t lds = static_cast<size_t>(a.k) * 4;
    SHV_REQUIRE(lds <= 64 * 1024, "gemv: k = %d does not fit the staging of x", a.k);
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_any_kernel<TYPE>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised = true;
    }
    SHV_LAUNCH(ctx, gemv_any_kernel<TYPE>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), lds, a);
    return SHV_OK;
}

}  // namespace

int shv_launch_gemv(shv_ctx *ctx, const shv_gemv_args *pa) {
    const shv_gemv_args &a = *pa;
    SHV_REQUIRE(a.w && a.x && a.y, "gemv: NULL w, x or y");
    SHV_REQUIRE(a.n > 0 && a.k > 0, "gemv: %d x %d", a.n, a.k);
    const int blk = a.type == SHV_GGML_Q4_K || a.type == SHV_GGML_Q5_K || a.type == SHV_GGML_Q6_K ? 256 : 32;
    SHV_REQUIRE(row_bytes(a.type, a.k) > 0 && a.k % blk == 0, "gemv: rows of %d elements of ggml type %d (not a type the loader accepts, or not whole blocks)", a.k, a.type);
    switch (a.type) {
        case SHV_GGML_F32: return launch_type<SHV_GGML_F32>(ctx, a);
        case SHV_GGML_F16: return launch_type<SHV_GGML_F16>(ctx, a);
        case SHV_GGML_BF16: return launch_type<SHV_GGML_BF16>(ctx, a);
        case SHV_GGML_Q8_0: return launch_type<SHV_GGML_Q8_0>(ctx, a);
        case SHV_GGML_Q4_1: return launch_type<SHV_GGML_Q4_1>(ctx, a);
        case SHV_GGML_Q5_0: return launch_type<SHV_GGML_Q5_0>(ctx, a);
        case SHV_GGML_Q5_1: return launch_type<SHV_GGML_Q5_1>(ctx, a);
        case SHV_GGML_IQ4_NL: return launch_type<SHV_GGML_IQ4_NL>(ctx, a);
        case SHV_GGML_Q4_K: return launch_type<SHV_GGML_Q4_K>(ctx, a);
        case SHV_GGML_Q5_K: return launch_type<SHV_GGML_Q5_K>(ctx, a);
        case SHV_GGML_Q6_K: return launch_type<SHV_GGML_Q6_K>(ctx, a);
    }
    return shv_set_error(SHV_E_INVALID, "gemv: ggml type %d", a.type);
}
