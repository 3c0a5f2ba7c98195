// Dequantisers for the GGUF tensor types a checkpoint mixes with Q4_K (gguf/dequant.go:52-98 and the
// arms below it): what a loader needs to bring a tensor of any accepted type to float32 on the
// device.  One thread per 32 output elements (a block of the 32-element types, an eighth of a
// K-quant super-block); every product, sum and difference is rounded on its own, as on a CPU that
// never fuses a multiply-add, so the bits are ggml's.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

__device__ __forceinline__ float half_at(const uint8_t *b) { return f16_bits_to_f32(static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8)); }
__device__ __forceinline__ uint32_t u32_at(const uint8_t *b) {
    return static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8) | (static_cast<uint32_t>(b[2]) << 16) | (static_cast<uint32_t>(b[3]) << 24);
}

// ggml's get_scale_min_k4 (gguf/dequant.go:238-243)
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

// Group g (32 outputs) of a run of n elements starting at src, written to o.
__device__ __forceinline__ void dequant_group(int type, const uint8_t *src, long long g, long long n, float *o) {
    switch (type) {
        case SHV_GGML_F32: {
            const int m = n - g * 32 < 32 ? static_cast<int>(n - g * 32) : 32;
            for (int j = 0; j < m; j++) o[j] = __uint_as_float(u32_at(src + (g * 32 + j) * 4));
            break;
        }
        case SHV_GGML_F16: {
            const int m = n - g * 32 < 32 ? static_cast<int>(n - g * 32) : 32;
            for (int j = 0; j < m; j++) o[j] = half_at(src + (g * 32 + j) * 2);
            break;
        }
        case SHV_GGML_BF16: {
            const int m = n - g * 32 < 32 ? static_cast<int>(n - g * 32) : 32;
            for (int j = 0; j < m; j++) {
                const uint8_t *b = src + (g * 32 + j) * 2;
                o[j] = __uint_as_float((static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8)) << 16);
            }
            break;
        }
        case SHV_GGML_Q8_0: {  // gguf/dequant.go:128-137
            const uint8_t *b = src + g * 34;
            const float d = half_at(b);
            for (int j = 0; j < 32; j++) o[j] = __fmul_rn(static_cast<float>(static_cast<int8_t>(b[2 + j])), d);
            break;
        }
        case SHV_GGML_Q4_1: {  // :146-161
            const uint8_t *b = src + g * 20;
            const float d = half_at(b), m = half_at(b + 2);
            for (int j = 0; j < 16; j++) {
                o[j] = __fadd_rn(__fmul_rn(static_cast<float>(b[4 + j] & 0x0F), d), m);
                o[j + 16] = __fadd_rn(__fmul_rn(static_cast<float>(b[4 + j] >> 4), d), m);
            }
            break;
        }
        case SHV_GGML_Q5_0: {  // :171-190
            const uint8_t *b = src + g * 22;
            const float d = half_at(b);
            const uint32_t qh = u32_at(b + 2);
            for (int j = 0; j < 16; j++) {
                const int x0 = static_cast<int>((b[6 + j] & 0x0Fu) | (((qh >> j) << 4) & 0x10u)) - 16;
                const int x1 = static_cast<int>((b[6 + j] >> 4) | ((qh >> (j + 12)) & 0x10u)) - 16;
                o[j] = __fmul_rn(static_cast<float>(x0), d);
                o[j + 16] = __fmul_rn(static_cast<float>(x1), d);
            }
            break;
        }
        case SHV_GGML_Q5_1: {  // :197-217
            const uint8_t *b = src + g * 24;
            const float d = half_at(b), m = half_at(b + 2);
            const uint32_t qh = u32_at(b + 4);
            for (int j = 0; j < 16; j++) {
                const uint32_t x0 = (b[8 + j] & 0x0Fu) | (((qh >> j) << 4) & 0x10u);
                const uint32_t x1 = (b[8 + j] >> 4) | ((qh >> (j + 12)) & 0x10u);
                o[j] = __fadd_rn(__fmul_rn(static_cast<float>(x0), d), m);
                o[j + 16] = __fadd_rn(__fmul_rn(static_cast<float>(x1), d), m);
            }
            break;
        }
        case SHV_GGML_IQ4_NL: {  // :222-234
            const uint8_t *b = src + g * 18;
            const float d = half_at(b);
            for (int j = 0; j < 16; j++) {
                o[j] = __fmul_rn(d, static_cast<float>(kValuesIQ4NL[b[2 + j] & 0xF]));
                o[j + 16] = __fmul_rn(d, static_cast<float>(kValuesIQ4NL[b[2 + j] >> 4]));
            }
            break;
        }
        case SHV_GGML_Q4_K:    // :252-276
        case SHV_GGML_Q5_K: {  // :282-317
            const bool five = type == SHV_GGML_Q5_K;
            const int sub = static_cast<int>(g & 7);  // sub-block of 32: low nibbles when even, high when odd
            const uint8_t *b = src + (g >> 3) * (five ? 176 : 144);
            const float d = half_at(b), dmin = half_at(b + 2);
            uint32_t sc, m;
            scale_min_k4(sub, b + 4, sc, m);
            const float d1 = __fmul_rn(d, static_cast<float>(sc)), m1 = __fmul_rn(dmin, static_cast<float>(m));
            const uint8_t *ql = b + (five ? 48 : 16) + (sub >> 1) * 32, *qh = b + 16;
            const uint32_t bit = 1u << sub;  // u1, u2 of the reference: 1,2 then 4,8 ...
            for (int l = 0; l < 32; l++) {
                uint32_t v = (sub & 1) ? ql[l] >> 4 : ql[l] & 0xFu;
                if (five && (qh[l] & bit)) v += 16;
                o[l] = __fsub_rn(__fmul_rn(d1, static_cast<float>(v)), m1);
            }
            break;
        }
        case SHV_GGML_Q6_K: {  // :331-356
            const int sub = static_cast<int>(g & 7);  // outputs 32*sub .. +31 of the super-block
            const uint8_t *b = src + (g >> 3) * 210;
            const uint8_t *ql = b, *qh = b + 128, *scs = b + 192;
            const float d = half_at(b + 208);
            const int n0 = (sub >> 2) * 128, quarter = sub & 3;  // the 128-element pass and which of its four quarters
            for (int l = 0; l < 32; l++) {
                const uint32_t h = qh[n0 / 4 + l];
                const uint32_t lo = ql[n0 / 2 + l + (quarter & 1) * 32];
                const uint32_t nib = quarter >= 2 ? lo >> 4 : lo & 0xFu;
                const int q = static_cast<int>(nib | (((h >> (2 * quarter)) & 3u) << 4)) - 32;
                const float s = static_cast<float>(static_cast<int8_t>(scs[n0 / 16 + l / 16 + 2 * quarter]));
                o[l] = __fmul_rn(__fmul_rn(d, s), static_cast<float>(q));
            }
            break;
        }
    }
}

__global__ __launch_bounds__(256) void dequant_kernel(int type, const uint8_t *src, float *dst, long long n) {
    const long long g = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;  // group of 32 outputs
    if (g * 32 >= n) return;
    dequant_group(type, src, g, n, dst + g * 32);
}

// Embedding rows out of a table kept in the checkpoint's own type: row id_t expanded as
// Tensor.DequantizeRow does (llm/model.go:125-131, gguf/dequant.go:119-124).  grid (groups/64, n_tok).
__global__ __launch_bounds__(64) void embed_typed_kernel(shv_embed_args a, long long row_bytes) {
    const int t = blockIdx.y;
    const int g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g * 32 >= a.n_embd) return;
    const int id = a.ids[(a.pos ? a.pos[0] : 0) + t];
    float *o = a.x + static_cast<size_t>(t) * a.x_stride + g * 32;
    if (id < 0 || id >= a.vocab) {
        const int m = a.n_embd - g * 32 < 32 ? a.n_embd - g * 32 : 32;
        for (int j = 0; j < m; j++) o[j] = __int_as_float(0x7fc00000);
        return;
    }
    dequant_group(a.type, static_cast<const uint8_t *>(a.table) + static_cast<long long>(id) * row_bytes, g, a.n_embd, o);
}

}  // namespace

// Bytes of n elements of a type, or -1 for a type the loader refuses / a count that is not whole blocks.
long long shv_type_bytes(int type, long long n) {
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

int shv_launch_dequant(shv_ctx *ctx, const shv_dequant_args *a) {
    SHV_REQUIRE(a->src && a->dst, "dequant: NULL src or dst");
    SHV_REQUIRE(a->n > 0 && shv_type_bytes(a->type, a->n) > 0, "dequant: %lld elements of ggml type %d (not a type the loader accepts, or not whole blocks)",
                static_cast<long long>(a->n), a->type);
    const long long groups = (a->n + 31) / 32, blocks = (groups + 255) / 256;
    SHV_REQUIRE(blocks < (1ll << 31), "dequant: %lld elements is too many for one launch", static_cast<long long>(a->n));
    SHV_LAUNCH(ctx, dequant_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, a->type, static_cast<const uint8_t *>(a->src), a->dst,
               static_cast<long long>(a->n));
    return SHV_OK;
}

int shv_launch_embed_typed(shv_ctx *ctx, const shv_embed_args *a) {
    const long long row_bytes = shv_type_bytes(a->type, a->n_embd);
    SHV_REQUIRE(row_bytes > 0, "embed: a row of %d elements of ggml type %d (not a type the loader accepts, or not whole blocks)", a->n_embd, a->type);
    SHV_LAUNCH(ctx, embed_typed_kernel, dim3((a->n_embd / 32 + 63) / 64, a->n_tok), dim3(64), 0, *a, row_bytes);
    return SHV_OK;
}
