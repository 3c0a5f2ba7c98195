// Format-level kernels: bit-exact Q4_K dequantisation and on-device synthetic fill.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

// One thread per 64-weight group: 32 payload bytes -> 64 floats, written as the reference's
// dequantQ4_K orders them (32 low nibbles, then 32 high nibbles).  d*sc and dmin*m are formed
// first and the product and difference are rounded separately, so the bits are the reference's.
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t *w, float *dst, long long n_groups) {
    const long long gid = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (gid >= n_groups) return;
    const long long blk = gid >> 2;
    const int g = static_cast<int>(gid & 3);
    const uint8_t *bp = w + blk * SHV_Q4K_BYTES;
    const uint4 hdr = *reinterpret_cast<const uint4 *>(bp);
    uint32_t sc, mn;
    q4k_group_scale_min(hdr, g, sc, mn);
    const float d = f16_bits_to_f32(hdr.x), dmin = f16_bits_to_f32(hdr.x >> 16);
    const float d1 = __fmul_rn(d, static_cast<float>(sc & 0xFFu)), m1 = __fmul_rn(dmin, static_cast<float>(mn & 0xFFu));
    const float d2 = __fmul_rn(d, static_cast<float>(sc >> 8)), m2 = __fmul_rn(dmin, static_cast<float>(mn >> 8));
    const uint4 q0 = *reinterpret_cast<const uint4 *>(bp + 16 + g * 32);
    const uint4 q1 = *reinterpret_cast<const uint4 *>(bp + 32 + g * 32);
    const uint32_t q[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    float *o = dst + blk * SHV_Q4K_BLOCK + g * 64;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t byte = (q[i] >> (8 * b)) & 0xFFu;
            o[4 * i + b] = __fsub_rn(__fmul_rn(d1, static_cast<float>(byte & 0xFu)), m1);
            o[32 + 4 * i + b] = __fsub_rn(__fmul_rn(d2, static_cast<float>(byte >> 4)), m2);
        }
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// dst[i] = mean + std * z_i, z_i from Box-Muller on the two halves of splitmix64(seed, i).
__global__ __launch_bounds__(256) void fill_normal_kernel(float *dst, long long n, uint64_t seed, float mean, float std) {
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + static_cast<uint64_t>(i));
        const float u1 = (static_cast<float>(static_cast<uint32_t>(r >> 40)) + 1.0f) * (1.0f / 16777216.0f);
        const float u2 = static_cast<float>(static_cast<uint32_t>(r) >> 8) * (1.0f / 16777216.0f);
        const float rad = sqrtf(-2.0f * logf(u1));
        dst[i] = mean + std * rad * cosf(6.28318530717958647692f * u2);
    }
}

}  // namespace

int shv_launch_dequant_q4k(shv_ctx *ctx, const shv_dequant_q4k_args *a) {
    SHV_REQUIRE(a->w && a->dst, "dequant_q4k: NULL w or dst");
    SHV_REQUIRE(a->rows > 0 && a->k > 0 && a->k % SHV_Q4K_BLOCK == 0, "dequant_q4k: rows %lld, k %d", static_cast<long long>(a->rows), a->k);
    SHV_REQUIRE(shv_aligned16(a->w), "dequant_q4k: w must be 16-byte aligned");
    const long long groups = a->rows * (a->k / 64);
    const long long blocks = (groups + 255) / 256;
    SHV_REQUIRE(blocks < (1ll << 31), "dequant_q4k: %lld groups is too many for one launch", groups);
    hipLaunchKernelGGL(dequant_q4k_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx->stream,
                       static_cast<const uint8_t *>(a->w), a->dst, groups);
    SHV_HIP_CHECK(hipGetLastError());
    return SHV_OK;
}

int shv_launch_fill_normal(shv_ctx *ctx, const shv_fill_normal_args *a) {
    SHV_REQUIRE(a->dst && a->n > 0, "fill_normal: NULL dst or n = %lld", static_cast<long long>(a->n));
    long long blocks = (a->n + 255) / 256;
    const long long cap = static_cast<long long>(ctx->prop.multiProcessorCount) * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(fill_normal_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, ctx->stream, a->dst,
                       static_cast<long long>(a->n), a->seed, a->mean, a->std);
    SHV_HIP_CHECK(hipGetLastError());
    return SHV_OK;
}
