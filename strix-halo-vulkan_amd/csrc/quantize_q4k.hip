// The reference's round-to-nearest Q4_K quantiser (ggml quantize_row_q4_K_ref) on the device, so a
// synthetic model of any size can be drawn and quantised in HBM.  The arithmetic is kept
// operation for operation in float32 — this file is compiled with floating-point contraction off
// — because the 21-rung scale search picks its rung by comparing near-equal float32 sums.
//
// 256 threads take 32 super-blocks: 8 threads per super-block, one per 32-weight group.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

constexpr int kGroup = 32;
constexpr int kNmax = 15;

__device__ __forceinline__ float nearest_int(float v) { return rintf(v); }

__device__ __forceinline__ float clamp_level(float f) {
    float l = nearest_int(f);
    if (l < 0.f) l = 0.f;
    if (l > static_cast<float>(kNmax)) l = static_cast<float>(kNmax);
    return l;
}

// make_qkx2_quants with (rmin, rdelta, nstep) = (-1, 0.1, 20); returns scale, the_min = -min.
__device__ void make_qkx_quants(const float *x, const float *w, float &scale_out, float &min_out) {
    float mn = x[0], mx = x[0];
    float sumW = w[0], sumX = w[0] * x[0];
    for (int i = 1; i < kGroup; i++) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        sumW += w[i];
        sumX += w[i] * x[i];
    }
    if (mn > 0.f) mn = 0.f;
    if (mx <= mn) {
        scale_out = 0.f;
        min_out = -mn;
        return;
    }
    float iscale = static_cast<float>(kNmax) / (mx - mn);
    float scale = 1.f / iscale;
    float bestErr = 0.f;
    for (int i = 0; i < kGroup; i++) {
        const float l = clamp_level(iscale * (x[i] - mn));
        const float diff = scale * l + mn - x[i];
        bestErr += w[i] * diff * diff;
    }
    // `mn` is the running best minimum: a rung that improves the fit moves it, and the rungs
    // after it are cut against the moved value, as in ggml.
    for (int is = 0; is <= 20; is++) {
        const float cur = mn;
        iscale = (-1.0f + 0.1f * static_cast<float>(is) + static_cast<float>(kNmax)) / (mx - cur);
        float sumL = 0.f, sumL2 = 0.f, sumXL = 0.f;
        for (int i = 0; i < kGroup; i++) {
            const float fl = clamp_level(iscale * (x[i] - cur));
            sumL += w[i] * fl;
            sumL2 += w[i] * fl * fl;
            sumXL += w[i] * fl * x[i];
        }
        const float det = sumW * sumL2 - sumL * sumL;
        if (det <= 0.f) continue;
        float thisScale = (sumW * sumXL - sumX * sumL) / det;
        float thisMin = (sumL2 * sumX - sumL * sumXL) / det;
        if (thisMin > 0.f) {
            thisMin = 0.f;
            thisScale = sumXL / sumL2;
        }
        float err = 0.f;
        for (int i = 0; i < kGroup; i++) {
            const float fl = clamp_level(iscale * (x[i] - cur));
            const float diff = thisScale * fl + thisMin - x[i];
            err += w[i] * diff * diff;
        }
        if (err < bestErr) {
            bestErr = err;
            scale = thisScale;
            mn = thisMin;
        }
    }
    scale_out = scale;
    min_out = -mn;
}

__device__ __forceinline__ int clamp63(float v) { return v < 0.f ? 0 : (v > 63.f ? 63 : static_cast<int>(v)); }

__global__ __launch_bounds__(256) void quantize_q4k_kernel(const float *src, uint8_t *dst, long long n_blocks) {
    __shared__ uint8_t lv[32][256];
    __shared__ uint8_t ls[32][8], lm[32][8];
    __shared__ uint32_t dd[32];
    const int tid = threadIdx.x, sbl = tid >> 3, j = tid & 7;
    const long long blk = static_cast<long long>(blockIdx.x) * 32 + sbl;
    const bool live = blk < n_blocks;
    float x[kGroup], w[kGroup];
    float scale = 0.f, themin = 0.f;
    if (live) {
        const float4 *p = reinterpret_cast<const float4 *>(src + blk * SHV_Q4K_BLOCK + j * kGroup);
#pragma unroll
        for (int i = 0; i < kGroup / 4; i++) {
            const float4 f = p[i];
            x[4 * i] = f.x; x[4 * i + 1] = f.y; x[4 * i + 2] = f.z; x[4 * i + 3] = f.w;
        }
        float sum2 = 0.f;
        for (int i = 0; i < kGroup; i++) sum2 += x[i] * x[i];
        const float q = sum2 / static_cast<float>(kGroup);
        const float avx = q <= 0.f ? 0.f : sqrtf(q);
        for (int i = 0; i < kGroup; i++) w[i] = avx + fabsf(x[i]);
        make_qkx_quants(x, w, scale, themin);
    }
    // maxima over the 8 groups of the super-block (8 consecutive lanes)
    float maxScale = scale, maxMin = themin;
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) {
        maxScale = fmaxf(maxScale, __shfl_xor(maxScale, off, 64));
        maxMin = fmaxf(maxMin, __shfl_xor(maxMin, off, 64));
    }
    // the reference starts both maxima at +0 and replaces them only by something greater, so a
    // group minimum of -0.0 must not survive as the super-block's
    if (!(maxScale > 0.f)) maxScale = 0.f;
    if (!(maxMin > 0.f)) maxMin = 0.f;
    const float invScale = maxScale > 0.f ? 63.f / maxScale : 0.f;
    const float invMin = maxMin > 0.f ? 63.f / maxMin : 0.f;
    const int LS = clamp63(nearest_int(invScale * scale));
    const int LM = clamp63(nearest_int(invMin * themin));
    const __half dh = __float2half_rn(maxScale / 63.f), dmh = __float2half_rn(maxMin / 63.f);
    const float DF = __half2float(dh), DMinF = __half2float(dmh);
    if (live) {
        const float ds = DF * static_cast<float>(LS), dm = DMinF * static_cast<float>(LM);
        for (int i = 0; i < kGroup; i++) {
            float l = 0.f;
            if (ds != 0.f) {
                l = nearest_int((x[i] + dm) / ds);
                if (l < 0.f) l = 0.f;
                if (l > static_cast<float>(kNmax)) l = static_cast<float>(kNmax);
            }
            lv[sbl][j * kGroup + i] = static_cast<uint8_t>(l);
        }
        ls[sbl][j] = static_cast<uint8_t>(LS);
        lm[sbl][j] = static_cast<uint8_t>(LM);
        if (j == 0) dd[sbl] = static_cast<uint32_t>(__half_as_ushort(dh)) | (static_cast<uint32_t>(__half_as_ushort(dmh)) << 16);
    }
    __syncthreads();
    if (!live) return;
    // pack: thread j writes 16 payload bytes j*16..j*16+15, and threads 0..3 a header dword each
    uint8_t *rec = dst + blk * SHV_Q4K_BYTES;
    {
        const int h = j >> 1, l0 = (j & 1) * 16;
        uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t lo = lv[sbl][h * 64 + l0 + i], hi = lv[sbl][h * 64 + 32 + l0 + i];
            out[i >> 2] |= ((lo & 0xFu) | ((hi & 0xFu) << 4)) << (8 * (i & 3));
        }
        *reinterpret_cast<uint4 *>(rec + 16 + j * 16) = make_uint4(out[0], out[1], out[2], out[3]);
    }
    if (j == 0) {
        *reinterpret_cast<uint32_t *>(rec) = dd[sbl];
    } else if (j <= 3) {
        // scale bytes 4(j-1)..4(j-1)+3 of the 12, ggml's packing (get_scale_min_k4 inverted)
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int idx = (j - 1) * 4 + b;
            uint32_t v;
            if (idx < 4) v = ls[sbl][idx] | ((ls[sbl][idx + 4] >> 4) << 6);
            else if (idx < 8) v = lm[sbl][idx - 4] | ((lm[sbl][idx] >> 4) << 6);
            else v = (ls[sbl][idx - 4] & 0xFu) | ((lm[sbl][idx - 4] & 0xFu) << 4);
            word |= (v & 0xFFu) << (8 * b);
        }
        *reinterpret_cast<uint32_t *>(rec + 4 + (j - 1) * 4) = word;
    }
}

}  // namespace

int shv_launch_quantize_q4k(shv_ctx *ctx, const shv_quantize_q4k_args *a) {
    SHV_REQUIRE(a->src && a->dst, "quantize_q4k: NULL src or dst");
    SHV_REQUIRE(a->rows > 0 && a->k > 0 && a->k % SHV_Q4K_BLOCK == 0, "quantize_q4k: rows %lld, k %d", static_cast<long long>(a->rows), a->k);
    SHV_REQUIRE(shv_aligned16(a->src) && shv_aligned16(a->dst), "quantize_q4k: src and dst must be 16-byte aligned");
    const long long n_blocks = a->rows * (a->k / SHV_Q4K_BLOCK);
    const long long grid = (n_blocks + 31) / 32;
    SHV_REQUIRE(grid < (1ll << 31), "quantize_q4k: %lld super-blocks is too many for one launch", n_blocks);
    SHV_LAUNCH(ctx, quantize_q4k_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, a->src,
                       static_cast<uint8_t *>(a->dst), n_blocks);
    return SHV_OK;
}
