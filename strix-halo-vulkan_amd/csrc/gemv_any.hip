// y = W x for a weight matrix in any tensor type the reference's loader accepts: the CPU path's
// matvec over Tensor.DequantizeRow (llm/hc.go:255-264, gguf/dequant.go:119-124) for the tensors
// of a checkpoint that are not Q4_K (a UD-Q4_K_XL file keeps dense projections in Q8_0 and some
// banks in Q5_K / Q6_K).  HBM-bound like the Q4_K kernel, not yet tuned like it: a lane takes one
// 32-element group of a row, dequantises it exactly as the format's CPU arm does and multiplies
// it with its 32 activations from LDS; a wave owns a row at a time and adds the lanes up.
#include "group_dot.hpp"

namespace {

using namespace shv;
using namespace shv_any;

constexpr int kBlock = 256;
constexpr int kRowsPerWave = 4;  // rows a wave has in flight
constexpr int kTokMax = 4;       // activation rows a launch multiplies with one reading of the weights

// grid: ceil(n / (4 waves * kRowsPerWave)) blocks; the launch's rows of x staged once per block in LDS, with the
// RMSNorm's gamma if there is one (the norm's factor goes onto the finished sums)
template <int TYPE>
__global__ __launch_bounds__(kBlock) void gemv_any_kernel(shv_gemv_args a, int t0, int nt) {
    extern __shared__ __align__(16) float xs[];  // [nt][k]
    __shared__ float red[kTokMax][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int xst = a.x_stride > 0 ? a.x_stride : a.k, yst = a.y_stride > 0 ? a.y_stride : a.n;
    for (int t = 0; t < nt; t++) {
        const float *x = a.x + static_cast<size_t>(t0 + t) * xst;
        float ss = 0.f;
        for (int c = tid; c < a.k; c += kBlock) {
            const float v = x[c];
            ss = fmaf(v, v, ss);
            xs[t * a.k + c] = a.gamma ? v * a.gamma[c] : v;
        }
        ss = wave_sum_all(ss);
        if (lane == 0) red[t][wave] = ss;
    }
    __syncthreads();
    float scale[kTokMax];
#pragma unroll
    for (int t = 0; t < kTokMax; t++)
        scale[t] = (a.gamma && t < nt) ? 1.f / sqrtf(((red[t][0] + red[t][1]) + (red[t][2] + red[t][3])) / static_cast<float>(a.k) + a.eps) : 1.f;
    const long long rb = row_bytes(TYPE, a.k);
    const int groups = a.k / 32;
    const long long row0 = (static_cast<long long>(blockIdx.x) * 4 + wave) * kRowsPerWave;
#pragma unroll
    for (int r = 0; r < kRowsPerWave; r++) {
        const long long row = row0 + r;
        if (row >= a.n) break;
        const uint8_t *rp = static_cast<const uint8_t *>(a.w) + row * rb;
        for (int t = 0; t < nt; t++) {
            float acc = 0.f;
            for (int g = lane; g < groups; g += 64) acc += group_dot<TYPE>(rp, g, xs + t * a.k + g * 32);
            acc = wave_sum_all(acc) * scale[t];
            const size_t at = static_cast<size_t>(t0 + t) * yst + row;
            if (lane == 0) a.y[at] = a.residual ? acc + a.residual[at] : acc;
        }
    }
}

template <int TYPE>
int launch_type(shv_ctx *ctx, const shv_gemv_args &a) {
    const long long per_block = 4ll * kRowsPerWave;
    const long long blocks = (a.n + per_block - 1) / per_block;
    SHV_REQUIRE(blocks < (1ll << 31), "gemv: %d rows is too many for one launch", a.n);
    const int rows = a.n_tok > 0 ? a.n_tok : 1;
    SHV_REQUIRE(static_cast<size_t>(a.k) * 4 <= 64 * 1024, "gemv: k = %d does not fit the staging of x", a.k);
    const int per = 16384 / a.k >= kTokMax ? kTokMax : 16384 / a.k >= 1 ? 16384 / a.k : 1;  // rows a launch stages: up to 64 KB of them
    for (int t0 = 0; t0 < rows; t0 += per) {
        const int nt = rows - t0 < per ? rows - t0 : per;
        const size_t lds = static_cast<size_t>(a.k) * 4 * nt;
        static std::atomic<size_t> raised{0};
        if (lds > 48 * 1024 && lds > raised.load(std::memory_order_acquire)) {
            SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_any_kernel<TYPE>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            raised.store(lds, std::memory_order_release);
        }
        SHV_LAUNCH(ctx, gemv_any_kernel<TYPE>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), lds, a, t0, nt);
    }
    return SHV_OK;
}

}  // namespace

int shv_launch_gemv(shv_ctx *ctx, const shv_gemv_args *pa) {
    const shv_gemv_args &a = *pa;
    SHV_REQUIRE(a.w && a.x && a.y, "gemv: NULL w, x or y");
    SHV_REQUIRE(a.n > 0 && a.k > 0, "gemv: %d x %d", a.n, a.k);
    SHV_REQUIRE(a.n_tok >= 0 && a.n_tok <= 4096, "gemv: n_tok %d", a.n_tok);
    SHV_REQUIRE(a.n_tok <= 1 || ((a.x_stride == 0 || a.x_stride >= a.k) && (a.y_stride == 0 || a.y_stride >= a.n)), "gemv: rows %d and %d floats apart for k %d, n %d",
                a.x_stride, a.y_stride, a.k, a.n);
    SHV_REQUIRE(shv_aligned16(a.w), "gemv: the weight matrix must be 16-byte aligned");
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
