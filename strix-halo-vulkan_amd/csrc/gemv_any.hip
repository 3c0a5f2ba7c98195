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
    static std::atomic<bool> raised{false};
    if (lds > 48 * 1024 && !raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_any_kernel<TYPE>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised.store(true, std::memory_order_release);
    }
    SHV_LAUNCH(ctx, gemv_any_kernel<TYPE>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), lds, a);
    return SHV_OK;
}

}  // namespace

int shv_launch_gemv(shv_ctx *ctx, const shv_gemv_args *pa) {
    const shv_gemv_args &a = *pa;
    SHV_REQUIRE(a.w && a.x && a.y, "gemv: NULL w, x or y");
    SHV_REQUIRE(a.n > 0 && a.k > 0, "gemv: %d x %d", a.n, a.k);
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
