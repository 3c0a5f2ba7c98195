// The router's rows carried through the output projection that feeds them.
//
// A decode step's layer ends its mixer with y = x + W pro(v) (W the Q4_K output projection) and
// starts its MoE block with logits = R (gamma * y) * f, f = rsqrt(mean(y^2) + eps) the RMSNorm's
// factor and R the float32 router with the shared gate as its last row (llm/moe.go:219-232,
// 396-402; llm/hc.go:176-190).  Up to f the logits are linear in [pro(v) | x]:
//     R diag(gamma) y = (R diag(gamma) W) pro(v) + (R diag(gamma)) x
// so with the table [R diag(gamma) W | R diag(gamma)] made once here, the output projection's
// launch can form them beside its own rows and the router needs no launch of its own.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

// out[e][k + i] = R[e][i] * gamma[i]; grid (ceil(n_embd/256), rows)
__global__ __launch_bounds__(256) void router_fold_scale_kernel(shv_router_fold_args a, int rows) {
    const int i = blockIdx.x * 256 + threadIdx.x, e = blockIdx.y;
    if (i >= a.n_embd || e >= rows) return;
    const float *r = e < a.n_expert ? a.router + static_cast<size_t>(e) * a.n_embd : a.shared_gate;
    a.out[static_cast<size_t>(e) * (a.k + a.n_embd) + a.k + i] = r[i] * a.gamma[i];
}

// out[e][j] = sum_i out[e][k + i] * Wf[i][j], Wf the projection expanded to float32 [n_embd][k],
// accumulated in float64 and rounded once.  grid (k/256, ceil(rows/kE)); a thread owns column j
// for kE router rows, whose scaled entries come through LDS 256 at a time.
constexpr int kE = 16;
__global__ __launch_bounds__(256) void router_fold_product_kernel(shv_router_fold_args a, int rows) {
    __shared__ float rs[kE][256];
    const int j = blockIdx.x * 256 + threadIdx.x, e0 = blockIdx.y * kE;
    const size_t stride = static_cast<size_t>(a.k) + a.n_embd;
    double acc[kE];
#pragma unroll
    for (int e = 0; e < kE; e++) acc[e] = 0.0;
    for (int i0 = 0; i0 < a.n_embd; i0 += 256) {
        __syncthreads();
#pragma unroll
        for (int e = 0; e < kE; e++) {
            const int i = i0 + threadIdx.x;
            rs[e][threadIdx.x] = (e0 + e < rows && i < a.n_embd) ? a.out[static_cast<size_t>(e0 + e) * stride + a.k + i] : 0.f;
        }
        __syncthreads();
        const int ni = a.n_embd - i0 < 256 ? a.n_embd - i0 : 256;
        for (int ii = 0; ii < ni; ii++) {
            const double w = j < a.k ? static_cast<double>(a.scratch[static_cast<size_t>(i0 + ii) * a.k + j]) : 0.0;
#pragma unroll
            for (int e = 0; e < kE; e++) acc[e] = fma(static_cast<double>(rs[e][ii]), w, acc[e]);
        }
    }
    if (j < a.k) {
#pragma unroll
        for (int e = 0; e < kE; e++)
            if (e0 + e < rows) a.out[static_cast<size_t>(e0 + e) * stride + j] = static_cast<float>(acc[e]);
    }
}

}  // namespace

int shv_launch_router_fold(shv_ctx *ctx, const shv_router_fold_args *pa) {
    const shv_router_fold_args &a = *pa;
    SHV_REQUIRE(a.router && a.gamma && a.w_out && a.out && a.scratch, "router_fold: NULL argument");
    SHV_REQUIRE(a.n_expert >= 1 && a.n_embd >= 1 && a.k >= 256 && a.k % 256 == 0, "router_fold: n_expert %d, n_embd %d, k %d", a.n_expert, a.n_embd, a.k);
    SHV_REQUIRE(shv_aligned16(a.w_out), "router_fold: w_out must be 16-byte aligned");
    const int rows = a.n_expert + (a.shared_gate ? 1 : 0);
    shv_dequant_q4k_args d{a.w_out, a.scratch, a.n_embd, a.k};
    const int rc = shv_launch_dequant_q4k(ctx, &d);
    if (rc != SHV_OK) return rc;
    SHV_LAUNCH(ctx, router_fold_scale_kernel, dim3((a.n_embd + 255) / 256, rows), dim3(256), 0, a, rows);
    SHV_LAUNCH(ctx, router_fold_product_kernel, dim3(a.k / 256, (rows + kE - 1) / kE), dim3(256), 0, a, rows);
    return SHV_OK;
}
