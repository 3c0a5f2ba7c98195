// Expert banks in the checkpoint's own tensor types: the two expert-gathered GEMVs of the MoE
// block (llm/moe.go:289-409; llm_moe_gemv.comp's Q5_K / Q5_1 / Q8_0 / Q4_1 / IQ4_NL arms) for
// banks that are not Q4_K.  The routed banks and the shared expert may each be of another type;
// the type is uniform over a wave, so the choice of arm costs a scalar branch.  A lane takes one
// 32-element group of a row at a time, formed as the format's CPU arm forms it; HBM-streamed and
// correct, not tuned like the Q4_K kernels.
#include "group_dot.hpp"

namespace {

using namespace shv;
using namespace shv_any;

constexpr int kBlock = 256;
constexpr int kRowsPerWave = 4;
constexpr int kRowsPerBlock = 4 * kRowsPerWave;

__host__ __device__ inline int bank_type(int t) { return t == 0 ? SHV_GGML_Q4_K : t; }

// grid (ceil(ffn / 16), slots, n_tok), slot = blockIdx.y + slot0: act[t][slot][row] = silu(Wg row . xn[t]) * (Wu row . xn[t])
__global__ __launch_bounds__(kBlock) void moe_up_any_kernel(shv_moe_up_args a, int slot0, int rpw) {
    extern __shared__ __align__(16) float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int slot = blockIdx.y + slot0, t = blockIdx.z;
    const float *x = a.xn + static_cast<size_t>(t) * a.n_embd;
    for (int c = tid; c < a.n_embd; c += kBlock) xs[c] = x[c];
    __syncthreads();
    const bool routed = slot < a.n_used;
    const int gt = bank_type(routed ? a.gate_type : a.gate_sh_type), ut = bank_type(routed ? a.up_type : a.up_sh_type);
    const long long grb = row_bytes(gt, a.n_embd), urb = row_bytes(ut, a.n_embd);
    const long long e = routed ? a.topk[static_cast<size_t>(t) * a.n_used + slot] : 0;
    const uint8_t *gb = static_cast<const uint8_t *>(routed ? a.gate_exps : a.gate_sh) + e * a.ffn * grb;
    const uint8_t *ub = static_cast<const uint8_t *>(routed ? a.up_exps : a.up_sh) + e * a.ffn * urb;
    float *act = a.act + (static_cast<size_t>(t) * (a.n_used + 1) + slot) * a.ffn;
    const int groups = a.n_embd / 32;
    for (int r = 0; r < rpw; r++) {  // rpw rows a wave: fewer when the launch would otherwise leave CUs idle
        const int row = (blockIdx.x * 4 + wave) * rpw + r;
        if (row >= a.ffn) break;  // uniform over the wave
        float g = 0.f, u = 0.f;
        for (int q = lane; q < groups; q += 64) {
            g += group_dot_rt(gt, gb + row * grb, q, xs + q * 32);
            u += group_dot_rt(ut, ub + row * urb, q, xs + q * 32);
        }
        g = wave_sum_all(g);
        u = wave_sum_all(u);
        if (lane == 0) act[row] = siluf_dev(g) * u;
    }
}

// grid (ceil(n_embd / 4), n_tok), a wave per output row: out[t][row] = residual + sum_slot weights[t][slot] *
// (Wd_slot row . act[t][slot]).  The lanes of a wave share out the (slot, group) pairs of the row; the
// activations (a few KB a token, shared by every block) are read where they lie.
__global__ __launch_bounds__(kBlock) void moe_down_any_kernel(shv_moe_down_args a, int s_lo, int s_hi, int add) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.y, ns = a.n_used + 1;
    const int row = blockIdx.x * 4 + wave;
    if (row >= a.n_embd) return;  // uniform over the wave; the kernel has no barrier
    const float *acts = a.act + static_cast<size_t>(t) * ns * a.ffn;
    const int32_t *tk = a.topk + static_cast<size_t>(t) * a.n_used;
    const float *wt = a.weights + static_cast<size_t>(t) * ns;
    const int rt = bank_type(a.down_type), st = bank_type(a.down_sh_type);
    const long long rrb = row_bytes(rt, a.ffn), srb = row_bytes(st, a.ffn);
    // slots [s_lo, s_hi) only; add: on top of what out already holds (another launch wrote the other slots)
    const int gpr = a.ffn / 32, r_hi = s_hi < a.n_used ? s_hi : a.n_used, routed = (r_hi - s_lo) * gpr;
    float acc = 0.f;
    for (int p = lane; p < routed; p += 64) {
        const int slot = s_lo + p / gpr, q = p - (slot - s_lo) * gpr;
        const uint8_t *rp = static_cast<const uint8_t *>(a.down_exps) + (static_cast<long long>(tk[slot]) * a.n_embd + row) * rrb;
        acc = fmaf(wt[slot], group_dot_rt(rt, rp, q, acts + slot * a.ffn + q * 32), acc);
    }
    for (int q = lane; q < gpr && s_hi > a.n_used; q += 64)
        acc = fmaf(wt[a.n_used], group_dot_rt(st, static_cast<const uint8_t *>(a.down_sh) + row * srb, q, acts + a.n_used * a.ffn + q * 32), acc);
    acc = wave_sum_all(acc);
    if (lane == 0) {
        float *o = a.out + static_cast<size_t>(t) * a.out_stride + row;
        const float res = add ? *o : a.residual ? a.residual[static_cast<size_t>(t) * a.res_stride + row] : 0.f;
        *o = res + acc;
    }
}

}  // namespace

int shv_launch_moe_up_any(shv_ctx *ctx, const shv_moe_up_args *pa, int slot0, int slots) {
    const shv_moe_up_args &a = *pa;
    SHV_REQUIRE(!a.logits, "moe_up: banks of other types than Q4_K take the selection from the router, not from logits");
    const bool routed = slot0 < a.n_used, shared = slot0 + slots > a.n_used;
    const int types[4] = {routed ? bank_type(a.gate_type) : SHV_GGML_Q4_K, routed ? bank_type(a.up_type) : SHV_GGML_Q4_K,
                          shared ? bank_type(a.gate_sh_type) : SHV_GGML_Q4_K, shared ? bank_type(a.up_sh_type) : SHV_GGML_Q4_K};
    for (int t : types)
        SHV_REQUIRE(t != SHV_GGML_F32 && whole_rows(t, a.n_embd), "moe_up: rows of %d elements of ggml type %d (not a type a bank can be, or not whole blocks)", a.n_embd, t);
    SHV_REQUIRE(shv_aligned16(a.gate_exps) && shv_aligned16(a.up_exps) && shv_aligned16(a.gate_sh) && shv_aligned16(a.up_sh),
                "moe_up: weight banks must be 16-byte aligned");
    const size_t lds = static_cast<size_t>(a.n_embd) * 4;
    SHV_REQUIRE(lds <= 48 * 1024, "moe_up: n_embd %d does not fit the staging of a row", a.n_embd);
    const long long tall = static_cast<long long>((a.ffn + kRowsPerBlock - 1) / kRowsPerBlock) * slots * a.n_tok;
    const int rpw = tall >= 2 * ctx->prop.multiProcessorCount ? kRowsPerWave : 1;
    SHV_LAUNCH(ctx, moe_up_any_kernel, dim3((a.ffn + 4 * rpw - 1) / (4 * rpw), slots, a.n_tok), dim3(kBlock), lds, a, slot0, rpw);
    return SHV_OK;
}

int shv_launch_moe_down_any(shv_ctx *ctx, const shv_moe_down_args *pa, int s_lo, int s_hi, int add) {
    const shv_moe_down_args &a = *pa;
    const int types[2] = {s_lo < a.n_used ? bank_type(a.down_type) : SHV_GGML_Q4_K, s_hi > a.n_used ? bank_type(a.down_sh_type) : SHV_GGML_Q4_K};
    for (int t : types)
        SHV_REQUIRE(t != SHV_GGML_F32 && whole_rows(t, a.ffn), "moe_down: rows of %d elements of ggml type %d (not a type a bank can be, or not whole blocks)", a.ffn, t);
    SHV_REQUIRE(shv_aligned16(a.down_exps) && shv_aligned16(a.down_sh) && shv_aligned16(a.act), "moe_down: weight banks and activations must be 16-byte aligned");
    SHV_LAUNCH(ctx, moe_down_any_kernel, dim3((a.n_embd + 3) / 4, a.n_tok), dim3(kBlock), 0, a, s_lo, s_hi, add);
    return SHV_OK;
}
