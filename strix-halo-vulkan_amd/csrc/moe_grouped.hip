// The experts of a pass of many rows, grouped by expert on the matrix cores (the prompt side of
// MoETrace.Experts, llm/moe.go:289-409; the reference batches a chunk's tokens per expert in
// llm_moe_gemv.comp's multi-row arm).  The per-(token, expert) GEMV reads and unpacks an expert's
// weights once per token that chose it, this path once per 16 such tokens: it pays when tokens
// outnumber experts (2048 rows choosing 10 of 512: 40 tokens an expert), not at 64 rows (1.9).
//
//   moe_group_kernel          per-expert lists of (token, slot) pairs from topk, tokens ascending
//   moe_up_grouped_kernel     a block = (expert, half of its ffn rows): the listed tokens' xn rows
//                             are gathered into LDS as matrix-core operands (two halves hi + lo,
//                             as the projections do), each wave streams one gate tile and the
//                             matching up tile of 16 rows, SwiGLU in registers, act[pair] out
//   moe_down_grouped_kernel   a block = (expert, quarter of n_embd rows): act rows gathered the
//                             same way, each wave two tiles, raw products to pairout[pair]
//   moe_combine_kernel        out[t] = residual[t] + sum over slots of weights[t][s]*pairout[t][s],
//                             slots in order
// The shared expert is an expert every token lists: its blocks take 16 tokens each.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kTok = 16;          // tokens a block multiplies at a time: one matrix-core tile
constexpr int kFrag = 64 * 16;    // one operand: a lane's eight halves
constexpr int kMaxExperts = 1024;

// The caller's `group` workspace: [0, n_expert] start of each expert's list (one more: the total),
// then n_tok * n_used pair ids (token * (n_used + 1) + slot).  A list's order is whatever the
// arrivals made it; every pair's products are formed in a matrix-core column of their own, so no
// value depends on it.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *topk, int n_tok, int n_used, int n_expert, int32_t *group) {
    __shared__ int32_t s_cnt[kMaxExperts + 1];
    const int tid = threadIdx.x, n_pairs = n_tok * n_used;
    for (int e = tid; e <= n_expert; e += blockDim.x) s_cnt[e] = 0;
    __syncthreads();
    for (int i = tid; i < n_pairs; i += blockDim.x) {
        const int e = topk[i];
        if (e >= 0 && e < n_expert) atomicAdd(&s_cnt[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int at = 0;
        for (int e = 0; e < n_expert; e++) {
            const int c = s_cnt[e];
            s_cnt[e] = at;
            at += c;
        }
        s_cnt[n_expert] = at;
    }
    __syncthreads();
    for (int e = tid; e <= n_expert; e += blockDim.x) group[e] = s_cnt[e];
    __syncthreads();
    int32_t *list = group + n_expert + 1;
    for (int i = tid; i < n_pairs; i += blockDim.x) {
        const int e = topk[i];
        if (e >= 0 && e < n_expert) list[atomicAdd(&s_cnt[e], 1)] = (i / n_used) * (n_used + 1) + i % n_used;
    }
}

// Rows src[i] (each K floats) of up to 16 listed rows into operand order: fragment (sub-block, part)
// is 64 lanes x 16 bytes, lane = row + 16 * (k block of 8 columns), the eight columns in slot order
// [0, 2, 1, 3, 4, 6, 5, 7]; sxs[sub][row] is the sub-block's sum of x.
template <int K>
__device__ __forceinline__ void gather_rows(const float *const *rows_s, int m, char *frags, float *sxs) {
    constexpr int QPR = K / 4;                 // quads a row
    constexpr int RPI = kThreads / QPR;        // rows an iteration of the block covers
    const int tid = threadIdx.x;
    const int c = 4 * (tid % QPR);
    const int sub = c >> 5, kb = (c & 31) >> 3, qh = (c & 7) >> 2;
    for (int i0 = 0; i0 < m; i0 += RPI) {
        const int i = i0 + tid / QPR;
        const bool on = i < m;
        float4 v = {0.f, 0.f, 0.f, 0.f};
        if (on) v = *reinterpret_cast<const float4 *>(rows_s[i] + c);
        float sum = (v.x + v.y) + (v.z + v.w);
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        sum += __shfl_xor(sum, 4, 64);
        if (on) {
            if ((c & 31) == 0) sxs[sub * kTok + i] = sum;
            const float o[4] = {v.x, v.z, v.y, v.w};
            half4_t h, l;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const _Float16 hi = static_cast<_Float16>(o[j]);
                h[j] = hi;
                l[j] = static_cast<_Float16>(o[j] - static_cast<float>(hi));
            }
            char *e = frags + static_cast<size_t>(sub * 2) * kFrag + (kb * 16 + i) * 16 + qh * 8;
            *reinterpret_cast<half4_t *>(e) = h;
            *reinterpret_cast<half4_t *>(e + kFrag) = l;
        }
    }
}

struct SbLoads {
    uint4 hdr;
    uint2 q[4];
    __device__ __forceinline__ void load(const char *sb, int kb) {
        hdr = *reinterpret_cast<const uint4 *>(sb);
#pragma unroll
        for (int g = 0; g < 4; g++) q[g] = *reinterpret_cast<const uint2 *>(sb + 16 + g * 32 + kb * 8);
    }
};

// y[r][j] += sum over the row's K columns of W[row of tile r][.] * x[token 4 kb + j][.] for R row
// tiles whose lane rows start at rp[r]; the operands of the 16 tokens are in LDS.
template <int K, int R>
__device__ __forceinline__ void tiles_times_rows(const char *const (&rp)[R], const char *frags, const float *sxs, int lane, float4_t (&y)[R]) {
    constexpr int SBS = K / SHV_Q4K_BLOCK;
    const int kb = lane >> 4;
    const NibbleConsts nc = nibble_consts();
    SbLoads ld[R];
#pragma unroll
    for (int r = 0; r < R; r++) ld[r].load(rp[r], kb);
#pragma unroll 1
    for (int sb = 0; sb < SBS; sb++) {
        SbLoads cur[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            cur[r] = ld[r];
            // the last super-block asks for itself again, so that the loads are unconditional
            ld[r].load(rp[r] + static_cast<size_t>(sb + 1 < SBS ? sb + 1 : sb) * SHV_Q4K_BYTES, kb);
        }
#pragma unroll
        for (int g = 0; g < 4; g++) {
            uint32_t sc[R], mn[R];
#pragma unroll
            for (int r = 0; r < R; r++) q4k_group_scale_min(cur[r].hdr, g, sc[r], mn[r]);
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {
                const int sub = sb * 8 + g * 2 + hi;
                const char *f = frags + static_cast<size_t>(sub * 2) * kFrag + lane * 16;
                const half8_t xh = *reinterpret_cast<const half8_t *>(f);
                const half8_t xl = *reinterpret_cast<const half8_t *>(f + kFrag);
                const float4 sx = *reinterpret_cast<const float4 *>(sxs + sub * kTok + 4 * kb);
                const float sxv[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const uint32_t q0 = cur[r].q[g].x, q1 = cur[r].q[g].y;
                    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                    u32x4 v;
                    if (hi == 0) {
                        v.x = ((q0 << 4) & nc.mask) | nc.one; v.y = ((q0 >> 4) & nc.mask) | nc.one;
                        v.z = ((q1 << 4) & nc.mask) | nc.one; v.w = ((q1 >> 4) & nc.mask) | nc.one;
                    } else {
                        v.x = (q0 & nc.mask) | nc.one; v.y = ((q0 >> 8) & nc.mask) | nc.one;
                        v.z = (q1 & nc.mask) | nc.one; v.w = ((q1 >> 8) & nc.mask) | nc.one;
                    }
                    const half8_t b = __builtin_bit_cast(half8_t, v);
                    const float dd = f16_bits_to_f32(cur[r].hdr.x), dmin = f16_bits_to_f32(cur[r].hdr.x >> 16);
                    const float ds = dd * static_cast<float>(hi ? sc[r] >> 8 : sc[r] & 0xFFu);
                    const float e = fmaf(64.f, ds, dmin * static_cast<float>(hi ? mn[r] >> 8 : mn[r] & 0xFFu));
                    float4_t acc = {0.f, 0.f, 0.f, 0.f};
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, b, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, b, acc, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; j++) y[r][j] = fmaf(-e, sxv[j], fmaf(ds, acc[j], y[r][j]));
                }
            }
        }
    }
}

// Which expert, which part of its rows and which of its tokens a block takes.  The first
// parts * ceil(n_tok / 16) blocks are the shared expert, one per (part, tile of 16 tokens); the
// rest are the routed experts (every token tile of the expert's list in turn).
struct Unit {
    int expert;   // -1: the shared expert
    int part;
    int first, count;  // positions in the expert's list (routed) or token numbers (shared)
};
__device__ __forceinline__ Unit unit_of(int b, int parts, int n_expert, int n_tok, const int32_t *group) {
    Unit u;
    const int shared = parts * ((n_tok + kTok - 1) / kTok);  // the shared expert's blocks come first: all of them have work
    if (b >= shared) {
        b -= shared;
        u.expert = b / parts;
        u.part = b % parts;
        u.first = group[u.expert];
        u.count = group[u.expert + 1] - u.first;
    } else {
        u.expert = -1;
        u.part = b % parts;
        u.first = (b / parts) * kTok;
        u.count = n_tok - u.first < kTok ? n_tok - u.first : kTok;
    }
    return u;
}

// grid: n_expert * 2 + 2 * ceil(n_tok / 16) blocks of 16 waves; K = n_embd; ffn = 512: a half is
// 256 rows = 16 tiles, wave w takes gate tile w and up tile w.
template <int K>
__global__ __launch_bounds__(kThreads) void moe_up_grouped_kernel(shv_moe_up_args a) {
    const int32_t *group = a.group;
    extern __shared__ __align__(16) char smem[];
    constexpr int SUBS = K / 32;
    char *frags = smem;
    float *sxs = reinterpret_cast<float *>(smem + static_cast<size_t>(SUBS) * 2 * kFrag);
    const float **rows_s = reinterpret_cast<const float **>(sxs + SUBS * kTok);
    int32_t *pair_s = reinterpret_cast<int32_t *>(rows_s + kTok);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int parts = a.ffn / 256;
    const Unit u = unit_of(blockIdx.x, parts, a.n_expert, a.n_tok, group);
    if (u.count <= 0) return;
    const size_t row_bytes = static_cast<size_t>(K / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES;
    const int row = u.part * 256 + wave * 16 + n;   // this lane's row of the expert, gate and up alike
    const size_t wrow = static_cast<size_t>(u.expert < 0 ? 0 : u.expert) * a.ffn + row;
    const char *rp[2] = {static_cast<const char *>(u.expert < 0 ? a.gate_sh : a.gate_exps) + wrow * row_bytes,
                         static_cast<const char *>(u.expert < 0 ? a.up_sh : a.up_exps) + wrow * row_bytes};
    for (int t0 = 0; t0 < u.count; t0 += kTok) {
        const int m = u.count - t0 < kTok ? u.count - t0 : kTok;
        if (tid < m) {
            const int pair = u.expert < 0 ? (u.first + t0 + tid) * (a.n_used + 1) + a.n_used : group[a.n_expert + 1 + u.first + t0 + tid];
            pair_s[tid] = pair;
            rows_s[tid] = a.xn + static_cast<size_t>(pair / (a.n_used + 1)) * K;
        }
        __syncthreads();
        gather_rows<K>(rows_s, m, frags, sxs);
        __syncthreads();
        float4_t y[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
        tiles_times_rows<K, 2>(rp, frags, sxs, lane, y);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = 4 * kb + j;
            if (i < m) {
                const float gv = y[0][j];
                a.act[static_cast<size_t>(pair_s[i]) * a.ffn + row] = gv * sigmoid_exact(gv) * y[1][j];
            }
        }
        __syncthreads();
    }
}

// grid: n_expert * parts + parts * ceil(n_tok / 16) blocks, parts = n_embd / 512: a part is 512
// output rows = 32 tiles, wave w takes tiles 2w and 2w + 1.  K = ffn.
template <int K>
__global__ __launch_bounds__(kThreads) void moe_down_grouped_kernel(shv_moe_down_args a) {
    const int32_t *group = a.group;
    float *pairout = a.pairs;
    extern __shared__ __align__(16) char smem[];
    constexpr int SUBS = K / 32;
    char *frags = smem;
    float *sxs = reinterpret_cast<float *>(smem + static_cast<size_t>(SUBS) * 2 * kFrag);
    const float **rows_s = reinterpret_cast<const float **>(sxs + SUBS * kTok);
    int32_t *pair_s = reinterpret_cast<int32_t *>(rows_s + kTok);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int parts = a.n_embd / 512;
    const Unit u = unit_of(blockIdx.x, parts, a.n_expert, a.n_tok, group);
    if (u.count <= 0) return;
    const size_t row_bytes = static_cast<size_t>(K / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES;
    const int row0 = u.part * 512 + wave * 32 + n;
    const char *base = static_cast<const char *>(u.expert < 0 ? a.down_sh : a.down_exps) +
                       (static_cast<size_t>(u.expert < 0 ? 0 : u.expert) * a.n_embd + row0) * row_bytes;
    const char *rp[2] = {base, base + 16 * row_bytes};
    for (int t0 = 0; t0 < u.count; t0 += kTok) {
        const int m = u.count - t0 < kTok ? u.count - t0 : kTok;
        if (tid < m) {
            const int pair = u.expert < 0 ? (u.first + t0 + tid) * (a.n_used + 1) + a.n_used : group[a.n_expert + 1 + u.first + t0 + tid];
            pair_s[tid] = pair;
            rows_s[tid] = a.act + static_cast<size_t>(pair) * K;
        }
        __syncthreads();
        gather_rows<K>(rows_s, m, frags, sxs);
        __syncthreads();
        float4_t y[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
        tiles_times_rows<K, 2>(rp, frags, sxs, lane, y);
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = 4 * kb + j;
                if (i < m) pairout[static_cast<size_t>(pair_s[i]) * a.n_embd + row0 + r * 16] = y[r][j];
            }
        __syncthreads();
    }
}

// grid: (ceil(n_embd / 1024), n_tok), 256 threads, four outputs a thread.
__global__ __launch_bounds__(256) void moe_combine_kernel(shv_moe_down_args a) {
    const float *pairout = a.pairs;
    const int t = blockIdx.y, c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= a.n_embd) return;
    const float *w = a.weights + static_cast<size_t>(t) * (a.n_used + 1);
    float4 v = {0.f, 0.f, 0.f, 0.f};
    if (a.residual) v = *reinterpret_cast<const float4 *>(a.residual + static_cast<size_t>(t) * a.res_stride + c);
    for (int s = 0; s <= a.n_used; s++) {
        const float ws = w[s];
        const float4 p = *reinterpret_cast<const float4 *>(pairout + (static_cast<size_t>(t) * (a.n_used + 1) + s) * a.n_embd + c);
        v.x = fmaf(ws, p.x, v.x); v.y = fmaf(ws, p.y, v.y); v.z = fmaf(ws, p.z, v.z); v.w = fmaf(ws, p.w, v.w);
    }
    *reinterpret_cast<float4 *>(a.out + static_cast<size_t>(t) * a.out_stride + c) = v;
}

template <int K>
constexpr size_t grouped_lds() {
    return static_cast<size_t>(K / 32) * 2 * kFrag + static_cast<size_t>(K / 32) * kTok * 4 + kTok * sizeof(float *) + kTok * 4;
}

template <typename Kern>
int raise_lds(Kern kern, size_t lds) {
    SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
    return SHV_OK;
}

bool shapes_covered(const shv_ctx *ctx, int n_tok, int n_embd, int ffn, int n_used, int n_expert) {
    return n_tok >= ctx->moe_group_min && n_embd == 2048 && ffn == 512 && n_expert >= 1 && n_expert <= kMaxExperts && n_used >= 1 &&
           static_cast<long long>(n_tok) * (n_used + 1) < (1ll << 30) / 2048;
}

}  // namespace

// Whether a pass takes the grouped path: a workspace from the caller, rows enough for experts to
// repeat, the shapes the kernels are built for, and a selection that is already made (topk from
// the router).  The launchers in moe.hip have checked that every bank is Q4_K.
bool shv_moe_up_grouped_covers(const shv_ctx *ctx, const shv_moe_up_args &a) {
    return a.group && !a.logits && shv_aligned16(a.xn) && shapes_covered(ctx, a.n_tok, a.n_embd, a.ffn, a.n_used, a.n_expert);
}

bool shv_moe_down_grouped_covers(const shv_ctx *ctx, const shv_moe_down_args &a) {
    return a.group && a.pairs && shv_aligned16(a.act) && shv_aligned16(a.pairs) && shapes_covered(ctx, a.n_tok, a.n_embd, a.ffn, a.n_used, a.n_expert);
}

// Lists, then the grouped gate/up products.
int shv_launch_moe_up_grouped(shv_ctx *ctx, const shv_moe_up_args &a) {
    SHV_LAUNCH(ctx, moe_group_kernel, dim3(1), dim3(1024), 0, a.topk, a.n_tok, a.n_used, a.n_expert, a.group);
    constexpr size_t lds = grouped_lds<2048>();
    static const int raised = raise_lds(&moe_up_grouped_kernel<2048>, lds);
    if (raised != SHV_OK) return raised;
    const int parts = a.ffn / 256, tiles = (a.n_tok + kTok - 1) / kTok;
    SHV_LAUNCH(ctx, moe_up_grouped_kernel<2048>, dim3(a.n_expert * parts + parts * tiles), dim3(kThreads), lds, a);
    return SHV_OK;
}

// The down projection makes its own lists from the same selection (the gate/up products may have
// gone another road: banks of other types), writes every pair's products to the caller's `pairs`
// and folds them per token in slot order.
int shv_launch_moe_down_grouped(shv_ctx *ctx, const shv_moe_down_args &a) {
    SHV_REQUIRE(a.n_embd % 4 == 0 && a.out_stride % 4 == 0 && shv_aligned16(a.out) &&
                    (!a.residual || (a.res_stride % 4 == 0 && shv_aligned16(a.residual))),
                "moe_down: the grouped path moves 16 bytes at a time");
    SHV_LAUNCH(ctx, moe_group_kernel, dim3(1), dim3(1024), 0, a.topk, a.n_tok, a.n_used, a.n_expert, const_cast<int32_t *>(a.group));
    constexpr size_t lds = grouped_lds<512>();
    static const int raised = raise_lds(&moe_down_grouped_kernel<512>, lds);
    if (raised != SHV_OK) return raised;
    const int parts = a.n_embd / 512, tiles = (a.n_tok + kTok - 1) / kTok;
    SHV_LAUNCH(ctx, moe_down_grouped_kernel<512>, dim3(a.n_expert * parts + parts * tiles), dim3(kThreads), lds, a);
    SHV_LAUNCH(ctx, moe_combine_kernel, dim3((a.n_embd + 1023) / 1024, a.n_tok), dim3(256), 0, a);
    return SHV_OK;
}
