// MoE FFN decode step: router logits, softmax/top-k selection, expert-gathered
// gate/up GEMV with SwiGLU, down GEMV with weighting and combine.  Only the rows of the selected
// experts (and the shared one) are read from HBM.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kMaxUsed = 16;
inline bool is_q4k(int ggml_type) { return ggml_type == 0 || ggml_type == SHV_GGML_Q4_K; }  // 0: the type field left unset
constexpr float kWeightsSumFloor = 6.103515625e-5f;  // 2^-14

// ---------------------------------------------------------------------------- router ---------

// Candidates are ordered by (probability, lower index first): the pair (bits of p, 0x7FFFFFFF-idx)
// compared lexicographically.  Probabilities are positive, so their bit patterns order as they do.
__device__ __forceinline__ bool pair_gt(uint32_t ah, uint32_t al, uint32_t bh, uint32_t bl) {
    return ah > bh || (ah == bh && al > bl);
}

template <int CTRL>
__device__ __forceinline__ void pair_max_step(uint32_t &hi, uint32_t &lo) {
    const uint32_t oh = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(hi), CTRL, 0xF, 0xF, false));
    const uint32_t ol = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(lo), CTRL, 0xF, 0xF, false));
    const bool take = pair_gt(oh, ol, hi, lo);
    hi = take ? oh : hi;
    lo = take ? ol : lo;
}

// Maximum pair over the wave, in every lane: DPP within the rows of 16, then the four row
// winners are read out as scalars.
__device__ __forceinline__ void wave_pair_max(uint32_t &hi, uint32_t &lo) {
    pair_max_step<kDppXor1>(hi, lo);
    pair_max_step<kDppXor2>(hi, lo);
    pair_max_step<kDppHalfMirror>(hi, lo);
    pair_max_step<kDppMirror>(hi, lo);
    uint32_t bh = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(hi), 0));
    uint32_t bl = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(lo), 0));
#pragma unroll
    for (int r = 16; r < 64; r += 16) {
        const uint32_t oh = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(hi), r));
        const uint32_t ol = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(lo), r));
        const bool take = pair_gt(oh, ol, bh, bl);
        bh = take ? oh : bh;
        bl = take ? ol : bl;
    }
    hi = bh;
    lo = bl;
}

// n_used rounds of arg-max over the wave's candidates: the general selection, used when ties make
// the shortcut below ambiguous.  kh/kl hold (bits of p, 0x7FFFFFFF - index); (0, 0) is empty.
template <int PER>
__device__ void select_by_rounds(uint32_t *kh, uint32_t *kl, int n_used, int32_t *sel_e, float *sel_w) {
    const int lane = threadIdx.x & 63;
#pragma unroll 1
    for (int k = 0; k < n_used; k++) {
        uint32_t bh = 0u, bl = 0u;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const bool take = pair_gt(kh[i], kl[i], bh, bl);
            bh = take ? kh[i] : bh;
            bl = take ? kl[i] : bl;
        }
        wave_pair_max(bh, bl);
#pragma unroll
        for (int i = 0; i < PER; i++)
            if (kh[i] == bh && kl[i] == bl) kh[i] = kl[i] = 0u;
        if (lane == 0) {
            sel_e[k] = 0x7FFFFFFF - static_cast<int>(bl);
            sel_w[k] = __uint_as_float(bh);
        }
    }
}

// One wave routes one token: softmax over n_expert logits (n_expert <= 64*PER), the n_used largest
// probabilities in descending order with ties to the lower index, their sum in slot order clamped
// at 2^-14, the normalised weights.  Probabilities are formed as the reference forms them (exp of
// the logit minus the maximum, times the reciprocal of their sum) so equal logits stay equal
// probabilities; the reference adds the exponentials one after another where a tree is used
// here, which moves only the last bits of a factor common to every probability.
//
// Selection: the n_used-th largest of 16 group maxima bounds the n_used-th largest key from
// below, so only keys at or above it can be selected.  Those few candidates (found by a bitwise
// search with wave ballots) are compacted into LDS and ranked against each other.
// lds: scratch of at least 192 floats.
template <int PER, bool AGENT>
__device__ void route_token(const float *logits, int n_expert, int n_used, int32_t *topk, float *weights, float *lds, float scale = 1.f) {
    const int lane = threadIdx.x & 63;
    uint32_t *cand_p = reinterpret_cast<uint32_t *>(lds);       // [64]
    int32_t *cand_e = reinterpret_cast<int32_t *>(lds + 64);    // [64]
    int32_t *sel_e = reinterpret_cast<int32_t *>(lds + 128);    // [kMaxUsed]
    float *sel_w = lds + 128 + kMaxUsed;                        // [kMaxUsed]
    float l[PER];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int e = lane + i * 64;
        l[i] = e < n_expert ? (AGENT ? load_agent(logits + e) : logits[e]) * scale : -INFINITY;  // scale: a factor the logits still lack
        mx = fmaxf(mx, l[i]);
    }
    mx = wave_max_all(mx);
    float ex[PER];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int e = lane + i * 64;
        ex[i] = e < n_expert ? expf(l[i] - mx) : 0.f;
        sum += ex[i];
    }
    sum = wave_sum_all(sum);
    const float inv = 1.f / sum;
    uint32_t kh[PER], kl[PER];
    uint32_t lane_max = 0u;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int e = lane + i * 64;
        kh[i] = e < n_expert ? __float_as_uint(ex[i] * inv) : 0u;
        kl[i] = e < n_expert ? static_cast<uint32_t>(0x7FFFFFFF - e) : 0u;
        lane_max = kh[i] > lane_max ? kh[i] : lane_max;
    }
    // thr = the n_used-th largest of the 16 maxima of four neighbouring lanes: n_used different
    // groups hold a key at or above it, so the n_used largest keys all are.  Every lane ranks one
    // group's maximum among the 16 (ties by group, so the ranks are distinct); the group of rank
    // n_used-1 holds the threshold.
    uint32_t thr = 0u;
    {
        uint32_t gm = lane_max;
        const uint32_t o1 = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(gm), kDppXor1, 0xF, 0xF, false));
        gm = o1 > gm ? o1 : gm;
        const uint32_t o2 = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(gm), kDppXor2, 0xF, 0xF, false));
        gm = o2 > gm ? o2 : gm;
        uint32_t *lm = cand_p;  // the candidate table is not in use yet
        if ((lane & 3) == 0) lm[lane >> 2] = gm;
        __builtin_amdgcn_wave_barrier();
        const int grp = lane & 15;
        const uint32_t mine = lm[grp];
        int rank = 0;
#pragma unroll
        for (int j4 = 0; j4 < 4; j4++) {
            const uint4 o = *reinterpret_cast<const uint4 *>(lm + 4 * j4);
            const uint32_t ov[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
            for (int j = 0; j < 4; j++) rank += (ov[j] > mine || (ov[j] == mine && 4 * j4 + j < grp)) ? 1 : 0;
        }
        uint32_t *thr_slot = reinterpret_cast<uint32_t *>(sel_e);
        if (lane < 16 && rank == n_used - 1) *thr_slot = mine;
        __builtin_amdgcn_wave_barrier();
        thr = *thr_slot;
        __builtin_amdgcn_wave_barrier();
    }
    // compact the keys at or above it
    int total = 0;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const bool pred = kl[i] != 0u && kh[i] >= thr;
        const unsigned long long mask = __ballot(pred);
        const int pos = total + static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                                 __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u)));
        if (pred && pos < 64) {
            cand_p[pos] = kh[i];
            cand_e[pos] = lane + i * 64;
        }
        total += __popcll(mask);
    }
    if (total > 64 || n_expert < 64) {
        // many equal probabilities (or fewer experts than lanes): take the general road
        select_by_rounds<PER>(kh, kl, n_used, sel_e, sel_w);
    } else {
        __builtin_amdgcn_wave_barrier();
        const uint32_t my_p = lane < total ? cand_p[lane] : 0u;
        const int my_e = lane < total ? cand_e[lane] : 0x7FFFFFFF;
        // rank of candidate j = how many candidates come before it: its key goes round as two
        // scalars, every lane answers, and the answers are counted (no memory on the way)
        int rank = 0;
        for (int j = 0; j < total; j++) {
            const uint32_t pj = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(my_p), j));
            const int ej = __builtin_amdgcn_readlane(my_e, j);
            const int before = __popcll(__ballot(my_p > pj || (my_p == pj && my_e < ej)));
            rank = lane == j ? before : rank;
        }
        if (lane < total && rank < n_used) {
            sel_e[rank] = my_e;
            sel_w[rank] = __uint_as_float(my_p);
        }
    }
    __builtin_amdgcn_wave_barrier();
    // lane k holds slot k; the sum runs over the slots in order, in float32: the reference's sum
    const float w_mine = lane < n_used ? sel_w[lane] : 0.f;
    const int32_t e_mine = lane < n_used ? sel_e[lane] : 0;
    float wsum = 0.f;
    for (int k = 0; k < n_used; k++) wsum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_mine), k));
    if (wsum < kWeightsSumFloor) wsum = kWeightsSumFloor;
    if (lane < n_used) {
        topk[lane] = e_mine;
        weights[lane] = w_mine / wsum;
    }
}

// grid: (ceil((n_expert+1)/(4 RW)), ceil(n_tok/tpb)) blocks of 4 waves, RW float32 router rows per
// wave, tpb tokens per block.  Tokens go through in groups of kRouterGroup: one set of block-wide
// waits per group, not per token.  A pass of few tokens spreads the router over many small
// blocks (RW = 1, 4 tokens a block); a prompt pass, where every block reads every token's row and
// every token's block reads the router, takes RW = 4 and 8 to 32 tokens a block.
constexpr int kRouterGroup = 4;
constexpr int kRouterTokens = 4;
constexpr int kRouterTokensMany = 32;
template <int H, int RW>
__global__ __launch_bounds__(kBlock) void moe_router_kernel(shv_moe_router_args a, int tpb) {
    __shared__ __align__(16) float xs[kRouterGroup][H];
    __shared__ float red[kRouterGroup][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = (blockIdx.x * 4 + wave) * RW;  // n_expert = the shared-gate row
    const int t_first = blockIdx.y * tpb;
    const int t_end = t_first + tpb < a.n_tok ? t_first + tpb : a.n_tok;
    // Loads come back in the order they were asked for: the first tokens' rows and gamma go first
    // (they come from cache, and the normalising below is over by the time the router rows arrive
    // instead of queueing behind them); a later group's rows are asked for while the group before
    // it is being multiplied.
    float v[kRouterGroup][H / kBlock];
    auto fetch = [&](int t0) {
        const int ng = t_end - t0 < kRouterGroup ? t_end - t0 : kRouterGroup;
#pragma unroll
        for (int g = 0; g < kRouterGroup; g++) {
            if (g >= ng) break;
            const float *h = a.h + static_cast<size_t>(t0 + g) * a.h_stride;
#pragma unroll
            for (int i = 0; i < H / kBlock; i++) v[g][i] = h[tid + i * kBlock];
        }
    };
    fetch(t_first);
    float gm[H / kBlock];
#pragma unroll
    for (int i = 0; i < H / kBlock; i++) gm[i] = a.gamma ? a.gamma[tid + i * kBlock] : 1.f;
    // the wave's router rows stay in registers for every token
    float4 wrow[RW][H / 256];
    bool has_row[RW];
#pragma unroll
    for (int j = 0; j < RW; j++) {
        const int row = row0 + j;
        has_row[j] = row <= a.n_expert && (row < a.n_expert || a.shared_gate);
        const float *w = row < a.n_expert ? a.router + static_cast<size_t>(row) * H : a.shared_gate;
#pragma unroll
        for (int i = 0; i < H / 256; i++)
            wrow[j][i] = has_row[j] ? *reinterpret_cast<const float4 *>(w + (i * 64 + lane) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int t0 = t_first; t0 < t_end; t0 += kRouterGroup) {
        const int ng = t_end - t0 < kRouterGroup ? t_end - t0 : kRouterGroup;
        if (a.gamma) {
#pragma unroll
            for (int g = 0; g < kRouterGroup; g++) {
                if (g >= ng) break;
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < H / kBlock; i++) ss = fmaf(v[g][i], v[g][i], ss);
                ss = wave_sum_all(ss);
                if (lane == 0) red[g][wave] = ss;
            }
            __syncthreads();
        }
#pragma unroll
        for (int g = 0; g < kRouterGroup; g++) {
            if (g >= ng) break;
            float scale = 1.f;
            if (a.gamma) scale = __builtin_amdgcn_rsqf(((red[g][0] + red[g][1]) + (red[g][2] + red[g][3])) / static_cast<float>(H) + a.eps);
#pragma unroll
            for (int i = 0; i < H / kBlock; i++) {
                const int c = tid + i * kBlock;
                const float x = a.gamma ? v[g][i] * scale * gm[i] : v[g][i];
                xs[g][c] = x;
                if (blockIdx.x == 0 && a.xn) a.xn[static_cast<size_t>(t0 + g) * H + c] = x;
            }
        }
        __syncthreads();
        if (t0 + kRouterGroup < t_end) fetch(t0 + kRouterGroup);
#pragma unroll
        for (int g = 0; g < kRouterGroup; g++) {
            if (g >= ng) break;
            float acc[RW];
#pragma unroll
            for (int j = 0; j < RW; j++) acc[j] = 0.f;
#pragma unroll
            for (int i = 0; i < H / 256; i++) {
                const int c = (i * 64 + lane) * 4;
                const float4 xv = *reinterpret_cast<const float4 *>(&xs[g][c]);
#pragma unroll
                for (int j = 0; j < RW; j++) {
                    const float4 wv = wrow[j][i];
                    acc[j] = fmaf(wv.x, xv.x, acc[j]);
                    acc[j] = fmaf(wv.y, xv.y, acc[j]);
                    acc[j] = fmaf(wv.z, xv.z, acc[j]);
                    acc[j] = fmaf(wv.w, xv.w, acc[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < RW; j++) {
                const float sum = wave_sum_all(acc[j]);
                if (lane == 0 && has_row[j]) a.logits[static_cast<size_t>(t0 + g) * (a.n_expert + 1) + row0 + j] = sum;
            }
        }
        if (t0 + kRouterGroup < t_end) __syncthreads();
    }
}

// grid: n_tok blocks of one wave: the selection for one token from its finished logits.
__global__ __launch_bounds__(64) void moe_route_kernel(shv_moe_router_args a) {
    __shared__ __align__(16) float probs[192];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *lg = a.logits + static_cast<size_t>(t) * (a.n_expert + 1);
    float *wt = a.weights + static_cast<size_t>(t) * (a.n_used + 1);
    route_token<8, false>(lg, a.n_expert, a.n_used, a.topk + static_cast<size_t>(t) * a.n_used, wt, probs);
    if (lane == 0) wt[a.n_used] = a.shared_gate ? sigmoid_exact(lg[a.n_expert]) : 0.f;
}

// The same selection with a thread per expert (grid: n_tok blocks of 512 threads): the one wave
// above spends most of its 4 us in dependent instructions (eight exponentials, eight ballots, the
// candidates' ranks), which eight waves do side by side.  Same rule: probabilities as the
// reference forms them, the n_used largest in descending order with ties to the lower index,
// their sum in slot order clamped at 2^-14.  The threshold is the n_used-th largest of the 16
// half-wave maxima; the few keys at or above it are compacted and ranked by the first wave.
// Rows with more than 64 candidates (many equal probabilities) take the one-wave road.
constexpr int kRouteBlock = 512;
__global__ __launch_bounds__(kRouteBlock) void moe_route_block_kernel(shv_moe_router_args a) {
    __shared__ __align__(16) float probs[192];  // the one-wave road's scratch
    __shared__ float s_max[8], s_sum[8];
    __shared__ uint32_t s_gm[16];
    __shared__ uint32_t s_thr;
    __shared__ int s_cnt[8];
    __shared__ uint32_t cand_p[64];
    __shared__ int32_t cand_e[64];
    __shared__ int32_t sel_e[kMaxUsed];
    __shared__ float sel_w[kMaxUsed];
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lg = a.logits + static_cast<size_t>(t) * (a.n_expert + 1);
    float *wt = a.weights + static_cast<size_t>(t) * (a.n_used + 1);
    int32_t *topk = a.topk + static_cast<size_t>(t) * a.n_used;
    const int e = tid;
    const bool has = e < a.n_expert;
    const float l = has ? lg[e] : -INFINITY;
    // the shared gate's logit is asked for with the rest
    const float lsh = (tid == kRouteBlock - 1 && a.shared_gate) ? lg[a.n_expert] : 0.f;
    float mx = wave_max_all(l);
    if (lane == 0) s_max[wave] = mx;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 8; w++) mx = fmaxf(mx, s_max[w]);
    const float ex = has ? expf(l - mx) : 0.f;
    const float ws = wave_sum_all(ex);
    if (lane == 0) s_sum[wave] = ws;
    // half-wave maxima of the unnormalised exponentials give the same threshold as the
    // probabilities' would (one common positive factor), but the keys compared below are the
    // probabilities themselves, as the reference's are
    __syncthreads();
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 8; w++) sum += s_sum[w];
    const float inv = 1.f / sum;
    const uint32_t kh = has ? __float_as_uint(ex * inv) : 0u;
    uint32_t gm = kh;
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) {
        const uint32_t o = static_cast<uint32_t>(__shfl_xor(static_cast<int>(gm), off, 64));
        gm = o > gm ? o : gm;
    }
    if ((lane & 31) == 0) s_gm[tid >> 5] = gm;
    if (tid == 0) s_thr = 0u;
    __syncthreads();
    if (tid < 16) {
        const uint32_t mine = s_gm[tid];
        int rank = 0;
#pragma unroll
        for (int j = 0; j < 16; j++) rank += (s_gm[j] > mine || (s_gm[j] == mine && j < tid)) ? 1 : 0;
        if (rank == a.n_used - 1) s_thr = mine;
    }
    __syncthreads();
    const uint32_t thr = s_thr;
    const bool pred = has && kh >= thr;
    const unsigned long long mask = __ballot(pred);
    if (lane == 0) s_cnt[wave] = __popcll(mask);
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        before += w < wave ? s_cnt[w] : 0;
        total += s_cnt[w];
    }
    if (total > 64 || a.n_expert < 64 || a.n_used > 16) {
        // uniform over the block: many equal probabilities, or a shape the threshold does not cover
        if (wave == 0) {
            route_token<8, false>(lg, a.n_expert, a.n_used, topk, wt, probs);
            if (lane == 0) wt[a.n_used] = a.shared_gate ? sigmoid_exact(lg[a.n_expert]) : 0.f;
        }
        return;
    }
    if (pred) {
        const int pos = before + static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u)));
        cand_p[pos] = kh;
        cand_e[pos] = e;
    }
    if (tid == kRouteBlock - 1) wt[a.n_used] = a.shared_gate ? sigmoid_exact(lsh) : 0.f;
    __syncthreads();
    if (wave != 0) return;
    // candidates are in expert order; rank of candidate j = how many come before it (as in route_token)
    const uint32_t my_p = lane < total ? cand_p[lane] : 0u;
    const int my_e = lane < total ? cand_e[lane] : 0x7FFFFFFF;
    int rank = 0;
    for (int j = 0; j < total; j++) {
        const uint32_t pj = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(my_p), j));
        const int ej = __builtin_amdgcn_readlane(my_e, j);
        const int bef = __popcll(__ballot(my_p > pj || (my_p == pj && my_e < ej)));
        rank = lane == j ? bef : rank;
    }
    if (lane < total && rank < a.n_used) {
        sel_e[rank] = my_e;
        sel_w[rank] = __uint_as_float(my_p);
    }
    __builtin_amdgcn_wave_barrier();
    const float w_mine = lane < a.n_used ? sel_w[lane] : 0.f;
    const int32_t e_mine = lane < a.n_used ? sel_e[lane] : 0;
    float wsum = 0.f;
    for (int k = 0; k < a.n_used; k++) wsum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_mine), k));
    if (wsum < kWeightsSumFloor) wsum = kWeightsSumFloor;
    if (lane < a.n_used) {
        topk[lane] = e_mine;
        wt[lane] = w_mine / wsum;
    }
}

// The same selection inside a kernel that routes its own token before it can ask for its expert's
// rows.  Every block of the launch repeats it and all of them at once, so what counts is how few
// instructions it takes: the block's first 256 threads take two experts each (tid and tid + 256);
// any further waves only keep the block-wide waits (three) and, like the first four, rank the
// candidates for themselves at the end, so that no wave waits for another's result.
// Candidates are the keys whose logit is at or just below the n_used-th largest of the 16 group
// maxima, compacted into a table and ranked by (logit, lower index first).  The softmax sum is not
// formed: a routing weight is p_k / sum over the selected p_j, in which the sum over all experts
// cancels, so the weights are exp(l_k - max) / sum over the selected exp(l_j - max) (to rounding
// what the routing kernel's p_k / sum p_j gives), and the reference's floor of 2^-14 on the sum of
// the selected probabilities cannot engage with at most 512 experts (the largest probability is
// at least 1/512).  Two different logits whose probabilities round to the same float would be
// ordered by index in the reference and are ordered by logit here: a tie of the last bit.
// sel_e [kMaxUsed] / sel_w [kMaxUsed + 1] receive experts, weights and the shared expert's gate;
// probs is the one-wave road's scratch.  On return every wave can read sel_e / sel_w (each has
// written the same values there itself).
constexpr int kCandMax = 64;

// A float's bits as an unsigned integer that orders as the float does.
__device__ __forceinline__ uint32_t ordered_bits(float v) {
    const uint32_t b = __float_as_uint(v);
    return b ^ (static_cast<uint32_t>(static_cast<int32_t>(b) >> 31) | 0x80000000u);
}
__device__ __forceinline__ float from_ordered_bits(uint32_t u) {
    return __uint_as_float(u ^ ((u >> 31) ? 0x80000000u : 0xFFFFFFFFu));
}

// rank += (key of the lane k to the right in the row of 16, cyclically) > own key
template <int K>
__device__ __forceinline__ void count_greater_ror(uint32_t key, int &rank) {
    const uint32_t o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(key), 0x120 + K, 0xF, 0xF, false));
    rank += o > key ? 1 : 0;
}

// NORM: the logits still lack the RMSNorm's factor of the token row (they came with the output
// projection's launch); the block's waves have left their sums of squares of the row's k columns in
// `red` before the call, and the factor, which changes no order, goes into the weights alone.
template <bool NORM>
__device__ __forceinline__ void route_block256(const float *lg, int n_expert, int n_used, bool shared_gate, int32_t *sel_e, float *sel_w, float *probs,
                                               const float *red = nullptr, float mean_div = 1.f, float eps = 0.f) {
    __shared__ float s_max[4];
    __shared__ __align__(16) float s_gm[16];
    __shared__ int s_cnt[4];
    __shared__ __align__(16) unsigned long long cand[kCandMax];  // (logit as ordered bits << 32) | (0x7FFFFFFF - expert)
    __shared__ unsigned long long s_sel[16][kMaxUsed];            // per wave: the selected keys in slot order
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool routing = tid < 256;
    const int e0 = tid, e1 = tid + 256;
    const bool has0 = routing && e0 < n_expert, has1 = routing && e1 < n_expert;
    const float l0 = has0 ? lg[e0] : -INFINITY, l1 = has1 ? lg[e1] : -INFINITY;
    const float lsh = (lane == 63 && shared_gate) ? lg[n_expert] : 0.f;  // every wave keeps the shared gate for itself
    if (routing) {  // the block's maximum and the maxima of 16 groups of 16 threads
        float gm = fmaxf(l0, l1);
        gm = fmaxf(gm, dpp_f32<kDppXor1>(gm));
        gm = fmaxf(gm, dpp_f32<kDppXor2>(gm));
        gm = fmaxf(gm, dpp_f32<kDppHalfMirror>(gm));
        gm = fmaxf(gm, dpp_f32<kDppMirror>(gm));
        if ((lane & 15) == 0) s_gm[tid >> 4] = gm;
        // the wave's maximum from its four rows' (no exchange through LDS)
        const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gm), 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gm), 16));
        const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gm), 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gm), 48));
        if (lane == 0) s_max[wave] = fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
    }
    __syncthreads();
    const float mx = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    float scale = 1.f;
    if constexpr (NORM) scale = __builtin_amdgcn_rsqf(((red[0] + red[1]) + (red[2] + red[3])) * mean_div + eps);
    unsigned long long m0 = 0ull, m1 = 0ull;
    bool p0 = false, p1 = false;
    int n0 = 0;
    if (routing) {
        // A lower bound of the n_used-th largest key: the n_used-th largest group maximum.  Every
        // routing wave finds it for itself: the 16 maxima in the lanes of a row, as integers that
        // order as the floats do with the group's number in the low four bits (which makes them
        // distinct and rounds the bound down, never up); a lane's rank is how many of the other
        // fifteen are greater, counted over the row's rotations.
        const uint32_t key = (ordered_bits(s_gm[lane & 15]) & ~15u) | static_cast<uint32_t>(15 - (lane & 15));
        int ra = 0, rb = 0, rc = 0;  // three chains, so that the adds do not wait for one another
        count_greater_ror<1>(key, ra);  count_greater_ror<2>(key, rb);  count_greater_ror<3>(key, rc);
        count_greater_ror<4>(key, ra);  count_greater_ror<5>(key, rb);  count_greater_ror<6>(key, rc);
        count_greater_ror<7>(key, ra);  count_greater_ror<8>(key, rb);  count_greater_ror<9>(key, rc);
        count_greater_ror<10>(key, ra); count_greater_ror<11>(key, rb); count_greater_ror<12>(key, rc);
        count_greater_ror<13>(key, ra); count_greater_ror<14>(key, rb); count_greater_ror<15>(key, rc);
        const int rank = ra + rb + rc;
        const unsigned long long hit = __ballot(lane < 16 && rank == n_used - 1);
        float thr_l = -INFINITY;
        if (hit) thr_l = from_ordered_bits(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(key & ~15u), __ffsll(static_cast<long long>(hit)) - 1)));
        // (a bound of -inf, fewer than n_used groups holding anything, rounds down to a NaN pattern)
        if (!(thr_l == thr_l)) thr_l = -INFINITY;
        p0 = has0 && l0 >= thr_l;
        p1 = has1 && l1 >= thr_l;
        m0 = __ballot(p0);
        m1 = __ballot(p1);
        n0 = __popcll(m0);
        if (lane == 0) s_cnt[wave] = n0 + __popcll(m1);
    }
    __syncthreads();
    const int c0 = s_cnt[0], c1 = s_cnt[1], c2 = s_cnt[2], c3 = s_cnt[3];
    const int total = c0 + c1 + c2 + c3;
    if (total > kCandMax || total < n_used || n_expert < 64 || n_used > 16) {
        // uniform over the block: many equal logits, or a shape the threshold does not cover
        if (wave == 0) {
            route_token<8, false>(lg, n_expert, n_used, sel_e, sel_w, probs, scale);
            if (lane == 0) sel_w[n_used] = shared_gate ? sigmoid_exact(lg[n_expert] * scale) : 0.f;
        }
        __syncthreads();
        return;
    }
    if (routing) {
        // the table's order does not matter to the ranks: each wave writes its candidates after
        // those of the waves before it
        const int before = (wave > 0 ? c0 : 0) + (wave > 1 ? c1 : 0) + (wave > 2 ? c2 : 0);
        if (p0) {
            const int pos = before + static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(m0 >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(m0), 0u)));
            cand[pos] = (static_cast<unsigned long long>(ordered_bits(l0)) << 32) | static_cast<uint32_t>(0x7FFFFFFF - e0);
        }
        if (p1) {
            const int pos = before + n0 + static_cast<int>(__builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(m1 >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(m1), 0u)));
            cand[pos] = (static_cast<unsigned long long>(ordered_bits(l1)) << 32) | static_cast<uint32_t>(0x7FFFFFFF - e1);
        }
    }
    __syncthreads();
    // every wave: lane i owns candidate i; its rank is how many candidates are larger (the keys are
    // distinct: the expert is part of them).  The table is read sixteen entries at a time, all of a
    // batch's reads in flight together; entries past `total` hold old keys and are masked out.
    const unsigned long long mine = lane < total ? cand[lane] : 0ull;
    int r4[4] = {0, 0, 0, 0};  // four chains of counts
    for (int c = 0; c < total; c += 16) {
        ulonglong2 o[8];
#pragma unroll
        for (int j2 = 0; j2 < 8; j2++) o[j2] = *reinterpret_cast<const ulonglong2 *>(&cand[c + 2 * j2]);
#pragma unroll
        for (int j2 = 0; j2 < 8; j2++) {
            r4[(2 * j2) & 3] += (c + 2 * j2 < total && o[j2].x > mine) ? 1 : 0;
            r4[(2 * j2 + 1) & 3] += (c + 2 * j2 + 1 < total && o[j2].y > mine) ? 1 : 0;
        }
    }
    const int rank = (r4[0] + r4[1]) + (r4[2] + r4[3]);
    // slot k's key goes to lane k through the wave's own table; the selected experts' exponentials,
    // then their sum over the slots in order, in float32: the reference's order of additions
    if (lane < total && rank < n_used) s_sel[wave][rank] = mine;
    __builtin_amdgcn_wave_barrier();
    const unsigned long long sk = lane < n_used ? s_sel[wave][lane] : 0ull;
    const float ex_k = lane < n_used ? expf(from_ordered_bits(static_cast<uint32_t>(sk >> 32)) * scale - mx * scale) : 0.f;
    const int e_k = 0x7FFFFFFF - static_cast<int>(static_cast<uint32_t>(sk));
    float wsum = 0.f;
    for (int k = 0; k < n_used; k++) wsum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ex_k), k));
    if (lane < n_used) {
        sel_e[lane] = e_k;
        sel_w[lane] = ex_k / wsum;
    }
    if (lane == 63) sel_w[n_used] = shared_gate ? sigmoid_exact(lsh * scale) : 0.f;
    __builtin_amdgcn_wave_barrier();  // the wave reads what it has written itself (all waves write the same)
}

// ------------------------------------------------------------------------------- up ----------

// grid: (ffn/RPP/4/P row groups, n_used+1 slots, n_tok).  A pass of a wave is RPP gate rows and the
// same RPP up rows of one expert, six 16-byte loads per lane in flight together.  P: passes a wave
// makes over the staged activation row; a launch of many tokens has blocks to spare and uses
// them to stage the row an eighth as often (64-row chunk: 148 to 119 us a layer).
// NORM: a.xn is the row before its RMSNorm and a.logits lack the norm's factor (see route_block256):
// the row is staged as x * gamma, the factor comes from the block's own sum of squares and goes
// onto the finished gate and up products.
template <int K, int P, bool NORM = false>
__global__ __launch_bounds__(kBlock) void moe_up_kernel(shv_moe_up_args a, int slot0) {
    constexpr int LPR = K / 64, RPP = 64 / LPR;
    constexpr int ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    constexpr int NV = K / 4 / kBlock;
    static_assert(NV >= 1 || K == 512, "a thread stages whole float4s");
    __shared__ __align__(16) float xs[lds_padded(K)];
    __shared__ __align__(16) float xsum[K / 32];
    __shared__ __align__(16) float probs[192];
    __shared__ int32_t s_topk[kMaxUsed];
    __shared__ float s_w[kMaxUsed + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int slot = blockIdx.y + slot0, t = blockIdx.z;  // slot0: a launch over a part of the slots only
    const int gi = lane % LPR, rsub = lane / LPR, sb = gi >> 2, g = gi & 3;
    const int row0 = (blockIdx.x * 4 + wave) * P * RPP + rsub;  // row within the expert, first pass

    // the activation row is requested before anything else and staged further down
    const float *x = a.xn + static_cast<size_t>(t) * K;
    constexpr int NVr = NV >= 1 ? NV : 1;
    float4 xv[NVr];
    __shared__ float red[4];
#pragma unroll
    for (int j = 0; j < NVr; j++) {
        const int c = 4 * (tid + kBlock * j);
        xv[j] = c < K ? *reinterpret_cast<const float4 *>(x + c) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if constexpr (NORM) {
        float4 gm[NVr];
#pragma unroll
        for (int j = 0; j < NVr; j++) {
            const int c = 4 * (tid + kBlock * j);
            gm[j] = c < K ? *reinterpret_cast<const float4 *>(a.gamma + c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NVr; j++) {
            const float4 v = xv[j];
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
            xv[j] = make_float4(v.x * gm[j].x, v.y * gm[j].y, v.z * gm[j].z, v.w * gm[j].w);
        }
        ss = wave_sum_all(ss);
        if (lane == 0) red[wave] = ss;  // read behind the next block-wide wait, wherever that is
    }
    // the shared expert's gate from the staged row, by the first of the shared expert's blocks
    const bool gate_here = NORM && a.shared_gate && slot == a.n_used && blockIdx.x == 0;
    __shared__ float red_sg[4];
    if constexpr (NORM) {
        if (gate_here) {
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < NVr; j++) {
                const int c = 4 * (tid + kBlock * j);
                const float4 sg = c < K ? *reinterpret_cast<const float4 *>(a.shared_gate + c) : make_float4(0.f, 0.f, 0.f, 0.f);
                dot = fmaf(sg.x, xv[j].x, fmaf(sg.y, xv[j].y, fmaf(sg.z, xv[j].z, fmaf(sg.w, xv[j].w, dot))));
            }
            dot = wave_sum_all(dot);
            if (lane == 0) red_sg[wave] = dot;
        }
    }

    // the shared expert's blocks need no selection (the block that stores it is a routed slot's)
    if (a.logits && slot < a.n_used) {
        // route this block's token from the router's logits, all four waves together
        const float *lg = a.logits + static_cast<size_t>(t) * (a.n_expert + 1);
        route_block256<NORM>(lg, a.n_expert, a.n_used, a.no_shared_gate == 0 && !(NORM && a.shared_gate), s_topk, s_w, probs, red, 1.f / static_cast<float>(K), a.eps);
        if (blockIdx.x == 0 && blockIdx.y == 0) {
            if (tid < a.n_used) a.topk[static_cast<size_t>(t) * a.n_used + tid] = s_topk[tid];
            if (tid < a.n_used + ((NORM && a.shared_gate) ? 0 : 1)) a.weights[static_cast<size_t>(t) * (a.n_used + 1) + tid] = s_w[tid];
        }
    }

    // the weight loads go out next: they do not depend on the staged vector
    const char *gbase, *ubase;
    if (slot < a.n_used) {
        int e;
        if (a.logits) e = min(max(s_topk[slot], 0), a.n_expert - 1);  // whatever the selection gave, the address stays inside the bank
        else e = a.topk[static_cast<size_t>(t) * a.n_used + slot];
        gbase = static_cast<const char *>(a.gate_exps) + static_cast<size_t>(e) * a.ffn * ROWB;
        ubase = static_cast<const char *>(a.up_exps) + static_cast<size_t>(e) * a.ffn * ROWB;
    } else {
        gbase = static_cast<const char *>(a.gate_sh);
        ubase = static_cast<const char *>(a.up_sh);
    }
    Q4kLane wg[2], wu[2];
    {
        const size_t roff = static_cast<size_t>(row0 < a.ffn ? row0 : 0) * ROWB + sb * SHV_Q4K_BYTES;
        wg[0].load(gbase + roff, g);
        wu[0].load(ubase + roff, g);
    }

#pragma unroll
    for (int j = 0; j < NVr; j++) {
        const int c = 4 * (tid + kBlock * j);
        if (c < K) {
            *reinterpret_cast<float4 *>(&xs[lds_slot(c)]) = xv[j];
            const float s8 = sum8_all((xv[j].x + xv[j].y) + (xv[j].z + xv[j].w));
            if ((lane & 7) == 0) xsum[c >> 5] = s8;
        }
    }
    __syncthreads();
    float scale = 1.f;
    if constexpr (NORM) {
        scale = __builtin_amdgcn_rsqf(((red[0] + red[1]) + (red[2] + red[3])) / static_cast<float>(K) + a.eps);
        if (gate_here && tid == 0) a.weights[static_cast<size_t>(t) * (a.n_used + 1) + a.n_used] = sigmoid_exact(((red_sg[0] + red_sg[1]) + (red_sg[2] + red_sg[3])) * scale);
    }
    float xr[64], xs_lo, xs_hi;
    load_x_slice_presummed(xs, xsum, gi, xr, xs_lo, xs_hi);
    const NibbleConsts nc = nibble_consts();
#pragma unroll
    for (int p = 0; p < P; p++) {
        const int row = row0 + p * RPP;
        if (p + 1 < P) {
            // the next pass's weights are on their way while this pass multiplies
            const size_t roff = static_cast<size_t>(row + RPP < a.ffn ? row + RPP : 0) * ROWB + sb * SHV_Q4K_BYTES;
            wg[(p + 1) & 1].load(gbase + roff, g);
            wu[(p + 1) & 1].load(ubase + roff, g);
        }
        float gv = wg[p & 1].dot(g, nc, xr, xs_lo, xs_hi);
        float uv = wu[p & 1].dot(g, nc, xr, xs_lo, xs_hi);
        gv = group_sum<LPR>(gv) * scale;
        uv = group_sum<LPR>(uv) * scale;
        if (row < a.ffn && group_sum_owner<LPR>(lane)) {
            const float s = gv * sigmoid_exact(gv);
            a.act[(static_cast<size_t>(t) * (a.n_used + 1) + slot) * a.ffn + row] = s * uv;
        }
    }
}

// ------------------------------------------------------------------------------ down ---------

// grid: (n_embd/RPP/P row groups, n_tok).  A block owns P * RPP output rows of one token; its four
// waves split the n_used+1 slots, each lane scales its partial dot by the slot's weight, and the
// block adds the four waves' sums (and the residual) at the end.  P: passes over the staged
// activation rows, as in the up projection (eight for many tokens, taken slot after slot).
template <int K, int MAXS, int P>
__global__ __launch_bounds__(kBlock) void moe_down_kernel(shv_moe_down_args a, int s_lo, int s_hi) {
    constexpr int LPR = K / 64, RPP = 64 / LPR;
    constexpr int ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    constexpr int SPW = (MAXS + 3) / 4;  // slots per wave
    __shared__ __align__(16) float xs[MAXS][lds_padded(K)];
    __shared__ float part[4][P * RPP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.y;
    const int ns = a.n_used + 1;
    const int gi = lane % LPR, rsub = lane / LPR, sb = gi >> 2, g = gi & 3;
    const int row0 = blockIdx.x * P * RPP + rsub;
    // the residual of the row this thread will write at the end is asked for now
    float res = 0.f;
    if (a.residual && tid < P * RPP && blockIdx.x * P * RPP + tid < a.n_embd) res = a.residual[static_cast<size_t>(t) * a.res_stride + blockIdx.x * P * RPP + tid];

    Q4kLane w[2][SPW];
    float wt[SPW];
    const char *base[SPW];
#pragma unroll
    for (int i = 0; i < SPW; i++) {
        const int s = wave + 4 * i;
        wt[i] = 0.f;
        base[i] = static_cast<const char *>(a.down_sh);
        if (s >= s_lo && s < s_hi) {  // [s_lo, s_hi): the slots this launch adds up
            if (s < a.n_used) {
                const int e = a.topk[static_cast<size_t>(t) * a.n_used + s];
                base[i] = static_cast<const char *>(a.down_exps) + static_cast<size_t>(e) * a.n_embd * ROWB;
            }
            w[0][i].load(base[i] + static_cast<size_t>(row0 < a.n_embd ? row0 : 0) * ROWB + sb * SHV_Q4K_BYTES, g);
            wt[i] = a.weights[static_cast<size_t>(t) * ns + s];
        }
    }
    // each wave stages the activations of its own slots only, so no block-wide hand-over is
    // needed before the dot products: all loads first, then the LDS writes
    const float *act = a.act + static_cast<size_t>(t) * ns * K;
    constexpr int F4 = K / 4 / 64;  // float4 per lane per slot
    float4 stage[SPW][F4];
#pragma unroll
    for (int i = 0; i < SPW; i++) {
        const int s = wave + 4 * i;
#pragma unroll
        for (int j = 0; j < F4; j++)
            stage[i][j] = s >= s_lo && s < s_hi ? *reinterpret_cast<const float4 *>(act + static_cast<size_t>(s) * K + (j * 64 + lane) * 4)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < SPW; i++) {
        const int s = wave + 4 * i;
        if (s >= s_lo && s < s_hi) {
#pragma unroll
            for (int j = 0; j < F4; j++) {
                const int c = (j * 64 + lane) * 4;  // four consecutive columns never straddle a 64-slice
                *reinterpret_cast<float4 *>(&xs[s][lds_slot(c)]) = stage[i][j];
            }
        }
    }
    __builtin_amdgcn_wave_barrier();  // LDS operations of one wave complete in order

    const NibbleConsts nc = nibble_consts();
    if constexpr (P <= 2) {
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int row = row0 + p * RPP;
            if (p + 1 < P) {
                // the next pass's weights are on their way while this pass multiplies
                const size_t roff = static_cast<size_t>(row + RPP < a.n_embd ? row + RPP : 0) * ROWB + sb * SHV_Q4K_BYTES;
#pragma unroll
                for (int i = 0; i < SPW; i++)
                    if (wave + 4 * i >= s_lo && wave + 4 * i < s_hi) w[(p + 1) & 1][i].load(base[i] + roff, g);
            }
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < SPW; i++) {
                const int s = wave + 4 * i;
                if (s >= s_lo && s < s_hi) {
                    float xr[64], xs_lo, xs_hi;
                    load_x_slice(xs[s], gi, xr, xs_lo, xs_hi);
                    acc = fmaf(wt[i], w[p & 1][i].dot(g, nc, xr, xs_lo, xs_hi), acc);
                }
            }
            acc = group_sum<LPR>(acc);
            if (group_sum_owner<LPR>(lane)) part[wave][p * RPP + rsub] = acc;
        }
    } else {
        // Many passes: slot after slot, so that a slot's 64 activations come out of LDS once for all
        // of the block's rows instead of once per pass (that re-reading was a third of the kernel at
        // 64 tokens).  Each output row still adds its slots up in slot order.
        float acc[P];
#pragma unroll
        for (int p = 0; p < P; p++) acc[p] = 0.f;
#pragma unroll
        for (int i = 0; i < SPW; i++) {
            const int s = wave + 4 * i;
            if (s >= s_lo && s < s_hi) {
                float xr[64], xs_lo, xs_hi;
                load_x_slice(xs[s], gi, xr, xs_lo, xs_hi);
                Q4kLane ww[2];
                ww[0] = w[0][i];
#pragma unroll
                for (int p = 0; p < P; p++) {
                    const int row = row0 + p * RPP;
                    if (p + 1 < P) ww[(p + 1) & 1].load(base[i] + static_cast<size_t>(row + RPP < a.n_embd ? row + RPP : 0) * ROWB + sb * SHV_Q4K_BYTES, g);
                    acc[p] = fmaf(wt[i], ww[p & 1].dot(g, nc, xr, xs_lo, xs_hi), acc[p]);
                }
            }
        }
#pragma unroll
        for (int p = 0; p < P; p++) {
            const float v = group_sum<LPR>(acc[p]);
            if (group_sum_owner<LPR>(lane)) part[wave][p * RPP + rsub] = v;
        }
    }
    __syncthreads();
    if (tid < P * RPP) {
        const int r = blockIdx.x * P * RPP + tid;
        if (r < a.n_embd) {
            float v = (part[0][tid] + part[1][tid]) + (part[2][tid] + part[3][tid]);
            a.out[static_cast<size_t>(t) * a.out_stride + r] = v + res;
        }
    }
}


// The down projection of a pass of few tokens (the decode step): a chain of latencies, so every
// slot gets a wave of its own (a block is n_used+1 waves over P passes of RPP output rows) instead
// of four waves walking three slots each, the slot's activations are asked for first (loads come
// back in the order they were issued, and the weights take longest), and the sums of every 32
// activations the min term needs are made once at staging, not by every lane.  The waves' products
// are added in slot order by the block's first threads, with the residual.
// grid: (n_embd / (P * RPP), n_tok), (s_hi - s_lo) * 64 threads.
template <int K, int P>
__global__ __launch_bounds__(768) void moe_down_slots_kernel(shv_moe_down_args a, int s_lo, int s_hi) {
    constexpr int LPR = K / 64, RPP = 64 / LPR, ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES, NV = K / 4 / 64;
    constexpr int kMaxSlots = 12;
    __shared__ __align__(16) float xs[kMaxSlots][lds_padded(K)];
    __shared__ __align__(16) float xsum[kMaxSlots][K / 32];
    __shared__ float part[kMaxSlots][P * RPP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.y, s = s_lo + wave, ns = a.n_used + 1;
    const int gi = lane % LPR, rsub = lane / LPR, sb = gi >> 2, g = gi & 3;
    const int row0 = blockIdx.x * P * RPP + rsub;
    // this slot's activations, then its expert and weight (scalar loads), then the weights
    const float *act = a.act + (static_cast<size_t>(t) * ns + s) * K;
    float4 av[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) av[j] = *reinterpret_cast<const float4 *>(act + 4 * (lane + 64 * j));
    const char *base = static_cast<const char *>(a.down_sh);
    if (s < a.n_used) base = static_cast<const char *>(a.down_exps) + static_cast<size_t>(a.topk[static_cast<size_t>(t) * a.n_used + s]) * a.n_embd * ROWB;
    const float wt = a.weights[static_cast<size_t>(t) * ns + s];
    Q4kLane w[P];
#pragma unroll
    for (int p = 0; p < P; p++) {
        const int row = row0 + p * RPP;
        w[p].load(base + static_cast<size_t>(row < a.n_embd ? row : 0) * ROWB + sb * SHV_Q4K_BYTES, g);
    }
    float res = 0.f;
    const int out_row = blockIdx.x * P * RPP + tid;
    if (a.residual && tid < P * RPP && out_row < a.n_embd) res = a.residual[static_cast<size_t>(t) * a.res_stride + out_row];
    // the wave stages its own slot: no block-wide wait before the products
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int c = 4 * (lane + 64 * j);
        *reinterpret_cast<float4 *>(&xs[wave][lds_slot(c)]) = av[j];
        const float s8 = sum8_all((av[j].x + av[j].y) + (av[j].z + av[j].w));
        if ((lane & 7) == 0) xsum[wave][c >> 5] = s8;
    }
    __builtin_amdgcn_wave_barrier();  // LDS operations of one wave complete in order
    float xr[64], xs_lo, xs_hi;
    load_x_slice_presummed(xs[wave], xsum[wave], gi, xr, xs_lo, xs_hi);
    const NibbleConsts nc = nibble_consts();
#pragma unroll
    for (int p = 0; p < P; p++) {
        float acc = group_sum<LPR>(w[p].dot(g, nc, xr, xs_lo, xs_hi));
        if (group_sum_owner<LPR>(lane)) part[wave][p * RPP + rsub] = wt * acc;
    }
    __syncthreads();
    if (tid < P * RPP && out_row < a.n_embd) {
        float v = 0.f;
        for (int i = 0; i < s_hi - s_lo; i++) v += part[i][tid];  // slot order
        a.out[static_cast<size_t>(t) * a.out_stride + out_row] = v + res;
    }
}

}  // namespace

int shv_launch_moe_router(shv_ctx *ctx, const shv_moe_router_args *pa) {
    const shv_moe_router_args &a = *pa;
    SHV_REQUIRE(a.h && a.router && a.logits, "moe_router: NULL h, router or logits");
    SHV_REQUIRE(a.defer_route || (a.topk && a.weights), "moe_router: NULL topk or weights");
    SHV_REQUIRE(a.n_tok >= 1, "moe_router: n_tok %d", a.n_tok);
    SHV_REQUIRE(a.n_expert >= 1 && a.n_expert <= 512, "moe_router: n_expert %d, the routing wave covers up to 512", a.n_expert);
    SHV_REQUIRE(a.n_used >= 1 && a.n_used <= kMaxUsed && a.n_used <= a.n_expert, "moe_router: n_used %d of %d (at most %d)", a.n_used, a.n_expert, kMaxUsed);
    SHV_REQUIRE(a.h_stride >= a.n_embd, "moe_router: h_stride %d < n_embd %d", a.h_stride, a.n_embd);
    SHV_REQUIRE(shv_aligned16(a.router) && shv_aligned16(a.shared_gate), "moe_router: router and shared_gate must be 16-byte aligned");
    // a pass of many rows: the logits on the matrix cores
    if (shv_router_wide_covers(ctx, a)) {
        const int rc = shv_launch_router_wide(ctx, a);
        if (rc != SHV_OK) return rc;
        if (!a.defer_route) {
            if (a.n_expert > 64 && a.n_expert <= kRouteBlock) SHV_LAUNCH(ctx, moe_route_block_kernel, dim3(a.n_tok), dim3(kRouteBlock), 0, a);
            else SHV_LAUNCH(ctx, moe_route_kernel, dim3(a.n_tok), dim3(64), 0, a);
        }
        return SHV_OK;
    }
    // four rows a wave only where that still leaves a few hundred blocks
    const bool many = a.n_tok >= 128;
    const int rw = many ? 4 : 1, tpb = a.n_tok >= 512 ? kRouterTokensMany : many ? 8 : kRouterTokens;
    const dim3 blocks((a.n_expert + 1 + 4 * rw - 1) / (4 * rw), (a.n_tok + tpb - 1) / tpb);
    SHV_REQUIRE(blocks.y <= 65535, "moe_router: n_tok %d", a.n_tok);
    switch (a.n_embd) {
        case 2048:
            if (many) SHV_LAUNCH(ctx, (moe_router_kernel<2048, 4>), blocks, dim3(kBlock), 0, a, tpb);
            else SHV_LAUNCH(ctx, (moe_router_kernel<2048, 1>), blocks, dim3(kBlock), 0, a, tpb);
            break;
        case 1024:
            if (many) SHV_LAUNCH(ctx, (moe_router_kernel<1024, 4>), blocks, dim3(kBlock), 0, a, tpb);
            else SHV_LAUNCH(ctx, (moe_router_kernel<1024, 1>), blocks, dim3(kBlock), 0, a, tpb);
            break;
        case 512:
            if (many) SHV_LAUNCH(ctx, (moe_router_kernel<512, 4>), blocks, dim3(kBlock), 0, a, tpb);
            else SHV_LAUNCH(ctx, (moe_router_kernel<512, 1>), blocks, dim3(kBlock), 0, a, tpb);
            break;
        default: return shv_set_error(SHV_E_INVALID, "moe_router: n_embd = %d; built for 512, 1024 and 2048", a.n_embd);
    }
    // the selection needs every logit of the token, i.e. the whole grid above: a second, tiny
    // launch is cheaper than handing the logits to one block inside the first
    if (!a.defer_route) {
        if (a.n_expert > 64 && a.n_expert <= kRouteBlock) SHV_LAUNCH(ctx, moe_route_block_kernel, dim3(a.n_tok), dim3(kRouteBlock), 0, a);
        else SHV_LAUNCH(ctx, moe_route_kernel, dim3(a.n_tok), dim3(64), 0, a);
    }
    return SHV_OK;
}

int shv_launch_moe_up(shv_ctx *ctx, const shv_moe_up_args *pa) {
    const shv_moe_up_args &a = *pa;
    SHV_REQUIRE(a.xn && a.topk && a.gate_exps && a.up_exps && a.gate_sh && a.up_sh && a.act, "moe_up: NULL argument");
    if (a.logits) {
        SHV_REQUIRE(a.weights, "moe_up: routing from logits needs somewhere to store the weights");
        SHV_REQUIRE(a.n_expert >= 1 && a.n_expert <= 512 && a.n_used <= a.n_expert, "moe_up: n_expert %d, n_used %d", a.n_expert, a.n_used);
    }
    SHV_REQUIRE(a.n_tok >= 1 && a.n_tok <= 65535, "moe_up: n_tok %d", a.n_tok);
    SHV_REQUIRE(a.n_used >= 1 && a.n_used <= kMaxUsed, "moe_up: n_used %d", a.n_used);
    SHV_REQUIRE(a.ffn >= 1, "moe_up: ffn %d", a.ffn);
    SHV_REQUIRE(!a.shared_gate || (a.gamma && shv_aligned16(a.shared_gate)), "moe_up: shared_gate goes with gamma (the row normalised inside the launch), 16-byte aligned");
    if (a.gamma)
        SHV_REQUIRE(a.logits && a.n_tok <= 4 && a.n_embd == 2048 && shv_aligned16(a.gamma) && shv_aligned16(a.xn) && is_q4k(a.gate_type) && is_q4k(a.up_type) &&
                        is_q4k(a.gate_sh_type) && is_q4k(a.up_sh_type),
                    "moe_up: the RMSNorm of the row inside the launch (gamma) goes with logits, one to four rows of 2048 and Q4_K banks");
    ctx->moe_stamp = {};  // only the grouped launch leaves lists or operands behind, and says so itself
    // Banks of other types than Q4_K go through their own arms; a block whose routed banks and
    // shared expert differ in that takes one launch each, over its part of the slots.
    const bool r_other = !is_q4k(a.gate_type) || !is_q4k(a.up_type), s_other = !is_q4k(a.gate_sh_type) || !is_q4k(a.up_sh_type);
    if (r_other && s_other) return shv_launch_moe_up_any(ctx, pa, 0, a.n_used + 1);
    if (r_other || s_other) SHV_REQUIRE(!a.logits, "moe_up: banks of other types than Q4_K take the selection from the router, not from logits");
    const int slot0 = r_other ? a.n_used : 0, slots = r_other ? 1 : s_other ? a.n_used : a.n_used + 1;  // the Q4_K part
    SHV_REQUIRE(shv_aligned16(a.gate_exps) && shv_aligned16(a.up_exps) && shv_aligned16(a.gate_sh) && shv_aligned16(a.up_sh),
                "moe_up: weight banks must be 16-byte aligned");
    // a pass of many rows whose selection is made: the experts' weights once per 48 tokens
    if (!r_other && !s_other && shv_moe_up_grouped_covers(ctx, a)) return shv_launch_moe_up_grouped(ctx, a);
    dim3 block(kBlock);
    // enough tokens to fill the chip with blocks eight passes tall; not when the blocks route
    // for themselves, which they do once per block
    const bool many = a.n_tok >= ctx->moe_tall_min && !a.logits;
    switch (a.n_embd) {
        case 2048: {
            constexpr int RPP = 64 / (2048 / 64);
            if (many) {
                dim3 grid((a.ffn + RPP * 32 - 1) / (RPP * 32), slots, a.n_tok);
                SHV_LAUNCH(ctx, (moe_up_kernel<2048, 8>), grid, block, 0, a, slot0);
            } else {
                // a block routes and stages for itself before its rows' weights matter: one pass a wave for the
                // decode step, whose blocks all fit the chip at once; two from two rows on (3 rows: 2112 blocks
                // in three rounds against 1056; 14.4 to 12.5 us a layer)
                // (four passes a wave at four rows that route for themselves: four sequences a pass 2.86 to 2.76 ms; at three rows no change)
                const int pp = (a.n_tok == 4 && a.gamma) ? 4 : a.n_tok >= 2 ? 2 : 1;
                dim3 grid((a.ffn + RPP * 4 * pp - 1) / (RPP * 4 * pp), slots, a.n_tok);
                if (pp == 4) SHV_LAUNCH(ctx, (moe_up_kernel<2048, 4, true>), grid, block, 0, a, slot0);
                else if (pp == 2) {
                    if (a.gamma) SHV_LAUNCH(ctx, (moe_up_kernel<2048, 2, true>), grid, block, 0, a, slot0);
                    else SHV_LAUNCH(ctx, (moe_up_kernel<2048, 2>), grid, block, 0, a, slot0);
                } else if (a.gamma) SHV_LAUNCH(ctx, (moe_up_kernel<2048, 1, true>), grid, block, 0, a, slot0);
                else SHV_LAUNCH(ctx, (moe_up_kernel<2048, 1>), grid, block, 0, a, slot0);
            }
            break;
        }
        case 1024: {
            constexpr int RPP = 64 / (1024 / 64);
            if (many) {
                dim3 grid((a.ffn + RPP * 32 - 1) / (RPP * 32), slots, a.n_tok);
                SHV_LAUNCH(ctx, (moe_up_kernel<1024, 8>), grid, block, 0, a, slot0);
            } else {
                dim3 grid((a.ffn + RPP * 4 - 1) / (RPP * 4), slots, a.n_tok);
                SHV_LAUNCH(ctx, (moe_up_kernel<1024, 1>), grid, block, 0, a, slot0);
            }
            break;
        }
        case 512: {
            constexpr int RPP = 64 / (512 / 64);
            if (many) {
                dim3 grid((a.ffn + RPP * 32 - 1) / (RPP * 32), slots, a.n_tok);
                SHV_LAUNCH(ctx, (moe_up_kernel<512, 8>), grid, block, 0, a, slot0);
            } else {
                dim3 grid((a.ffn + RPP * 4 - 1) / (RPP * 4), slots, a.n_tok);
                SHV_LAUNCH(ctx, (moe_up_kernel<512, 1>), grid, block, 0, a, slot0);
            }
            break;
        }
        default: return shv_set_error(SHV_E_INVALID, "moe_up: n_embd = %d; built for 512, 1024 and 2048", a.n_embd);
    }
    if (r_other) return shv_launch_moe_up_any(ctx, pa, 0, a.n_used);
    if (s_other) return shv_launch_moe_up_any(ctx, pa, a.n_used, 1);
    return SHV_OK;
}

int shv_launch_moe_down(shv_ctx *ctx, const shv_moe_down_args *pa) {
    const shv_moe_down_args &a = *pa;
    SHV_REQUIRE(a.act && a.topk && a.weights && a.down_exps && a.down_sh && a.out, "moe_down: NULL argument");
    SHV_REQUIRE(a.n_tok >= 1 && a.n_tok <= 65535, "moe_down: n_tok %d", a.n_tok);
    SHV_REQUIRE(a.n_used >= 1 && a.n_used + 1 <= 12, "moe_down: n_used %d; built for up to 11 routed experts", a.n_used);
    SHV_REQUIRE(a.n_embd >= 1 && a.out_stride >= a.n_embd && (!a.residual || a.res_stride >= a.n_embd), "moe_down: strides");
    SHV_REQUIRE(a.ffn >= 1, "moe_down: ffn %d", a.ffn);
    // act as matrix-core operands is read by the grouped Q4_K launch alone: every other road below
    // takes floats, so the flag and what the gate/up launch really left must agree with the road
    {
        const bool packed_here = ctx->moe_stamp.packed && ctx->moe_stamp.act == a.act;
        const bool grouped_road = is_q4k(a.down_type) && is_q4k(a.down_sh_type) && shv_moe_down_grouped_covers(ctx, a);
        // (a pass too short to be grouped ignores the flag in both launches: act is floats then)
        SHV_REQUIRE(!packed_here || (a.act_packed && grouped_road),
                    "moe_down: the shv_moe_up before this call left act as matrix-core operands (its act_packed); this call %s",
                    a.act_packed ? "does not take the grouped Q4_K path that reads them (bank types, workspaces)" : "reads floats (act_packed is not set)");
    }
    // as in the up projection: the Q4_K part of the slots here, the rest through the other arms,
    // which then add to what this launch has written
    const bool r_other = !is_q4k(a.down_type), s_other = !is_q4k(a.down_sh_type);
    if (r_other && s_other) return shv_launch_moe_down_any(ctx, pa, 0, a.n_used + 1, 0);
    const int s_lo = r_other ? a.n_used : 0, s_hi = s_other ? a.n_used : a.n_used + 1;
    SHV_REQUIRE(shv_aligned16(a.down_exps) && shv_aligned16(a.down_sh), "moe_down: weight banks must be 16-byte aligned");
    if (!r_other && !s_other && shv_moe_down_grouped_covers(ctx, a)) return shv_launch_moe_down_grouped(ctx, a);
    dim3 block(kBlock);
    switch (a.ffn) {
        case 512: {
            constexpr int RPP = 64 / (512 / 64);
            if (a.n_tok >= ctx->moe_tall_min) SHV_LAUNCH(ctx, (moe_down_kernel<512, 12, 8>), dim3((a.n_embd + RPP * 8 - 1) / (RPP * 8), a.n_tok), block, 0, a, s_lo, s_hi);
            else if (a.n_tok >= 3 && a.n_tok < 8 && a.n_embd % (4 * RPP) == 0 && shv_aligned16(a.act)) SHV_LAUNCH(ctx, (moe_down_slots_kernel<512, 4>),  // three rows and more: four
                dim3(a.n_embd / (4 * RPP), a.n_tok), dim3((s_hi - s_lo) * 64), 0, a, s_lo, s_hi);  // passes a wave (a 3-row verification pass 2.48 to 2.43 ms; at two rows 2.14 becomes 2.19)
            else if (a.n_tok >= 2 && a.n_tok < 8 && a.n_embd % (2 * RPP) == 0 && shv_aligned16(a.act)) SHV_LAUNCH(ctx, (moe_down_slots_kernel<512, 2>),  // verification passes: one round of blocks
                dim3(a.n_embd / (2 * RPP), a.n_tok), dim3((s_hi - s_lo) * 64), 0, a, s_lo, s_hi);
            else if (a.n_tok < 8 && a.n_embd % (1 * RPP) == 0 && shv_aligned16(a.act)) SHV_LAUNCH(ctx, (moe_down_slots_kernel<512, 1>),  // the decode step and verification passes
                dim3(a.n_embd / (1 * RPP), a.n_tok), dim3((s_hi - s_lo) * 64), 0, a, s_lo, s_hi);
            else if (a.n_tok >= 8 && a.n_tok <= 12 && a.n_embd % (4 * RPP) == 0 && shv_aligned16(a.act)) SHV_LAUNCH(ctx, (moe_down_slots_kernel<512, 4>),  // eight sequences
                dim3(a.n_embd / (4 * RPP), a.n_tok), dim3((s_hi - s_lo) * 64), 0, a, s_lo, s_hi);                      // decoded together: a wave a slot, one round of blocks (4.32 to 4.25 ms a pass; two passes a wave 4.31, eight 4.48)
            else if (a.n_tok >= 8) SHV_LAUNCH(ctx, (moe_down_kernel<512, 12, 4>),  // eight sequences decoded together: 5.31 to 5.19 ms a pass
                dim3((a.n_embd + RPP * 4 - 1) / (RPP * 4), a.n_tok), block, 0, a, s_lo, s_hi);
            else SHV_LAUNCH(ctx, (moe_down_kernel<512, 12, 1>), dim3((a.n_embd + RPP - 1) / RPP, a.n_tok), block, 0, a, s_lo, s_hi);
            break;
        }
        case 256: {
            constexpr int RPP = 64 / (256 / 64);
            if (a.n_tok >= ctx->moe_tall_min) SHV_LAUNCH(ctx, (moe_down_kernel<256, 12, 8>), dim3((a.n_embd + RPP * 8 - 1) / (RPP * 8), a.n_tok), block, 0, a, s_lo, s_hi);
            else SHV_LAUNCH(ctx, (moe_down_kernel<256, 12, 1>), dim3((a.n_embd + RPP - 1) / RPP, a.n_tok), block, 0, a, s_lo, s_hi);
            break;
        }
        default: return shv_set_error(SHV_E_INVALID, "moe_down: ffn = %d; built for 256 and 512", a.ffn);
    }
    if (r_other) return shv_launch_moe_down_any(ctx, pa, 0, a.n_used, 1);
    if (s_other) return shv_launch_moe_down_any(ctx, pa, a.n_used, a.n_used + 1, 1);
    return SHV_OK;
}
