// The experts of a pass of many rows, grouped by expert on the matrix cores (the prompt side of
// MoETrace.Experts, llm/moe.go:289-409; the reference batches a chunk's tokens per expert in
// llm_moe_gemv.comp's multi-row arm).  The per-(token, expert) GEMV reads and unpacks an expert's
// weights once per token that chose it, this path once per 48 such tokens: it pays when tokens
// outnumber experts (2048 rows choosing 10 of 512: 40 tokens an expert), not at 64 rows (1.9).
//
//   moe_group_kernel          per-expert lists of (token, slot) pairs from topk (one block; long passes:
//                             moe_group_count_kernel + moe_group_place_kernel, sixteen blocks)
//   moe_up_grouped_kernel     a block = (expert, half of its ffn rows) and up to 48 of its tokens
//                             at a time: their xn rows go through LDS as matrix-core operands
//                             (two halves hi + lo, as the projections do) in slabs of 512 columns,
//                             each wave streams two gate tiles of 16 rows and the matching up
//                             tiles, forms a sub-block's weights once (as the whole numbers n * sc,
//                             exact in binary16) for all three token tiles, keeps one matrix
//                             accumulator per super-block, SwiGLU in registers, act[pair] out
//   moe_down_grouped_kernel   a block = (expert, quarter of n_embd rows): act rows staged the
//                             same way (one slab), each wave two tiles, raw products to pairs[pair]
//   moe_combine_kernel        out[t] = residual[t] + sum over slots of weights[t][s]*pairs[t][s],
//                             slots in order
// The shared expert is an expert every token lists: its blocks take 48 tokens each.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;       // 256 registers a lane: the streams, the accumulators of four row tiles and the operands fit without spilling
constexpr int kThreads = kWaves * 64;
constexpr int kTT = 3;            // matrix-core tiles of 16 tokens a block multiplies per pass over the weights
constexpr int kTok = 16 * kTT;    // tokens of such a pass
constexpr int kTiles = 4;         // weight row tiles of 16 a wave owns
constexpr int kSlab = 512;        // columns of the tokens' rows staged at a time
constexpr int kSlabSubs = kSlab / 32;
constexpr int kFrag = 64 * 16;    // one operand: a lane's eight halves
constexpr int kMaxExperts = 1024;

// The caller's `group` workspace: [0, n_expert] start of each expert's list (one more: the total),
// then n_tok * n_used pair ids (token * (n_used + 1) + slot), then the experts in the order their
// blocks are launched: longest list first, so that the blocks which walk their weights two or
// three times start early and the launch does not end on them.  A list's order is whatever the
// arrivals made it; every pair's products are formed in a matrix-core column of their own, so no
// value depends on it.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *topk, int n_tok, int n_used, int n_expert, int32_t *group) {
    __shared__ int32_t s_cnt[kMaxExperts + 1];
    __shared__ __align__(16) int32_t s_len[kMaxExperts];
    const int tid = threadIdx.x, n_pairs = n_tok * n_used;
    for (int e = tid; e <= n_expert; e += blockDim.x) s_cnt[e] = 0;
    for (int e = tid; e < kMaxExperts; e += blockDim.x) s_len[e] = -1;  // past n_expert: shorter than any list
    // A thread's selections are asked for once, all together, and stay in registers for both passes (the count and
    // the placement): up to NQ quads of four a thread, i.e. 4096 * NQ pairs; a longer pass reads the rest again.
    constexpr int NQ = 8;
    // whole quads of an aligned table; the tail and what does not fit the registers go one by one
    const int n_quads = (reinterpret_cast<uintptr_t>(topk) & 15) == 0 ? n_pairs / 4 : 0;
    int4 q[NQ];
#pragma unroll
    for (int b = 0; b < NQ; b++) {
        const int i = tid + b * 1024;
        q[b] = i < n_quads ? reinterpret_cast<const int4 *>(topk)[i] : make_int4(-1, -1, -1, -1);
    }
    const int rest0 = (n_quads < NQ * 1024 ? n_quads : NQ * 1024) * 4;
    __syncthreads();
    auto count = [&](int e) {
        if (e >= 0 && e < n_expert) atomicAdd(&s_cnt[e], 1);
    };
#pragma unroll
    for (int b = 0; b < NQ; b++) {
        count(q[b].x);
        count(q[b].y);
        count(q[b].z);
        count(q[b].w);
    }
    for (int i = rest0 + tid; i < n_pairs; i += 1024) count(topk[i]);
    __syncthreads();
    {
        // starts = running sum of the counts: thread e takes expert e (the block has a thread for each)
        __shared__ int32_t s_wsum[16];
        const int lane = tid & 63, wave = tid >> 6;
        const int c = tid < n_expert ? s_cnt[tid] : 0;
        int incl = c;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        if (lane == 63) s_wsum[wave] = incl;
        __syncthreads();
        int base = 0;
        for (int w = 0; w < wave; w++) base += s_wsum[w];
        if (tid < n_expert) {
            s_cnt[tid] = base + incl - c;
            s_len[tid] = c;
        }
        if (tid == n_expert - 1) s_cnt[n_expert] = base + incl;
    }
    __syncthreads();
    for (int e = tid; e <= n_expert; e += blockDim.x) group[e] = s_cnt[e];
    // rank by list length, longer first, equal lengths by index: an expert's place in the launch.  32 threads an
    // expert, each against every 32nd length, 32 experts a round: with a thread an expert half the block idles
    // through E comparisons each.
    int32_t *order = group + n_expert + 1 + n_pairs;
    {
        const int part = tid & 31;
        for (int e = tid >> 5; e < n_expert; e += 32) {
            const int ce = s_len[e];
            int rank = 0;
            for (int o = part; o < n_expert; o += 32) {
                const int co = s_len[o];
                rank += (co > ce || (co == ce && o < e)) ? 1 : 0;
            }
            rank += __shfl_xor(rank, 16, 64);
            rank += __shfl_xor(rank, 8, 64);
            rank += __shfl_xor(rank, 4, 64);
            rank += __shfl_xor(rank, 2, 64);
            rank += __shfl_xor(rank, 1, 64);
            if (part == 0) order[rank] = e;
        }
    }
    __syncthreads();  // the starts are copied out before the placement moves them
    int32_t *list = group + n_expert + 1;
    auto place = [&](int e, int i) {
        if (e >= 0 && e < n_expert) list[atomicAdd(&s_cnt[e], 1)] = (i / n_used) * (n_used + 1) + i % n_used;
    };
#pragma unroll
    for (int b = 0; b < NQ; b++) {
        const int i = 4 * (tid + b * 1024);
        place(q[b].x, i);
        place(q[b].y, i + 1);
        place(q[b].z, i + 2);
        place(q[b].w, i + 3);
    }
    for (int i = rest0 + tid; i < n_pairs; i += 1024) place(topk[i], i);
}

// The same lists by several blocks in two launches, for passes long enough that one block's count and placement
// (one compute unit's scattered stores) are most of the grouping: block b takes pairs [b * chunk, (b + 1) * chunk).
// First launch: every block's count of its pairs per expert, to counts[b][e].  Second: every block adds up the
// counts (an expert's total, and what the blocks before it hold of it), forms the starts, and places its own pairs
// behind those of the blocks before it; block 0 also writes the starts and the experts' launch order.
constexpr int kGroupBlocks = 16;
__global__ __launch_bounds__(1024) void moe_group_count_kernel(const int32_t *topk, int n_pairs, int chunk, int n_expert, int32_t *counts) {
    __shared__ int32_t s_cnt[kMaxExperts];
    const int tid = threadIdx.x;
    for (int e = tid; e < n_expert; e += 1024) s_cnt[e] = 0;
    __syncthreads();
    const int lo = blockIdx.x * chunk, hi = lo + chunk < n_pairs ? lo + chunk : n_pairs;
    for (int i = lo + tid; i < hi; i += 1024) {
        const int e = topk[i];
        if (e >= 0 && e < n_expert) atomicAdd(&s_cnt[e], 1);
    }
    __syncthreads();
    for (int e = tid; e < n_expert; e += 1024) counts[blockIdx.x * n_expert + e] = s_cnt[e];
}

__global__ __launch_bounds__(1024) void moe_group_place_kernel(const int32_t *topk, int n_pairs, int chunk, int n_used, int n_expert, const int32_t *counts,
                                                               int32_t *group) {
    __shared__ int32_t s_cnt[kMaxExperts + 1];
    __shared__ __align__(16) int32_t s_len[kMaxExperts];
    __shared__ int32_t s_wsum[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nb = gridDim.x, b = blockIdx.x;
    // thread e: expert e's total, and the pairs of it the blocks before this one hold
    int c = 0, before = 0;
    if (tid < n_expert) {
        // all of them asked for together: one after the other they are sixteen trips to memory
        int v[kGroupBlocks];
#pragma unroll
        for (int o = 0; o < kGroupBlocks; o++) v[o] = o < nb ? counts[o * n_expert + tid] : 0;
#pragma unroll
        for (int o = 0; o < kGroupBlocks; o++) {
            c += v[o];
            before += o < b ? v[o] : 0;
        }
    }
    int incl = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) s_wsum[wave] = incl;
    s_len[tid] = tid < n_expert ? c : -1;   // past n_expert: shorter than any list
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; w++) base += s_wsum[w];
    const int start = base + incl - c;
    if (tid < n_expert) s_cnt[tid] = start + before;
    if (b == 0) {
        if (tid < n_expert) group[tid] = start;
        if (tid == n_expert - 1) group[n_expert] = start + c;
    }
    // An expert's place in the launch: longer lists first, equal lengths by index.  Each block ranks its share of
    // the experts, 32 threads an expert (each against every 32nd length), instead of one block all of them with a
    // thread an expert: E^2 comparisons are most of what one block would spend on a pass's lists.
    {
        const int per = (n_expert + nb - 1) / nb, e0 = b * per;
        const int part = tid & 31;
        for (int eb = tid >> 5; eb < per; eb += 32) {
            const int e = e0 + eb;
            const bool live = e < n_expert;
            const int ce = live ? s_len[e] : 0;
            int rank = 0;
            for (int o = part; o < n_expert; o += 32) {
                const int co = s_len[o];
                rank += (co > ce || (co == ce && o < e)) ? 1 : 0;
            }
            rank += __shfl_xor(rank, 16, 64);
            rank += __shfl_xor(rank, 8, 64);
            rank += __shfl_xor(rank, 4, 64);
            rank += __shfl_xor(rank, 2, 64);
            rank += __shfl_xor(rank, 1, 64);
            if (live && part == 0) group[n_expert + 1 + n_pairs + rank] = e;
        }
    }
    __syncthreads();
    int32_t *list = group + n_expert + 1;
    const int lo = b * chunk, hi = lo + chunk < n_pairs ? lo + chunk : n_pairs;
    for (int i = lo + tid; i < hi; i += 1024) {
        const int e = topk[i];
        if (e >= 0 && e < n_expert) list[atomicAdd(&s_cnt[e], 1)] = (i / n_used) * (n_used + 1) + i % n_used;
    }
}

// Columns [col0, col0 + kSlab) of up to kTok listed rows (each a row of floats at rows_s[i]) into
// operand order: the fragment of (sub-block, part hi / lo, token tile) is 64 lanes x 16 bytes,
// lane = token in the tile + 16 * (k block of 8 columns), the eight columns in slot order
// [0, 2, 1, 3, 4, 6, 5, 7]; sxs[sub][token] is the sub-block's sum of x.
__device__ __forceinline__ void gather_slab(const float *const *rows_s, int m, int col0, char *frags, float *sxs) {
    constexpr int QPR = kSlab / 4;             // quads a row's slab
    constexpr int RPI = kThreads / QPR;        // rows an iteration of the block covers
    const int tid = threadIdx.x;
    const int c = 4 * (tid % QPR);
    const int sub = c >> 5, kb = (c & 31) >> 3, qh = (c & 7) >> 2;
    // six rows' quads are asked for before the first is used: two memory latencies a slab, not one a row
    constexpr int NI = kTok / RPI, NB = 6;
    static_assert(kTok % RPI == 0 && NI % NB == 0, "whole batches");
#pragma unroll 1
    for (int b0 = 0; b0 < NI; b0 += NB) {
        if (b0 * RPI >= m) break;
        float4 vv[NB];
#pragma unroll
        for (int it = 0; it < NB; it++) {
            const int i = (b0 + it) * RPI + tid / QPR;
            vv[it] = *reinterpret_cast<const float4 *>(rows_s[i < m ? i : 0] + col0 + c);
        }
#pragma unroll
        for (int it = 0; it < NB; it++) {
            const int i = (b0 + it) * RPI + tid / QPR;
            const bool on = i < m;
            float4 v = vv[it];
            if (!on) v = float4{0.f, 0.f, 0.f, 0.f};
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
                char *e = frags + static_cast<size_t>((sub * 2) * kTT + (i >> 4)) * kFrag + (kb * 16 + (i & 15)) * 16 + qh * 8;
                *reinterpret_cast<half4_t *>(e) = h;
                *reinterpret_cast<half4_t *>(e + kTT * kFrag) = l;
            }
        }
    }
}

// A wave's place in its R weight rows' streams: the header of the super-block it is in, the next
// super-block's header and the payload of the next 64-weight group, both on their way.
template <int R>
struct RowStream {
    uint4 hdr[R], hdr_next[R];
    uint2 q_next[R];
    // group G = 4 * super-block + g, clamped to the last one so that the loads are unconditional
    __device__ __forceinline__ void ask_group(const char *const (&rp)[R], int G, int G_last, int kb) {
        const int Gc = G < G_last ? G : G_last;
#pragma unroll
        for (int r = 0; r < R; r++)
            q_next[r] = *reinterpret_cast<const uint2 *>(rp[r] + static_cast<size_t>(Gc >> 2) * SHV_Q4K_BYTES + 16 + (Gc & 3) * 32 + kb * 8);
    }
    // A lane's 16 bytes of a PAIR of groups (pair Pg = groups 2 Pg, 2 Pg + 1: 64 payload bytes a row, one line's
    // worth in one load where two 8-byte loads of a group each took a half line apiece): lane (row, kb) holds bytes
    // 16 kb .. 16 kb + 15 of the pair, i.e. columns 16 (kb & 1) .. + 15 of group 2 Pg + (kb >> 1), low and high nibbles.
    uint4 pair_next[R];
    __device__ __forceinline__ void ask_pair(const char *const (&rp)[R], int Pg, int P_last, int kb) {
        const int Pc = Pg < P_last ? Pg : P_last;
#pragma unroll
        for (int r = 0; r < R; r++)
            pair_next[r] = *reinterpret_cast<const uint4 *>(rp[r] + static_cast<size_t>(Pc >> 1) * SHV_Q4K_BYTES + 16 + (Pc & 1) * 64 + kb * 16);
    }
    __device__ __forceinline__ void ask_header(const char *const (&rp)[R], int sb, int sb_last) {
        const int sc = sb < sb_last ? sb : sb_last;
#pragma unroll
        for (int r = 0; r < R; r++) hdr_next[r] = *reinterpret_cast<const uint4 *>(rp[r] + static_cast<size_t>(sc) * SHV_Q4K_BYTES);
    }
};

// The 64-weight groups [G0, G0 + NG) of R row tiles (lane rows at rp[r]) against the staged slab,
// whose first sub-block is the first of group G0:
// y[r][tt][j] += sum over those columns of W[row of tile r][.] * x[token 16 tt + 4 kb + j][.].
// A sub-block's eight weights per lane are formed once, as the whole numbers n * sc, and multiplied
// with every token tile; the matrix accumulators run over a super-block and take its d at its end,
// the min term is subtracted per sub-block: y = sum_sb d * (sum x * n * sc) - sum_sub dmin * m * sum(x).
template <int NG, int R, int SXS = kTok>
__device__ __forceinline__ void slab_times_tiles(const char *const (&rp)[R], RowStream<R> &st, int G0, int G_last, const char *frags,
                                                 const float *sxs, int lane, int n_tt, float4_t (&acc)[R][kTT], float4_t (&y)[R][kTT]) {
    const int kb = lane >> 4;
    const NibbleConsts nc = nibble_consts();
#pragma unroll 1
    for (int gi = 0; gi < NG; gi++) {
        const int G = G0 + gi, g = G & 3;
        uint2 q[R];
#pragma unroll
        for (int r = 0; r < R; r++) q[r] = st.q_next[r];
        st.ask_group(rp, G + 1, G_last, kb);
        uint32_t sc[R], mn[R];
        float dmin[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            q4k_group_scale_min(st.hdr[r], g, sc[r], mn[r]);
            dmin[r] = f16_bits_to_f32(st.hdr[r].x >> 16);
        }
#pragma unroll
        for (int hi = 0; hi < 2; hi++) {
            const int sub = gi * 2 + hi;
            half8_t b[R];
            float dm[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t q0 = q[r].x, q1 = q[r].y;
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                u32x4 v;
                if (hi == 0) {
                    v.x = ((q0 << 4) & nc.mask) | nc.one; v.y = ((q0 >> 4) & nc.mask) | nc.one;
                    v.z = ((q1 << 4) & nc.mask) | nc.one; v.w = ((q1 >> 4) & nc.mask) | nc.one;
                } else {
                    v.x = (q0 & nc.mask) | nc.one; v.y = ((q0 >> 8) & nc.mask) | nc.one;
                    v.z = (q1 & nc.mask) | nc.one; v.w = ((q1 >> 8) & nc.mask) | nc.one;
                }
                // the halves 64 + n become n * sc: whole numbers up to 15 * 63, exact in binary16 (as is
                // 64 * sc, should the two steps be fused), so one accumulator runs over the super-block
                const _Float16 s16 = static_cast<_Float16>(static_cast<float>(hi ? sc[r] >> 8 : sc[r] & 0xFFu));
                b[r] = (__builtin_bit_cast(half8_t, v) - static_cast<half8_t>(static_cast<_Float16>(64.f))) * static_cast<half8_t>(s16);
                dm[r] = dmin[r] * static_cast<float>(hi ? mn[r] >> 8 : mn[r] & 0xFFu);
            }
#pragma unroll
            for (int tt = 0; tt < kTT; tt++) {
                if (tt >= n_tt) break;
                const char *f = frags + static_cast<size_t>((sub * 2) * kTT + tt) * kFrag + lane * 16;
                const half8_t xh = *reinterpret_cast<const half8_t *>(f);
                const half8_t xl = *reinterpret_cast<const half8_t *>(f + kTT * kFrag);
                float sxv[4];
                if constexpr (SXS > 0) {
                    const float4 sx = *reinterpret_cast<const float4 *>(sxs + sub * SXS + 16 * tt + 4 * kb);
                    sxv[0] = sx.x, sxv[1] = sx.y, sxv[2] = sx.z, sxv[3] = sx.w;
                } else {
                    // the sub-block's sum of x per token, from the operands themselves: a product
                    // with ones leaves token 4 kb + j's sum in register j of every lane
                    const half8_t ones = static_cast<half8_t>(static_cast<_Float16>(1.f));
                    float4_t s4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, ones, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    s4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, ones, s4, 0, 0, 0);
                    sxv[0] = s4[0], sxv[1] = s4[1], sxv[2] = s4[2], sxv[3] = s4[3];
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    acc[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, b[r], acc[r][tt], 0, 0, 0);
                    acc[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, b[r], acc[r][tt], 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; j++) y[r][tt][j] = fmaf(-dm[r], sxv[j], y[r][tt][j]);
                }
            }
        }
        if (g == 3) {
            // the super-block ends: its sums take its d, the next one's header moves in
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float dd = f16_bits_to_f32(st.hdr[r].x);
#pragma unroll
                for (int tt = 0; tt < kTT; tt++) {
#pragma unroll
                    for (int j = 0; j < 4; j++) y[r][tt][j] = fmaf(dd, acc[r][tt][j], y[r][tt][j]);
                    acc[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
                }
            }
            // asked for only now: a header a super-block ahead costs sixteen registers these kernels do not have
            st.ask_header(rp, (G >> 2) + 1, G_last >> 2);
#pragma unroll
            for (int r = 0; r < R; r++) st.hdr[r] = st.hdr_next[r];
        }
    }
}

// All K columns of up to kTok listed rows against a wave's kTiles row tiles: the rows go through
// LDS a slab at a time, the weights of the next super-block are on their way while a slab is staged.
template <int K>
__device__ __forceinline__ void rows_times_tiles(const char *const (&rp)[kTiles], const float *const *rows_s, int m, char *frags, float *sxs,
                                                 int lane, float4_t (&y)[kTiles][kTT]) {
    constexpr int GROUPS = K / 64, NG = kSlab / 64;
    static_assert(K % kSlab == 0, "whole slabs");
    const int n_tt = (m + 15) >> 4;
#pragma unroll
    for (int r = 0; r < kTiles; r++)
#pragma unroll
        for (int tt = 0; tt < kTT; tt++) y[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t acc[kTiles][kTT];
#pragma unroll
    for (int r = 0; r < kTiles; r++)
#pragma unroll
        for (int tt = 0; tt < kTT; tt++) acc[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
    RowStream<kTiles> st;
    st.ask_header(rp, 0, GROUPS / 4 - 1);
#pragma unroll
    for (int r = 0; r < kTiles; r++) st.hdr[r] = st.hdr_next[r];
    st.ask_group(rp, 0, GROUPS - 1, lane >> 4);
#pragma unroll 1
    for (int sl = 0; sl < K / kSlab; sl++) {
        __syncthreads();   // the list is written / the slab before this one has been multiplied
        gather_slab(rows_s, m, sl * kSlab, frags, sxs);
        __syncthreads();
        slab_times_tiles<NG, kTiles>(rp, st, sl * NG, GROUPS - 1, frags, sxs, lane, n_tt, acc, y);
    }
}

// The same product over rows that a launch before this one has made into operands, a row's
// own bytes together (moe_stage_kernel): [row][sub-block][part hi, lo][block of 8 columns] x 16
// bytes, 128 bytes a sub-block, the eight columns in slot order.  A slab of 256 columns is 48
// fragments which the loads place in LDS themselves, a lane's 16 bytes each from the listed row it
// stands for (the four lanes of a row read 64 bytes in a line, the other part the line's other
// half), so staging costs no vector work and no registers, and the next slab is on its way while
// this one is multiplied.  Wave w asks for sub-block w of the slab: its two parts for every token
// tile.  The sub-blocks' sums of x come from the operands (slab_times_tiles with SXS 0).
// tok_s: the listed rows' numbers in the staged array.
// The masks and exponents of the two nibble positions a weight is read from.
struct NibbleMasks {
    uint32_t m0, m4;  // bits 0..3, 4..7 of both halves
    uint32_t o0, o4;  // the halves 1024, 64
};
__device__ __forceinline__ NibbleMasks nibble_masks() {
    NibbleMasks c;
    c.m0 = 0x000F000Fu, c.m4 = 0x00F000F0u;
    c.o0 = 0x64006400u, c.o4 = 0x54005400u;
    // opaque to the optimiser: a mask in a scalar register and an exponent in a vector one make (q & m) | o one instruction
    asm volatile("" : "+s"(c.m0), "+s"(c.m4));
    asm volatile("" : "+v"(c.o0), "+v"(c.o4));
    return c;
}

typedef const __attribute__((address_space(1))) void *global_ptr_t;
typedef __attribute__((address_space(3))) void *lds_ptr_t;
constexpr int kStWaves = kWaves;                 // waves of a block of the staged kernels: two such blocks share a compute unit, one's waits under the other's work
constexpr int kStThreads = kStWaves * 64;
constexpr int kStSubs = kStWaves;             // sub-blocks of a staged slab: one a wave
constexpr int kStQuarter = 1024 / (32 * kStSubs);  // slabs in the 1024 columns one min-term product covers
constexpr int kStSlab = 32 * kStSubs;
constexpr int kStFrags = kStSubs * 2 * kTT * kFrag;
constexpr int kStSubBytes = 128;              // a row's sub-block: 2 parts x 4 column blocks x 16 bytes
constexpr int kStSumFrags = kTT * 2 * kFrag;   // the sums of a quarter of the columns (four super-blocks): [token tile][part]
constexpr int kStMinHdrs = kStWaves * kTiles * kFrag;   // every lane's row header of its super-block of the quarter, a wave's own
constexpr size_t kStagedLds = 2 * static_cast<size_t>(kStFrags) + 2 * kStSumFrags + kStMinHdrs + 2 * kTok * 4;

// After the rows, every row's sums of x over its sub-blocks, as operands too: [row][super-block]
// x 32 bytes, the eight sums' binary16 values and then what those leave.
__host__ __device__ constexpr size_t staged_sums_offset(int rows, int k) { return static_cast<size_t>(rows) * (k / 32) * 128; }
__host__ __device__ constexpr size_t staged_bytes(int rows, int k) { return staged_sums_offset(rows, k) + static_cast<size_t>(rows) * (k / 256) * 32; }

// grid: (k / 1024, rows), 256 threads, a quad of columns each.
__global__ __launch_bounds__(256) void moe_stage_kernel(const float *x, int x_stride, int k, int rows, char *staged) {
    const int t = blockIdx.y, c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= k) return;
    const float4 v = *reinterpret_cast<const float4 *>(x + static_cast<size_t>(t) * x_stride + c);
    const float o[4] = {v.x, v.z, v.y, v.w};
    half4_t h, l;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const _Float16 hi = static_cast<_Float16>(o[j]);
        h[j] = hi;
        l[j] = static_cast<_Float16>(o[j] - static_cast<float>(hi));
    }
    char *e = staged + (static_cast<size_t>(t) * (k / 32) + (c >> 5)) * kStSubBytes + ((c & 31) >> 3) * 16 + ((c & 7) >> 2) * 8;
    *reinterpret_cast<half4_t *>(e) = h;
    *reinterpret_cast<half4_t *>(e + 64) = l;
    // the sub-block's sum: eight neighbouring lanes (k is a multiple of 32, so they are all here)
    float sum = (v.x + v.y) + (v.z + v.w);
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    sum += __shfl_xor(sum, 4, 64);
    if ((c & 31) == 0) {
        const _Float16 hi = static_cast<_Float16>(sum);
        _Float16 *sp = reinterpret_cast<_Float16 *>(staged + staged_sums_offset(rows, k) + (static_cast<size_t>(t) * (k / 256) + (c >> 8)) * 32) + ((c >> 5) & 7);
        sp[0] = hi;
        sp[8] = static_cast<_Float16>(sum - static_cast<float>(hi));
    }
}

template <int K>
__device__ __forceinline__ void ask_staged_slab(const char *staged, const int32_t *tok_s, int m, int n_tt, int sl, char *buf, int lane, int wave) {
    // Wave w asks for product w of the slab's eight: pair w / 4 of its groups, the pair's low (0) or high (1) nibbles,
    // the first or second eight of a lane's sixteen bytes.  Its lane (token, kb) stands where the weights' lane
    // (row, kb) does: sub-block 2 (group of the lane) + nibble, columns 16 (kb & 1) + 8 (half) .. + 7 of it.
    const int n = lane & 15, kb = lane >> 4;
    const int pr = wave >> 2, hi = (wave >> 1) & 1, half = wave & 1;
    const int sg = sl * kStSubs + 4 * pr + 2 * (kb >> 1) + hi;  // the sub-block this lane's eight columns lie in
    const int cb = 2 * (kb & 1) + half;                          // and which eight of its 32
#pragma unroll
    for (int tt = 0; tt < kTT; tt++) {
        if (tt >= n_tt) break;
        const int i = 16 * tt + n;
        const int t = tok_s[i < m ? i : 0];  // a column past the list repeats the first row; nobody reads its products
        const char *g = staged + (static_cast<size_t>(t) * (K / 32) + sg) * kStSubBytes + cb * 16;
        char *f = buf + ((wave * 2) * kTT + tt) * kFrag;
        __builtin_amdgcn_global_load_lds((global_ptr_t)(g), (lds_ptr_t)(f), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((global_ptr_t)(g + 64), (lds_ptr_t)(f + kTT * kFrag), 16, 0, 0);
    }
}

// The sums of x of columns [1024 q, 1024 q + 1024), four super-blocks, as the operands of the
// min term: fragment (token tile, part), lane = token in the tile + 16 * (super-block of the four).
// The waves share the fragments out.
template <int K>
__device__ __forceinline__ void ask_staged_sums(const char *sums, const int32_t *tok_s, int m, int n_tt, int q, char *buf, int lane, int wave) {
    const int n = lane & 15, kb = lane >> 4;
    const int sb = 4 * q + kb < K / 256 ? 4 * q + kb : K / 256 - 1;  // past the row: a real sum against a zero weight
    for (int f = wave; f < 2 * n_tt; f += kStWaves) {
        const int tt = f >> 1, part = f & 1;
        const int i = 16 * tt + n;
        const int t = tok_s[i < m ? i : 0];
        const char *g = sums + (static_cast<size_t>(t) * (K / 256) + sb) * 32 + part * 16;
        __builtin_amdgcn_global_load_lds((global_ptr_t)(g), (lds_ptr_t)(buf + f * kFrag), 16, 0, 0);
    }
}

// The headers min_terms reads, on their way a slab ahead: lane (row, kb) asks for its R rows'
// headers of super-block 4 q + kb, into the wave's own kTiles fragments at hbuf.
template <int K, int R>
__device__ __forceinline__ void ask_min_headers(const char *const (&rp)[R], int q, char *hbuf, int lane) {
    const int sb = 4 * q + (lane >> 4) < K / 256 ? 4 * q + (lane >> 4) : 0;
#pragma unroll
    for (int r = 0; r < R; r++)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(rp[r] + static_cast<size_t>(sb) * SHV_Q4K_BYTES), (lds_ptr_t)(hbuf + r * kFrag), 16, 0, 0);
}

// y -= sum over the quarter's sub-blocks of dmin * m * sum(x), on the matrix cores: lane (row,
// kb) forms its row's eight -dmin * m of super-block 4 q + kb as two halves each (the product has
// 17 significant bits), the tokens' sums come as two halves too, and three products (the small
// halves' one is below float32's last bit) add to the accumulators what the vector units would
// subtract sub-block by sub-block.
template <int K, int R, int NTT>
__device__ __forceinline__ void min_terms(int q, const char *sfr, const char *hbuf, int lane, float4_t (&y)[R][NTT]) {
    const int kb = lane >> 4;
    const bool on = 4 * q + kb < K / 256;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const uint4 h = *reinterpret_cast<const uint4 *>(hbuf + r * kFrag + lane * 16);
        const float nd = on ? -f16_bits_to_f32(h.x >> 16) : 0.f;
        const uint32_t m03 = h.z & 0x3F3F3F3Fu, m47 = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
        half8_t bh, bl;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float p = nd * static_cast<float>(((j < 4 ? m03 : m47) >> (8 * (j & 3))) & 0xFFu);
            const _Float16 hi = static_cast<_Float16>(p);
            bh[j] = hi;
            bl[j] = static_cast<_Float16>(p - static_cast<float>(hi));
        }
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) {
            const half8_t sh = *reinterpret_cast<const half8_t *>(sfr + (tt * 2) * kFrag + lane * 16);
            const half8_t sl = *reinterpret_cast<const half8_t *>(sfr + (tt * 2 + 1) * kFrag + lane * 16);
            y[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sh, bh, y[r][tt], 0, 0, 0);
            y[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sl, bh, y[r][tt], 0, 0, 0);
            y[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sh, bl, y[r][tt], 0, 0, 0);
        }
    }
}

// slab_times_tiles for staged rows and NTT token tiles, without the min term (min_terms has it):
// the (sub-block, token tile) steps of a 64-weight group run as one pipeline in which the
// fragments of the step after this one are read from LDS before this step's products are issued,
// so no product waits for an LDS read.
template <int NG, int R, int NTT, typename Ask>
__device__ __forceinline__ void staged_slab_times_tiles(const char *const (&rp)[R], RowStream<R> &st, int G0, int G_last, const char *frags, const char *hbuf,
                                                        int lane, float4_t (&acc)[R][NTT], float4_t (&y)[R][NTT], Ask &&ask_next) {
    static_assert(NG == 4, "a slab is one super-block: its header is read once, where the slab begins");
    const int kb = lane >> 4;
    const NibbleMasks nc = nibble_masks();
    // The rows' headers of this super-block are in LDS already: min_terms' loads brought the quarter's (lane (row, kb)
    // holds super-block 4 q + kb's), a slab and more ahead.  Asked for from memory where a super-block ends they were
    // waited for where the next begins; kept in registers they cost sixteen, so each pair of groups reads them again.
    typedef uint32_t u32x4_lds __attribute__((ext_vector_type(4)));
    const __attribute__((address_space(3))) char *hl = (const __attribute__((address_space(3))) char *)(hbuf) + ((lane & 15) + 16 * ((G0 >> 2) & 3)) * 16;
    // LDS addresses are 32 bits wide: kept as such, a fragment's place costs no 64-bit arithmetic
    typedef const __attribute__((address_space(3))) char *lds_bytes_t;
    typedef const __attribute__((address_space(3))) half8_t *lds_half8_t;
    const lds_bytes_t fl = (lds_bytes_t)(frags) + lane * 16;
    half8_t nh = *(lds_half8_t)(fl), nl = *(lds_half8_t)(fl + kTT * kFrag);
#pragma unroll 1
    for (int pi = 0; pi < NG / 2; pi++) {
        const int Pg = (G0 >> 1) + pi;                                          // the pair of groups: 2 Pg, 2 Pg + 1
        const lds_bytes_t fp = fl + pi * (8 * kTT * kFrag);                     // this pair's four products
        const lds_bytes_t fn = pi + 1 < NG / 2 ? fp + 8 * kTT * kFrag : fl;    // the pair after it (the slab's first again past its last, unused)
        uint4 q[R];
#pragma unroll
        for (int r = 0; r < R; r++) q[r] = st.pair_next[r];
        // the pair's bytes are here: only now the loads that nothing in this slab waits for (a
        // wait for loaded registers also waits for every load issued before them)
        asm volatile("" : "+v"(q[0].x), "+v"(q[1].x), "+v"(q[2].x), "+v"(q[3].x));
        // this lane's group of the pair, within the super-block: its scales, and the rows' d
        const int g = (2 * Pg + (kb >> 1)) & 3;
        uint32_t sc[R], dd16[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const u32x4_lds h = *reinterpret_cast<const __attribute__((address_space(3))) u32x4_lds *>(hl + r * kFrag);
            uint32_t mn;
            q4k_group_scale_min(make_uint4(h.x, h.y, h.z, h.w), g, sc[r], mn);
            dd16[r] = h.x;
        }
        // read to the end before the loads of the quarter after this one may be asked for (they land in the same place)
        asm volatile("" : "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]), "+v"(dd16[0]), "+v"(dd16[1]), "+v"(dd16[2]), "+v"(dd16[3]));
        // the next pair's bytes first: a wait for them then does not wait for the slab's loads behind them
        st.ask_pair(rp, Pg + 1, G_last >> 1, kb);
        ask_next(pi);
        __builtin_amdgcn_sched_barrier(0);  // the loads stay up here, a pair ahead of their use
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int hi = u >> 1;  // products 0, 1: the low nibbles of bytes 0..7 and 8..15; 2, 3: the high nibbles
            half8_t b[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t q0 = (u & 1) ? q[r].z : q[r].x, q1 = (u & 1) ? q[r].w : q[r].y;
                typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                // A nibble in the low bits of a half's mantissa reads, under the right exponent, as
                // C + n: bits 0..3 under 1024's, bits 4..7 under 64's (the odd bytes' nibbles take
                // one shift down there).  One fused multiply-add then makes (C + n) * sc - C * sc =
                // n * sc: a whole number up to 15 * 63, exact in binary16, as are C * sc.
                const _Float16 s1 = static_cast<_Float16>(static_cast<float>(hi ? sc[r] >> 8 : sc[r] & 0xFFu));
                const half2_t s2 = {s1, s1};
                half2_t w[4], c[4];
                if (hi == 0) {
                    w[0] = __builtin_bit_cast(half2_t, (q0 & nc.m0) | nc.o0); w[1] = __builtin_bit_cast(half2_t, ((q0 >> 4) & nc.m4) | nc.o4);
                    w[2] = __builtin_bit_cast(half2_t, (q1 & nc.m0) | nc.o0); w[3] = __builtin_bit_cast(half2_t, ((q1 >> 4) & nc.m4) | nc.o4);
                    c[0] = c[2] = s2 * static_cast<half2_t>(static_cast<_Float16>(-1024.f));
                    c[1] = c[3] = s2 * static_cast<half2_t>(static_cast<_Float16>(-64.f));
                } else {
                    w[0] = __builtin_bit_cast(half2_t, (q0 & nc.m4) | nc.o4); w[1] = __builtin_bit_cast(half2_t, ((q0 >> 8) & nc.m4) | nc.o4);
                    w[2] = __builtin_bit_cast(half2_t, (q1 & nc.m4) | nc.o4); w[3] = __builtin_bit_cast(half2_t, ((q1 >> 8) & nc.m4) | nc.o4);
                    c[0] = c[1] = c[2] = c[3] = s2 * static_cast<half2_t>(static_cast<_Float16>(-64.f));
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const half2_t p = __builtin_elementwise_fma(w[i], s2, c[i]);
                    b[r][2 * i] = p[0];
                    b[r][2 * i + 1] = p[1];
                }
            }
            // the matrix instructions of a step win the SIMD's issue slot over the other wave's vector
            // instructions, which then run under them instead of between them
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int tt = 0; tt < NTT; tt++) {
                const half8_t xh = nh, xl = nl;
                // the step after this one: the next token tile, the next product's first, or (past
                // the slab's last) the first again, unused
                const int ntt = tt + 1 < NTT ? tt + 1 : 0;
                const lds_bytes_t f = tt + 1 < NTT ? fp + ((u * 2) * kTT + ntt) * kFrag : (u < 3 ? fp + ((u + 1) * 2) * kTT * kFrag : fn);
                nh = *(lds_half8_t)(f);
                nl = *(lds_half8_t)(f + kTT * kFrag);
#pragma unroll
                for (int r = 0; r < R; r++) acc[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, b[r], acc[r][tt], 0, 0, 0);
#pragma unroll
                for (int r = 0; r < R; r++) acc[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, b[r], acc[r][tt], 0, 0, 0);
            }
            __builtin_amdgcn_s_setprio(0);
        }
        if (Pg & 1) {
            // the super-block ends: its sums take its d
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float dd = f16_bits_to_f32(dd16[r]);
#pragma unroll
                for (int tt = 0; tt < NTT; tt++) {
#pragma unroll
                    for (int j = 0; j < 4; j++) y[r][tt][j] = fmaf(dd, acc[r][tt][j], y[r][tt][j]);
                    acc[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
                }
            }
        }
    }
}

template <int K, int NTT>
__device__ __forceinline__ void staged_times_tiles(const char *const (&rp)[kTiles], const char *staged, const char *sums, const int32_t *tok_s, int m,
                                                   char *bufs, int lane, int wave, float4_t (&y)[kTiles][NTT]) {
    constexpr int GROUPS = K / 64, NG = kStSlab / 64, SLABS = K / kStSlab;
    static_assert(K % kStSlab == 0, "whole slabs");
#pragma unroll
    for (int r = 0; r < kTiles; r++)
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) y[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float4_t acc[kTiles][NTT];
#pragma unroll
    for (int r = 0; r < kTiles; r++)
#pragma unroll
        for (int tt = 0; tt < NTT; tt++) acc[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
    char *sum_bufs = bufs + 2 * kStFrags;
    char *hbuf = sum_bufs + 2 * kStSumFrags + wave * (kTiles * kFrag);
    ask_staged_slab<K>(staged, tok_s, m, NTT, 0, bufs, lane, wave);
    ask_staged_sums<K>(sums, tok_s, m, NTT, 0, sum_bufs, lane, wave);
    ask_min_headers<K, kTiles>(rp, 0, hbuf, lane);
    RowStream<kTiles> st;
    st.ask_pair(rp, 0, GROUPS / 2 - 1, lane >> 4);
#pragma unroll 1
    for (int sl = 0; sl < SLABS; sl++) {
        char *buf = bufs + (sl & 1) * kStFrags;
        // this wave's loads have landed, then everybody's: the slab is whole, and the buffer the
        // next one goes to has been read to its end
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        if (sl % kStQuarter == 0) min_terms<K, kTiles, NTT>(sl / kStQuarter, sum_bufs + ((sl / kStQuarter) & 1) * kStSumFrags, hbuf, lane, y);
        staged_slab_times_tiles<NG, kTiles, NTT>(rp, st, sl * NG, GROUPS - 1, buf, hbuf, lane, acc, y, [&](int pi) {
            // the next slab at the slab's first pair of groups; the next quarter's sums and headers at its second, behind
            // the last reading of this quarter's headers
            if (sl + 1 < SLABS) {
                if (pi == 0) ask_staged_slab<K>(staged, tok_s, m, NTT, sl + 1, bufs + ((sl + 1) & 1) * kStFrags, lane, wave);
                if (pi == 1 && (sl + 1) % kStQuarter == 0) {
                    const int q = (sl + 1) / kStQuarter;
                    ask_staged_sums<K>(sums, tok_s, m, NTT, q, sum_bufs + (q & 1) * kStSumFrags, lane, wave);
                    ask_min_headers<K, kTiles>(rp, q, hbuf, lane);
                }
            }
        });
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
__device__ __forceinline__ Unit unit_of(int b, int parts, int n_expert, int n_tok, int n_used, const int32_t *group) {
    Unit u;
    const int shared = parts * ((n_tok + kTok - 1) / kTok);  // the shared expert's blocks come first: all of them have work
    if (b >= shared) {
        b -= shared;
        u.expert = group[n_expert + 1 + n_tok * n_used + b / parts];
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

struct Staging {
    char *frags;
    float *sxs;
    const float **rows_s;
    int32_t *pair_s;
    __device__ __forceinline__ explicit Staging(char *smem) {
        frags = smem;
        sxs = reinterpret_cast<float *>(smem + static_cast<size_t>(kSlabSubs) * 2 * kTT * kFrag);
        rows_s = reinterpret_cast<const float **>(sxs + kSlabSubs * kTok);
        pair_s = reinterpret_cast<int32_t *>(rows_s + kTok);
    }
};
constexpr size_t kGroupedLds = static_cast<size_t>(kSlabSubs) * 2 * kTT * kFrag + static_cast<size_t>(kSlabSubs) * kTok * 4 + kTok * sizeof(float *) + kTok * 4;

// Where the grouped down projection finds a pair's act row when it comes as operands: the row's
// own 4 * ffn bytes of act in the staged layout, and its sub-blocks' sums in the library's scratch.
__host__ __device__ constexpr size_t packed_sums_bytes(long long pairs, int ffn) { return static_cast<size_t>(pairs) * (ffn / 256) * 32; }

// One pass of a block of the gate/up kernel over up to 16 NTT of its tokens: the products, SwiGLU, act out
// (as floats, or, packed, as the operands the grouped down projection stages from).
template <int K, int NTT>
__device__ __forceinline__ void up_pass(const shv_moe_up_args &a, const char *const (&rp)[kTiles], const char *staged, const int32_t *tok_s,
                                        const int32_t *pair_s, int m, char *smem, int row, char *act_sums) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, kb = lane >> 4, n = lane & 15;
    float4_t y[kTiles][NTT];
    staged_times_tiles<K, NTT>(rp, staged, staged + staged_sums_offset(a.n_tok, K), tok_s, m, smem, lane, wave, y);
    // this wave's 32 columns are one sub-block of the down projection's rows
    const int sub = row >> 5;   // row = 32 * sub + n
    // column 16 r + n of the sub-block: block of 8 columns 2 r + n / 8, slot of [0, 2, 1, 3, 4, 6, 5, 7]
    const int p8 = n & 7, slot = (p8 & 4) | ((p8 & 1) << 1) | ((p8 & 2) >> 1);
#pragma unroll
    for (int tt = 0; tt < NTT; tt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = 16 * tt + 4 * kb + j;
            float v[2];
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const float gv = y[r][tt][j];
                v[r] = gv * sigmoid_exact(gv) * y[2 + r][tt][j];
            }
            if (!a.act_packed) {
                if (i < m) {
#pragma unroll
                    for (int r = 0; r < 2; r++) a.act[static_cast<size_t>(pair_s[i]) * a.ffn + row + 16 * r] = v[r];
                }
            } else {
                // the sub-block's sum: both tiles, the 16 lanes of the token
                float sum = v[0] + v[1];
                sum += __shfl_xor(sum, 1, 64);
                sum += __shfl_xor(sum, 2, 64);
                sum += __shfl_xor(sum, 4, 64);
                sum += __shfl_xor(sum, 8, 64);
                if (i < m) {
                    const size_t pair = static_cast<size_t>(pair_s[i]);
                    char *e = reinterpret_cast<char *>(a.act) + (pair * (a.ffn / 32) + sub) * kStSubBytes + (n >> 3) * 16 + slot * 2;
#pragma unroll
                    for (int r = 0; r < 2; r++) {
                        const _Float16 hi = static_cast<_Float16>(v[r]);
                        *reinterpret_cast<_Float16 *>(e + r * 32) = hi;
                        *reinterpret_cast<_Float16 *>(e + r * 32 + 64) = static_cast<_Float16>(v[r] - static_cast<float>(hi));
                    }
                    if (n == 0) {
                        const _Float16 hi = static_cast<_Float16>(sum);
                        _Float16 *sp = reinterpret_cast<_Float16 *>(act_sums + (pair * (a.ffn / 256) + (sub >> 3)) * 32) + (sub & 7);
                        sp[0] = hi;
                        sp[8] = static_cast<_Float16>(sum - static_cast<float>(hi));
                    }
                }
            }
        }
}

// grid: n_expert * parts + parts * ceil(n_tok / 48) blocks of 8 waves, parts = ffn / 256; K = n_embd.
// A part is 256 gate rows and the same 256 up rows = 16 + 16 tiles; wave w takes gate tiles 2w and
// 2w + 1 and the up tiles of the same rows, so SwiGLU stays in registers.
template <int K>
__global__ __launch_bounds__(kStThreads, 2) void moe_up_grouped_kernel(shv_moe_up_args a, const char *staged, char *act_sums) {
    extern __shared__ __align__(16) char smem[];
    // the two slab buffers, then the listed rows' pair and token numbers
    int32_t *pair_s = reinterpret_cast<int32_t *>(smem + 2 * kStFrags + 2 * kStSumFrags + kStMinHdrs);
    int32_t *tok_s = pair_s + kTok;
    const int32_t *group = a.group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15;
    const int parts = a.ffn / (32 * kStWaves);
    const Unit u = unit_of(blockIdx.x, parts, a.n_expert, a.n_tok, a.n_used, group);
    if (u.count <= 0) return;
    const size_t row_bytes = static_cast<size_t>(K / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES;
    const int row = u.part * (32 * kStWaves) + wave * 32 + n;   // this lane's first row of the expert, gate and up alike; its second is 16 on
    const size_t wrow = static_cast<size_t>(u.expert < 0 ? 0 : u.expert) * a.ffn + row;
    const char *gp = static_cast<const char *>(u.expert < 0 ? a.gate_sh : a.gate_exps) + wrow * row_bytes;
    const char *up = static_cast<const char *>(u.expert < 0 ? a.up_sh : a.up_exps) + wrow * row_bytes;
    const char *rp[kTiles] = {gp, gp + 16 * row_bytes, up, up + 16 * row_bytes};
    for (int t0 = 0; t0 < u.count; t0 += kTok) {
        const int m = u.count - t0 < kTok ? u.count - t0 : kTok;
        if (tid < m) {
            const int pair = u.expert < 0 ? (u.first + t0 + tid) * (a.n_used + 1) + a.n_used : group[a.n_expert + 1 + u.first + t0 + tid];
            pair_s[tid] = pair;
            tok_s[tid] = pair / (a.n_used + 1);
        }
        __syncthreads();   // the list is written; the pass before this one has read its last slab
        const int n_tt = (m + 15) >> 4;
        if (n_tt == 3) up_pass<K, 3>(a, rp, staged, tok_s, pair_s, m, smem, row, act_sums);
        else if (n_tt == 2) up_pass<K, 2>(a, rp, staged, tok_s, pair_s, m, smem, row, act_sums);
        else up_pass<K, 1>(a, rp, staged, tok_s, pair_s, m, smem, row, act_sums);
        __syncthreads();   // the list is read to the end before the next one replaces it
    }
}

// grid: n_expert * parts + parts * ceil(n_tok / 48) blocks, parts = n_embd / 512: a part is 512
// output rows = 32 tiles, wave w takes tiles 4w .. 4w + 3.  K = ffn.
template <int K>
__global__ __launch_bounds__(kThreads) void moe_down_grouped_kernel(shv_moe_down_args a) {
    extern __shared__ __align__(16) char smem[];
    const Staging st(smem);
    const int32_t *group = a.group;
    float *pairout = a.pairs;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int parts = a.n_embd / 512;
    const Unit u = unit_of(blockIdx.x, parts, a.n_expert, a.n_tok, a.n_used, group);
    if (u.count <= 0) return;
    const size_t row_bytes = static_cast<size_t>(K / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES;
    const int row0 = u.part * 512 + wave * 64 + n;
    const char *base = static_cast<const char *>(u.expert < 0 ? a.down_sh : a.down_exps) +
                       (static_cast<size_t>(u.expert < 0 ? 0 : u.expert) * a.n_embd + row0) * row_bytes;
    const char *rp[kTiles] = {base, base + 16 * row_bytes, base + 32 * row_bytes, base + 48 * row_bytes};
    for (int t0 = 0; t0 < u.count; t0 += kTok) {
        const int m = u.count - t0 < kTok ? u.count - t0 : kTok;
        if (tid < m) {
            const int pair = u.expert < 0 ? (u.first + t0 + tid) * (a.n_used + 1) + a.n_used : group[a.n_expert + 1 + u.first + t0 + tid];
            st.pair_s[tid] = pair;
            st.rows_s[tid] = a.act + static_cast<size_t>(pair) * K;
        }
        float4_t y[kTiles][kTT];
        rows_times_tiles<K>(rp, st.rows_s, m, st.frags, st.sxs, lane, y);
#pragma unroll
        for (int tt = 0; tt < kTT; tt++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = 16 * tt + 4 * kb + j;
                if (i < m) {
                    float *dst = pairout + static_cast<size_t>(st.pair_s[i]) * a.n_embd + row0;
#pragma unroll
                    for (int r = 0; r < kTiles; r++) dst[16 * r] = y[r][tt][j];
                }
            }
        __syncthreads();
    }
}

// One pass of a block of the staged down kernel: the products of up to 16 NTT listed pairs, raw, to pairs[pair].
template <int K, int NTT>
__device__ __forceinline__ void down_pass(const shv_moe_down_args &a, const char *const (&rp)[kTiles], const char *act_sums, const int32_t *pair_s,
                                          int m, char *smem, int row0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, kb = lane >> 4;
    float4_t y[kTiles][NTT];
    staged_times_tiles<K, NTT>(rp, reinterpret_cast<const char *>(a.act), act_sums, pair_s, m, smem, lane, wave, y);
#pragma unroll
    for (int tt = 0; tt < NTT; tt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = 16 * tt + 4 * kb + j;
            if (i < m) {
                float *dst = a.pairs + static_cast<size_t>(pair_s[i]) * a.n_embd + row0;
#pragma unroll
                for (int r = 0; r < kTiles; r++) dst[16 * r] = y[r][tt][j];
            }
        }
}

// The down projection over act rows that the gate/up kernel left as operands (act_packed): the
// same blocks and tiles as moe_down_grouped_kernel, the rows staged by the loads themselves.
template <int K>
__global__ __launch_bounds__(kStThreads, 2) void moe_down_staged_kernel(shv_moe_down_args a, const char *act_sums) {
    extern __shared__ __align__(16) char smem[];
    int32_t *pair_s = reinterpret_cast<int32_t *>(smem + 2 * kStFrags + 2 * kStSumFrags + kStMinHdrs);
    const int32_t *group = a.group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15;
    const int parts = a.n_embd / (64 * kStWaves);
    const Unit u = unit_of(blockIdx.x, parts, a.n_expert, a.n_tok, a.n_used, group);
    if (u.count <= 0) return;
    const size_t row_bytes = static_cast<size_t>(K / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES;
    const int row0 = u.part * (64 * kStWaves) + wave * 64 + n;
    const char *base = static_cast<const char *>(u.expert < 0 ? a.down_sh : a.down_exps) +
                       (static_cast<size_t>(u.expert < 0 ? 0 : u.expert) * a.n_embd + row0) * row_bytes;
    const char *rp[kTiles] = {base, base + 16 * row_bytes, base + 32 * row_bytes, base + 48 * row_bytes};
    for (int t0 = 0; t0 < u.count; t0 += kTok) {
        const int m = u.count - t0 < kTok ? u.count - t0 : kTok;
        if (tid < m) pair_s[tid] = u.expert < 0 ? (u.first + t0 + tid) * (a.n_used + 1) + a.n_used : group[a.n_expert + 1 + u.first + t0 + tid];
        __syncthreads();   // the list is written; the pass before this one has read its last slab
        const int n_tt = (m + 15) >> 4;
        if (n_tt == 3) down_pass<K, 3>(a, rp, act_sums, pair_s, m, smem, row0);
        else if (n_tt == 2) down_pass<K, 2>(a, rp, act_sums, pair_s, m, smem, row0);
        else down_pass<K, 1>(a, rp, act_sums, pair_s, m, smem, row0);
        __syncthreads();   // the list is read to the end before the next one replaces it
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

// The per-expert lists of a pass: one block for short passes of few experts, kGroupBlocks in two launches from 2048
// pairs or 128 experts on (ranking the experts by length is E^2 comparisons, a block's share of them a sixteenth)
// (their counts meet in the library's scratch, which nothing else on the stream is using between the two).
int launch_group(shv_ctx *ctx, const int32_t *topk, int n_tok, int n_used, int n_expert, int32_t *group) {
    const int n_pairs = n_tok * n_used;
    if ((n_pairs < 2048 && n_expert < 128) || !ctx->gemm_part || ctx->moe_group_one_block) {
        SHV_LAUNCH(ctx, moe_group_kernel, dim3(1), dim3(1024), 0, topk, n_tok, n_used, n_expert, group);
        return SHV_OK;
    }
    static_assert(static_cast<size_t>(kGroupBlocks) * kMaxExperts * 4 <= static_cast<size_t>(shv_ctx::kGemmPartBytes), "the blocks' counts fit the scratch");
    int32_t *counts = reinterpret_cast<int32_t *>(ctx->gemm_part);
    const int chunk = (n_pairs + kGroupBlocks - 1) / kGroupBlocks;
    SHV_LAUNCH(ctx, moe_group_count_kernel, dim3(kGroupBlocks), dim3(1024), 0, topk, n_pairs, chunk, n_expert, counts);
    SHV_LAUNCH(ctx, moe_group_place_kernel, dim3(kGroupBlocks), dim3(1024), 0, topk, n_pairs, chunk, n_used, n_expert, counts, group);
    return SHV_OK;
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
    return a.group && !a.logits && shv_aligned16(a.xn) && shapes_covered(ctx, a.n_tok, a.n_embd, a.ffn, a.n_used, a.n_expert) && ctx->gemm_stage &&
           staged_bytes(a.n_tok, a.n_embd) <= static_cast<size_t>(shv_ctx::kGemmStageBytes);
}

bool shv_moe_down_grouped_covers(const shv_ctx *ctx, const shv_moe_down_args &a) {
    return a.group && a.pairs && shv_aligned16(a.act) && shv_aligned16(a.pairs) && shapes_covered(ctx, a.n_tok, a.n_embd, a.ffn, a.n_used, a.n_expert);
}

// Lists, the rows as operands, then the grouped gate/up products.
int shv_launch_moe_up_grouped(shv_ctx *ctx, const shv_moe_up_args &a) {
    // refused before anything is enqueued: an error return leaves no half pass on the stream
    SHV_REQUIRE(!a.act_packed || (ctx->gemm_part && packed_sums_bytes(static_cast<long long>(a.n_tok) * (a.n_used + 1), a.ffn) <= static_cast<size_t>(shv_ctx::kGemmPartBytes)),
                "moe_up: %d rows are too many for act_packed", a.n_tok);
    if (const int rc = launch_group(ctx, a.topk, a.n_tok, a.n_used, a.n_expert, a.group); rc != SHV_OK) return rc;
    SHV_LAUNCH(ctx, moe_stage_kernel, dim3((a.n_embd + 1023) / 1024, a.n_tok), dim3(256), 0, a.xn, a.n_embd, a.n_embd, a.n_tok, ctx->gemm_stage);
    constexpr size_t lds = kStagedLds;
    static const int raised = raise_lds(&moe_up_grouped_kernel<2048>, lds);
    if (raised != SHV_OK) return raised;
    const int parts = a.ffn / (32 * kStWaves), tiles = (a.n_tok + kTok - 1) / kTok;
    SHV_LAUNCH(ctx, moe_up_grouped_kernel<2048>, dim3(a.n_expert * parts + parts * tiles), dim3(kStThreads), lds, a, static_cast<const char *>(ctx->gemm_stage),
               reinterpret_cast<char *>(ctx->gemm_part));
    ctx->moe_stamp = {a.topk, a.group, a.act, a.n_tok, a.n_used, true, a.act_packed != 0};
    return SHV_OK;
}

// The down projection makes its own lists from the same selection (the gate/up products may have
// gone another road: banks of other types), writes every pair's products to the caller's `pairs`
// and folds them per token in slot order.
int shv_launch_moe_down_grouped(shv_ctx *ctx, const shv_moe_down_args &a) {
    SHV_REQUIRE(a.n_embd % 4 == 0 && a.out_stride % 4 == 0 && shv_aligned16(a.out) &&
                    (!a.residual || (a.res_stride % 4 == 0 && shv_aligned16(a.residual))),
                "moe_down: the grouped path moves 16 bytes at a time");
    // the lists are this pass's only if the grouped gate/up launch of this very pass made them
    const shv_ctx::MoeStamp &st = ctx->moe_stamp;
    const bool lists = a.group_ready && st.grouped && st.topk == a.topk && st.group == a.group && st.n_tok == a.n_tok && st.n_used == a.n_used;
    SHV_REQUIRE(!a.act_packed || (lists && st.packed && st.act == a.act && ctx->gemm_part),
                "moe_down: act_packed, but the shv_moe_up before this call did not leave act as operands for this pass");
    if (!lists) {
        if (const int rc = launch_group(ctx, a.topk, a.n_tok, a.n_used, a.n_expert, const_cast<int32_t *>(a.group)); rc != SHV_OK) return rc;
    }
    const int parts = a.n_embd / 512, tiles = (a.n_tok + kTok - 1) / kTok;
    if (a.act_packed) {
        constexpr size_t lds = kStagedLds;
        static const int raised = raise_lds(&moe_down_staged_kernel<512>, lds);
        if (raised != SHV_OK) return raised;
        static_assert(64 * kStWaves == 512, "a part is 512 rows");
        SHV_LAUNCH(ctx, moe_down_staged_kernel<512>, dim3(a.n_expert * parts + parts * tiles), dim3(kStThreads), lds, a, reinterpret_cast<const char *>(ctx->gemm_part));
    } else {
        constexpr size_t lds = kGroupedLds;
        static const int raised = raise_lds(&moe_down_grouped_kernel<512>, lds);
        if (raised != SHV_OK) return raised;
        SHV_LAUNCH(ctx, moe_down_grouped_kernel<512>, dim3(a.n_expert * parts + parts * tiles), dim3(kThreads), lds, a);
    }
    SHV_LAUNCH(ctx, moe_combine_kernel, dim3((a.n_embd + 1023) / 1024, a.n_tok), dim3(256), 0, a);
    return SHV_OK;
}
