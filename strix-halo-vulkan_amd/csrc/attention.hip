// Gated full-attention decode over an fp16 KV cache, GQA with 8 query heads per KV head, one or
// two consecutive rows of a sequence per launch.
//
// HBM-bound on the cache: a block owns one KV head and one slice of the cells and serves all the
// query heads of that KV head, for both rows, from a single pass over K and a single pass over V.
//   start     the wave's first K and V rows are requested before anything else
//   prologue  per-head RMS norm + rotary of the block's query heads into LDS; the block whose slice
//             holds a new cell also normalises/rotates K, rounds K and V to binary16 and appends them
//   per chunk of 64 cells, every wave on its own 16 cells with no block-wide synchronisation:
//     scores (32 lanes a cell, 16-byte loads of K, eight partial dots a lane reduced with a
//     transposing butterfly), a running max and sum per (row, head) kept by the wave, P*V with 64
//     lanes across the 256 dims of a V row
//   epilogue  the four waves' (max, sum, accumulator) are merged through LDS and go to scratch
// A second, small kernel merges the slices: one block a (row, head), one thread a dim, every
// slice's value requested at once.  (Merging in the last block to arrive instead costs more than
// the launch: that block walks all the records alone, a few dependent round trips to memory.)
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kD = 256;        // head dimension the kernel is built for
constexpr int kRep = 8;        // query heads per KV head
#ifndef SHV_ATTN_WAVE_CELLS
#define SHV_ATTN_WAVE_CELLS 16
#endif
constexpr int kWaveCells = SHV_ATTN_WAVE_CELLS; // cells a wave scores together
constexpr int kChunk = 4 * kWaveCells;
constexpr int kMaxSplits = 512;
constexpr int kRec = kRep * (kD + 2);  // floats of one (slice, row) record: per head d values, max, sum

// v[8] per lane -> the sum over the 32 lanes of an aligned half-wave of v[head], where
// head = bit4(li)*4 + bit3(li)*2 + bit2(li); every lane of the half-wave gets one head's total.
__device__ __forceinline__ float reduce8_over32(const float *v, int li) {
    const bool b4 = (li & 16) != 0, b3 = (li & 8) != 0, b2 = (li & 4) != 0;
    float r[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float keep = b4 ? v[i + 4] : v[i];
        const float send = b4 ? v[i] : v[i + 4];
        r[i] = keep + __shfl_xor(send, 16, 64);
    }
    float r2[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float keep = b3 ? r[i + 2] : r[i];
        const float send = b3 ? r[i] : r[i + 2];
        r2[i] = keep + __shfl_xor(send, 8, 64);
    }
    const float keep = b2 ? r2[1] : r2[0];
    const float send = b2 ? r2[0] : r2[1];
    float t = keep + __shfl_xor(send, 4, 64);
    t += dpp_f32<kDppXor2>(t);
    t += dpp_f32<kDppXor1>(t);
    return t;
}

__device__ __forceinline__ float2 half2_bits_to_float2(uint32_t u) {
    const f16x2_native h = __builtin_bit_cast(f16x2_native, u);
    return make_float2(static_cast<float>(h.x), static_cast<float>(h.y));
}

// RMS norm over the 256 dims of one head by one wave (4 dims per lane), then NeoX rotary on the
// first rope_dims dims through LDS.  dst is 256 floats of LDS.
__device__ __forceinline__ void norm_rope_head(const float *src, const float *gamma, const float *rope_row, int rope_dims,
                                               float eps, float *dst, int lane) {
    const float4 v = *reinterpret_cast<const float4 *>(src + 4 * lane);
    const float ss = wave_sum_all(fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w))));
    const float sc = 1.f / sqrtf(ss / static_cast<float>(kD) + eps);
    const float4 g = *reinterpret_cast<const float4 *>(gamma + 4 * lane);
    dst[4 * lane + 0] = v.x * sc * g.x;
    dst[4 * lane + 1] = v.y * sc * g.y;
    dst[4 * lane + 2] = v.z * sc * g.z;
    dst[4 * lane + 3] = v.w * sc * g.w;
    __builtin_amdgcn_wave_barrier();
    const int half = rope_dims / 2;
    if (lane < half) {
        const float x0 = dst[lane], x1 = dst[lane + half];
        const float cs = rope_row[lane], sn = rope_row[half + lane];
        dst[lane] = x0 * cs - x1 * sn;
        dst[lane + half] = x0 * sn + x1 * cs;
    }
    __builtin_amdgcn_wave_barrier();
}

// LDS of one block, R rows a launch.
template <int R>
struct Smem {
    float qh[R][kRep][kD];                    // normalised, rotated queries
    float sc[4][R][kWaveCells][kRep];         // per wave: scores, then probabilities, of its cells
    float al[4][R][kRep];                     // per wave: the factor the running sums shrink by
    float big[4][kRep][kD];                   // the waves' accumulators of one row, to be merged
    float wm[4][kRep], wl[4][kRep];           // the waves' running max and sum of one row
    float kv_tmp[R][kD];
};

// grid: (n_splits, n_head_kv, n_seq); rows row0..row0+R-1 of each sequence.
template <int R>
__global__ __launch_bounds__(kBlock) void attn_decode_kernel(shv_attn_decode_args a, int row0) {
    extern __shared__ __align__(16) char smem_raw[];
    Smem<R> &sm = *reinterpret_cast<Smem<R> *>(smem_raw);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int split = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int p_first = (a.pos ? a.pos[seq] : 0) + row0;  // position of the launch's first row
    const int n_cells = p_first + R;                       // cells the last row sees
    // The grid is sized for the cache's capacity; how many of its slices take part depends on how
    // many cells the sequence holds now: about kChunk cells a slice while there are slices to
    // spare, so that a short context is not mostly merge and a long one covers the whole chip.
    int n_active = (n_cells + kChunk - 1) / kChunk;
    if (n_active > a.n_splits) n_active = a.n_splits;
    if (split >= n_active) return;
    int cps = (n_cells + n_active - 1) / n_active;
    cps = (cps + 7) & ~7;
    const int c0 = split * cps;
    const int c1 = c0 + cps < n_cells ? c0 + cps : n_cells;
    const int nc = c1 > c0 ? c1 - c0 : 0;

    const int kvw = a.n_head_kv * kD;
    uint16_t *kc = static_cast<uint16_t *>(a.kcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;
    uint16_t *vc = static_cast<uint16_t *>(a.vcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;
    const int li = lane & 31, cg = lane >> 5;

    // ---- the wave's first K and V rows: cells c0 + 16*wave + .. ; only cells that existed before
    //      this launch may be read this early ----
    uint4 kq[kWaveCells / 2];
    uint2 vq[kWaveCells];
    auto load_k = [&](int ch0, bool old_only) {
#pragma unroll
        for (int u = 0; u < kWaveCells / 2; u++) {
            const int c = c0 + ch0 + wave * kWaveCells + 2 * u + cg;
            if (c < c1 && (!old_only || c < p_first))
                kq[u] = *reinterpret_cast<const uint4 *>(kc + static_cast<size_t>(c) * kvw + 8 * li);
            else if (!old_only || c >= c1)
                kq[u] = make_uint4(0u, 0u, 0u, 0u);
        }
    };
    auto load_v = [&](int ch0, bool old_only) {
#pragma unroll
        for (int u = 0; u < kWaveCells; u++) {
            const int c = c0 + ch0 + wave * kWaveCells + u;
            if (c < c1 && (!old_only || c < p_first))
                vq[u] = *reinterpret_cast<const uint2 *>(vc + static_cast<size_t>(c) * kvw + 4 * lane);
            else if (!old_only || c >= c1)
                vq[u] = make_uint2(0u, 0u);
        }
    };
    load_k(0, true);
    load_v(0, true);

    // ---- prologue ----
    const float *qkv0 = a.qkv + static_cast<size_t>(seq * a.seq_len + row0) * a.qkv_stride;
#pragma unroll
    for (int j = 0; j < R; j++) {
        const float *qkv = qkv0 + static_cast<size_t>(j) * a.qkv_stride;
        const int p = p_first + j;
        const float *rope_row = a.rope + static_cast<size_t>(p) * a.rope_dims;
        if (nc > 0) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int hh = wave * 2 + i;
                norm_rope_head(qkv + static_cast<size_t>(kvh * kRep + hh) * 2 * kD, a.q_norm, rope_row, a.rope_dims, a.eps, sm.qh[j][hh], lane);
            }
        }
        if (p >= c0 && p < c1) {
            // the new cell of row j lies in this slice: waves 2j and 2j+1 (mod 4) append its K and V
            if (wave == ((2 * j) & 3)) {
                const float *ksrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvh * kD;
                norm_rope_head(ksrc, a.k_norm, rope_row, a.rope_dims, a.eps, sm.kv_tmp[j], lane);
                uint16_t *dst = kc + static_cast<size_t>(p) * kvw;
#pragma unroll
                for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(sm.kv_tmp[j][4 * lane + i]));
            } else if (wave == ((2 * j + 1) & 3)) {
                const float *vsrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvw + kvh * kD;
                uint16_t *dst = vc + static_cast<size_t>(p) * kvw;
#pragma unroll
                for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(vsrc[4 * lane + i]));
            }
        }
    }
    __threadfence_block();
    __syncthreads();
    // the cells this launch appended can be read now
    if (c1 > p_first) {
#pragma unroll
        for (int u = 0; u < kWaveCells / 2; u++) {
            const int c = c0 + wave * kWaveCells + 2 * u + cg;
            if (c >= p_first && c < c1) kq[u] = *reinterpret_cast<const uint4 *>(kc + static_cast<size_t>(c) * kvw + 8 * li);
        }
#pragma unroll
        for (int u = 0; u < kWaveCells; u++) {
            const int c = c0 + wave * kWaveCells + u;
            if (c >= p_first && c < c1) vq[u] = *reinterpret_cast<const uint2 *>(vc + static_cast<size_t>(c) * kvw + 4 * lane);
        }
    }

    // per lane: accumulators of 4 dims for every (row, head); the wave's running max and sum of
    // (row, head = lane%8), the same in the eight lanes that share the head
    float acc[R][kRep][4];
    float m_run[R], l_run[R];
#pragma unroll
    for (int j = 0; j < R; j++) {
        m_run[j] = -INFINITY;
        l_run[j] = 0.f;
#pragma unroll
        for (int hh = 0; hh < kRep; hh++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][hh][i] = 0.f;
    }
    const float scale = 1.f / sqrtf(static_cast<float>(kD));
    const int my_head = ((li >> 4) & 1) * 4 + ((li >> 3) & 1) * 2 + ((li >> 2) & 1);

    for (int ch0 = 0; ch0 < nc; ch0 += kChunk) {
        const int wc0 = c0 + ch0 + wave * kWaveCells;  // this wave's first cell of the chunk
        if (ch0 > 0) {
            load_k(ch0, false);
            load_v(ch0, false);
        }
        if (wc0 < c1) {
#pragma unroll
            for (int j = 0; j < R; j++) {
                // (a) scores of row j: its queries come back from LDS, 8 dims of every head a lane
                float qr[kRep][8];
#pragma unroll
                for (int hh = 0; hh < kRep; hh++) {
                    const float4 q0 = *reinterpret_cast<const float4 *>(&sm.qh[j][hh][8 * li]);
                    const float4 q1 = *reinterpret_cast<const float4 *>(&sm.qh[j][hh][8 * li + 4]);
                    qr[hh][0] = q0.x; qr[hh][1] = q0.y; qr[hh][2] = q0.z; qr[hh][3] = q0.w;
                    qr[hh][4] = q1.x; qr[hh][5] = q1.y; qr[hh][6] = q1.z; qr[hh][7] = q1.w;
                }
#pragma unroll
                for (int u = 0; u < kWaveCells / 2; u++) {
                    const int cl = 2 * u + cg, c = wc0 + cl;
                    const float2 k01 = half2_bits_to_float2(kq[u].x), k23 = half2_bits_to_float2(kq[u].y);
                    const float2 k45 = half2_bits_to_float2(kq[u].z), k67 = half2_bits_to_float2(kq[u].w);
                    float part[kRep];
#pragma unroll
                    for (int hh = 0; hh < kRep; hh++) {
                        float sdot = qr[hh][0] * k01.x;
                        sdot = fmaf(qr[hh][1], k01.y, sdot);
                        sdot = fmaf(qr[hh][2], k23.x, sdot);
                        sdot = fmaf(qr[hh][3], k23.y, sdot);
                        sdot = fmaf(qr[hh][4], k45.x, sdot);
                        sdot = fmaf(qr[hh][5], k45.y, sdot);
                        sdot = fmaf(qr[hh][6], k67.x, sdot);
                        sdot = fmaf(qr[hh][7], k67.y, sdot);
                        part[hh] = sdot;
                    }
                    const float tot = reduce8_over32(part, li);
                    // causal: row j sees cells up to its own position
                    if ((li & 3) == 0) sm.sc[wave][j][cl][my_head] = (c < c1 && c <= p_first + j) ? tot * scale : -INFINITY;
                }
                __builtin_amdgcn_wave_barrier();
                // (b) the wave's running max and sum: lane = (cell pair g, g+8 ; head)
                {
                    const int hh = lane & 7, g = lane >> 3;
                    const float s0 = sm.sc[wave][j][g][hh], s1 = kWaveCells > 8 ? sm.sc[wave][j][(g + 8) % kWaveCells][hh] : -INFINITY;
                    float mx = fmaxf(s0, s1);
                    mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
                    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                    const float m_new = fmaxf(m_run[j], mx);
                    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // nothing visible yet: all weights 0
                    const float e0 = __expf(s0 - m_use), e1 = __expf(s1 - m_use);
                    sm.sc[wave][j][g][hh] = e0;
                    if (kWaveCells > 8) sm.sc[wave][j][(g + 8) % kWaveCells][hh] = e1;
                    float sum = e0 + e1;
                    sum += __shfl_xor(sum, 8, 64);
                    sum += __shfl_xor(sum, 16, 64);
                    sum += __shfl_xor(sum, 32, 64);
                    const float alpha = __expf(m_run[j] - m_use);  // 0 while the old max is -inf
                    l_run[j] = l_run[j] * alpha + sum;
                    m_run[j] = m_new;
                    if (g == 0) sm.al[wave][j][hh] = alpha;
                }
                __builtin_amdgcn_wave_barrier();
                // (c) acc = acc*alpha + P*V over the wave's cells
                {
                    const float4 a0 = *reinterpret_cast<const float4 *>(&sm.al[wave][j][0]);
                    const float4 a1 = *reinterpret_cast<const float4 *>(&sm.al[wave][j][4]);
                    const float alv[kRep] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
                    for (int hh = 0; hh < kRep; hh++)
#pragma unroll
                        for (int i = 0; i < 4; i++) acc[j][hh][i] *= alv[hh];
                }
#pragma unroll
                for (int u = 0; u < kWaveCells; u++) {
                    const float2 v01 = half2_bits_to_float2(vq[u].x), v23 = half2_bits_to_float2(vq[u].y);
                    const float4 p0 = *reinterpret_cast<const float4 *>(&sm.sc[wave][j][u][0]);
                    const float4 p1 = *reinterpret_cast<const float4 *>(&sm.sc[wave][j][u][4]);
                    const float pr[kRep] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
#pragma unroll
                    for (int hh = 0; hh < kRep; hh++) {
                        acc[j][hh][0] = fmaf(pr[hh], v01.x, acc[j][hh][0]);
                        acc[j][hh][1] = fmaf(pr[hh], v01.y, acc[j][hh][1]);
                        acc[j][hh][2] = fmaf(pr[hh], v23.x, acc[j][hh][2]);
                        acc[j][hh][3] = fmaf(pr[hh], v23.y, acc[j][hh][3]);
                    }
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
    // ---- the four waves' results of each row are merged and go to scratch ----
    float *part_base = a.partial + ((static_cast<size_t>(seq) * a.n_head_kv + kvh) * a.n_splits + split) * R * kRec;
#pragma unroll
    for (int j = 0; j < R; j++) {
        if (lane < kRep) {
            sm.wm[wave][lane] = m_run[j];
            sm.wl[wave][lane] = l_run[j];
        }
#pragma unroll
        for (int hh = 0; hh < kRep; hh++)
            *reinterpret_cast<float4 *>(&sm.big[wave][hh][4 * lane]) = make_float4(acc[j][hh][0], acc[j][hh][1], acc[j][hh][2], acc[j][hh][3]);
        __syncthreads();
        {
            // thread = (head, 8 dims) here as in the merge below
            const int hh = tid >> 5, d0 = (tid & 31) * 8;
            float M = fmaxf(fmaxf(sm.wm[0][hh], sm.wm[1][hh]), fmaxf(sm.wm[2][hh], sm.wm[3][hh]));
            float w[4], L = 0.f;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                w[k] = sm.wm[k][hh] == -INFINITY ? 0.f : __expf(sm.wm[k][hh] - M);
                L = fmaf(w[k], sm.wl[k][hh], L);
            }
            float *rec = part_base + j * kRec + hh * (kD + 2);
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                float v0 = 0.f, v1 = 0.f;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    v0 = fmaf(w[k], sm.big[k][hh][d0 + i], v0);
                    v1 = fmaf(w[k], sm.big[k][hh][d0 + i + 1], v1);
                }
                *reinterpret_cast<float2 *>(rec + d0 + i) = make_float2(v0, v1);
            }
            if ((tid & 31) == 0) *reinterpret_cast<float2 *>(rec + kD) = make_float2(M, L);
        }
        __syncthreads();
    }
}

// grid: (n_head * 4, R, n_seq), one wave = 64 dims of one head.  The slices' records of that
// (row, head) are combined with a running max; all of a batch's loads are in flight together.
template <int R>
__global__ __launch_bounds__(64) void attn_merge_kernel(shv_attn_decode_args a, int row0) {
    const int head = blockIdx.x >> 2, d = (blockIdx.x & 3) * 64 + threadIdx.x, j = blockIdx.y, seq = blockIdx.z;
    const int kvh = head / kRep, hh = head % kRep;
    const int n_cells = (a.pos ? a.pos[seq] : 0) + row0 + R;
    int n_active = (n_cells + kChunk - 1) / kChunk;
    if (n_active > a.n_splits) n_active = a.n_splits;
    const float *pin = a.partial + (static_cast<size_t>(seq) * a.n_head_kv + kvh) * a.n_splits * R * kRec + j * kRec + hh * (kD + 2);
    constexpr int MB = 64;
    float num = 0.f, den = 0.f, M = -INFINITY;
    for (int s0 = 0; s0 < n_active; s0 += MB) {
        float v[MB];
        float2 ml[MB];
#pragma unroll
        for (int u = 0; u < MB; u++) {
            const int sidx = s0 + u < n_active ? s0 + u : s0;
            const float *rec = pin + static_cast<size_t>(sidx) * R * kRec;
            v[u] = rec[d];
            ml[u] = *reinterpret_cast<const float2 *>(rec + kD);
        }
#pragma unroll
        for (int u = 0; u < MB; u++) {
            if (s0 + u >= n_active || ml[u].x == -INFINITY) continue;
            const float Mn = fmaxf(M, ml[u].x);
            const float shrink = __expf(M - Mn), w = __expf(ml[u].x - Mn);  // shrink is 0 while M is -inf
            den = fmaf(den, shrink, w * ml[u].y);
            num = fmaf(num, shrink, w * v[u]);
            M = Mn;
        }
    }
    a.out[static_cast<size_t>(seq * a.seq_len + row0 + j) * a.n_head * kD + static_cast<size_t>(head) * kD + d] = num / den;
}

template <int R>
int launch_rows(shv_ctx *ctx, const shv_attn_decode_args &a, int row0) {
    static bool raised = false;
    if (sizeof(Smem<R>) > 48 * 1024 && !raised) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_decode_kernel<R>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          static_cast<int>(sizeof(Smem<R>))));
        raised = true;
    }
    dim3 grid(a.n_splits, a.n_head_kv, a.n_seq);
    SHV_LAUNCH(ctx, (attn_decode_kernel<R>), grid, dim3(kBlock), sizeof(Smem<R>), a, row0);
    SHV_LAUNCH(ctx, (attn_merge_kernel<R>), dim3(a.n_head * 4, R, a.n_seq), dim3(64), 0, a, row0);
    return SHV_OK;
}

}  // namespace

int shv_launch_attn_decode(shv_ctx *ctx, const shv_attn_decode_args *pa) {
    const shv_attn_decode_args &a = *pa;
    SHV_REQUIRE(a.qkv && a.q_norm && a.k_norm && a.rope && a.kcache && a.vcache && a.partial && a.out, "attn_decode: NULL argument");
    SHV_REQUIRE(a.head_dim == kD, "attn_decode: head_dim %d; built for %d", a.head_dim, kD);
    SHV_REQUIRE(a.n_head_kv >= 1 && a.n_head == a.n_head_kv * kRep, "attn_decode: %d query heads over %d KV heads; built for %d per KV head",
                a.n_head, a.n_head_kv, kRep);
    SHV_REQUIRE(a.rope_dims >= 0 && a.rope_dims <= 128 && a.rope_dims % 2 == 0, "attn_decode: rope_dims %d", a.rope_dims);
    SHV_REQUIRE(a.n_seq >= 1 && a.seq_len >= 1, "attn_decode: %d sequences of %d rows", a.n_seq, a.seq_len);
    SHV_REQUIRE(a.n_seq <= 65535, "attn_decode: %d sequences", a.n_seq);
    SHV_REQUIRE(a.n_splits >= 1 && a.n_splits <= kMaxSplits, "attn_decode: %d slices; 1..%d", a.n_splits, kMaxSplits);
    SHV_REQUIRE(a.qkv_stride >= a.n_head * 2 * kD + 2 * a.n_head_kv * kD, "attn_decode: qkv_stride %d", a.qkv_stride);
    SHV_REQUIRE(shv_aligned16(a.qkv) && shv_aligned16(a.kcache) && shv_aligned16(a.vcache) && shv_aligned16(a.q_norm) &&
                    shv_aligned16(a.k_norm) && shv_aligned16(a.out) && shv_aligned16(a.partial) && a.qkv_stride % 4 == 0,
                "attn_decode: qkv, caches, norms, partial and out must be 16-byte aligned");
    // the rows of a sequence go two at a time: both see one pass over the cache
    for (int i = 0; i < a.seq_len; i += 2) {
        const int rc = a.seq_len - i >= 2 ? launch_rows<2>(ctx, a, i) : launch_rows<1>(ctx, a, i);
        if (rc != SHV_OK) return rc;
    }
    return SHV_OK;
}
