// Gated full-attention decode over an fp16 KV cache, GQA with 8 query heads per KV head.
//
// HBM-bound on the cache: a block owns one KV head and one slice of the cells and serves all the
// query heads of that KV head from a single pass over K and a single pass over V.
//   prologue  per-head RMS norm + rotary of the block's query heads into LDS; the block that owns
//             the new cell also normalises/rotates K, rounds K and V to binary16 and appends them
//   per chunk of 128 cells (flash-decoding with a running max):
//     (a) the chunk's V rows are requested, (b) scores: 32 lanes per cell (16-byte loads of K),
//     eight partial dots per lane reduced with a transposing butterfly so every lane ends with
//     one head's score, (c) running max and exponentials per head in LDS, (d) P*V: 64 lanes
//     across the 256 dims of a V row, eight heads' accumulators per lane
//   epilogue  the block's (max, sum, accumulator) goes to scratch; the last block of the KV head
//             to arrive merges the slices
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kD = 256;        // head dimension the kernel is built for
constexpr int kRep = 8;        // query heads per KV head
constexpr int kChunk = 128;    // cells scored together; also what a slice is given while slices are to spare
constexpr int kMaxSplits = 512; // slices the merge has LDS for
constexpr int kPlane = kMaxSplits * kRep;

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

// grid: (n_splits, n_head_kv, n_seq); row_i is the row of each sequence this launch handles.
__global__ __launch_bounds__(kBlock) void attn_decode_kernel(shv_attn_decode_args a, int row_i, int32_t *counters) {
    __shared__ __align__(16) float qh[kRep][kD];         // 8 KB: normalised, rotated queries
    __shared__ __align__(16) float sc[kChunk][kRep];     // 4 KB: scores, then probabilities, of a chunk
    __shared__ __align__(16) float big[4 * kRep * kD];   // 32 KB: cross-wave sums, then the merge's weights
    __shared__ __align__(16) float kv_tmp[kD];
    __shared__ float red[4][kRep];
    __shared__ float mrun[kRep], lrun[kRep], alpha[kRep];
    __shared__ float stat[2][kRep];
    __shared__ int is_last;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int split = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int p = (a.pos ? a.pos[seq] : 0) + row_i;
    const int row = seq * a.seq_len + row_i;
    const int n_cells = p + 1;
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
    const bool owner = p >= c0 && p < c1;

    const float *qkv = a.qkv + static_cast<size_t>(row) * a.qkv_stride;
    const float *rope_row = a.rope + static_cast<size_t>(p) * a.rope_dims;
    const int kvw = a.n_head_kv * kD;
    uint16_t *kc = static_cast<uint16_t *>(a.kcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;
    uint16_t *vc = static_cast<uint16_t *>(a.vcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;

    // ---- prologue ----
    if (nc > 0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int hh = wave * 2 + i;
            const int head = kvh * kRep + hh;
            norm_rope_head(qkv + static_cast<size_t>(head) * 2 * kD, a.q_norm, rope_row, a.rope_dims, a.eps, qh[hh], lane);
        }
    }
    if (owner) {
        if (wave == 0) {
            const float *ksrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvh * kD;
            norm_rope_head(ksrc, a.k_norm, rope_row, a.rope_dims, a.eps, kv_tmp, lane);
            uint16_t *dst = kc + static_cast<size_t>(p) * kvw;
#pragma unroll
            for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(kv_tmp[4 * lane + i]));
        } else if (wave == 1) {
            const float *vsrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvw + kvh * kD;
            uint16_t *dst = vc + static_cast<size_t>(p) * kvw;
#pragma unroll
            for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(vsrc[4 * lane + i]));
        }
        __threadfence_block();
    }
    if (tid < kRep) {
        mrun[tid] = -INFINITY;
        lrun[tid] = 0.f;
    }
    __syncthreads();

    // The slice is walked in chunks of kChunk cells, flash-decoding style: the chunk's V rows are
    // requested first and arrive while its scores are being formed.
    float acc[kRep][4];
#pragma unroll
    for (int hh = 0; hh < kRep; hh++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[hh][i] = 0.f;

    const int li = lane & 31, cg = lane >> 5;
    float qr[kRep][8];
    if (nc > 0) {
#pragma unroll
        for (int hh = 0; hh < kRep; hh++) {
            const float4 q0 = *reinterpret_cast<const float4 *>(&qh[hh][8 * li]);
            const float4 q1 = *reinterpret_cast<const float4 *>(&qh[hh][8 * li + 4]);
            qr[hh][0] = q0.x; qr[hh][1] = q0.y; qr[hh][2] = q0.z; qr[hh][3] = q0.w;
            qr[hh][4] = q1.x; qr[hh][5] = q1.y; qr[hh][6] = q1.z; qr[hh][7] = q1.w;
        }
    }
    const float scale = 1.f / sqrtf(static_cast<float>(kD));
    const int my_head = ((li >> 4) & 1) * 4 + ((li >> 3) & 1) * 2 + ((li >> 2) & 1);

    for (int ch0 = 0; ch0 < nc; ch0 += kChunk) {
        const int cn = nc - ch0 < kChunk ? nc - ch0 : kChunk;
        // (a) V rows of this wave's cells of the chunk: cells wave, wave+4, ... (4 dims a lane)
        constexpr int VPW = kChunk / 4;
        uint2 vq[VPW];
#pragma unroll
        for (int u = 0; u < VPW; u++) {
            const int c = wave + 4 * u;
            vq[u] = *reinterpret_cast<const uint2 *>(vc + static_cast<size_t>(c0 + ch0 + (c < cn ? c : 0)) * kvw + 4 * lane);
        }
        // (b) scores: 32 lanes a cell, 8 dims a lane, eight passes of the wave loaded together
        constexpr int PB = 8;
#pragma unroll
        for (int half = 0; half < kChunk / (8 * PB); half++) {
            const int cb0 = half * 8 * PB + wave * 2;
            if (cb0 < cn) {
                uint4 kq[PB];
#pragma unroll
                for (int u = 0; u < PB; u++) {
                    const int c = cb0 + 8 * u + cg;
                    kq[u] = *reinterpret_cast<const uint4 *>(kc + static_cast<size_t>(c0 + ch0 + (c < cn ? c : 0)) * kvw + 8 * li);
                }
#pragma unroll
                for (int u = 0; u < PB; u++) {
                    const int c = cb0 + 8 * u + cg;
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
                    if (c < cn && (li & 3) == 0) sc[c][my_head] = tot * scale;
                }
            }
        }
        __syncthreads();
        // (c) running max, the chunk's exponentials and their sum, per head
        {
            const int hh = tid & 7, stripe = tid >> 3;  // 32 stripes of cells
            float mx = -INFINITY;
            for (int c = stripe; c < cn; c += 32) mx = fmaxf(mx, sc[c][hh]);
            mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            if (lane < kRep) red[wave][lane] = mx;
            const float m_old = mrun[hh];
            __syncthreads();
            const float m_new = fmaxf(m_old, fmaxf(fmaxf(red[0][hh], red[1][hh]), fmaxf(red[2][hh], red[3][hh])));
            __syncthreads();
            float sum = 0.f;
            for (int c = stripe; c < cn; c += 32) {
                const float e = __expf(sc[c][hh] - m_new);
                sc[c][hh] = e;
                sum += e;
            }
            sum += __shfl_xor(sum, 8, 64);
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            if (lane < kRep) red[wave][lane] = sum;
            __syncthreads();
            if (tid < kRep) {
                const float al = __expf(m_old - m_new);  // 0 on the first chunk (m_old = -inf)
                alpha[tid] = al;
                lrun[tid] = lrun[tid] * al + ((red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]));
                mrun[tid] = m_new;
            }
            __syncthreads();
        }
        // (d) acc = acc*alpha + P*V over this wave's cells of the chunk
#pragma unroll
        for (int hh = 0; hh < kRep; hh++) {
            const float al = alpha[hh];
#pragma unroll
            for (int i = 0; i < 4; i++) acc[hh][i] *= al;
        }
#pragma unroll
        for (int u = 0; u < VPW; u++) {
            const int c = wave + 4 * u;
            if (c < cn) {
                const float2 v01 = half2_bits_to_float2(vq[u].x), v23 = half2_bits_to_float2(vq[u].y);
                const float4 p0 = *reinterpret_cast<const float4 *>(&sc[c][0]);
                const float4 p1 = *reinterpret_cast<const float4 *>(&sc[c][4]);
                const float pr[kRep] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
#pragma unroll
                for (int hh = 0; hh < kRep; hh++) {
                    acc[hh][0] = fmaf(pr[hh], v01.x, acc[hh][0]);
                    acc[hh][1] = fmaf(pr[hh], v01.y, acc[hh][1]);
                    acc[hh][2] = fmaf(pr[hh], v23.x, acc[hh][2]);
                    acc[hh][3] = fmaf(pr[hh], v23.y, acc[hh][3]);
                }
            }
        }
        __syncthreads();
    }
    const float m_head = tid < kRep ? mrun[tid] : 0.f, l_head = tid < kRep ? lrun[tid] : 0.f;
    // cross-wave sum through LDS: buf[wave][head][dim]
    float *buf = big;
#pragma unroll
    for (int hh = 0; hh < kRep; hh++)
        *reinterpret_cast<float4 *>(buf + (wave * kRep + hh) * kD + 4 * lane) =
            make_float4(acc[hh][0], acc[hh][1], acc[hh][2], acc[hh][3]);
    if (tid < kRep) {
        stat[0][tid] = m_head;
        stat[1][tid] = l_head;
    }
    __syncthreads();
    // partial record of this block: per head, d accumulators then (max, sum)
    float *part_out = a.partial + ((static_cast<size_t>(seq) * a.n_head_kv + kvh) * a.n_splits + split) * kRep * (kD + 2);
    // thread = (head, 8 dims) here as in the merge below
    {
        const int hh = tid >> 5, d0 = (tid & 31) * 8;
        float *rec = part_out + hh * (kD + 2) + d0;
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const float v0 = (buf[(0 * kRep + hh) * kD + d0 + i] + buf[(1 * kRep + hh) * kD + d0 + i]) +
                             (buf[(2 * kRep + hh) * kD + d0 + i] + buf[(3 * kRep + hh) * kD + d0 + i]);
            const float v1 = (buf[(0 * kRep + hh) * kD + d0 + i + 1] + buf[(1 * kRep + hh) * kD + d0 + i + 1]) +
                             (buf[(2 * kRep + hh) * kD + d0 + i + 1] + buf[(3 * kRep + hh) * kD + d0 + i + 1]);
            store_agent2(rec + i, v0, v1);
        }
    }
    if (tid < kRep) store_agent2(part_out + tid * (kD + 2) + kD, stat[0][tid], stat[1][tid]);
    // ---- the last slice of this (sequence, KV head) to arrive merges them all ----
    if (!arrive_last(counters + seq * a.n_head_kv + kvh, n_active, &is_last)) return;
    const float *pin = a.partial + (static_cast<size_t>(seq) * a.n_head_kv + kvh) * a.n_splits * kRep * (kD + 2);
    // weights of the slices: w[s][h] = exp(m_s - M_h), and the merged denominator per head
    float *wbuf = big;  // [n_active][kRep], and a second plane of the same size
    for (int i = tid; i < n_active * kRep; i += kBlock) {
        const int sidx = i / kRep, hh = i % kRep;
        wbuf[i] = load_agent(pin + (static_cast<size_t>(sidx) * kRep + hh) * (kD + 2) + kD);
    }
    __syncthreads();
    if (tid < kRep) {
        float M = -INFINITY;
        for (int sidx = 0; sidx < n_active; sidx++) M = fmaxf(M, wbuf[sidx * kRep + tid]);
        stat[0][tid] = M;
    }
    __syncthreads();
    for (int i = tid; i < n_active * kRep; i += kBlock) {
        const int sidx = i / kRep, hh = i % kRep;
        const float ms = wbuf[i];
        const float w = ms == -INFINITY ? 0.f : __expf(ms - stat[0][hh]);
        wbuf[i] = w;
        // the slice's sum of exponentials, scaled, goes to a second plane
        wbuf[kPlane + i] = w * load_agent(pin + (static_cast<size_t>(sidx) * kRep + hh) * (kD + 2) + kD + 1);
    }
    __syncthreads();
    if (tid < kRep) {
        float den = 0.f;
        for (int sidx = 0; sidx < n_active; sidx++) den += wbuf[kPlane + sidx * kRep + tid];
        stat[1][tid] = den;
    }
    __syncthreads();
    // thread = (head, 8 dims): n_active records of two float4 each, eight slices in flight
    {
        const int hh = tid >> 5, d0 = (tid & 31) * 8;
        float num[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        constexpr int MB = 16;
        for (int s0 = 0; s0 < n_active; s0 += MB) {
            float4 r0[MB], r1[MB];
#pragma unroll
            for (int u = 0; u < MB; u++) {
                const int sidx = s0 + u < n_active ? s0 + u : s0;
                const float *rec = pin + (static_cast<size_t>(sidx) * kRep + hh) * (kD + 2) + d0;
                // records are 258 floats long, so only 8-byte alignment holds
                const float2 a0 = load_agent2(rec), a1 = load_agent2(rec + 2);
                const float2 a2 = load_agent2(rec + 4), a3 = load_agent2(rec + 6);
                r0[u] = make_float4(a0.x, a0.y, a1.x, a1.y);
                r1[u] = make_float4(a2.x, a2.y, a3.x, a3.y);
            }
#pragma unroll
            for (int u = 0; u < MB; u++) {
                if (s0 + u >= n_active) break;
                const float w = wbuf[(s0 + u) * kRep + hh];
                num[0] = fmaf(w, r0[u].x, num[0]); num[1] = fmaf(w, r0[u].y, num[1]);
                num[2] = fmaf(w, r0[u].z, num[2]); num[3] = fmaf(w, r0[u].w, num[3]);
                num[4] = fmaf(w, r1[u].x, num[4]); num[5] = fmaf(w, r1[u].y, num[5]);
                num[6] = fmaf(w, r1[u].z, num[6]); num[7] = fmaf(w, r1[u].w, num[7]);
            }
        }
        const float inv = 1.f / stat[1][hh];
        float *o = a.out + static_cast<size_t>(row) * a.n_head * kD + static_cast<size_t>(kvh * kRep + hh) * kD + d0;
        *reinterpret_cast<float4 *>(o) = make_float4(num[0] * inv, num[1] * inv, num[2] * inv, num[3] * inv);
        *reinterpret_cast<float4 *>(o + 4) = make_float4(num[4] * inv, num[5] * inv, num[6] * inv, num[7] * inv);
    }
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
    SHV_REQUIRE(a.n_seq * a.n_head_kv <= ctx->n_counters - shv_ctx::kCounterAttn, "attn_decode: %d sequences is more than the library tracks", a.n_seq);
    SHV_REQUIRE(a.n_splits >= 1 && a.n_splits <= kMaxSplits, "attn_decode: %d slices; 1..%d", a.n_splits, kMaxSplits);
    SHV_REQUIRE(a.qkv_stride >= a.n_head * 2 * kD + 2 * a.n_head_kv * kD, "attn_decode: qkv_stride %d", a.qkv_stride);
    SHV_REQUIRE(shv_aligned16(a.qkv) && shv_aligned16(a.kcache) && shv_aligned16(a.vcache) && shv_aligned16(a.q_norm) &&
                    shv_aligned16(a.k_norm) && shv_aligned16(a.out) && shv_aligned16(a.partial) && a.qkv_stride % 4 == 0,
                "attn_decode: qkv, caches, norms, partial and out must be 16-byte aligned");
    dim3 grid(a.n_splits, a.n_head_kv, a.n_seq);
    for (int i = 0; i < a.seq_len; i++) {
        SHV_LAUNCH(ctx, attn_decode_kernel, grid, dim3(kBlock), 0, a, i, ctx->counters + shv_ctx::kCounterAttn);
    }
    return SHV_OK;
}
