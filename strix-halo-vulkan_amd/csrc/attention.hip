// Gated full-attention decode over an fp16 KV cache, GQA with 8 query heads per KV head.
//
// HBM-bound on the cache: a block owns one KV head and one slice of the cells and serves all the
// query heads of that KV head from a single pass over K and a single pass over V.
//   prologue  per-head RMS norm + rotary of the block's query heads into LDS; the block that owns
//             the new cell also normalises/rotates K, rounds K and V to binary16 and appends them
//   phase 1   scores: 32 lanes per cell (16-byte loads of K), eight partial dots per lane reduced
//             with a transposing butterfly so every lane ends with one head's score
//   phase 2   the slice's max and exponentials per head (in LDS)
//   phase 3   P*V: 64 lanes across the 256 dims of a V row, eight heads' accumulators per lane
//   epilogue  the block's (max, sum, accumulator) goes to scratch; the last block of the KV head
//             to arrive merges the slices
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kD = 256;        // head dimension the kernel is built for
constexpr int kRep = 8;        // query heads per KV head
constexpr int kMaxCells = 1024; // cells one block can take (its scores live in LDS)

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
    __shared__ __align__(16) float qh[kRep][kD];          // 8 KB: normalised, rotated queries
    __shared__ __align__(16) float sc[kMaxCells][kRep];   // 32 KB: scores, then probabilities; reused for the merge
    __shared__ __align__(16) float kv_tmp[2][kD];
    __shared__ float red[4][kRep];
    __shared__ float stat[2][kRep];
    __shared__ int is_last;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int split = blockIdx.x, kvh = blockIdx.y, seq = blockIdx.z;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int p = (a.pos ? a.pos[seq] : 0) + row_i;
    const int row = seq * a.seq_len + row_i;
    const int n_cells = p + 1;
    int cps = (n_cells + a.n_splits - 1) / a.n_splits;
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
            norm_rope_head(ksrc, a.k_norm, rope_row, a.rope_dims, a.eps, kv_tmp[0], lane);
            uint16_t *dst = kc + static_cast<size_t>(p) * kvw;
#pragma unroll
            for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(kv_tmp[0][4 * lane + i]));
        } else if (wave == 1) {
            const float *vsrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvw + kvh * kD;
            uint16_t *dst = vc + static_cast<size_t>(p) * kvw;
#pragma unroll
            for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(vsrc[4 * lane + i]));
        }
        __threadfence_block();
    }
    __syncthreads();

    float m_head = -INFINITY, l_head = 0.f;  // meaningful in threads tid < kRep after phase 2
    if (nc > 0) {
        // ---- phase 1: scores ----
        const int li = lane & 31, cg = lane >> 5;
        float qr[kRep][8];
#pragma unroll
        for (int hh = 0; hh < kRep; hh++) {
            const float4 q0 = *reinterpret_cast<const float4 *>(&qh[hh][8 * li]);
            const float4 q1 = *reinterpret_cast<const float4 *>(&qh[hh][8 * li + 4]);
            qr[hh][0] = q0.x; qr[hh][1] = q0.y; qr[hh][2] = q0.z; qr[hh][3] = q0.w;
            qr[hh][4] = q1.x; qr[hh][5] = q1.y; qr[hh][6] = q1.z; qr[hh][7] = q1.w;
        }
        const float scale = 1.f / sqrtf(static_cast<float>(kD));
        const int my_head = ((li >> 4) & 1) * 4 + ((li >> 3) & 1) * 2 + ((li >> 2) & 1);
        for (int cb = wave * 2; cb < nc; cb += 8) {
            const int c = cb + cg;
            const bool live = c < nc;
            const uint16_t *kp = kc + static_cast<size_t>(c0 + (live ? c : 0)) * kvw + 8 * li;
            const uint4 kq = *reinterpret_cast<const uint4 *>(kp);
            const float2 k01 = half2_bits_to_float2(kq.x), k23 = half2_bits_to_float2(kq.y);
            const float2 k45 = half2_bits_to_float2(kq.z), k67 = half2_bits_to_float2(kq.w);
            float part[kRep];
#pragma unroll
            for (int hh = 0; hh < kRep; hh++) {
                float s = qr[hh][0] * k01.x;
                s = fmaf(qr[hh][1], k01.y, s);
                s = fmaf(qr[hh][2], k23.x, s);
                s = fmaf(qr[hh][3], k23.y, s);
                s = fmaf(qr[hh][4], k45.x, s);
                s = fmaf(qr[hh][5], k45.y, s);
                s = fmaf(qr[hh][6], k67.x, s);
                s = fmaf(qr[hh][7], k67.y, s);
                part[hh] = s;
            }
            const float tot = reduce8_over32(part, li);
            if (live && (li & 3) == 0) sc[c][my_head] = tot * scale;
        }
        __syncthreads();
        // ---- phase 2: max, exponentials and their sum per head over the slice ----
        {
            const int hh = tid & 7, stripe = tid >> 3;  // 32 stripes of cells
            float mx = -INFINITY;
            for (int c = stripe; c < nc; c += 32) mx = fmaxf(mx, sc[c][hh]);
            mx = fmaxf(mx, __shfl_xor(mx, 8, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            if (lane < kRep) red[wave][lane] = mx;
            __syncthreads();
            mx = fmaxf(fmaxf(red[0][hh], red[1][hh]), fmaxf(red[2][hh], red[3][hh]));
            __syncthreads();
            float sum = 0.f;
            for (int c = stripe; c < nc; c += 32) {
                const float e = __expf(sc[c][hh] - mx);
                sc[c][hh] = e;
                sum += e;
            }
            sum += __shfl_xor(sum, 8, 64);
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            if (lane < kRep) red[wave][lane] = sum;
            __syncthreads();
            if (tid < kRep) {
                m_head = mx;
                l_head = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
            }
        }
        __syncthreads();
    }
    // ---- phase 3: P*V, 4 dims per lane, the block's cells dealt round-robin to its waves ----
    float acc[kRep][4];
#pragma unroll
    for (int hh = 0; hh < kRep; hh++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[hh][i] = 0.f;
    for (int c = wave; c < nc; c += 4) {
        const uint2 vq = *reinterpret_cast<const uint2 *>(vc + static_cast<size_t>(c0 + c) * kvw + 4 * lane);
        const float2 v01 = half2_bits_to_float2(vq.x), v23 = half2_bits_to_float2(vq.y);
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
    __syncthreads();
    // cross-wave sum through LDS (the score buffer is free now): buf[wave][head][dim]
    float *buf = &sc[0][0];
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
#pragma unroll
    for (int hh = 0; hh < kRep; hh++) {
        const float v = (buf[(0 * kRep + hh) * kD + tid] + buf[(1 * kRep + hh) * kD + tid]) +
                        (buf[(2 * kRep + hh) * kD + tid] + buf[(3 * kRep + hh) * kD + tid]);
        part_out[hh * (kD + 2) + tid] = v;
    }
    if (tid < kRep) {
        part_out[tid * (kD + 2) + kD] = stat[0][tid];
        part_out[tid * (kD + 2) + kD + 1] = stat[1][tid];
    }
    // ---- the last slice of this (sequence, KV head) to arrive merges them all ----
    __threadfence();
    __syncthreads();
    int32_t *counter = counters + seq * a.n_head_kv + kvh;
    if (tid == 0) {
        const int prev = __hip_atomic_fetch_add(counter, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        is_last = prev == a.n_splits - 1;
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();
    if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float *pin = a.partial + (static_cast<size_t>(seq) * a.n_head_kv + kvh) * a.n_splits * kRep * (kD + 2);
    for (int hh = 0; hh < kRep; hh++) {
        float M = -INFINITY;
        for (int s = 0; s < a.n_splits; s++) M = fmaxf(M, pin[(static_cast<size_t>(s) * kRep + hh) * (kD + 2) + kD]);
        float num = 0.f, den = 0.f;
        for (int s = 0; s < a.n_splits; s++) {
            const float *rec = pin + (static_cast<size_t>(s) * kRep + hh) * (kD + 2);
            const float ms = rec[kD];
            if (ms == -INFINITY) continue;
            const float w = __expf(ms - M);
            num = fmaf(w, rec[tid], num);
            den = fmaf(w, rec[kD + 1], den);
        }
        a.out[static_cast<size_t>(row) * a.n_head * kD + static_cast<size_t>(kvh * kRep + hh) * kD + tid] = num / den;
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
    SHV_REQUIRE(a.n_splits >= 1 && static_cast<long long>(a.n_splits) * kMaxCells >= a.max_cells,
                "attn_decode: %d splits cannot cover %d cells at %d cells a block", a.n_splits, a.max_cells, kMaxCells);
    SHV_REQUIRE(a.qkv_stride >= a.n_head * 2 * kD + 2 * a.n_head_kv * kD, "attn_decode: qkv_stride %d", a.qkv_stride);
    SHV_REQUIRE(shv_aligned16(a.qkv) && shv_aligned16(a.kcache) && shv_aligned16(a.vcache) && shv_aligned16(a.q_norm) &&
                    shv_aligned16(a.k_norm) && a.qkv_stride % 4 == 0,
                "attn_decode: qkv, caches and norms must be 16-byte aligned");
    dim3 grid(a.n_splits, a.n_head_kv, a.n_seq);
    for (int i = 0; i < a.seq_len; i++) {
        hipLaunchKernelGGL(attn_decode_kernel, grid, dim3(kBlock), 0, ctx->stream, a, i, ctx->counters + shv_ctx::kCounterAttn);
        SHV_HIP_CHECK(hipGetLastError());
    }
    return SHV_OK;
}
