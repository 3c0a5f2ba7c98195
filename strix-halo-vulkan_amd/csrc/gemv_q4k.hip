// Q4_K dequant-fused GEMV for batch-1..4 decode: y[t] = W * pro(x[t]) (+ residual[t]).
//
// HBM-bound: every weight byte is read once with 128-bit loads and nothing else of size moves.
// Work split (wave64): a lane owns one 64-weight group of a row — 32 contiguous payload bytes
// (two 16-byte loads) plus the row's 16-byte super-block header — and keeps the 64 activations of
// those columns in registers for every row it visits.  K/64 lanes cover a row, so a wave covers
// 64/(K/64) rows per pass and reduces each row across its lanes with DPP.  Passes of a wave are
// unrolled so all of its loads are in flight before the first is consumed.
//
// The input vector is staged once per 256-thread block through LDS, where the optional prologue
// (RMSNorm, DeltaNet's gated per-head norm, or attention's sigmoid gate) is applied.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxTok = 4;

// U consecutive passes of one wave.  load() issues every 128-bit load of the batch; compute()
// consumes them.  The kernel keeps two batches alive so that the loads of the next one are in
// flight while the current one is being multiplied.
template <int K, int NT, int U>
struct GemvBatch {
    static constexpr int LPR = K / 64;
    static constexpr int RPP = 64 / LPR;
    static constexpr int ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    uint4 hdr[U], q0[U], q1[U];
    int row[U];
    float res[U][NT];  // the residual of the rows this lane writes, requested with the weights

    // the batch's passes are `stride` apart: pass, pass + stride, ...
    __device__ __forceinline__ void load(const shv_gemv_q4k_args &a, const char *wbase, int g, int rsub, int lane, long long pass,
                                         long long stride, int n, int t0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const long long r = (pass + u * stride) * RPP + rsub;
            row[u] = r < n ? static_cast<int>(r) : -1;
            const char *rp = wbase + static_cast<size_t>(row[u] < 0 ? 0 : row[u]) * ROWB;
            hdr[u] = load_stream16(rp);
            q0[u] = load_stream16(rp + 16 + g * 32);
            q1[u] = load_stream16(rp + 32 + g * 32);
        }
        if (a.residual) {
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int t = 0; t < NT; t++)
                    res[u][t] = row[u] >= 0 && group_sum_owner<LPR>(lane) ? a.residual[static_cast<size_t>(t0 + t) * a.y_stride + row[u]] : 0.f;
        }
    }

    // AMAX: the lane also keeps the best (value, row) of what it stores (one row of activations)
    template <bool AMAX = false>
    __device__ __forceinline__ void compute(const shv_gemv_q4k_args &a, int g, int lane, const NibbleConsts &nc,
                                            const float (*xr)[64], const float *xs_lo, const float *xs_hi,
                                            const size_t *y_off, int t0, float *bv = nullptr, int *bi = nullptr) const {
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                float acc = q4k_group_dot(hdr[u], q0[u], q1[u], g, nc, xr[t], xs_lo[t], xs_hi[t]);
                acc = group_sum<LPR>(acc);
                if (row[u] >= 0 && group_sum_owner<LPR>(lane)) {
                    float r = acc;
                    if (a.residual) r += res[u][t];
                    a.y[y_off[t] + row[u]] = r;
                    if (a.y_flat) a.y_flat[row[u]] = r;  // one row (the launcher checks)
                    if constexpr (AMAX) {
                        if (amax_better(r, row[u], *bv, *bi)) { *bv = r; *bi = row[u]; }
                    }
                }
            }
        }
    }
};

// The grid's waves share the passes round-robin: wave w takes passes w, w + W, w + 2W, ... (W waves
// in the grid), so at any moment the chip streams one contiguous window of rows and no wave has
// more than one pass more than another.  U passes are loaded together; n_batches batches a wave.
// AMAX (one row): every block leaves the best (value, row) of the rows it wrote, and the block that
// arrives last names the row's first maximum as the next token, as the arg-max launch would.
template <int K, int NT, int U, bool AMAX = false>
__global__ __launch_bounds__(kBlock) void gemv_q4k_kernel(shv_gemv_q4k_args a, int n_batches, int t0, float *amax_val = nullptr,
                                                          int32_t *amax_idx = nullptr, int32_t *amax_counter = nullptr) {
    constexpr int LPR = K / 64;   // lanes per row
    constexpr int XPAD = K + K / 64 * 4;
    extern __shared__ float smem[];
    float(*xs)[XPAD] = reinterpret_cast<float(*)[XPAD]>(smem);
    __shared__ float red[4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gi = lane % LPR;   // 64-weight group of the row
    const int rsub = lane / LPR; // which of the pass's rows
    const int sb = gi >> 2, g = gi & 3;
    const char *wbase = static_cast<const char *>(a.w) + sb * SHV_Q4K_BYTES;
    const int n = a.n;
    const long long first_pass = static_cast<long long>(blockIdx.x) * kWavesPerBlock + wave;
    const long long stride = static_cast<long long>(gridDim.x) * kWavesPerBlock;

    // The first batch of weights does not depend on the activations: its loads go out before
    // the prologue so that HBM latency and the staging of x overlap.
    GemvBatch<K, NT, U> A, B;
    A.load(a, wbase, g, rsub, lane, first_pass, stride, n, t0);

    // where each row's ring slot is (its sequence's position and slot): asked for now, used by
    // the gated-norm prologue or by the final store
    int ring_row[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        ring_row[t] = 0;
        if (a.ring_slots > 0) {
            const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
            const int s = (t0 + t) / sl, i = (t0 + t) % sl;
            const int p = a.pos ? a.pos[s] : 0;
            const int slot = a.slot ? a.slot[s] : s;
            ring_row[t] = slot * a.ring_slots + (p + i) % a.ring_slots;
        }
    }

    // ---- stage pro(x) in LDS ----
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const float *x = a.x + static_cast<size_t>(t0 + t) * a.x_stride;
        if (a.prologue == SHV_PRO_RMSNORM) {
            float v[K / kBlock], gm[K / kBlock];  // gamma is asked for before the block-wide sum, not after it
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < K / kBlock; i++) {
                v[i] = x[tid + i * kBlock];
                gm[i] = a.gamma[tid + i * kBlock];
            }
#pragma unroll
            for (int i = 0; i < K / kBlock; i++) ss = fmaf(v[i], v[i], ss);
            ss = block_sum_256(ss, red);
            const float scale = 1.f / sqrtf(ss / static_cast<float>(K) + a.eps);
#pragma unroll
            for (int i = 0; i < K / kBlock; i++) xs[t][lds_slot(tid + i * kBlock)] = v[i] * scale * gm[i];
        } else if (a.prologue == SHV_PRO_GATED_NORM) {
            // thread owns K/256 consecutive columns; a head of head_dim columns spans
            // head_dim/(K/256) consecutive threads (a power of two <= 64).
            constexpr int PER = K / kBlock;
            const float *z = a.z + static_cast<size_t>(t0 + t) * a.z_stride;
            if (a.z_ring) z = a.z + static_cast<size_t>(ring_row[t]) * a.ring_stride;
            float v[PER], zv[PER], gm[PER];
            float ss = 0.f;
            const HeadSplit hs(a.head_dim);
#pragma unroll
            for (int i = 0; i < PER; i++) {
                v[i] = x[tid * PER + i];
                zv[i] = z[tid * PER + i];
                gm[i] = a.gamma[hs.dim(tid * PER + i)];
            }
#pragma unroll
            for (int i = 0; i < PER; i++) ss = fmaf(v[i], v[i], ss);
            const int span = a.head_dim / PER;
            for (int off = 1; off < span; off <<= 1) ss += __shfl_xor(ss, off, 64);
            const float scale = 1.f / sqrtf(ss / static_cast<float>(a.head_dim) + a.eps);
#pragma unroll
            for (int i = 0; i < PER; i++) {
                const int c = tid * PER + i;
                xs[t][lds_slot(c)] = v[i] * scale * gm[i] * sigmoid_fast(zv[i]);
            }
        } else if (a.prologue == SHV_PRO_RMSNORM_PAIR) {
            // two K/2-wide vectors, each with its own RMS, side by side
            if constexpr (K >= 2 * kBlock) {
                constexpr int HALF = K / kBlock / 2;
                const float *z = a.z + static_cast<size_t>(t0 + t) * a.z_stride;
                float v[2 * HALF], gm[2 * HALF];
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int i = 0; i < HALF; i++) {
                    v[i] = x[tid + i * kBlock];
                    v[HALF + i] = z[tid + i * kBlock];
                }
#pragma unroll
                for (int i = 0; i < 2 * HALF; i++) gm[i] = a.gamma[tid + i * kBlock];
#pragma unroll
                for (int i = 0; i < HALF; i++) {
                    s0 = fmaf(v[i], v[i], s0);
                    s1 = fmaf(v[HALF + i], v[HALF + i], s1);
                }
                s0 = block_sum_256(s0, red);
                s1 = block_sum_256(s1, red);
                const float sc0 = 1.f / sqrtf(s0 / static_cast<float>(K / 2) + a.eps);
                const float sc1 = 1.f / sqrtf(s1 / static_cast<float>(K / 2) + a.eps);
#pragma unroll
                for (int i = 0; i < 2 * HALF; i++) {
                    const int c = tid + i * kBlock;
                    xs[t][lds_slot(c)] = v[i] * (i < HALF ? sc0 : sc1) * gm[i];
                }
            }
        } else if (a.prologue == SHV_PRO_MUL_SIGMOID) {
            const float *z = a.z + static_cast<size_t>(t0 + t) * a.z_stride;
            const HeadSplit hs(a.head_dim > 0 ? a.head_dim : 1);
            float v[K / kBlock], zv[K / kBlock];
#pragma unroll
            for (int i = 0; i < K / kBlock; i++) {
                const int c = tid + i * kBlock;
                // head_dim > 0: z rows are [q (head_dim) | gate (head_dim)] per head and the gate
                // half is the one wanted (the fused query projection, llm/attn.go:162-166)
                const int zi = a.head_dim > 0 ? hs.head(c) * 2 * a.head_dim + a.head_dim + hs.dim(c) : c;
                v[i] = x[c];
                zv[i] = z[zi];
            }
#pragma unroll
            for (int i = 0; i < K / kBlock; i++) xs[t][lds_slot(tid + i * kBlock)] = v[i] * sigmoid_fast(zv[i]);
        } else {
#pragma unroll
            for (int i = 0; i < K / kBlock; i++) {
                const int c = tid + i * kBlock;
                xs[t][lds_slot(c)] = x[c];
            }
        }
    }
    __syncthreads();

    // ---- this lane's 64 activations per token ----
    float xr[NT][64];
    float xs_lo[NT], xs_hi[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) load_x_slice(xs[t], gi, xr[t], xs_lo[t], xs_hi[t]);

    size_t y_off[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        if (a.ring_slots > 0 && !a.z_ring) {
            y_off[t] = static_cast<size_t>(ring_row[t]) * a.ring_stride;
        } else {
            y_off[t] = static_cast<size_t>(t0 + t) * a.y_stride;
        }
    }

    const NibbleConsts nc = nibble_consts();
    const int nb = n_batches;  // double-buffered
    // "no candidate" is (-inf, n): any real element beats it, including -inf at a lower index
    float bv = -INFINITY;
    int bi = n;
    for (int b = 0; b < nb; b += 2) {
        const bool has_b = b + 1 < nb;
        if (has_b) B.load(a, wbase, g, rsub, lane, first_pass + static_cast<long long>(b + 1) * U * stride, stride, n, t0);
        A.template compute<AMAX>(a, g, lane, nc, xr, xs_lo, xs_hi, y_off, t0, &bv, &bi);
        if (has_b) {
            if (b + 2 < nb) A.load(a, wbase, g, rsub, lane, first_pass + static_cast<long long>(b + 2) * U * stride, stride, n, t0);
            B.template compute<AMAX>(a, g, lane, nc, xr, xs_lo, xs_hi, y_off, t0, &bv, &bi);
        }
    }
    if constexpr (AMAX) {
        __shared__ float sv[kWavesPerBlock];
        __shared__ int si[kWavesPerBlock];
        __shared__ int is_last;
        const int nblk = static_cast<int>(gridDim.x);
        amax_wave(bv, bi);
        if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
        __syncthreads();
        if (tid == 0) {
#pragma unroll
            for (int w = 1; w < kWavesPerBlock; w++)
                if (amax_better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
            store_agent(amax_val + blockIdx.x, bv);
            store_agent(amax_idx + blockIdx.x, bi);
        }
        if (!arrive_last(amax_counter, nblk, &is_last)) return;
        bv = -INFINITY;
        bi = n;
        for (int b = tid; b < nblk; b += kBlock) {
            const float v = load_agent(amax_val + b);
            const int i = load_agent(amax_idx + b);
            if (amax_better(v, i, bv, bi)) { bv = v; bi = i; }
        }
        amax_wave(bv, bi);
        if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
        __syncthreads();
        if (tid == 0) {
#pragma unroll
            for (int w = 1; w < kWavesPerBlock; w++)
                if (amax_better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
            if (bi >= n) bi = 0;  // a row of NaN has no element that is `>` -inf: the reference returns 0 there
            a.amax_best[0] = bi;
            if (a.amax_ids && a.amax_pos) {
                const int p = a.amax_pos[0] + (a.amax_advance > 0 ? a.amax_advance : 1);
                a.amax_ids[p] = bi;
                a.amax_pos[0] = p;
            }
        }
    }
}


// ---- one activation row (the decode step) ------------------------------------------------------
// A short launch is a chain of latencies, so this kernel keeps the chain short: the weights of all
// of a wave's passes are requested first; the input row is staged by all threads, four consecutive
// columns each (128-bit loads and LDS stores), together with the sums of every 32 columns, which
// the lanes would otherwise each add up again; there is ONE block-wide wait; and an RMS norm's
// scale, a scalar, is applied to the finished dot products instead of to the staged vector, so
// that the sum of squares does not stand between the loads and the staging.
// WAVES waves a block, P passes a wave (pass = 64/(K/64) rows); grid = ceil(passes / (WAVES*P)).
// STAGED (a variant kept for comparison): the lane of a super-block's first group decodes all
// eight (d*sc, dmin*m) pairs of the header and leaves them in LDS for the four lanes of the
// super-block, instead of every lane decoding its own group's from the header it holds anyway.
// FOLD: the launch also forms the router's logits of the MoE block that follows (a.fold: rows of
// k + n floats, [R diag(gamma) W | R diag(gamma)], against [pro(x) | residual]; see router_fold.hip).
// Every block takes two of those rows beside its own, four waves a row: a wave takes a quarter of
// the row's first k entries against the staged pro(x) and a quarter of its last n against the
// residual row, which it reads from memory itself (so y must be another buffer).
template <int K, int WAVES, int P, int PRO, bool STAGED = false, bool FOLD = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_row_kernel(shv_gemv_q4k_args a) {
    constexpr int T = WAVES * 64, LPR = K / 64, RPP = 64 / LPR, ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    constexpr int NV = K / 4 / T;  // float4 a thread stages
    static_assert(NV >= 1 && K % (4 * T) == 0, "threads of a block each stage whole float4s");
    constexpr int FN = 2048;                         // FOLD: the residual row's length
    constexpr int FA = K / 4 / 256, FB = FN / 4 / 256;  // float4 a lane loads of a wave's quarter: against pro(x), against the residual
    static_assert(!FOLD || (WAVES == 8 && K % 1024 == 0), "a fold row is split over four waves");
    __shared__ __align__(16) float xs[lds_padded(K)];
    __shared__ __align__(16) float xsum[K / 32];
    __shared__ float red[WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gi = lane % LPR, rsub = lane / LPR, sb = gi >> 2, g = gi & 3;
    const char *wbase = static_cast<const char *>(a.w) + sb * SHV_Q4K_BYTES;
    const long long pass0 = (static_cast<long long>(blockIdx.x) * WAVES + wave) * P;

    // Loads return in the order they were asked for, so the input row goes first: it comes from
    // cache in a fraction of the weights' latency, and the staging below (and the block-wide wait)
    // is over by the time the first weights arrive, instead of queueing behind all of them.
    int ring_row = 0;  // the ring slot of the row (its sequence's position and slot)
    if (a.ring_slots > 0) {
        const int p = a.pos ? a.pos[0] : 0;
        const int slot = a.slot ? a.slot[0] : 0;
        ring_row = slot * a.ring_slots + p % a.ring_slots;
    }
    float4 xv[NV], gv[NV], zv[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int c = 4 * (tid + T * j);
        xv[j] = *reinterpret_cast<const float4 *>(a.x + c);
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            gv[j] = *reinterpret_cast<const float4 *>(a.gamma + c);
        } else if constexpr (PRO == SHV_PRO_GATED_NORM) {
            const float *z = a.z_ring ? a.z + static_cast<size_t>(ring_row) * a.ring_stride : a.z;
            zv[j] = *reinterpret_cast<const float4 *>(z + c);
            gv[j] = *reinterpret_cast<const float4 *>(a.gamma + (c & (a.head_dim - 1)));
        } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
            // head_dim > 0: z rows are [q (head_dim) | gate (head_dim)] per head and the gate half is
            // the one wanted (the fused query projection, llm/attn.go:162-166)
            const HeadSplit hs(a.head_dim > 0 ? a.head_dim : 1);
            const int zi = a.head_dim > 0 ? hs.head(c) * 2 * a.head_dim + a.head_dim + hs.dim(c) : c;
            zv[j] = *reinterpret_cast<const float4 *>(a.z + zi);
        }
    }
    // FOLD: the wave's quarter of the residual row, asked for with the other inputs
    const int fold_row = static_cast<int>(blockIdx.x) * 2 + (wave >> 2), fold_q = wave & 3;
    float4 fx[FOLD ? FB : 1];
    if constexpr (FOLD) {
#pragma unroll
        for (int j = 0; j < FB; j++) fx[j] = *reinterpret_cast<const float4 *>(a.residual + fold_q * (FN / 4) + (j * 64 + lane) * 4);
    }
    Q4kLane w[P];
    int row[P];
#pragma unroll
    for (int u = 0; u < P; u++) {
        const long long r = (pass0 + u) * RPP + rsub;
        row[u] = r < a.n ? static_cast<int>(r) : -1;
        w[u].load(wbase + static_cast<size_t>(row[u] < 0 ? 0 : row[u]) * ROWB, g);
    }
    float res[P];
#pragma unroll
    for (int u = 0; u < P; u++) res[u] = (a.residual && row[u] >= 0 && group_sum_owner<LPR>(lane)) ? a.residual[row[u]] : 0.f;
    // the wave's quarter of its fold row, behind the weights
    float4 fw[FOLD ? FA + FB : 1];
    if constexpr (FOLD) {
        const float *fr = a.fold + static_cast<size_t>(fold_row < a.fold_rows ? fold_row : 0) * (K + FN);
#pragma unroll
        for (int j = 0; j < FA; j++) fw[j] = *reinterpret_cast<const float4 *>(fr + fold_q * (K / 4) + (j * 64 + lane) * 4);
#pragma unroll
        for (int j = 0; j < FB; j++) fw[FA + j] = *reinterpret_cast<const float4 *>(fr + K + fold_q * (FN / 4) + (j * 64 + lane) * 4);
    }

    // ---- stage pro(x): thread i of the block takes columns 4*(i + T*j) .. +3 ----
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int c = 4 * (tid + T * j);
        float4 v = xv[j];
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            const float4 gm = gv[j];
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
            v = make_float4(v.x * gm.x, v.y * gm.y, v.z * gm.z, v.w * gm.w);
        } else if constexpr (PRO == SHV_PRO_GATED_NORM) {
            // a head of head_dim columns is head_dim/4 consecutive threads (a power of two, 8..64)
            const float4 gm = gv[j], z4 = zv[j];
            float hs = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w)));
            const int span = a.head_dim >> 2;
            hs = sum8_all(hs);
            if (span >= 16) hs += dpp_f32<kDppMirror>(hs);
            if (span >= 32) hs += __shfl_xor(hs, 16, 64);
            if (span >= 64) hs += __shfl_xor(hs, 32, 64);
            const float sc = __builtin_amdgcn_rsqf(hs / static_cast<float>(a.head_dim) + a.eps);  // one instruction, one unit in the last place: this sits between the loads and the staging
            v = make_float4(v.x * sc * gm.x * sigmoid_fast(z4.x), v.y * sc * gm.y * sigmoid_fast(z4.y),
                            v.z * sc * gm.z * sigmoid_fast(z4.z), v.w * sc * gm.w * sigmoid_fast(z4.w));
        } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
            const float4 z4 = zv[j];
            v = make_float4(v.x * sigmoid_fast(z4.x), v.y * sigmoid_fast(z4.y), v.z * sigmoid_fast(z4.z), v.w * sigmoid_fast(z4.w));
        }
        *reinterpret_cast<float4 *>(&xs[lds_slot(c)]) = v;
        const float s8 = sum8_all((v.x + v.y) + (v.z + v.w));
        if ((lane & 7) == 0) xsum[c >> 5] = s8;
    }
    if constexpr (PRO == SHV_PRO_RMSNORM) {
        ss = wave_sum_all(ss);
        if (lane == 0) red[wave] = ss;
    }
    __syncthreads();
    float scale = 1.f;
    if constexpr (PRO == SHV_PRO_RMSNORM) {
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < WAVES; i++) tot += red[i];
        scale = __builtin_amdgcn_rsqf(tot / static_cast<float>(K) + a.eps);
    }

    float xr[64], xs_lo, xs_hi;
    load_x_slice_presummed(xs, xsum, gi, xr, xs_lo, xs_hi);
    float *y = a.y;
    if (a.ring_slots > 0 && !a.z_ring) y += static_cast<size_t>(ring_row) * a.ring_stride;
    const NibbleConsts nc = nibble_consts();
    __shared__ float4 staged_sc[STAGED ? WAVES * P * 64 : 1];
    if constexpr (STAGED) {
#pragma unroll
        for (int u = 0; u < P; u++) {
            if (g == 0) {
                const float d = f16_bits_to_f32(w[u].hdr.x), dmin = f16_bits_to_f32(w[u].hdr.x >> 16);
#pragma unroll
                for (int gg = 0; gg < 4; gg++) {
                    uint32_t sc, mn;
                    q4k_group_scale_min(w[u].hdr, gg, sc, mn);
                    staged_sc[(wave * P + u) * 64 + lane + gg] = make_float4(d * static_cast<float>(sc & 0xFFu), d * static_cast<float>(sc >> 8),
                                                                              dmin * static_cast<float>(mn & 0xFFu), dmin * static_cast<float>(mn >> 8));
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int u = 0; u < P; u++) {
        float acc;
        if constexpr (STAGED) acc = q4k_group_dot_scaled(w[u].q0, w[u].q1, staged_sc[(wave * P + u) * 64 + lane], nc, xr, xs_lo, xs_hi);
        else acc = w[u].dot(g, nc, xr, xs_lo, xs_hi);
        acc = group_sum<LPR>(acc);
        if (row[u] >= 0 && group_sum_owner<LPR>(lane)) {
            const float v = fmaf(acc, scale, res[u]);
            y[row[u]] = v;
            if (a.y_flat) a.y_flat[row[u]] = v;
        }
    }
    if constexpr (FOLD) {
        // the quarter row against the same columns of [pro(x) | residual]; the four quarters meet in
        // LDS and are added in a fixed order
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < FA; j++) {
            const float4 xv4 = *reinterpret_cast<const float4 *>(&xs[lds_slot(fold_q * (K / 4) + (j * 64 + lane) * 4)]);
            acc = fmaf(fw[j].x, xv4.x, fmaf(fw[j].y, xv4.y, fmaf(fw[j].z, xv4.z, fmaf(fw[j].w, xv4.w, acc))));
        }
#pragma unroll
        for (int j = 0; j < FB; j++) acc = fmaf(fw[FA + j].x, fx[j].x, fmaf(fw[FA + j].y, fx[j].y, fmaf(fw[FA + j].z, fx[j].z, fmaf(fw[FA + j].w, fx[j].w, acc))));
        acc = wave_sum_all(acc);
        __syncthreads();  // red is free again: every wave has its scale
        if (lane == 0) red[wave] = acc;
        __syncthreads();
        if ((tid & 255) == 0 && fold_row < a.fold_rows) a.fold_out[fold_row] = (red[wave] + red[wave + 1]) + (red[wave + 2] + red[wave + 3]);
    }
}

// ---- two to four activation rows (a verification pass, a short prompt tail, a few sequences' steps) ------
// The one-row kernel's shape with the rows side by side: every row's inputs first, the weights of
// the wave's passes once, each row staged with its sums, one block-wide wait, then the lane walks
// the rows with its weights in registers (a row's 64 activations come from LDS when its turn comes).
template <int K, int WAVES, int P, int PRO, int NT, bool FOLD = false>
__global__ __launch_bounds__(WAVES * 64) void gemv_fewrows_kernel(shv_gemv_q4k_args a) {
    constexpr int T = WAVES * 64, LPR = K / 64, RPP = 64 / LPR, ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    constexpr int NV = K / 4 / T;
    static_assert(NV >= 1 && K % (4 * T) == 0, "threads of a block each stage whole float4s");
    // FOLD: the router's rows beside the block's own, as in the one-row kernel, against every row
    constexpr int FN = 2048, FA = K / 4 / 256, FB = FN / 4 / 256;
    static_assert(!FOLD || (WAVES == 8 && K % 1024 == 0), "a fold row is split over four waves");
    __shared__ __align__(16) float xs[NT][lds_padded(K)];
    __shared__ __align__(16) float xsum[NT][K / 32];
    __shared__ float red[NT][WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gi = lane % LPR, rsub = lane / LPR, sb = gi >> 2, g = gi & 3;
    const char *wbase = static_cast<const char *>(a.w) + sb * SHV_Q4K_BYTES;
    const long long pass0 = (static_cast<long long>(blockIdx.x) * WAVES + wave) * P;
    // row t is row t % seq_len of sequence t / seq_len: its ring row follows that sequence's position and slot
    const int seq_rows = a.seq_len > 0 ? a.seq_len : a.n_tok;
    int ring_row[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        ring_row[t] = 0;
        if (a.ring_slots > 0) {
            const int s = t / seq_rows;
            ring_row[t] = (a.slot ? a.slot[s] : s) * a.ring_slots + ((a.pos ? a.pos[s] : 0) + t % seq_rows) % a.ring_slots;
        }
    }
    float4 xv[NT][NV], gv[NV], zv[NT][NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int c = 4 * (tid + T * j);
        if constexpr (PRO == SHV_PRO_RMSNORM) gv[j] = *reinterpret_cast<const float4 *>(a.gamma + c);
        else if constexpr (PRO == SHV_PRO_GATED_NORM) gv[j] = *reinterpret_cast<const float4 *>(a.gamma + (c & (a.head_dim - 1)));
#pragma unroll
        for (int t = 0; t < NT; t++) {
            xv[t][j] = *reinterpret_cast<const float4 *>(a.x + static_cast<size_t>(t) * a.x_stride + c);
            if constexpr (PRO == SHV_PRO_GATED_NORM) {
                const float *z = a.z_ring ? a.z + static_cast<size_t>(ring_row[t]) * a.ring_stride
                                          : a.z + static_cast<size_t>(t) * a.z_stride;
                zv[t][j] = *reinterpret_cast<const float4 *>(z + c);
            } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
                const HeadSplit hs(a.head_dim > 0 ? a.head_dim : 1);
                const int zi = a.head_dim > 0 ? hs.head(c) * 2 * a.head_dim + a.head_dim + hs.dim(c) : c;
                zv[t][j] = *reinterpret_cast<const float4 *>(a.z + static_cast<size_t>(t) * a.z_stride + zi);
            }
        }
    }
    const int fold_row = static_cast<int>(blockIdx.x) * 2 + (wave >> 2), fold_q = wave & 3;
    float4 fx[FOLD ? NT : 1][FOLD ? FB : 1];
    if constexpr (FOLD) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int j = 0; j < FB; j++) fx[t][j] = *reinterpret_cast<const float4 *>(a.residual + static_cast<size_t>(t) * a.y_stride + fold_q * (FN / 4) + (j * 64 + lane) * 4);
    }
    Q4kLane w[P];
    int row[P];
#pragma unroll
    for (int u = 0; u < P; u++) {
        const long long r = (pass0 + u) * RPP + rsub;
        row[u] = r < a.n ? static_cast<int>(r) : -1;
        w[u].load(wbase + static_cast<size_t>(row[u] < 0 ? 0 : row[u]) * ROWB, g);
    }
    float res[NT][P];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int u = 0; u < P; u++)
            res[t][u] = (a.residual && row[u] >= 0 && group_sum_owner<LPR>(lane)) ? a.residual[static_cast<size_t>(t) * a.y_stride + row[u]] : 0.f;
    float4 fw[FOLD ? FA + FB : 1];
    if constexpr (FOLD) {
        const float *fr = a.fold + static_cast<size_t>(fold_row < a.fold_rows ? fold_row : 0) * (K + FN);
#pragma unroll
        for (int j = 0; j < FA; j++) fw[j] = *reinterpret_cast<const float4 *>(fr + fold_q * (K / 4) + (j * 64 + lane) * 4);
#pragma unroll
        for (int j = 0; j < FB; j++) fw[FA + j] = *reinterpret_cast<const float4 *>(fr + K + fold_q * (FN / 4) + (j * 64 + lane) * 4);
    }

#pragma unroll
    for (int t = 0; t < NT; t++) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int c = 4 * (tid + T * j);
            float4 v = xv[t][j];
            if constexpr (PRO == SHV_PRO_RMSNORM) {
                const float4 gm = gv[j];
                ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
                v = make_float4(v.x * gm.x, v.y * gm.y, v.z * gm.z, v.w * gm.w);
            } else if constexpr (PRO == SHV_PRO_GATED_NORM) {
                const float4 gm = gv[j], z4 = zv[t][j];
                float hs = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w)));
                const int span = a.head_dim >> 2;
                hs = sum8_all(hs);
                if (span >= 16) hs += dpp_f32<kDppMirror>(hs);
                if (span >= 32) hs += __shfl_xor(hs, 16, 64);
                if (span >= 64) hs += __shfl_xor(hs, 32, 64);
                const float sc = __builtin_amdgcn_rsqf(hs / static_cast<float>(a.head_dim) + a.eps);
                v = make_float4(v.x * sc * gm.x * sigmoid_fast(z4.x), v.y * sc * gm.y * sigmoid_fast(z4.y),
                                v.z * sc * gm.z * sigmoid_fast(z4.z), v.w * sc * gm.w * sigmoid_fast(z4.w));
            } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
                const float4 z4 = zv[t][j];
                v = make_float4(v.x * sigmoid_fast(z4.x), v.y * sigmoid_fast(z4.y), v.z * sigmoid_fast(z4.z), v.w * sigmoid_fast(z4.w));
            }
            *reinterpret_cast<float4 *>(&xs[t][lds_slot(c)]) = v;
            const float s8 = sum8_all((v.x + v.y) + (v.z + v.w));
            if ((lane & 7) == 0) xsum[t][c >> 5] = s8;
        }
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            ss = wave_sum_all(ss);
            if (lane == 0) red[t][wave] = ss;
        }
    }
    __syncthreads();
    const NibbleConsts nc = nibble_consts();
#pragma unroll
    for (int t = 0; t < NT; t++) {
        float scale = 1.f;
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            float tot = 0.f;
#pragma unroll
            for (int i = 0; i < WAVES; i++) tot += red[t][i];
            scale = __builtin_amdgcn_rsqf(tot / static_cast<float>(K) + a.eps);
        }
        float xr[64], xs_lo, xs_hi;
        load_x_slice_presummed(xs[t], xsum[t], gi, xr, xs_lo, xs_hi);
        float *y = a.y + static_cast<size_t>(t) * a.y_stride;
        if (a.ring_slots > 0 && !a.z_ring) y = a.y + static_cast<size_t>(ring_row[t]) * a.ring_stride;
#pragma unroll
        for (int u = 0; u < P; u++) {
            float acc = w[u].dot(g, nc, xr, xs_lo, xs_hi);
            acc = group_sum<LPR>(acc);
            if (row[u] >= 0 && group_sum_owner<LPR>(lane)) y[row[u]] = fmaf(acc, scale, res[t][u]);
        }
    }
    if constexpr (FOLD) {
        float facc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < FA; j++) {
                const float4 xv4 = *reinterpret_cast<const float4 *>(&xs[t][lds_slot(fold_q * (K / 4) + (j * 64 + lane) * 4)]);
                acc = fmaf(fw[j].x, xv4.x, fmaf(fw[j].y, xv4.y, fmaf(fw[j].z, xv4.z, fmaf(fw[j].w, xv4.w, acc))));
            }
#pragma unroll
            for (int j = 0; j < FB; j++) acc = fmaf(fw[FA + j].x, fx[t][j].x, fmaf(fw[FA + j].y, fx[t][j].y, fmaf(fw[FA + j].z, fx[t][j].z, fmaf(fw[FA + j].w, fx[t][j].w, acc))));
            facc[t] = wave_sum_all(acc);
        }
        __syncthreads();  // red is free again: every wave has its scales
        if (lane == 0) {
#pragma unroll
            for (int t = 0; t < NT; t++) red[t][wave] = facc[t];
        }
        __syncthreads();
        // a.fold_stride floats from one row's products to the next
        if ((tid & 255) < NT && fold_row < a.fold_rows) {
            const int t = tid & 255;
            a.fold_out[static_cast<size_t>(t) * a.fold_stride + fold_row] = (red[t][wave] + red[t][wave + 1]) + (red[t][wave + 2] + red[t][wave + 3]);
        }
    }
}

template <int K, int WAVES, int P, int NT>
int launch_fewrows_kpn(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    constexpr int RPP = 64 / (K / 64);
    const long long passes = (static_cast<long long>(a.n) + RPP - 1) / RPP;
    const dim3 grid(static_cast<unsigned>((passes + WAVES * P - 1) / (WAVES * P))), block(WAVES * 64);
    switch (a.prologue) {
        case SHV_PRO_NONE: SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, P, SHV_PRO_NONE, NT>), grid, block, 0, a); break;
        case SHV_PRO_RMSNORM: SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, P, SHV_PRO_RMSNORM, NT>), grid, block, 0, a); break;
        case SHV_PRO_GATED_NORM: SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, P, SHV_PRO_GATED_NORM, NT>), grid, block, 0, a); break;
        default: SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, P, SHV_PRO_MUL_SIGMOID, NT>), grid, block, 0, a); break;
    }
    return SHV_OK;
}

template <int NT>
int launch_fewrows_fold(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    constexpr int K = 4096, WAVES = 8;
    const int rows_blocks = (a.n + WAVES - 1) / WAVES, fold_blocks = (a.fold_rows + 1) / 2;
    const dim3 grid(static_cast<unsigned>(rows_blocks > fold_blocks ? rows_blocks : fold_blocks)), block(WAVES * 64);
    if (a.prologue == SHV_PRO_GATED_NORM) SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, 1, SHV_PRO_GATED_NORM, NT, true>), grid, block, 0, a);
    else if (a.prologue == SHV_PRO_MUL_SIGMOID) SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, 1, SHV_PRO_MUL_SIGMOID, NT, true>), grid, block, 0, a);
    else SHV_LAUNCH(ctx, (gemv_fewrows_kernel<K, WAVES, 1, SHV_PRO_NONE, NT, true>), grid, block, 0, a);
    return SHV_OK;
}

template <int NT>
int launch_fewrows(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (a.fold) return launch_fewrows_fold<NT>(ctx, a);
    if (a.k == 4096) return launch_fewrows_kpn<4096, 8, 1, NT>(ctx, a);
    if (a.n <= 2 * 4 * 2 * ctx->prop.multiProcessorCount) return launch_fewrows_kpn<2048, 4, 1, NT>(ctx, a);
    return launch_fewrows_kpn<2048, 4, 2, NT>(ctx, a);
}

// Which one-row launches the kernel above takes: the decode step's projections (2048- and
// 4096-wide inputs).  A matrix of very many rows (the vocabulary projection) is a stream, not a
// latency, and stays on the looping kernel; so do the other widths and the pair-norm prologue.
template <int K, int WAVES, int P>
int launch_row_kp(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    constexpr int RPP = 64 / (K / 64);
    const long long passes = (static_cast<long long>(a.n) + RPP - 1) / RPP;
    const dim3 grid(static_cast<unsigned>((passes + WAVES * P - 1) / (WAVES * P))), block(WAVES * 64);
    if (ctx->gemv_scales_lds) {
        switch (a.prologue) {
            case SHV_PRO_NONE: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_NONE, true>), grid, block, 0, a); break;
            case SHV_PRO_RMSNORM: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_RMSNORM, true>), grid, block, 0, a); break;
            case SHV_PRO_GATED_NORM: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_GATED_NORM, true>), grid, block, 0, a); break;
            default: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_MUL_SIGMOID, true>), grid, block, 0, a); break;
        }
        return SHV_OK;
    }
    switch (a.prologue) {
        case SHV_PRO_NONE: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_NONE>), grid, block, 0, a); break;
        case SHV_PRO_RMSNORM: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_RMSNORM>), grid, block, 0, a); break;
        case SHV_PRO_GATED_NORM: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_GATED_NORM>), grid, block, 0, a); break;
        default: SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, P, SHV_PRO_MUL_SIGMOID>), grid, block, 0, a); break;
    }
    return SHV_OK;
}

// Two to four rows (of one sequence or of several) take the rows-side-by-side form of the same kernel.
bool fewrows_kernel_covers(const shv_ctx *ctx, const shv_gemv_q4k_args &a);

bool row_kernel_covers(const shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (a.n_tok != 1 || a.prologue == SHV_PRO_RMSNORM_PAIR) return false;
    if (a.k != 2048 && a.k != 4096) return false;
    if (!shv_aligned16(a.x) || (a.gamma && !shv_aligned16(a.gamma)) || (a.z && !shv_aligned16(a.z))) return false;
    if (a.prologue == SHV_PRO_GATED_NORM && (a.head_dim < 32 || a.head_dim > 256 || (a.z_ring && a.ring_stride % 4 != 0))) return false;
    if (a.prologue == SHV_PRO_MUL_SIGMOID && a.head_dim != 0 && a.head_dim < 4) return false;
    // more rounds of the chip than a few: a stream
    const long long passes = static_cast<long long>(a.n) / (64 / (a.k / 64));
    return passes <= static_cast<long long>(ctx->prop.multiProcessorCount) * 4 * 8;
}

bool fewrows_kernel_covers(const shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (a.n_tok < 2 || a.n_tok > 4 || a.y_flat) return false;
    // whole sequences of equal length (one of n_tok rows, or n_tok of one row each)
    const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
    if (sl < 1 || a.n_tok % sl != 0) return false;
    if (a.x_stride % 4 != 0 || ((a.prologue == SHV_PRO_GATED_NORM || a.prologue == SHV_PRO_MUL_SIGMOID) && !a.z_ring && a.z_stride % 4 != 0)) return false;
    shv_gemv_q4k_args one = a;
    one.n_tok = 1;
    return row_kernel_covers(ctx, one);
}

// The output projection of a decode step with the router's rows of the MoE block behind it.
int launch_row_fold(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    constexpr int K = 4096, WAVES = 8;
    const int rows_blocks = (a.n + WAVES - 1) / WAVES, fold_blocks = (a.fold_rows + 1) / 2;
    const dim3 grid(static_cast<unsigned>(rows_blocks > fold_blocks ? rows_blocks : fold_blocks)), block(WAVES * 64);
    if (a.prologue == SHV_PRO_GATED_NORM) SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, 1, SHV_PRO_GATED_NORM, false, true>), grid, block, 0, a);
    else if (a.prologue == SHV_PRO_MUL_SIGMOID) SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, 1, SHV_PRO_MUL_SIGMOID, false, true>), grid, block, 0, a);
    else SHV_LAUNCH(ctx, (gemv_row_kernel<K, WAVES, 1, SHV_PRO_NONE, false, true>), grid, block, 0, a);
    return SHV_OK;
}

int launch_row(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (a.fold) return launch_row_fold(ctx, a);
    if (a.k == 4096) return launch_row_kp<4096, 8, 1>(ctx, a);
    // two rows a pass at this width: one pass a wave up to a block a compute unit's worth of
    // rows, two above that
    if (a.n <= 2 * 4 * 2 * ctx->prop.multiProcessorCount) return launch_row_kp<2048, 4, 1>(ctx, a);
    return launch_row_kp<2048, 4, 2>(ctx, a);
}

template <int K, int NT, int U>
int launch_ntu(shv_ctx *ctx, const shv_gemv_q4k_args &a, dim3 grid, dim3 block, size_t lds, int ppw, int t0) {
    if (lds > 48 * 1024) {
        // above the default dynamic-LDS allowance the limit has to be raised once per kernel
        static std::atomic<bool> raised{false};
        if (!raised.load(std::memory_order_acquire)) {
            SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4k_kernel<K, NT, U>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            raised.store(true, std::memory_order_release);
        }
    }
    if constexpr (NT == 1) {
        if (a.amax_best) {
            SHV_REQUIRE(grid.x <= static_cast<unsigned>(shv_ctx::kGemvAmaxBlocks) && ctx->gemv_amax_val && ctx->gemv_amax_idx, "gemv_q4k: arg-max over %u blocks", grid.x);
            if (lds > 48 * 1024) SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4k_kernel<K, NT, U, true>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            SHV_LAUNCH(ctx, (gemv_q4k_kernel<K, NT, U, true>), grid, block, lds, a, ppw, t0, ctx->gemv_amax_val, ctx->gemv_amax_idx,
                       ctx->counters + shv_ctx::kCounterGemvAmax);
            return SHV_OK;
        }
    }
    SHV_LAUNCH(ctx, (gemv_q4k_kernel<K, NT, U>), grid, block, lds, a, ppw, t0, static_cast<float *>(nullptr), static_cast<int32_t *>(nullptr), static_cast<int32_t *>(nullptr));
    return SHV_OK;
}

template <int K, int NT>
int launch_nt(shv_ctx *ctx, const shv_gemv_q4k_args &a, dim3 grid, dim3 block, size_t lds, int ppw, int u, int t0) {
    switch (u) {
        case 1: return launch_ntu<K, NT, 1>(ctx, a, grid, block, lds, ppw, t0);
        case 2: return launch_ntu<K, NT, 2>(ctx, a, grid, block, lds, ppw, t0);
        case 3: return launch_ntu<K, NT, 3>(ctx, a, grid, block, lds, ppw, t0);
        default: return launch_ntu<K, NT, 4>(ctx, a, grid, block, lds, ppw, t0);
    }
}

template <int K>
int launch_k(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    constexpr int RPP = 64 / (K / 64);
    const long long passes = (static_cast<long long>(a.n) + RPP - 1) / RPP;
    // One round of resident blocks (two waves per SIMD at this kernel's register count, i.e. two
    // blocks per CU): every wave of the grid is on the chip at once.  Up to four passes of a wave
    // are loaded together; longer shares run as double-buffered batches of four.
    const long long resident = static_cast<long long>(ctx->prop.multiProcessorCount) * 2;
    long long blocks = (passes + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > resident) blocks = resident;
    // Every block stages (and for the gated prologues, transforms) the whole input row, which at
    // 4096 columns is a visible part of a short kernel: there a wave takes two passes and the
    // grid is half as many blocks.
    if (K >= 4096) {
        const long long half = (passes + 2 * kWavesPerBlock - 1) / (2 * kWavesPerBlock);
        if (half < blocks) blocks = half;
    }
    long long waves = blocks * kWavesPerBlock;
    long long iters = (passes + waves - 1) / waves;
    int u = iters < 4 ? static_cast<int>(iters) : 4;
    // A matrix of many rounds (the vocabulary projection: 37) is a stream, not a latency: one pass
    // at a time leaves registers for a third wave per SIMD, which hides more of the arithmetic
    // behind the loads (42 -> 36 us for 175 MB).
    if (iters >= 8 && a.n_tok == 1) {
        blocks = static_cast<long long>(ctx->prop.multiProcessorCount) * 3;
        waves = blocks * kWavesPerBlock;
        iters = (passes + waves - 1) / waves;
        u = 1;
    }
    const long long ppw = (iters + u - 1) / u;  // batches per wave
    SHV_REQUIRE(blocks > 0 && ppw < (1ll << 31), "gemv_q4k: grid of %lld blocks", blocks);
    dim3 grid(static_cast<unsigned>(blocks)), block(kBlock);
    // more than kMaxTok rows: several launches of up to kMaxTok rows each over the same weights
    for (int t0 = 0; t0 < a.n_tok; t0 += kMaxTok) {
        const int nt = a.n_tok - t0 < kMaxTok ? a.n_tok - t0 : kMaxTok;
        const size_t lds = static_cast<size_t>(nt) * (K + K / 64 * 4) * sizeof(float);
        int rc;
        switch (nt) {
            case 1: rc = launch_nt<K, 1>(ctx, a, grid, block, lds, static_cast<int>(ppw), u, t0); break;
            case 2: rc = launch_nt<K, 2>(ctx, a, grid, block, lds, static_cast<int>(ppw), u, t0); break;
            case 3: rc = launch_nt<K, 3>(ctx, a, grid, block, lds, static_cast<int>(ppw), u, t0); break;
            default: rc = launch_nt<K, 4>(ctx, a, grid, block, lds, static_cast<int>(ppw), u, t0); break;
        }
        if (rc != SHV_OK) return rc;
    }
    return SHV_OK;
}

}  // namespace

int shv_launch_gemv_q4k(shv_ctx *ctx, const shv_gemv_q4k_args *pa) {
    const shv_gemv_q4k_args &a = *pa;
    SHV_REQUIRE(a.w && a.x && a.y, "gemv_q4k: NULL w, x or y");
    SHV_REQUIRE(a.n > 0, "gemv_q4k: n = %d", a.n);
    SHV_REQUIRE(a.n_tok >= 1 && a.n_tok <= 4096, "gemv_q4k: n_tok %d; a pass carries 1..4096 rows", a.n_tok);
    SHV_REQUIRE(shv_aligned16(a.w), "gemv_q4k: w must be 16-byte aligned");
    const int x_width = a.prologue == SHV_PRO_RMSNORM_PAIR ? a.k / 2 : a.k;
    SHV_REQUIRE(a.x_stride >= x_width || a.n_tok == 1, "gemv_q4k: x_stride %d < %d", a.x_stride, x_width);
    SHV_REQUIRE(a.y_stride >= a.n || a.n_tok == 1 || a.ring_slots > 0, "gemv_q4k: y_stride %d < n %d", a.y_stride, a.n);
    SHV_REQUIRE(a.prologue >= SHV_PRO_NONE && a.prologue <= SHV_PRO_RMSNORM_PAIR, "gemv_q4k: prologue %d", a.prologue);
    if (a.prologue == SHV_PRO_RMSNORM_PAIR)
        SHV_REQUIRE(a.gamma && a.z && a.k >= 512 && (a.z_stride >= a.k / 2 || a.n_tok == 1), "gemv_q4k: pair-norm prologue needs gamma, z and k >= 512");
    if (a.prologue == SHV_PRO_RMSNORM) SHV_REQUIRE(a.gamma, "gemv_q4k: RMSNorm prologue without gamma");
    if (a.prologue == SHV_PRO_GATED_NORM) {
        SHV_REQUIRE(a.gamma && a.z, "gemv_q4k: gated-norm prologue without gamma or z");
        const int per = a.k / kBlock;
        SHV_REQUIRE(a.head_dim > 0 && a.k % a.head_dim == 0 && per > 0 && a.head_dim % per == 0 &&
                        a.head_dim / per <= 64 && ((a.head_dim / per) & (a.head_dim / per - 1)) == 0,
                    "gemv_q4k: gated-norm head_dim %d does not tile k %d", a.head_dim, a.k);
    }
    if (a.prologue == SHV_PRO_MUL_SIGMOID)
        SHV_REQUIRE(a.z && a.head_dim >= 0 && (a.head_dim & (a.head_dim - 1)) == 0, "gemv_q4k: sigmoid-gate prologue needs z and a head_dim that is 0 or a power of two (%d)", a.head_dim);
    if (a.z_ring) SHV_REQUIRE(a.prologue == SHV_PRO_GATED_NORM && a.ring_slots > 0, "gemv_q4k: z_ring needs the gated-norm prologue and a ring");
    SHV_REQUIRE(!a.y_flat || (a.n_tok == 1 && a.ring_slots > 0 && !a.z_ring), "gemv_q4k: y_flat goes with ring output of one row");
    if (a.ring_slots > 0) {
        const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
        SHV_REQUIRE((a.z_ring || (a.ring_stride >= a.n && !a.residual)) && sl <= a.ring_slots && a.n_tok % sl == 0,
                    "gemv_q4k: ring of %d slots, stride %d, sequences of %d in %d rows", a.ring_slots, a.ring_stride, sl, a.n_tok);
    }
    if (a.fold) {
        SHV_REQUIRE(a.n_tok >= 1 && a.n_tok <= 4 && a.k == 4096 && a.n == 2048 && a.residual && a.fold_out && a.fold_rows >= 1 && (a.ring_slots == 0 || a.z_ring),
                    "gemv_q4k: the router's rows ride on a 2048 x 4096 projection of one to four rows with a residual (n_tok %d, n %d, k %d)", a.n_tok, a.n, a.k);
        SHV_REQUIRE(a.prologue == SHV_PRO_NONE || a.prologue == SHV_PRO_GATED_NORM || a.prologue == SHV_PRO_MUL_SIGMOID, "gemv_q4k: fold with prologue %d", a.prologue);
        SHV_REQUIRE(a.residual != a.y && shv_aligned16(a.residual) && shv_aligned16(a.fold) && a.y_stride % 4 == 0,
                    "gemv_q4k: fold reads the whole residual row while y is written: they must be different, 16-byte aligned buffers");
        SHV_REQUIRE(a.n_tok == 1 || a.fold_stride >= a.fold_rows, "gemv_q4k: fold_stride %d < fold_rows %d", a.fold_stride, a.fold_rows);
        SHV_REQUIRE(!ctx->gemv_scales_lds && !ctx->mfma_rows_forced && (a.n_tok == 1 ? row_kernel_covers(ctx, a) : fewrows_kernel_covers(ctx, a)),
                    "gemv_q4k: fold needs the row kernels' shapes and alignment of x, gamma and z (whole sequences of equal length)");
    }
    if (a.amax_best) {
        SHV_REQUIRE(a.n_tok == 1 && a.ring_slots == 0 && !a.fold && !a.residual, "gemv_q4k: the arg-max in the launch goes with one plain row of outputs");
        SHV_REQUIRE((a.amax_ids == nullptr) == (a.amax_pos == nullptr) && a.amax_advance >= 0, "gemv_q4k: amax_ids and amax_pos go together");
        switch (a.k) {  // straight to the looping kernel: the short launches' kernel has no arg-max
            case 512: return launch_k<512>(ctx, a);
            case 1024: return launch_k<1024>(ctx, a);
            case 2048: return launch_k<2048>(ctx, a);
            case 4096: return launch_k<4096>(ctx, a);
            default: return shv_set_error(SHV_E_INVALID, "gemv_q4k: k = %d; built for 512, 1024, 2048 and 4096", a.k);
        }
    }
    // two to eight rows: every weight formed once for all of them, the products on the matrix cores; 4096 columns
    // wide, up to four rows are quicker side by side in the one-row kernel's shape (6.7 against
    // 8.0 us for three rows of a 2048 x 4096 output projection: a block there stages 16 K columns a row)
    const bool few = fewrows_kernel_covers(ctx, a) && !ctx->mfma_rows_forced;
    if (!ctx->mfma_rows_forced && !(few && a.k == 4096) && shv_gemv_mrows_covers(ctx, a)) return shv_launch_gemv_mrows(ctx, a);
    // (SHV_MFMA_MIN_ROWS at or below the row count sends few rows to the tiled matrix-core kernels instead, as before)
    if (few)
        return a.n_tok == 2 ? launch_fewrows<2>(ctx, a) : a.n_tok == 3 ? launch_fewrows<3>(ctx, a) : launch_fewrows<4>(ctx, a);
    if (a.n_tok >= (a.k > 2048 ? ctx->mfma_min_rows_wide : ctx->mfma_min_rows) && shv_gemm_q4k_covers(a)) return shv_launch_gemm_q4k(ctx, a);
    SHV_REQUIRE(a.n_tok <= 64, "gemv_q4k: %d rows: more than 64 go through the matrix-core kernel, which does not take this shape (k %d, prologue %d)",
                a.n_tok, a.k, a.prologue);
    if (row_kernel_covers(ctx, a)) return launch_row(ctx, a);
    switch (a.k) {
        case 512: return launch_k<512>(ctx, a);
        case 1024: return launch_k<1024>(ctx, a);
        case 2048: return launch_k<2048>(ctx, a);
        case 4096: return launch_k<4096>(ctx, a);
        default: return shv_set_error(SHV_E_INVALID, "gemv_q4k: k = %d; built for 512, 1024, 2048 and 4096", a.k);
    }
}
