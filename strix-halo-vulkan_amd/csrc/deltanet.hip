// Gated DeltaNet decode step: causal conv1d + SiLU + L2 norm of q/k, decay and write strength,
// and the delta-rule update of the 128x128 float32 state of each value head.
//
// HBM-bound on the state (read once, written once per call).  A 256-thread block owns 8 of a
// head's 128 state rows (row j holds column j of S, contiguous over the key axis): a wave holds
// two rows, 32 lanes x float4 each, in registers across all tokens of the call, and reduces the
// two dot products of the rule (against k, then against q) over those 32 lanes with DPP.  The
// cheap per-head prologue (conv, norm, gate) is recomputed by every block of the head so that no
// grid-wide hand-over is needed.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kD = 128;       // head dimension the kernel is built for
constexpr int kRowsPerBlock = 8;

// Sum over aligned groups of 32 lanes, result in every lane of the group.
__device__ __forceinline__ float sum32_all(float v) {
    v += dpp_f32<kDppXor1>(v);
    v += dpp_f32<kDppXor2>(v);
    v += dpp_f32<kDppHalfMirror>(v);
    v += dpp_f32<kDppMirror>(v);
    v += __shfl_xor(v, 16, 64);
    return v;
}

__device__ __forceinline__ float softplus_ref(float x) {
    // the add inside the log is float32 on purpose: below about -16.6 it returns exactly 0
    return x > 20.f ? x : logf(1.f + expf(x));
}

// Causal depthwise conv of kernel 4 for channel ch at position p: taps 0..3 meet positions
// p-3..p; rows before the sequence start are zero.
__device__ __forceinline__ float conv4(const float *ring, int ring_slots, int ring_stride, const float *taps, int ch, int p) {
    const float4 k = *reinterpret_cast<const float4 *>(taps + static_cast<size_t>(ch) * 4);
    const float kk[4] = {k.x, k.y, k.z, k.w};
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int pp = p + j - 3;
        const float x = pp < 0 ? 0.f : ring[static_cast<size_t>(pp % ring_slots) * ring_stride + ch];
        s += x * kk[j];
    }
    return s;
}

constexpr int kPrep = 8;  // rows of a sequence whose conv, norms and gates are prepared together

// grid: (128/(4*RW) row chunks, n_head_v, n_seq); RW state rows a wave (two, 32 lanes x float4 each;
// or four, two to a lane, for calls of several sequences, whose many small blocks would otherwise
// queue for the chip and prepare their heads twice as often).  The rows of a call go in groups of kPrep: first
// everything that does not depend on the state is worked out for the whole group, all threads
// busy (a thread keeps the sliding window of its channel's ring values, so a row costs one load);
// then the waves walk the group's rows with nothing between two rows but their own two
// reductions.
template <int RW>
__global__ __launch_bounds__(kBlock) void dn_step_kernel(shv_dn_step_args a) {
    constexpr int kRowsPerBlock = 4 * RW, NS = RW / 2;  // NS: state rows a lane holds four values of
    __shared__ __align__(16) float qs[kPrep][kD];
    __shared__ __align__(16) float ks[kPrep][kD];
    __shared__ float vs[kPrep][kRowsPerBlock];
    __shared__ float red[kPrep][4];
    __shared__ float gb[kPrep][2];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunk = blockIdx.x, h = blockIdx.y, seq = blockIdx.z;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int pos0 = a.pos ? a.pos[seq] : 0;
    const int hk = h % a.n_head_k;
    const int qk = a.n_head_k * kD, vw = a.n_head_v * kD;
    const int alpha_off = 2 * qk + 2 * vw, beta_off = alpha_off + a.n_head_v;
    const int rsub = lane >> 5, li = lane & 31;
    const int jl = wave * RW + rsub;          // first row of the lane within the block; its others follow two apart
    const int j = chunk * kRowsPerBlock + jl; // row of the head's state
    // a slot holds n_planes copies of the state; the committed one is read
    const int planes = a.n_planes > 1 ? a.n_planes : 1;
    const int cur = a.plane ? static_cast<int>(static_cast<unsigned>(a.plane[slot]) % static_cast<unsigned>(planes)) : 0;
    const size_t plane_floats = static_cast<size_t>(a.n_head_v) * kD * kD;
    float *sslot = a.state + static_cast<size_t>(slot) * planes * plane_floats + (static_cast<size_t>(h) * kD + j) * kD + li * 4;
    float *srow = sslot + cur * plane_floats;
    float4 s[NS];  // in flight while the first group is prepared
#pragma unroll
    for (int u = 0; u < NS; u++) s[u] = *reinterpret_cast<const float4 *>(srow + static_cast<size_t>(2 * u) * kD);

    const float *ring = a.ring + static_cast<size_t>(slot) * a.ring_slots * a.ring_stride;
    const float scale = 1.f / sqrtf(static_cast<float>(kD));
    // q (threads 0..127) and k (128..255) channels of key head hk
    const int ch = tid < kD ? hk * kD + tid : qk + hk * kD + (tid - kD);
    const float4 tp = *reinterpret_cast<const float4 *>(a.conv1d + static_cast<size_t>(ch) * 4);

    for (int i0 = 0; i0 < a.seq_len; i0 += kPrep) {
        const int nr = a.seq_len - i0 < kPrep ? a.seq_len - i0 : kPrep;
        const int p0 = pos0 + i0;
        // ---- the group's q and k: causal depthwise conv (taps 0..3 meet positions p-3..p; rows
        //      before the start of the sequence are zero), SiLU, sum of squares per key head ----
        float x[kPrep + 3];
        int rs = (p0 + a.ring_slots - 3) % a.ring_slots;  // ring row of position p0 - 3 (the ring holds more than 3 rows)
#pragma unroll
        for (int jj = 0; jj < kPrep + 3; jj++) {
            x[jj] = (jj < nr + 3 && p0 + jj - 3 >= 0) ? ring[static_cast<size_t>(rs) * a.ring_stride + ch] : 0.f;
            rs = rs + 1 == a.ring_slots ? 0 : rs + 1;
        }
        float act[kPrep];
#pragma unroll
        for (int r = 0; r < kPrep; r++) {
            if (r >= nr) break;
            float c = 0.f;
            c += x[r] * tp.x;
            c += x[r + 1] * tp.y;
            c += x[r + 2] * tp.z;
            c += x[r + 3] * tp.w;
            act[r] = c * sigmoid_exact(c);
            const float ss = wave_sum_all(act[r] * act[r]);
            if (lane == 0) red[r][wave] = ss;
        }
        // this block's eight v channels of each row, and each row's decay and write strength
        if (tid < nr * kRowsPerBlock) {
            const int r = tid / kRowsPerBlock, vr = tid % kRowsPerBlock;
            const int vch = 2 * qk + h * kD + chunk * kRowsPerBlock + vr;
            const float cv = conv4(ring, a.ring_slots, a.ring_stride, a.conv1d, vch, p0 + r);
            vs[r][vr] = cv * sigmoid_exact(cv);
        } else if (tid >= kBlock - kPrep && tid - (kBlock - kPrep) < nr) {
            const int r = tid - (kBlock - kPrep);
            const float *row = ring + static_cast<size_t>((p0 + r) % a.ring_slots) * a.ring_stride;
            const float asp = softplus_ref(row[alpha_off + h] + a.dt_bias[h]);
            gb[r][0] = expf(asp * a.a[h]);
            gb[r][1] = sigmoid_exact(row[beta_off + h]);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kPrep; r++) {
            if (r >= nr) break;
            const float ssq = tid < kD ? red[r][0] + red[r][1] : red[r][2] + red[r][3];
            const float nrm = a.qk_norm_max ? 1.f / fmaxf(sqrtf(ssq), a.eps) : 1.f / sqrtf(ssq + a.eps);
            if (tid < kD) qs[r][tid] = act[r] * nrm; else ks[r][tid - kD] = act[r] * nrm;
        }
        __syncthreads();
        // ---- the rule, row after row, the state in registers ----
        for (int r = 0; r < nr; r++) {
            const int i = i0 + r;
            const float4 k4 = *reinterpret_cast<const float4 *>(&ks[r][li * 4]);
            const float4 q4 = *reinterpret_cast<const float4 *>(&qs[r][li * 4]);
            const float g = gb[r][0], beta = gb[r][1];
#pragma unroll
            for (int u = 0; u < NS; u++) {
                float4 &su = s[u];
                const float vj = vs[r][jl + 2 * u];
                su.x *= g; su.y *= g; su.z *= g; su.w *= g;
                const float dk = sum32_all(fmaf(su.x, k4.x, fmaf(su.y, k4.y, fmaf(su.z, k4.z, su.w * k4.w))));
                const float delta = (vj - dk) * beta;
                su.x = fmaf(delta, k4.x, su.x);
                su.y = fmaf(delta, k4.y, su.y);
                su.z = fmaf(delta, k4.z, su.z);
                su.w = fmaf(delta, k4.w, su.w);
                const float oq = sum32_all(fmaf(su.x, q4.x, fmaf(su.y, q4.y, fmaf(su.z, q4.z, su.w * q4.w))));
                if (li == 0)
                    a.out[(static_cast<size_t>(seq) * a.seq_len + i) * vw + static_cast<size_t>(h) * kD + j + 2 * u] = oq * scale;
                // a rewindable pass keeps every prefix: the state after row i goes to its own plane
                if (a.spec) *reinterpret_cast<float4 *>(sslot + ((cur + 1 + i) % planes) * plane_floats + static_cast<size_t>(2 * u) * kD) = su;
            }
        }
        if (i0 + kPrep < a.seq_len) __syncthreads();  // the next group overwrites what the waves just read
    }
    if (!a.spec) {
#pragma unroll
        for (int u = 0; u < NS; u++) *reinterpret_cast<float4 *>(srow + static_cast<size_t>(2 * u) * kD) = s[u];
    }
}

// The same step for calls of many rows (prompt chunks), where the groups' preparation - not the
// rule - is most of the time of the kernel above: here eight more waves prepare group g+1 into a
// second set of LDS buffers while the four waves that hold the state walk group g, with one
// block-wide barrier a group.  A preparing wave owns whole vectors (the 128 q or k channels of a
// key head, two a lane), so the norms need no exchange between waves: the first half of them
// take q, two rows of the group each, the second half k; wave 0 also makes the block's eight v
// channels of every row, wave 1 the rows' decay and write strength.
// grid: (128/8 row chunks, n_head_v, n_seq), 256 + 64 * kPrepWaves threads.
constexpr int kPrepWaves = 8;                       // half of them for q, half for k
constexpr int kPrepRows = kPrep / (kPrepWaves / 2); // rows of a group a preparing wave takes
__global__ __launch_bounds__(kBlock + 64 * kPrepWaves) void dn_step_pipe_kernel(shv_dn_step_args a) {
    __shared__ __align__(16) float qs[2][kPrep][kD];
    __shared__ __align__(16) float ks[2][kPrep][kD];
    __shared__ float vs[2][kPrep][kRowsPerBlock];
    __shared__ float gb[2][kPrep][2];

    const int tid = threadIdx.x, lane = tid & 63;
    const bool producer = tid >= kBlock;
    const int wave = producer ? (tid - kBlock) >> 6 : tid >> 6;
    const int chunk = blockIdx.x, h = blockIdx.y, seq = blockIdx.z;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int pos0 = a.pos ? a.pos[seq] : 0;
    const int hk = h % a.n_head_k;
    const int qk = a.n_head_k * kD, vw = a.n_head_v * kD;
    const int alpha_off = 2 * qk + 2 * vw, beta_off = alpha_off + a.n_head_v;
    const float *ring = a.ring + static_cast<size_t>(slot) * a.ring_slots * a.ring_stride;
    const int groups = (a.seq_len + kPrep - 1) / kPrep;

    // ---- the preparing waves' constants ----
    const int kind = wave / (kPrepWaves / 2), r0 = (wave % (kPrepWaves / 2)) * kPrepRows;  // q or k; first of the wave's rows of a group
    const int ch0 = (kind ? qk : 0) + hk * kD + lane, ch1 = ch0 + 64;
    float4 tp0 = {0.f, 0.f, 0.f, 0.f}, tp1 = tp0;
    if (producer) {
        tp0 = *reinterpret_cast<const float4 *>(a.conv1d + static_cast<size_t>(ch0) * 4);
        tp1 = *reinterpret_cast<const float4 *>(a.conv1d + static_cast<size_t>(ch1) * 4);
    }
    auto prepare = [&](int g) {
        const int b = g & 1, i0 = g * kPrep;
        const int nr = a.seq_len - i0 < kPrep ? a.seq_len - i0 : kPrep;
        const int p0 = pos0 + i0;
        // sliding window of the wave's rows: positions p0 + r0 - 3 .. p0 + r0 + kPrepRows - 1
        float x0[kPrepRows + 3], x1[kPrepRows + 3];
        int rs = (p0 + r0 + a.ring_slots - 3) % a.ring_slots;
#pragma unroll
        for (int jj = 0; jj < kPrepRows + 3; jj++) {
            const bool on = r0 + jj - 3 < nr && p0 + r0 + jj - 3 >= 0;
            x0[jj] = on ? ring[static_cast<size_t>(rs) * a.ring_stride + ch0] : 0.f;
            x1[jj] = on ? ring[static_cast<size_t>(rs) * a.ring_stride + ch1] : 0.f;
            rs = rs + 1 == a.ring_slots ? 0 : rs + 1;
        }
        // the v channels and the gates are asked for before the q/k arithmetic
        float cv = 0.f, g_alpha = 0.f, g_beta = 0.f;
        const int vr_row = lane / kRowsPerBlock, vr = lane % kRowsPerBlock;
        if (wave == 0 && vr_row < nr) cv = conv4(ring, a.ring_slots, a.ring_stride, a.conv1d, 2 * qk + h * kD + chunk * kRowsPerBlock + vr, p0 + vr_row);
        if (wave == 1 && lane < nr) {
            const float *row = ring + static_cast<size_t>((p0 + lane) % a.ring_slots) * a.ring_stride;
            g_alpha = row[alpha_off + h];
            g_beta = row[beta_off + h];
        }
        float (*dst)[kD] = kind ? ks[b] : qs[b];
#pragma unroll
        for (int r = 0; r < kPrepRows; r++) {
            if (r0 + r >= nr) break;
            float c0 = 0.f, c1 = 0.f;
            c0 += x0[r] * tp0.x; c0 += x0[r + 1] * tp0.y; c0 += x0[r + 2] * tp0.z; c0 += x0[r + 3] * tp0.w;
            c1 += x1[r] * tp1.x; c1 += x1[r + 1] * tp1.y; c1 += x1[r + 2] * tp1.z; c1 += x1[r + 3] * tp1.w;
            const float a0 = c0 * sigmoid_exact(c0), a1 = c1 * sigmoid_exact(c1);
            const float ssq = wave_sum_all(fmaf(a0, a0, a1 * a1));
            const float nrm = a.qk_norm_max ? 1.f / fmaxf(sqrtf(ssq), a.eps) : 1.f / sqrtf(ssq + a.eps);
            dst[r0 + r][lane] = a0 * nrm;
            dst[r0 + r][lane + 64] = a1 * nrm;
        }
        if (wave == 0 && vr_row < nr) vs[b][vr_row][vr] = cv * sigmoid_exact(cv);
        if (wave == 1 && lane < nr) {
            const float asp = softplus_ref(g_alpha + a.dt_bias[h]);
            gb[b][lane][0] = expf(asp * a.a[h]);
            gb[b][lane][1] = sigmoid_exact(g_beta);
        }
    };

    // ---- the state-holding waves' constants ----
    const int rsub = lane >> 5, li = lane & 31;
    const int jl = wave * 2 + rsub;
    const int j = chunk * kRowsPerBlock + jl;
    const int planes = a.n_planes > 1 ? a.n_planes : 1;
    const int cur = a.plane ? static_cast<int>(static_cast<unsigned>(a.plane[slot]) % static_cast<unsigned>(planes)) : 0;
    const size_t plane_floats = static_cast<size_t>(a.n_head_v) * kD * kD;
    float *sslot = a.state + static_cast<size_t>(slot) * planes * plane_floats + (static_cast<size_t>(h) * kD + j) * kD + li * 4;
    float *srow = sslot + cur * plane_floats;
    float4 s = {0.f, 0.f, 0.f, 0.f};
    if (!producer) s = *reinterpret_cast<const float4 *>(srow);
    const float scale = 1.f / sqrtf(static_cast<float>(kD));

    if (producer) prepare(0);
    __syncthreads();
    for (int g = 0; g < groups; g++) {
        if (producer) {
            if (g + 1 < groups) prepare(g + 1);
        } else {
            const int b = g & 1, i0 = g * kPrep;
            const int nr = a.seq_len - i0 < kPrep ? a.seq_len - i0 : kPrep;
            for (int r = 0; r < nr; r++) {
                const int i = i0 + r;
                const float4 k4 = *reinterpret_cast<const float4 *>(&ks[b][r][li * 4]);
                const float4 q4 = *reinterpret_cast<const float4 *>(&qs[b][r][li * 4]);
                const float gg = gb[b][r][0], beta = gb[b][r][1], vj = vs[b][r][jl];
                s.x *= gg; s.y *= gg; s.z *= gg; s.w *= gg;
                const float dk = sum32_all(fmaf(s.x, k4.x, fmaf(s.y, k4.y, fmaf(s.z, k4.z, s.w * k4.w))));
                const float delta = (vj - dk) * beta;
                s.x = fmaf(delta, k4.x, s.x);
                s.y = fmaf(delta, k4.y, s.y);
                s.z = fmaf(delta, k4.z, s.z);
                s.w = fmaf(delta, k4.w, s.w);
                const float oq = sum32_all(fmaf(s.x, q4.x, fmaf(s.y, q4.y, fmaf(s.z, q4.z, s.w * q4.w))));
                if (li == 0)
                    a.out[(static_cast<size_t>(seq) * a.seq_len + i) * vw + static_cast<size_t>(h) * kD + j] = oq * scale;
                if (a.spec) *reinterpret_cast<float4 *>(sslot + ((cur + 1 + i) % planes) * plane_floats) = s;
            }
        }
        __syncthreads();  // group g has been read, group g+1 is ready
    }
    if (!producer && !a.spec) *reinterpret_cast<float4 *>(srow) = s;
}

}  // namespace

int shv_launch_dn_step(shv_ctx *ctx, const shv_dn_step_args *pa) {
    const shv_dn_step_args &a = *pa;
    SHV_REQUIRE(a.ring && a.conv1d && a.a && a.dt_bias && a.state && a.out, "dn_step: NULL argument");
    SHV_REQUIRE(a.head_dim == kD, "dn_step: head_dim %d; built for %d", a.head_dim, kD);
    SHV_REQUIRE(a.conv == 4, "dn_step: conv kernel %d; built for 4", a.conv);
    SHV_REQUIRE(a.n_head_k >= 1 && a.n_head_v >= a.n_head_k && a.n_head_v <= 65535, "dn_step: heads %d/%d", a.n_head_k, a.n_head_v);
    SHV_REQUIRE(a.n_seq >= 1 && a.n_seq <= 65535 && a.seq_len >= 1, "dn_step: %d sequences of %d", a.n_seq, a.seq_len);
    const int width = 2 * a.n_head_k * kD + 2 * a.n_head_v * kD + 2 * a.n_head_v;
    SHV_REQUIRE(a.ring_stride >= width, "dn_step: ring_stride %d < row width %d", a.ring_stride, width);
    SHV_REQUIRE(a.ring_slots >= a.seq_len + a.conv - 1, "dn_step: a ring of %d slots cannot hold %d tokens and %d of history",
                a.ring_slots, a.seq_len, a.conv - 1);
    SHV_REQUIRE(shv_aligned16(a.state) && shv_aligned16(a.conv1d), "dn_step: state and conv1d must be 16-byte aligned");
    SHV_REQUIRE(a.n_planes >= 0 && a.n_planes <= 64, "dn_step: %d state planes", a.n_planes);
    SHV_REQUIRE(!a.spec || (a.n_planes > 1 && a.seq_len < a.n_planes), "dn_step: a rewindable pass of %d rows needs more than %d state planes",
                a.seq_len, a.n_planes);
    SHV_REQUIRE(!a.work || a.work_floats >= 0, "dn_step: work_floats %lld", static_cast<long long>(a.work_floats));
    if (shv_dn_chunk_covers(a)) return shv_launch_dn_chunk(ctx, a);
    dim3 grid(kD / kRowsPerBlock, a.n_head_v, a.n_seq);
    // more than one group of rows: preparation and rule overlap
    if (a.seq_len > kPrep) SHV_LAUNCH(ctx, dn_step_pipe_kernel, grid, dim3(kBlock + 64 * kPrepWaves), 0, a);
    else if (a.n_seq >= 4) SHV_LAUNCH(ctx, dn_step_kernel<4>, dim3(kD / 16, a.n_head_v, a.n_seq), dim3(kBlock), 0, a);
    else SHV_LAUNCH(ctx, dn_step_kernel<2>, grid, dim3(kBlock), 0, a);
    return SHV_OK;
}
