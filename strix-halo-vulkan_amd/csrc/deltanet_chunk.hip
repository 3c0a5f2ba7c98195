// Gated DeltaNet over a prompt chunk, 64 rows at a time on the matrix cores.
//
// The rule of llm/deltanet.go:326-375 (S *= g; delta = (v - S k) beta; S += delta k^T; o = S q),
// row after row, is a chain of rank-one updates.  Over a chunk of C = 64 rows it has a closed form
// (the WY / UT form of the delta rule).  With G_t the running sum of log g inside the chunk and
// U the chunk's "pseudo values" (what the rule actually adds to the state, one row per token):
//
//     (I + A) U = B,   A[t][s] = beta_t e^(G_t - G_s) (k_t . k_s)  for s < t,
//                      B[t]    = beta_t (v_t - e^(G_t) S0 k_t)
//     o_t   = e^(G_t) S0 q_t + sum_{s<=t} e^(G_t - G_s) (q_t . k_s) U[s]
//     S_new = e^(G_C) S0 + sum_s e^(G_C - G_s) U[s] k_s^T
//
// so a chunk is a handful of 64x64x128 and 64x16x128 products plus one triangular solve, and the
// state is touched once per 64 rows instead of once per row.  Two kernels:
//
//   dn_prep_kernel   everything that does not depend on the state, once per pass: causal conv +
//                    SiLU of q, k, v, the L2 norm of q and k per key head, log g and beta
//   dn_chunk_kernel  (as producer, when the workspace has room) what a chunk needs that does not
//                    depend on the state either — A, M, the inverses of the diagonal blocks of I + A,
//                    G, beta — for every (value head, chunk) of the pass at once: the walk below is a
//                    chain, this part of it need not be, nor be repeated by a head's eight blocks
//   dn_chunk_kernel  a block owns 16 of a value head's 128 state rows (they evolve independently
//                    of the other rows) and walks the chunks of the pass with that slab in
//                    registers as float32; the solve is blocked 4 x 16: the four 16x16 diagonal
//                    blocks of (I + A) are inverted by substitution on the vector units (each lane
//                    a column, one wave, while the other three form the tiles of A below the
//                    diagonal), everything else is v_mfma_f32_16x16x16/32_f16
//
// float32 operands enter the matrix cores as a sum of two binary16 values (the low part scaled
// by 2^11 so that it stays normal), three products per term (hi*hi, hi*lo, lo*hi): about 22 bits
// of each operand, accumulated in float32.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kD = 128;   // head dimension
constexpr int kC = 64;    // rows of a chunk
constexpr int kJ = 16;    // state rows of a block
constexpr int kThreads = 256;
constexpr float kLoScale = 2048.f, kLoInv = 1.f / 2048.f;

__device__ __forceinline__ float softplus_ref(float x) {
    // the add inside the log is float32 on purpose: below about -16.6 it returns exactly 0
    return x > 20.f ? x : logf(1.f + expf(x));
}

__device__ __forceinline__ void split(float x, _Float16 &hi, _Float16 &lo) {
    hi = static_cast<_Float16>(x);
    lo = static_cast<_Float16>((x - static_cast<float>(hi)) * kLoScale);
}

// ------------------------------------------------------------------------------- prep --------
// One row of the result per pass row: [q^ (hk*d) | k^ (hk*d) | v (hv*d) | log g (hv) | beta (hv)]; q^ and k^ as
// binary16 pairs (value = hi + lo / 2048), every four columns' sixteen bytes holding their four hi, then their four lo.
// grid: (items, ceil(seq_len / 4), n_seq), 256 threads; an item is four (q or k, key head) vectors
// (a wave each), or 256 v channels, or the gates; a thread keeps the sliding window of its
// channel over the block's four rows.
constexpr int kPrepTok = 4;

__global__ __launch_bounds__(kThreads) void dn_prep_kernel(shv_dn_step_args a, float *prep, int pw) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int seq = blockIdx.z, t0 = blockIdx.y * kPrepTok;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int pos0 = a.pos ? a.pos[seq] : 0;
    const int qk = a.n_head_k * kD, vw = a.n_head_v * kD;
    const float *ring = a.ring + static_cast<size_t>(slot) * a.ring_slots * a.ring_stride;
    const int nr = a.seq_len - t0 < kPrepTok ? a.seq_len - t0 : kPrepTok;
    float *dst = prep + (static_cast<size_t>(seq) * a.seq_len + t0) * pw;
    const int qk_items = 2 * a.n_head_k / 4, v_items = vw / kThreads;
    const int item = blockIdx.x;
    const int p0 = pos0 + t0;
    if (item < qk_items + v_items) {
        const bool is_qk = item < qk_items;
        // q/k: the wave's vector, two channels a lane; v: one channel a thread
        const int vec = item * 4 + wave;  // (kind, head) of the wave
        const int ch0 = is_qk ? vec * kD + lane : 2 * qk + (item - qk_items) * kThreads + tid;
        const int ch1 = is_qk ? ch0 + 64 : ch0;
        const float4 tp0 = *reinterpret_cast<const float4 *>(a.conv1d + static_cast<size_t>(ch0) * 4);
        const float4 tp1 = *reinterpret_cast<const float4 *>(a.conv1d + static_cast<size_t>(ch1) * 4);
        float x0[kPrepTok + 3], x1[kPrepTok + 3];
        int rs = (p0 + a.ring_slots - 3) % a.ring_slots;
#pragma unroll
        for (int jj = 0; jj < kPrepTok + 3; jj++) {
            const bool on = jj - 3 < nr && p0 + jj - 3 >= 0;
            x0[jj] = on ? ring[static_cast<size_t>(rs) * a.ring_stride + ch0] : 0.f;
            x1[jj] = on && is_qk ? ring[static_cast<size_t>(rs) * a.ring_stride + ch1] : 0.f;
            rs = rs + 1 == a.ring_slots ? 0 : rs + 1;
        }
#pragma unroll
        for (int r = 0; r < kPrepTok; r++) {
            if (r >= nr) break;
            float c0 = 0.f, c1 = 0.f;
            c0 += x0[r] * tp0.x; c0 += x0[r + 1] * tp0.y; c0 += x0[r + 2] * tp0.z; c0 += x0[r + 3] * tp0.w;
            c1 += x1[r] * tp1.x; c1 += x1[r + 1] * tp1.y; c1 += x1[r + 2] * tp1.z; c1 += x1[r + 3] * tp1.w;
            const float a0 = c0 * sigmoid_exact(c0), a1 = c1 * sigmoid_exact(c1);
            if (is_qk) {
                const float ssq = wave_sum_all(fmaf(a0, a0, a1 * a1));
                const float nrm = a.qk_norm_max ? 1.f / fmaxf(sqrtf(ssq), a.eps) : 1.f / sqrtf(ssq + a.eps);
                // as the two halves the matrix cores take, split here once instead of by every block that stages the
                // row: four columns' large halves, then their small ones, in the sixteen bytes the four floats had
                char *seg = reinterpret_cast<char *>(dst + static_cast<size_t>(r) * pw + vec * kD);
                const float val[2] = {a0 * nrm, a1 * nrm};
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const int cc = lane + 64 * e;
                    _Float16 hi, lo;
                    split(val[e], hi, lo);
                    *reinterpret_cast<_Float16 *>(seg + (cc >> 2) * 16 + (cc & 3) * 2) = hi;
                    *reinterpret_cast<_Float16 *>(seg + (cc >> 2) * 16 + 8 + (cc & 3) * 2) = lo;
                }
            } else {
                dst[static_cast<size_t>(r) * pw + ch0] = a0;
            }
        }
    } else if (tid < nr * a.n_head_v) {
        const int r = tid / a.n_head_v, h = tid % a.n_head_v;
        const int alpha_off = 2 * qk + 2 * vw, beta_off = alpha_off + a.n_head_v;
        const float *row = ring + static_cast<size_t>((p0 + r) % a.ring_slots) * a.ring_stride;
        const float asp = softplus_ref(row[alpha_off + h] + a.dt_bias[h]);
        dst[static_cast<size_t>(r) * pw + 2 * qk + vw + h] = asp * a.a[h];
        dst[static_cast<size_t>(r) * pw + 2 * qk + vw + a.n_head_v + h] = sigmoid_exact(row[beta_off + h]);
    }
}

// ------------------------------------------------------------------------------ chunks -------
constexpr int kKS = kD + 8;    // halves between rows of the [64][128] operands (272 B: 16 rows cover all banks)
constexpr int kAS = kC + 8;    // halves between rows of the [64][64] and [16][64] operands
constexpr int kTS = 24;        // halves between rows of a 16x16 inverse

// What a chunk's solve and outputs need besides the state, q^ and k^: a function of the chunk's k^, q^, g and beta
// alone, so it can be formed for all chunks of a pass at once and handed over as one image of these bytes.
struct PreRec {
    _Float16 ah[kC][kAS], al[kC][kAS];                            // -A[t][s], s < t; in a stored record (I + A)^-1 [t][s], s <= t
    _Float16 mh[kC][kAS], ml[kC][kAS];                            // M[t][s] = e^(G_t - G_s) (q_t . k_s), s <= t
    _Float16 th[4][16][kTS], tl[4][16][kTS];                      // the inverses of the diagonal blocks of I + A
    float G[kC], beta[kC];
};
static_assert(sizeof(PreRec) % 16 == 0, "moved 16 bytes at a time");
constexpr int kPreVecs = sizeof(PreRec) / 16, kPrePerThread = (kPreVecs + kThreads - 1) / kThreads;

struct ChunkLds {
    _Float16 kh[kC][kKS], kl[kC][kKS], qh[kC][kKS], ql[kC][kKS];  // k^ and q^ of the chunk, hi and scaled lo
    _Float16 sh[kJ][kKS], sl[kJ][kKS];                            // the state slab S[j][i]
    alignas(16) PreRec pre;
    _Float16 uh[kJ][kAS], ul[kJ][kAS];                            // U transposed, [j][s]
    _Float16 dh[kJ][kAS], dl[kJ][kAS];                            // U e^(G_C - G_s) transposed
    _Float16 bth[kJ][kAS], btl[kJ][kAS];                          // B transposed, [j][t] (the walk over records)
    float adiag[4][16][16];                                       // the diagonal blocks of A in float32
    float v[kC][kJ];                                              // v of the chunk, the block's 16 columns
};

__device__ __forceinline__ float4_t mfma32(half8_t x, half8_t y, float4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, c, 0, 0, 0); }
__device__ __forceinline__ float4_t mfma16(half4_t x, half4_t y, float4_t c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(x, y, c, 0, 0, 0); }

// hi*hi into `main`, hi*lo + lo*hi into `low` (which carries the 2^11 of the scaled low parts)
__device__ __forceinline__ void mma32(half8_t xh, half8_t xl, half8_t yh, half8_t yl, float4_t &main, float4_t &low) {
    main = mfma32(xh, yh, main);
    low = mfma32(xh, yl, low);
    low = mfma32(xl, yh, low);
}
__device__ __forceinline__ void mma16(half4_t xh, half4_t xl, half4_t yh, half4_t yl, float4_t &main, float4_t &low) {
    main = mfma16(xh, yh, main);
    low = mfma16(xh, yl, low);
    low = mfma16(xl, yh, low);
}

// grid: (n_head_v * 8, n_seq): blocks that share a key head are neighbours (they read the same q^
// and k^); 256 threads.  Wave w owns rows 16w..16w+15 of the chunk in every [64][..] product and
// the state's columns 32w..32w+31.
// ROLE 0: the walk, every chunk's operands formed on the way.  ROLE 1: the walk with the chunks' records (PreRec)
// read from recs.  ROLE 2: the producer of those records, grid (n_head_v, ceil(chunks / per), n_seq): the block forms
// the records of `per` chunks in a row of its head by the very steps 1 and 2 of the walk (the next chunk's rows on
// their way meanwhile) and stores them; nothing of the state is touched.
constexpr int kWalk = 0, kWalkRecs = 1, kMakeRecs = 2;
template <int ROLE>
__global__ __launch_bounds__(kThreads, 1) void dn_chunk_kernel(shv_dn_step_args a, const float *prep, int pw, char *recs, int per) {
    extern __shared__ __align__(16) char smem_raw[];
    ChunkLds &L = *reinterpret_cast<ChunkLds *>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int seq = ROLE == kMakeRecs ? blockIdx.z : blockIdx.y;
    const int rep = a.n_head_v / a.n_head_k;
    const int hk = blockIdx.x % a.n_head_k, rest = blockIdx.x / a.n_head_k;
    const int h = ROLE == kMakeRecs ? static_cast<int>(blockIdx.x) : hk + a.n_head_k * (rest % rep), slab = ROLE == kMakeRecs ? 0 : rest / rep;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int qk = a.n_head_k * kD, vw = a.n_head_v * kD;
    const int planes = a.n_planes > 1 ? a.n_planes : 1;
    const int cur = a.plane ? static_cast<int>(static_cast<unsigned>(a.plane[slot]) % static_cast<unsigned>(planes)) : 0;
    const size_t plane_floats = static_cast<size_t>(a.n_head_v) * kD * kD;
    float *state = a.state + (static_cast<size_t>(slot) * planes + cur) * plane_floats + (static_cast<size_t>(h) * kD + slab * kJ) * kD;
    const float *rows = prep + static_cast<size_t>(seq) * a.seq_len * pw;
    const float scale = 1.f / sqrtf(static_cast<float>(kD));

    // the slab in float32: tiles of 16 columns i, tile 2w and 2w+1; element [r] is S[j = 4g + r][i = 16 tile + n]
    float4_t S[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if constexpr (ROLE != kMakeRecs) {
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) S[u][r] = state[static_cast<size_t>(4 * g + r) * kD + 16 * (2 * w + u) + n];
    }
    auto publish_state = [&]() {
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                _Float16 hi, lo;
                split(S[u][r], hi, lo);
                L.sh[4 * g + r][16 * (2 * w + u) + n] = hi;
                L.sl[4 * g + r][16 * (2 * w + u) + n] = lo;
            }
    };
    if constexpr (ROLE != kMakeRecs) publish_state();

    const int n_chunks = (a.seq_len + kC - 1) / kC;
    const int c_first = ROLE == kMakeRecs ? static_cast<int>(blockIdx.y) * per : 0;
    const int c_end = ROLE == kMakeRecs ? (c_first + per < n_chunks ? c_first + per : n_chunks) : n_chunks;
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    u32x4_t pr[ROLE == kWalkRecs ? kPrePerThread : 1];
    auto rec_of = [&](int c) { return recs + (static_cast<size_t>(seq * n_chunks + c) * a.n_head_v + h) * sizeof(PreRec); };
    // a thread's share of a chunk's q^ and k^: float4 f = tid + 256 u of the [64][32] float4s
    float4 kf[8], qf[8], vf;
    float gl = 0.f, bt = 0.f;
    auto fetch = [&](int c) {
        const int t0 = c * kC;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int f = tid + kThreads * u, row = f >> 5, c4 = (f & 31) * 4;
            const bool on = t0 + row < a.seq_len;
            const float *src = rows + static_cast<size_t>(on ? t0 + row : 0) * pw + hk * kD + c4;
            kf[u] = *reinterpret_cast<const float4 *>(src + qk);
            qf[u] = *reinterpret_cast<const float4 *>(src);
            if (!on) kf[u] = qf[u] = float4{0.f, 0.f, 0.f, 0.f};
        }
        {
            const int row = tid >> 2, c4 = (tid & 3) * 4;
            const bool on = t0 + row < a.seq_len;
            vf = *reinterpret_cast<const float4 *>(rows + static_cast<size_t>(on ? t0 + row : 0) * pw + 2 * qk + h * kD + slab * kJ + c4);
            if (!on) vf = float4{0.f, 0.f, 0.f, 0.f};
        }
        if (ROLE != kWalkRecs && tid < kC) {
            const bool on = t0 + tid < a.seq_len;
            const float *src = rows + static_cast<size_t>(on ? t0 + tid : 0) * pw + 2 * qk + vw;
            gl = on ? src[h] : 0.f;
            bt = on ? src[a.n_head_v + h] : 0.f;
        }
    };
    // the record of chunk c, this thread's sixteen-byte pieces of it (the last piece of the last threads repeats the first)
    const int last_piece = tid + kThreads * (kPrePerThread - 1) < kPreVecs ? kThreads * (kPrePerThread - 1) : -tid;
#define SHV_DN_FETCH_REC(c_)                                                                  \
    if constexpr (ROLE == kWalkRecs) {                                                        \
        const u32x4_t *src_ = reinterpret_cast<const u32x4_t *>(rec_of(c_)) + tid;                \
        _Pragma("unroll") for (int u = 0; u + 1 < kPrePerThread; u++) pr[u] = src_[kThreads * u]; \
        pr[kPrePerThread - 1] = src_[last_piece];                                             \
    }
    fetch(c_first);
    SHV_DN_FETCH_REC(c_first)

    for (int c = c_first; c < c_end; c++) {
        const int t0 = c * kC;
        // ---- 1: the chunk's operands into LDS ----
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int f = tid + kThreads * u, row = f >> 5, c4 = (f & 31) * 4;
            // the prepared rows hold q^ and k^ as halves already: four hi, four lo
            struct Halves { half4_t hi, lo; };
            const Halves kk = __builtin_bit_cast(Halves, kf[u]), qq = __builtin_bit_cast(Halves, qf[u]);
            *reinterpret_cast<half4_t *>(&L.kh[row][c4]) = kk.hi;
            *reinterpret_cast<half4_t *>(&L.kl[row][c4]) = kk.lo;
            *reinterpret_cast<half4_t *>(&L.qh[row][c4]) = qq.hi;
            *reinterpret_cast<half4_t *>(&L.ql[row][c4]) = qq.lo;
        }
        *reinterpret_cast<float4 *>(&L.v[tid >> 2][(tid & 3) * 4]) = vf;
        if constexpr (ROLE == kWalkRecs) {
            u32x4_t *dst = reinterpret_cast<u32x4_t *>(&L.pre) + tid;
#pragma unroll
            for (int u = 0; u + 1 < kPrePerThread; u++) dst[kThreads * u] = pr[u];
            if (last_piece > 0) dst[last_piece] = pr[kPrePerThread - 1];
        } else if (tid < kC) {
            // running sum of log g over the chunk: one wave, a prefix sum by shuffles
            float s = gl;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const float up = __shfl_up(s, o, 64);
                if (lane >= o) s += up;
            }
            L.pre.G[tid] = s;
            L.pre.beta[tid] = bt;
        }
        __syncthreads();

        // ---- 2: P = K K^T and R = Q K^T over the lower triangle of 4 x 4 tiles of 16 rows; A and M from them.
        //      First every wave its own diagonal tile; then, while wave 0 inverts the four diagonal
        //      blocks of I + A on the vector units, the other three take two of the six tiles below
        //      the diagonal each ----
        auto tile = [&](int tt, int st) {
            float4_t pm = {0.f, 0.f, 0.f, 0.f}, pl = pm, rm = pm, rl = pm;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const half8_t xkh = *reinterpret_cast<const half8_t *>(&L.kh[16 * tt + n][32 * ks + 8 * g]);
                const half8_t xkl = *reinterpret_cast<const half8_t *>(&L.kl[16 * tt + n][32 * ks + 8 * g]);
                const half8_t xqh = *reinterpret_cast<const half8_t *>(&L.qh[16 * tt + n][32 * ks + 8 * g]);
                const half8_t xql = *reinterpret_cast<const half8_t *>(&L.ql[16 * tt + n][32 * ks + 8 * g]);
                const half8_t bh = *reinterpret_cast<const half8_t *>(&L.kh[16 * st + n][32 * ks + 8 * g]);
                const half8_t bl = *reinterpret_cast<const half8_t *>(&L.kl[16 * st + n][32 * ks + 8 * g]);
                mma32(xkh, xkl, bh, bl, pm, pl);
                mma32(xqh, xql, bh, bl, rm, rl);
            }
            const float Gs = L.pre.G[16 * st + n];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int t = 16 * tt + 4 * g + r, s = 16 * st + n;
                const float Gtr = L.pre.G[t], btr = L.pre.beta[t];
                const float dec = __expf(Gtr - Gs);
                const float P = fmaf(pl[r], kLoInv, pm[r]), R = fmaf(rl[r], kLoInv, rm[r]);
                const float av = s < t ? btr * dec * P : 0.f;
                const float mv = s <= t ? dec * R : 0.f;
                _Float16 hi, lo;
                split(-av, hi, lo);
                L.pre.ah[t][s] = hi; L.pre.al[t][s] = lo;
                split(mv, hi, lo);
                L.pre.mh[t][s] = hi; L.pre.ml[t][s] = lo;
                if (st == tt) L.adiag[tt][4 * g + r][n] = av;
            }
        };
        if constexpr (ROLE != kWalkRecs) {
            tile(w, w);
            __syncthreads();
        }
        if (c + 1 < c_end) {
            fetch(c + 1);  // in flight under the rest of the chunk (the stores that read these registers have drained)
            SHV_DN_FETCH_REC(c + 1)
        }
        if (ROLE == kWalkRecs) {
            // the record holds it all
        } else if (w == 0) {
            // lane (b = g, column n): T = (I + A_bb)^-1 by forward substitution, the column in registers
            float T[16];
#pragma unroll
            for (int t = 0; t < 16; t++) {
                float s0 = t == n ? 1.f : 0.f, s1 = 0.f;
#pragma unroll
                for (int s = 0; s < t; s++) {
                    const float av = L.adiag[g][t][s];
                    if (s & 1) s1 = fmaf(-av, T[s], s1); else s0 = fmaf(-av, T[s], s0);
                }
                T[t] = s0 + s1;
                _Float16 hi, lo;
                split(T[t], hi, lo);
                L.pre.th[g][t][n] = hi;
                L.pre.tl[g][t][n] = lo;
            }
        } else if (w == 1) {
            tile(3, 0);
            tile(1, 0);
        } else if (w == 2) {
            tile(3, 1);
            tile(2, 0);
        } else {
            tile(3, 2);
            tile(2, 1);
        }

        if constexpr (ROLE == kMakeRecs) {
            __syncthreads();
            // The record carries (I + A)^-1 whole, so that the walk's solve is one product, U = (I + A)^-1 B, with one
            // wait before it instead of one per block row.  Wave w forms block column w of it, block rows w..3, by the
            // walk's own recurrence on the identity, X_c = T_cc (I_c - sum_{w <= b < c} A_cb X_b): a product's result is
            // already laid out as the next product's second operand, so the column never leaves the wave's registers.
            float4_t X[4];
            half4_t xbh[4], xbl[4];
#pragma unroll
            for (int cr = 0; cr < 4; cr++) {
                X[cr] = float4_t{0.f, 0.f, 0.f, 0.f};
                if (cr < w) continue;
                float4_t am = {0.f, 0.f, 0.f, 0.f}, alo = am;
#pragma unroll
                for (int b = 0; b < cr; b++) {
                    if (b < w) continue;
                    const half4_t xh = *reinterpret_cast<const half4_t *>(&L.pre.ah[16 * cr + n][16 * b + 4 * g]);
                    const half4_t xl = *reinterpret_cast<const half4_t *>(&L.pre.al[16 * cr + n][16 * b + 4 * g]);
                    mma16(xh, xl, xbh[b], xbl[b], am, alo);
                }
                half4_t bh, bl;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float e = (cr == w && 4 * g + r == n ? 1.f : 0.f) + fmaf(alo[r], kLoInv, am[r]);
                    _Float16 hi, lo;
                    split(e, hi, lo);
                    bh[r] = hi; bl[r] = lo;
                }
                const half4_t th = *reinterpret_cast<const half4_t *>(&L.pre.th[cr][n][4 * g]);
                const half4_t tl = *reinterpret_cast<const half4_t *>(&L.pre.tl[cr][n][4 * g]);
                float4_t um = {0.f, 0.f, 0.f, 0.f}, ul = um;
                mma16(th, tl, bh, bl, um, ul);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    X[cr][r] = fmaf(ul[r], kLoInv, um[r]);   // (I + A)^-1 [t = 16 cr + 4g + r][s = 16 w + n]
                    _Float16 hi, lo;
                    split(X[cr][r], hi, lo);
                    xbh[cr][r] = hi; xbl[cr][r] = lo;
                }
            }
            __syncthreads();   // every wave has read the last of -A
#pragma unroll
            for (int cr = 0; cr < 4; cr++) {
                if (cr < w) continue;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    L.pre.ah[16 * cr + 4 * g + r][16 * w + n] = xbh[cr][r];
                    L.pre.al[16 * cr + 4 * g + r][16 * w + n] = xbl[cr][r];
                }
            }
            __syncthreads();
            const uint4 *src = reinterpret_cast<const uint4 *>(&L.pre);
            uint4 *dst = reinterpret_cast<uint4 *>(rec_of(c));
            for (int i = tid; i < kPreVecs; i += kThreads) dst[i] = src[i];
            __syncthreads();   // stored before the next chunk's gates and tiles overwrite it
            continue;
        }

        // ---- 3: every wave's rows against the state ----
        half8_t akh[4], akl[4], aqh[4], aql[4];
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            akh[ks] = *reinterpret_cast<const half8_t *>(&L.kh[16 * w + n][32 * ks + 8 * g]);
            akl[ks] = *reinterpret_cast<const half8_t *>(&L.kl[16 * w + n][32 * ks + 8 * g]);
            aqh[ks] = *reinterpret_cast<const half8_t *>(&L.qh[16 * w + n][32 * ks + 8 * g]);
            aql[ks] = *reinterpret_cast<const half8_t *>(&L.ql[16 * w + n][32 * ks + 8 * g]);
        }
        float Gt[4], bt4[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            Gt[r] = L.pre.G[16 * w + 4 * g + r];
            bt4[r] = L.pre.beta[16 * w + 4 * g + r];
        }
        float4_t acc, accl = {0.f, 0.f, 0.f, 0.f}, w2;
        {
            float4_t w1m = {0.f, 0.f, 0.f, 0.f}, w1l = w1m, w2m = w1m, w2l = w1m;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const half8_t bh = *reinterpret_cast<const half8_t *>(&L.sh[n][32 * ks + 8 * g]);
                const half8_t bl = *reinterpret_cast<const half8_t *>(&L.sl[n][32 * ks + 8 * g]);
                mma32(akh[ks], akl[ks], bh, bl, w1m, w1l);
                mma32(aqh[ks], aql[ks], bh, bl, w2m, w2l);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float gam = __expf(Gt[r]);
                const float W1 = fmaf(w1l[r], kLoInv, w1m[r]);
                acc[r] = bt4[r] * (L.v[16 * w + 4 * g + r][n] - gam * W1);   // B[t][j], t = 16w + 4g + r, j = n
                w2[r] = gam * fmaf(w2l[r], kLoInv, w2m[r]);
            }
        }
        const float GC = L.pre.G[kC - 1];
        if constexpr (ROLE == kWalkRecs) {
            // ---- 4, with (I + A)^-1 in the record: U = (I + A)^-1 B.  Every wave's rows of B as second operands for all,
            //      one wait, then this wave's rows of U from the block rows up to its own ----
            {
                half4_t bh, bl;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    _Float16 hi, lo;
                    split(acc[r], hi, lo);
                    bh[r] = hi; bl[r] = lo;
                }
                *reinterpret_cast<half4_t *>(&L.bth[n][16 * w + 4 * g]) = bh;
                *reinterpret_cast<half4_t *>(&L.btl[n][16 * w + 4 * g]) = bl;
            }
            __syncthreads();
            float4_t um = {0.f, 0.f, 0.f, 0.f}, ul = um;
            for (int cb = 0; cb <= w; cb++) {
                const half4_t xh = *reinterpret_cast<const half4_t *>(&L.pre.ah[16 * w + n][16 * cb + 4 * g]);
                const half4_t xl = *reinterpret_cast<const half4_t *>(&L.pre.al[16 * w + n][16 * cb + 4 * g]);
                const half4_t yh = *reinterpret_cast<const half4_t *>(&L.bth[n][16 * cb + 4 * g]);
                const half4_t yl = *reinterpret_cast<const half4_t *>(&L.btl[n][16 * cb + 4 * g]);
                mma16(xh, xl, yh, yl, um, ul);
            }
            half4_t uh4, ul4, dh4, dl4;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float u = fmaf(ul[r], kLoInv, um[r]);   // U[s = 16 w + 4g + r][j = n]
                _Float16 hi, lo;
                split(u, hi, lo);
                uh4[r] = hi; ul4[r] = lo;
                split(u * __expf(GC - Gt[r]), hi, lo);
                dh4[r] = hi; dl4[r] = lo;
            }
            *reinterpret_cast<half4_t *>(&L.uh[n][16 * w + 4 * g]) = uh4;
            *reinterpret_cast<half4_t *>(&L.ul[n][16 * w + 4 * g]) = ul4;
            *reinterpret_cast<half4_t *>(&L.dh[n][16 * w + 4 * g]) = dh4;
            *reinterpret_cast<half4_t *>(&L.dl[n][16 * w + 4 * g]) = dl4;
            __syncthreads();
        } else {
        __syncthreads();

        // ---- 4: the solve, block row after block row ----
#pragma unroll
        for (int cb = 0; cb < 4; cb++) {
            if (w == cb) {
                // U_c = T_cc (B_c - sum_{b<c} A_cb U_b); the accumulator is already in second-operand order
                half4_t bh, bl;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    _Float16 hi, lo;
                    split(fmaf(accl[r], kLoInv, acc[r]), hi, lo);
                    bh[r] = hi; bl[r] = lo;
                }
                const half4_t th = *reinterpret_cast<const half4_t *>(&L.pre.th[cb][n][4 * g]);
                const half4_t tl = *reinterpret_cast<const half4_t *>(&L.pre.tl[cb][n][4 * g]);
                float4_t um = {0.f, 0.f, 0.f, 0.f}, ul = um;
                mma16(th, tl, bh, bl, um, ul);
                half4_t uh4, ul4, dh4, dl4;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float u = fmaf(ul[r], kLoInv, um[r]);   // U[s = 16 cb + 4g + r][j = n]
                    _Float16 hi, lo;
                    split(u, hi, lo);
                    uh4[r] = hi; ul4[r] = lo;
                    split(u * __expf(GC - Gt[r]), hi, lo);
                    dh4[r] = hi; dl4[r] = lo;
                }
                *reinterpret_cast<half4_t *>(&L.uh[n][16 * cb + 4 * g]) = uh4;
                *reinterpret_cast<half4_t *>(&L.ul[n][16 * cb + 4 * g]) = ul4;
                *reinterpret_cast<half4_t *>(&L.dh[n][16 * cb + 4 * g]) = dh4;
                *reinterpret_cast<half4_t *>(&L.dl[n][16 * cb + 4 * g]) = dl4;
            }
            __syncthreads();
            if (w > cb) {
                const half4_t xh = *reinterpret_cast<const half4_t *>(&L.pre.ah[16 * w + n][16 * cb + 4 * g]);
                const half4_t xl = *reinterpret_cast<const half4_t *>(&L.pre.al[16 * w + n][16 * cb + 4 * g]);
                const half4_t yh = *reinterpret_cast<const half4_t *>(&L.uh[n][16 * cb + 4 * g]);
                const half4_t yl = *reinterpret_cast<const half4_t *>(&L.ul[n][16 * cb + 4 * g]);
                mma16(xh, xl, yh, yl, acc, accl);
            }
        }
        }

        // ---- 5: the rows' outputs ----
        {
            float4_t om = {0.f, 0.f, 0.f, 0.f}, ol = om;
            for (int cb = 0; cb <= w; cb++) {
                const half4_t xh = *reinterpret_cast<const half4_t *>(&L.pre.mh[16 * w + n][16 * cb + 4 * g]);
                const half4_t xl = *reinterpret_cast<const half4_t *>(&L.pre.ml[16 * w + n][16 * cb + 4 * g]);
                const half4_t yh = *reinterpret_cast<const half4_t *>(&L.uh[n][16 * cb + 4 * g]);
                const half4_t yl = *reinterpret_cast<const half4_t *>(&L.ul[n][16 * cb + 4 * g]);
                mma16(xh, xl, yh, yl, om, ol);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int t = t0 + 16 * w + 4 * g + r;
                if (t < a.seq_len)
                    a.out[(static_cast<size_t>(seq) * a.seq_len + t) * vw + static_cast<size_t>(h) * kD + slab * kJ + n] =
                        (w2[r] + fmaf(ol[r], kLoInv, om[r])) * scale;
            }
        }

        // ---- 6: the state: S = e^(G_C) S + (U e^(G_C - G_s))^T K, this wave's 32 columns ----
        {
            const float gC = __expf(GC);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int i = 16 * (2 * w + u) + n;
                float4_t sm = {0.f, 0.f, 0.f, 0.f}, sl = sm;
#pragma unroll
                for (int cb = 0; cb < 4; cb++) {
                    const half4_t xh = *reinterpret_cast<const half4_t *>(&L.dh[n][16 * cb + 4 * g]);
                    const half4_t xl = *reinterpret_cast<const half4_t *>(&L.dl[n][16 * cb + 4 * g]);
                    half4_t yh, yl;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        yh[r] = L.kh[16 * cb + 4 * g + r][i];
                        yl[r] = L.kl[16 * cb + 4 * g + r][i];
                    }
                    mma16(xh, xl, yh, yl, sm, sl);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) S[u][r] = fmaf(gC, S[u][r], fmaf(sl[r], kLoInv, sm[r]));
            }
            publish_state();
        }
        __syncthreads();
    }
    if constexpr (ROLE != kMakeRecs) {
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) state[static_cast<size_t>(4 * g + r) * kD + 16 * (2 * w + u) + n] = S[u][r];
    }
}

}  // namespace

// Whether a call goes through the chunked kernels: a workspace was given, the pass is plain (no
// per-row state planes to keep) and long enough for a chunk to pay.
bool shv_dn_chunk_covers(const shv_dn_step_args &a) {
    if (!a.work || a.spec || a.seq_len <= 16) return false;
    const long long pw = 2ll * a.n_head_k * kD + static_cast<long long>(a.n_head_v) * kD + 2 * a.n_head_v;
    if (static_cast<long long>(a.n_seq) * a.seq_len * pw > a.work_floats) return false;
    return a.n_head_v % a.n_head_k == 0 && a.n_head_k % 2 == 0 && (a.n_head_v * kD) % kThreads == 0 && a.n_head_v * kPrepTok <= kThreads &&
           shv_aligned16(a.work) && shv_aligned16(a.out) && a.ring_stride % 4 == 0;
}

int shv_launch_dn_chunk(shv_ctx *ctx, const shv_dn_step_args &a) {
    const int pw = 2 * a.n_head_k * kD + a.n_head_v * kD + 2 * a.n_head_v;
    const int items = 2 * a.n_head_k / 4 + a.n_head_v * kD / kThreads + 1;
    SHV_LAUNCH(ctx, dn_prep_kernel, dim3(items, (a.seq_len + kPrepTok - 1) / kPrepTok, a.n_seq), dim3(kThreads), 0, a, a.work, pw);
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&dn_chunk_kernel<kWalk>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(sizeof(ChunkLds))));
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&dn_chunk_kernel<kWalkRecs>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(sizeof(ChunkLds))));
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&dn_chunk_kernel<kMakeRecs>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(sizeof(ChunkLds))));
        raised.store(true, std::memory_order_release);
    }
    // Room behind the prepared rows for a record per (sequence, chunk, value head): the chunks' state-independent
    // part is then formed for all of them at once, and the walk over the chunks only reads it.
    const long long prep_floats = (static_cast<long long>(a.n_seq) * a.seq_len * pw + 3) & ~3ll;
    const int n_chunks = (a.seq_len + kC - 1) / kC;
    const long long rec_floats = static_cast<long long>(a.n_seq) * n_chunks * a.n_head_v * static_cast<long long>(sizeof(PreRec) / 4);
    const dim3 grid(a.n_head_v * (kD / kJ), a.n_seq);
    if (n_chunks >= 2 && n_chunks <= 65535 && a.n_seq <= 65535 && prep_floats + rec_floats <= a.work_floats && !ctx->dn_chunk_no_recs) {
        char *recs = reinterpret_cast<char *>(a.work + prep_floats);
        // chunks a producer block takes in a row: as many as still leave a block for every compute unit (a block that
        // takes several has the next one's rows on their way while it works)
        int per = static_cast<int>(static_cast<long long>(a.n_head_v) * n_chunks * a.n_seq / ctx->prop.multiProcessorCount);
        per = per < 1 ? 1 : per > 8 ? 8 : per;
        SHV_LAUNCH(ctx, dn_chunk_kernel<kMakeRecs>, dim3(a.n_head_v, (n_chunks + per - 1) / per, a.n_seq), dim3(kThreads), sizeof(ChunkLds), a,
                   static_cast<const float *>(a.work), pw, recs, per);
        SHV_LAUNCH(ctx, dn_chunk_kernel<kWalkRecs>, grid, dim3(kThreads), sizeof(ChunkLds), a, static_cast<const float *>(a.work), pw, recs, 0);
    } else {
        SHV_LAUNCH(ctx, dn_chunk_kernel<kWalk>, grid, dim3(kThreads), sizeof(ChunkLds), a, static_cast<const float *>(a.work), pw, static_cast<char *>(nullptr), 0);
    }
    return SHV_OK;
}
