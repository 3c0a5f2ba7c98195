// Q4_K dequant-fused GEMM for passes of several rows: Y[t] = W * pro(X[t]) (+ residual[t]) on the
// matrix cores, with the GEMV's arguments and results (verification passes, batched decode rows,
// prompt chunks: llm/graph.go:1383-1429,1527-1666; the reference's form is llm_gemv.comp's
// multi-row arm).
//
// Still HBM-bound on the weights, which are read once for all rows of the pass.  A 64-lane wave
// owns a tile of 16 weight rows and walks along them one 256-column super-block at a time,
// multiplying by up to 16 activation rows with v_mfma_f32_16x16x16_f16:
//   A (tokens x k)  the activations, split into two halves hi + lo (lo = x - hi) so that the
//                   product keeps float32 accuracy.  The block stages them once into LDS, already
//                   in fragment order, and every wave reads them from there
//   B (k x rows)    the 4-bit levels as exact halves 64+n (a level sits in mantissa bits 4..7 of
//                   64.0); lane (row = lane%16, kb = lane/16) reads 8 payload bytes of each
//                   64-weight group, whose low nibbles feed the group's first 32 columns and whose
//                   high nibbles feed the other 32
//   C (tokens x rows) one 32-column sub-block at a time, because each has its own scale and min;
//                   the lane that loaded row n also holds C[.][n], so d*sc and dmin*m apply without
//                   any exchange:  y += d*sc*acc - (64*d*sc + dmin*m)*sum(x).
// Waves do not talk to one another while they stream, except that a matrix with few rows is also
// split along its columns (KS waves a tile), whose partial tiles meet in LDS at the end.
#include <algorithm>

#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;
constexpr int kDepth = 2;  // super-blocks of a tile requested ahead

// One wave's loads for one super-block of its row tile: the 16-byte header of the lane's row and
// 8 payload bytes of each of its four 64-weight groups.
struct SbLoads {
    uint4 hdr;
    uint2 q[4];
    __device__ __forceinline__ void load(const char *sb, int kb) {
        hdr = *reinterpret_cast<const uint4 *>(sb);
#pragma unroll
        for (int g = 0; g < 4; g++) q[g] = *reinterpret_cast<const uint2 *>(sb + 16 + g * 32 + kb * 8);
    }
};

__device__ __forceinline__ half4_t levels(uint32_t even, uint32_t odd) {
    // even = halves (byte0, byte2), odd = halves (byte1, byte3): k order [b0, b2, b1, b3]
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    u32x2 v;
    v.x = even;
    v.y = odd;
    return __builtin_bit_cast(half4_t, v);
}

// LDS: the activation fragments, the per-sub-block sums of x, scratch for the staging's reductions
// and for the column-split tiles.  TT is the pass's row capacity (4, 8 or 16).
template <int TT>
struct Lds {
    // fragment (sub-block s, chunk c, part p) is 4*TT entries of 8 bytes: entry kb*TT + token
    static __host__ __device__ constexpr size_t frag_bytes(int k) { return static_cast<size_t>(k / 32) * 4 * (4 * TT * 8); }
    static __host__ __device__ constexpr size_t sx_bytes(int k) { return static_cast<size_t>(k / 32) * TT * 4; }
    static __host__ __device__ constexpr size_t region(int k) { return frag_bytes(k) + sx_bytes(k); }  // what a pre-staged pass hands over
    static __host__ __device__ constexpr size_t total(int k, int waves) {
        return frag_bytes(k) + sx_bytes(k) + static_cast<size_t>(waves) * 64 * 16 /* tiles or reductions */ + TT * 8;
    }
};

// Stage pro(x) of rows t0..t0+nt into fragment order.  A thread takes quads of four consecutive
// columns of one row; quad q of the pass is row q / (K/4), columns 4*(q % (K/4)).., so a wave's quads
// lie in one row and a 32-column sub-block is eight neighbouring lanes.
template <int TT, int NTHR, int MAXQ>
__device__ __forceinline__ void stage(const shv_gemv_q4k_args &a, int t0, int nt, char *frags, float *sxs, float *red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = a.k, qpr = K / 4;              // quads per row
    const int n_quads = nt * qpr;
    float4 v[MAXQ], zv[MAXQ];  // MAXQ quads a thread at most: the launcher sizes the pass to fit
    const bool has_z = a.prologue == SHV_PRO_GATED_NORM || a.prologue == SHV_PRO_MUL_SIGMOID;
    const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
#pragma unroll
    for (int i = 0; i < MAXQ; i++) {
        const int q = tid + i * NTHR;
        if (q >= n_quads) continue;
        const int t = t0 + q / qpr, c = 4 * (q % qpr);
        v[i] = *reinterpret_cast<const float4 *>(a.x + static_cast<size_t>(t) * a.x_stride + c);
        if (has_z) {
            const float *z = a.z + static_cast<size_t>(t) * a.z_stride;
            if (a.z_ring) {
                const int s = t / sl, k = t % sl;
                const int p = a.pos ? a.pos[s] : 0;
                const int slot = a.slot ? a.slot[s] : s;
                z = a.z + (static_cast<size_t>(slot) * a.ring_slots + (p + k) % a.ring_slots) * a.ring_stride;
            }
            // sigmoid gate with head_dim: z rows are [q | gate] per head and the gate half is wanted
            // (head_dim is 0 or a power of two: the launcher of the row kernel checks)
            const int zi = a.prologue == SHV_PRO_MUL_SIGMOID && a.head_dim > 0 ? (c & ~(a.head_dim - 1)) * 2 + a.head_dim + (c & (a.head_dim - 1)) : c;
            zv[i] = *reinterpret_cast<const float4 *>(z + zi);
        }
    }
    if (a.prologue == SHV_PRO_RMSNORM) {
        // all 64 quads of a wave lie in one row (K/4 is a multiple of 64): red[row][piece] takes
        // the sum of squares of each 256-column piece, added up below in a fixed order
#pragma unroll
        for (int i = 0; i < MAXQ; i++) {
            const int q = tid + i * NTHR;
            float ss = q < n_quads ? fmaf(v[i].x, v[i].x, fmaf(v[i].y, v[i].y, fmaf(v[i].z, v[i].z, v[i].w * v[i].w))) : 0.f;
            ss = wave_sum_all(ss);
            const int q0 = wave * 64 + i * NTHR;
            if (lane == 0 && q0 < n_quads) red[(q0 / qpr) * 16 + (q0 % qpr) / 64] = ss;
        }
        __syncthreads();
        if (tid < nt) {
            float tot = 0.f;
            for (int pc = 0; pc < qpr / 64; pc++) tot += red[tid * 16 + pc];
            red[TT * 16 + tid] = 1.f / sqrtf(tot / static_cast<float>(K) + a.eps);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < MAXQ; i++) {
        const int q = tid + i * NTHR;
        const bool on = q < n_quads;
        const int tl = on ? q / qpr : 0, c = on ? 4 * (q % qpr) : 0;
        float x[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
        if (a.prologue == SHV_PRO_RMSNORM) {
            const float scale = red[TT * 16 + tl];
            const float4 g = *reinterpret_cast<const float4 *>(a.gamma + c);
            x[0] *= scale * g.x; x[1] *= scale * g.y; x[2] *= scale * g.z; x[3] *= scale * g.w;
        } else if (a.prologue == SHV_PRO_GATED_NORM) {
            float ss = on ? fmaf(x[0], x[0], fmaf(x[1], x[1], fmaf(x[2], x[2], x[3] * x[3]))) : 0.f;
            const int span = a.head_dim / 4;  // lanes a head spans
            for (int off = 1; off < span; off <<= 1) ss += __shfl_xor(ss, off, 64);
            const float scale = 1.f / sqrtf(ss / static_cast<float>(a.head_dim) + a.eps);
            const float zz[4] = {zv[i].x, zv[i].y, zv[i].z, zv[i].w};
            // head_dim is a power of two and a multiple of 4 here: the quad's four gammas are one load
            const float4 g4 = *reinterpret_cast<const float4 *>(a.gamma + (c & (a.head_dim - 1)));
            const float gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
            for (int j = 0; j < 4; j++) x[j] = x[j] * scale * gg[j] * sigmoid_fast(zz[j]);
        } else if (a.prologue == SHV_PRO_MUL_SIGMOID) {
            const float zz[4] = {zv[i].x, zv[i].y, zv[i].z, zv[i].w};
#pragma unroll
            for (int j = 0; j < 4; j++) x[j] *= sigmoid_fast(zz[j]);
        }
        // the sub-block's sum of x: eight neighbouring lanes
        float sum = on ? (x[0] + x[1]) + (x[2] + x[3]) : 0.f;
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        sum += __shfl_xor(sum, 4, 64);
        if (on) {
            const int sub = c >> 5, kb = (c & 31) >> 3, chunk = (c & 7) >> 2;
            if ((c & 31) == 0) sxs[sub * TT + tl] = sum;
            // k order of levels(): [x0, x2, x1, x3]
            const float o[4] = {x[0], x[2], x[1], x[3]};
            half4_t h, l;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const _Float16 hi = static_cast<_Float16>(o[j]);
                h[j] = hi;
                l[j] = static_cast<_Float16>(o[j] - static_cast<float>(hi));
            }
            char *e = frags + (static_cast<size_t>((sub * 2 + chunk) * 2) * (4 * TT) + kb * TT + tl) * 8;
            *reinterpret_cast<half4_t *>(e) = h;
            *reinterpret_cast<half4_t *>(e + 4 * TT * 8) = l;
        }
    }
}

// pro(x) of the four columns c..c+3 of activation row t; `scale` is the row's RMSNorm factor.
// Every lane of a wave calls it for the same row (the gated norm adds up across lanes).
__device__ __forceinline__ void pro_quad(const shv_gemv_q4k_args &a, int t, int c, float scale, float (&x)[4]) {
    const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
    const float4 v = *reinterpret_cast<const float4 *>(a.x + static_cast<size_t>(t) * a.x_stride + c);
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    if (a.prologue == SHV_PRO_RMSNORM) {
        const float4 g = *reinterpret_cast<const float4 *>(a.gamma + c);
        x[0] *= scale * g.x; x[1] *= scale * g.y; x[2] *= scale * g.z; x[3] *= scale * g.w;
    } else if (a.prologue == SHV_PRO_GATED_NORM || a.prologue == SHV_PRO_MUL_SIGMOID) {
        const float *z = a.z + static_cast<size_t>(t) * a.z_stride;
        if (a.z_ring) {
            const int s = t / sl, k = t % sl;
            const int p = a.pos ? a.pos[s] : 0;
            const int slot = a.slot ? a.slot[s] : s;
            z = a.z + (static_cast<size_t>(slot) * a.ring_slots + (p + k) % a.ring_slots) * a.ring_stride;
        }
        const int zi = a.prologue == SHV_PRO_MUL_SIGMOID && a.head_dim > 0 ? (c & ~(a.head_dim - 1)) * 2 + a.head_dim + (c & (a.head_dim - 1)) : c;
        const float4 zq = *reinterpret_cast<const float4 *>(z + zi);
        const float zz[4] = {zq.x, zq.y, zq.z, zq.w};
        if (a.prologue == SHV_PRO_GATED_NORM) {
            float ss = fmaf(x[0], x[0], fmaf(x[1], x[1], fmaf(x[2], x[2], x[3] * x[3])));
            const int span = a.head_dim / 4;  // lanes a head spans: a power of two up to 64
            for (int off = 1; off < span; off <<= 1) ss += __shfl_xor(ss, off, 64);
            const float scale = 1.f / sqrtf(ss / static_cast<float>(a.head_dim) + a.eps);
            const float4 g4 = *reinterpret_cast<const float4 *>(a.gamma + (c & (a.head_dim - 1)));
            const float gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
            for (int j = 0; j < 4; j++) x[j] = x[j] * scale * gg[j] * sigmoid_fast(zz[j]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) x[j] *= sigmoid_fast(zz[j]);
        }
    }
}

// The activations of a pass of many rows transformed once, for every block of the products to
// copy.  grid: (k/256, groups of `cap` rows), 256 threads: a block takes one super-block's worth of
// columns of its group's rows, a wave one row's 64 quads at a time, and writes fragments and sums
// straight into the group's region of `staged` (Lds<TT>::region(k) bytes, laid out as the product
// kernel lays out its LDS).  The per-row scale of the RMSNorm prologue needs the whole row: each
// wave adds up the rows it will serve, in a fixed order.
template <int TT>
__global__ __launch_bounds__(256) void gemm_stage_kernel(shv_gemv_q4k_args a, char *staged, int cap) {
    __shared__ float scale_s[TT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = a.k, kp = blockIdx.x, grp = blockIdx.y;
    const int t0 = grp * cap;
    const int nt = a.n_tok - t0 < cap ? a.n_tok - t0 : cap;
    char *frags = staged + static_cast<size_t>(grp) * Lds<TT>::region(K);
    float *sxs = reinterpret_cast<float *>(frags + Lds<TT>::frag_bytes(K));
    if (a.prologue == SHV_PRO_RMSNORM) {
        for (int tl = wave; tl < nt; tl += 4) {
            const float *x = a.x + static_cast<size_t>(t0 + tl) * a.x_stride;
            float ss = 0.f;
            for (int q = lane; q < K / 4; q += 64) {
                const float4 v = *reinterpret_cast<const float4 *>(x + 4 * q);
                ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
            }
            ss = wave_sum_all(ss);
            if (lane == 0) scale_s[tl] = 1.f / sqrtf(ss / static_cast<float>(K) + a.eps);
        }
        __syncthreads();
    }
    for (int tl = wave; tl < nt; tl += 4) {
        const int t = t0 + tl, c = kp * 256 + 4 * lane;
        float x[4];
        pro_quad(a, t, c, a.prologue == SHV_PRO_RMSNORM ? scale_s[tl] : 1.f, x);
        // the sub-block's sum of x: eight neighbouring lanes
        float sum = (x[0] + x[1]) + (x[2] + x[3]);
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        sum += __shfl_xor(sum, 4, 64);
        const int sub = c >> 5, kb = (c & 31) >> 3, chunk = (c & 7) >> 2;
        if ((c & 31) == 0) sxs[sub * TT + tl] = sum;
        // k order of levels(): [x0, x2, x1, x3]
        const float o[4] = {x[0], x[2], x[1], x[3]};
        half4_t h, l;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const _Float16 hi = static_cast<_Float16>(o[j]);
            h[j] = hi;
            l[j] = static_cast<_Float16>(o[j] - static_cast<float>(hi));
        }
        char *e = frags + (static_cast<size_t>((sub * 2 + chunk) * 2) * (4 * TT) + kb * TT + tl) * 8;
        *reinterpret_cast<half4_t *>(e) = h;
        *reinterpret_cast<half4_t *>(e + 4 * TT * 8) = l;
    }
}

// grid: blocks of NTHR/64 waves.  KS consecutive waves share a row tile, each over 1/KS of the
// columns.  t0: first activation row of this launch, nt: how many (<= TT).
template <int TT, int NTHR, int MAXQ>
__global__ __launch_bounds__(NTHR) void gemm_q4k_kernel(shv_gemv_q4k_args a, int t0, int nt, int n_tiles, int ks, const char *staged) {
    extern __shared__ __align__(16) char smem[];
    constexpr int NW = NTHR / 64;
    char *frags = smem;
    float *sxs = reinterpret_cast<float *>(smem + Lds<TT>::frag_bytes(a.k));
    float *ytile = sxs + a.k / 32 * TT;                         // [NW][64] float4, also the staging's reductions
    size_t *yoffs = reinterpret_cast<size_t *>(ytile + NW * 64 * 4);  // [TT]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;  // B: weight row of the tile, k block; C: row n, tokens 4kb..4kb+3
    const int sbs = a.k / SHV_Q4K_BLOCK;      // super-blocks a row
    const size_t row_bytes = static_cast<size_t>(sbs) * SHV_Q4K_BYTES;
    const int steps = sbs / ks, part = wave % ks;
    const int tiles_per_block = NW / ks;
    const char *wbase = static_cast<const char *>(a.w) + static_cast<size_t>(part * steps) * SHV_Q4K_BYTES;

    // the first tile's first super-blocks do not depend on the activations
    int tl = blockIdx.x * tiles_per_block + wave / ks;
    SbLoads ld[kDepth];
    {
        const int r = tl * kTileRows + n;
        const char *rp = wbase + static_cast<size_t>(r < a.n ? r : a.n - 1) * row_bytes;
#pragma unroll
        for (int d = 0; d < kDepth; d++)
            if (d < steps && tl < n_tiles) ld[d].load(rp + d * SHV_Q4K_BYTES, kb);
    }

    // where each activation row's outputs go (the DeltaNet projection ring, or plain rows)
    if (tid < nt) {
        const int t = t0 + tid;
        size_t off;
        if (a.ring_slots > 0 && !a.z_ring) {
            const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
            const int s = t / sl, i = t % sl;
            const int p = a.pos ? a.pos[s] : 0;
            const int slot = a.slot ? a.slot[s] : s;
            off = (static_cast<size_t>(slot) * a.ring_slots + (p + i) % a.ring_slots) * a.ring_stride;
        } else {
            off = static_cast<size_t>(t) * a.y_stride;
        }
        yoffs[tid] = off;
    }
    if (staged) {
        // the operands were made once for the whole pass: every block copies its rows' region
        const size_t region = Lds<TT>::region(a.k);
        const uint4 *src = reinterpret_cast<const uint4 *>(staged);
        uint4 *dst = reinterpret_cast<uint4 *>(smem);
        for (size_t i = tid; i < region / 16; i += NTHR) dst[i] = src[i];
    } else {
        stage<TT, NTHR, MAXQ>(a, t0, nt, frags, sxs, ytile);
    }
    __syncthreads();

    const NibbleConsts nc = nibble_consts();
    // this lane's fragment entry and its four tokens' sums; rows beyond the capacity alias real ones
    const char *my_frag = frags + (kb * TT + (n & (TT - 1))) * 8;
    const float *my_sx = sxs + ((4 * kb) & (TT - 1));
    constexpr int FRAG = 4 * TT * 8;  // bytes of one (sub-block, chunk, part) fragment
    const int stride = gridDim.x * tiles_per_block;
    const int iters = (n_tiles + stride - 1) / stride;
    for (int it = 0; it < iters; it++, tl += stride) {
        const bool live = tl < n_tiles;
        const int r = tl * kTileRows + n;
        const char *rp = wbase + static_cast<size_t>(r < a.n ? r : a.n - 1) * row_bytes;
        float4_t y = {0.f, 0.f, 0.f, 0.f};
        if (live) {
            // super-block j of a tile sits in slot j % depth; steps is a power of two, so is depth
            const int depth = steps < kDepth ? steps : kDepth;
            for (int st = 0; st < steps; st += depth) {
#pragma unroll
                for (int d = 0; d < kDepth; d++) {
                    if (d >= depth) break;
                    const SbLoads cur = ld[d];
                    // the same slot's next super-block, or the next tile's first ones
                    if (st + d + depth < steps) {
                        ld[d].load(rp + (st + d + depth) * SHV_Q4K_BYTES, kb);
                    } else {
                        const int tn = tl + stride;
                        const int dn = st + d + depth - steps;
                        if (tn < n_tiles) {
                            const int rn = tn * kTileRows + n;
                            ld[d].load(wbase + static_cast<size_t>(rn < a.n ? rn : a.n - 1) * row_bytes + dn * SHV_Q4K_BYTES, kb);
                        }
                    }
                    const int sb = part * steps + st + d;
                    const float dd = f16_bits_to_f32(cur.hdr.x), dmin = f16_bits_to_f32(cur.hdr.x >> 16);
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        uint32_t sc, mn;
                        q4k_group_scale_min(cur.hdr, g, sc, mn);
                        const uint32_t q0 = cur.q[g].x, q1 = cur.q[g].y;
#pragma unroll
                        for (int hi = 0; hi < 2; hi++) {
                            const int sub = sb * 8 + g * 2 + hi;
                            half4_t b0, b1;
                            if (hi == 0) {
                                b0 = levels(((q0 << 4) & nc.mask) | nc.one, ((q0 >> 4) & nc.mask) | nc.one);
                                b1 = levels(((q1 << 4) & nc.mask) | nc.one, ((q1 >> 4) & nc.mask) | nc.one);
                            } else {
                                b0 = levels((q0 & nc.mask) | nc.one, ((q0 >> 8) & nc.mask) | nc.one);
                                b1 = levels((q1 & nc.mask) | nc.one, ((q1 >> 8) & nc.mask) | nc.one);
                            }
                            const char *f = my_frag + static_cast<size_t>(sub) * 4 * FRAG;
                            const half4_t xh0 = *reinterpret_cast<const half4_t *>(f);
                            const half4_t xl0 = *reinterpret_cast<const half4_t *>(f + FRAG);
                            const half4_t xh1 = *reinterpret_cast<const half4_t *>(f + 2 * FRAG);
                            const half4_t xl1 = *reinterpret_cast<const half4_t *>(f + 3 * FRAG);
                            float4_t acc = {0.f, 0.f, 0.f, 0.f};
                            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xh0, b0, acc, 0, 0, 0);
                            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xh1, b1, acc, 0, 0, 0);
                            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xl0, b0, acc, 0, 0, 0);
                            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xl1, b1, acc, 0, 0, 0);
                            const float ds = dd * static_cast<float>(hi ? sc >> 8 : sc & 0xFFu);
                            const float e = fmaf(64.f, ds, dmin * static_cast<float>(hi ? mn >> 8 : mn & 0xFFu));
                            const float4 sx = *reinterpret_cast<const float4 *>(my_sx + sub * TT);
                            const float sxv[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
                            for (int j = 0; j < 4; j++) y[j] = fmaf(-e, sxv[j], fmaf(ds, acc[j], y[j]));
                        }
                    }
                }
            }
        }
        // ---- the column parts of a tile meet in LDS; then C[4kb+j][n] goes out ----
        if (ks > 1) {
            *reinterpret_cast<float4_t *>(ytile + (wave * 64 + lane) * 4) = y;
            __syncthreads();
            if (part == 0) {
                for (int p = 1; p < ks; p++) {
                    const float4_t o = *reinterpret_cast<const float4_t *>(ytile + ((wave + p) * 64 + lane) * 4);
                    y += o;
                }
            }
        }
        if (live && part == 0 && r < a.n) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int tok = 4 * kb + j;
                if (tok < nt) {
                    float v = y[j];
                    if (a.residual) v += a.residual[static_cast<size_t>(t0 + tok) * a.y_stride + r];
                    a.y[yoffs[tok] + r] = v;
                }
            }
        }
        if (ks > 1) __syncthreads();
    }
}

// ---------------------------------------------------------------- passes of 3 to 16 rows -------
// Several sequences decoded together, or the rows of a verification pass, against matrices of the
// decode step's widths: the weights are what the launch moves, the rest is what it waits for.  One
// block of sixteen waves a compute unit; every thread asks for its share of the activation rows,
// the gates and gammas that go with them and its wave's first super-blocks before anything is
// computed, the rows become matrix operands under those loads, and one block-wide wait later every
// wave multiplies: v_mfma_f32_16x16x32_f16 with the eight rows as A (binary16 pairs hi + lo, the
// tokens of the upper half of the tile repeat the lower) and a sub-block's weights as B, formed as
// the whole numbers n * sc by one fused multiply-add on halves, one accumulator a super-block
// (y += d * acc), the min term from the sub-blocks' sums of x.  The RMSNorm factor of a row is
// applied to its outputs, so nothing waits for a row's sum of squares.
// Operand order in LDS: fragment (sub-block, part) is 32 entries of 16 bytes, entry 8 kb + token
// holding columns 8 kb .. 8 kb + 7 of the sub-block in the order [0, 2, 1, 3, 4, 6, 5, 7]; a wave
// stages whole sub-blocks (lane = token + 8 * quad of the sub-block), so its writes fill a
// fragment's 512 bytes side by side.
__device__ __forceinline__ size_t out_offset(const shv_gemv_q4k_args &a, int t);
constexpr int kRowsTok = 8, kRowsWaves = 16, kRowsThreads = kRowsWaves * 64;
constexpr int kRowsFrag = 4 * kRowsTok * 16;  // bytes of one (sub-block, part) fragment

template <int K>
struct RowsLds {
    static constexpr size_t frags = static_cast<size_t>(K / 32) * 2 * kRowsFrag;
    static constexpr size_t sums = static_cast<size_t>(K / 32) * kRowsTok * 4;
    static constexpr size_t red = static_cast<size_t>(kRowsTok) * kRowsWaves * 4;
    static constexpr size_t ytile = static_cast<size_t>(kRowsWaves) * 64 * 16;
    static constexpr size_t total = frags + sums + red + ytile + kRowsTok * sizeof(size_t);
};

// grid: blocks of sixteen waves; KS consecutive waves share a 16-row tile of the matrix, each over
// 1/KS of its super-blocks.  t0: first activation row of this launch, nt: how many (<= 8).
template <int K, int PRO, int RD>
__global__ __launch_bounds__(kRowsThreads) void gemm_rows_kernel(shv_gemv_q4k_args a, int t0, int nt, int n_tiles, int ks_log2) {
    extern __shared__ __align__(16) char smem[];
    constexpr int SBS = K / SHV_Q4K_BLOCK;
    constexpr int WCOLS = K / kRowsWaves;   // columns a wave stages: 128 or 256
    constexpr int NQ = WCOLS / 32;          // sub-blocks a wave stages, one a step: a lane's quads
    char *frags = smem;
    float *sxs = reinterpret_cast<float *>(smem + RowsLds<K>::frags);
    float *red = reinterpret_cast<float *>(smem + RowsLds<K>::frags + RowsLds<K>::sums);          // [token][wave]
    float *ytile = red + kRowsTok * kRowsWaves;                                                 // [wave][64] float4
    size_t *yoffs = reinterpret_cast<size_t *>(ytile + kRowsWaves * 64 * 4);                    // [token]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;  // B: weight row of the tile, k block; C: row n, tokens 4 kb .. 4 kb + 3
    constexpr size_t row_bytes = static_cast<size_t>(SBS) * SHV_Q4K_BYTES;
    const int ks = 1 << ks_log2, steps_log2 = __builtin_ctz(SBS) - ks_log2, steps = 1 << steps_log2;
    const int part = wave & (ks - 1), tpb = kRowsWaves >> ks_log2;
    const int tl0 = blockIdx.x * tpb + (wave >> ks_log2), stride = gridDim.x * tpb;
    const int iters = (n_tiles + stride - 1) / stride;
    const int total = iters << steps_log2;  // (tile, super-block) steps of this wave, the same count for every wave
    const char *wbase = static_cast<const char *>(a.w) + static_cast<size_t>(part << steps_log2) * SHV_Q4K_BYTES;
    auto sb_of = [&](int idx) {
        const int tile = tl0 + (idx >> steps_log2) * stride, r = tile * kTileRows + n;
        return wbase + static_cast<size_t>(r < a.n ? r : a.n - 1) * row_bytes + static_cast<size_t>(idx & (steps - 1)) * SHV_Q4K_BYTES;
    };

    // ---- everything this thread will need, asked for at once: its quads of the rows first ----
    const int st_tok = lane & (kRowsTok - 1), st_quad = lane >> 3;  // token, quad of the sub-block
    const int t_ld = t0 + (st_tok < nt ? st_tok : nt - 1);          // rows past the pass repeat its last (their outputs are dropped)
    const int c0 = wave * WCOLS + 4 * st_quad;                      // step i: columns c0 + 32 i ..
    float4 xv[NQ], zv[NQ], gv[PRO == SHV_PRO_GATED_NORM ? 4 : NQ];
    {
        const float *xrow = a.x + static_cast<size_t>(t_ld) * a.x_stride;
        const float *zrow = a.z;
        if constexpr (PRO == SHV_PRO_GATED_NORM || PRO == SHV_PRO_MUL_SIGMOID) {
            zrow = a.z + static_cast<size_t>(t_ld) * a.z_stride;
            if (a.z_ring) {
                const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
                const int s = t_ld / sl, k = t_ld % sl;
                const int p = a.pos ? a.pos[s] : 0;
                const int slot = a.slot ? a.slot[s] : s;
                zrow = a.z + (static_cast<size_t>(slot) * a.ring_slots + (p + k) % a.ring_slots) * a.ring_stride;
            }
        }
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            const int c = c0 + 32 * i;
            xv[i] = *reinterpret_cast<const float4 *>(xrow + c);
            if constexpr (PRO == SHV_PRO_RMSNORM) gv[i] = *reinterpret_cast<const float4 *>(a.gamma + c);
            if constexpr (PRO == SHV_PRO_GATED_NORM) {
                // heads of 128 columns: the gammas of step i are those of step i + 4
                if (i < 4) gv[i] = *reinterpret_cast<const float4 *>(a.gamma + (c & 127));
                zv[i] = *reinterpret_cast<const float4 *>(zrow + c);
            }
            if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
                // z rows are [q | gate] per head and the gate half is wanted (head_dim 0: plain rows)
                const int zi = a.head_dim > 0 ? (c & ~(a.head_dim - 1)) * 2 + a.head_dim + (c & (a.head_dim - 1)) : c;
                zv[i] = *reinterpret_cast<const float4 *>(zrow + zi);
            }
        }
    }
    SbLoads ld[RD];
#pragma unroll
    for (int d = 0; d < RD; d++)
        if (d < total) ld[d].load(sb_of(d), kb);
    if (tid < nt) yoffs[tid] = out_offset(a, t0 + tid);

    // ---- the rows become operands ----
    {
        float ss = 0.f;
        float hs[NQ];
        if constexpr (PRO == SHV_PRO_GATED_NORM) {
            // a head is four steps of this lane and the eight lanes of its token
#pragma unroll
            for (int i = 0; i < NQ; i++) hs[i] = fmaf(xv[i].x, xv[i].x, fmaf(xv[i].y, xv[i].y, fmaf(xv[i].z, xv[i].z, xv[i].w * xv[i].w)));
#pragma unroll
            for (int h = 0; h < NQ; h += 4) {
                float t = (hs[h] + hs[h + 1]) + (hs[h + 2] + hs[h + 3]);
                t += __shfl_xor(t, 8, 64);
                t += __shfl_xor(t, 16, 64);
                t += __shfl_xor(t, 32, 64);
                hs[h] = __builtin_amdgcn_rsqf(t * (1.f / 128.f) + a.eps);
            }
        }
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            float4 v = xv[i];
            if constexpr (PRO == SHV_PRO_RMSNORM) {
                ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
                v = make_float4(v.x * gv[i].x, v.y * gv[i].y, v.z * gv[i].z, v.w * gv[i].w);
            } else if constexpr (PRO == SHV_PRO_GATED_NORM) {
                const float sc = hs[i & ~3];
                const float4 g = gv[i & 3], z = zv[i];
                v = make_float4(v.x * sc * g.x * sigmoid_fast(z.x), v.y * sc * g.y * sigmoid_fast(z.y),
                                v.z * sc * g.z * sigmoid_fast(z.z), v.w * sc * g.w * sigmoid_fast(z.w));
            } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
                const float4 z = zv[i];
                v = make_float4(v.x * sigmoid_fast(z.x), v.y * sigmoid_fast(z.y), v.z * sigmoid_fast(z.z), v.w * sigmoid_fast(z.w));
            }
            // the sub-block's sum of x: the eight lanes of this token
            float sum = (v.x + v.y) + (v.z + v.w);
            sum += __shfl_xor(sum, 8, 64);
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            const int sub = wave * NQ + i;
            if (st_quad == 0) sxs[sub * kRowsTok + st_tok] = sum;
            const float o[4] = {v.x, v.z, v.y, v.w};
            half4_t h, l;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const _Float16 hi = static_cast<_Float16>(o[j]);
                h[j] = hi;
                l[j] = static_cast<_Float16>(o[j] - static_cast<float>(hi));
            }
            char *e = frags + static_cast<size_t>(sub) * 2 * kRowsFrag + ((st_quad >> 1) * kRowsTok + st_tok) * 16 + (st_quad & 1) * 8;
            *reinterpret_cast<half4_t *>(e) = h;
            *reinterpret_cast<half4_t *>(e + kRowsFrag) = l;
        }
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            ss += __shfl_xor(ss, 8, 64);
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            if (st_quad == 0) red[st_tok * kRowsWaves + wave] = ss;
        }
    }
    // LDS writes only: the super-blocks asked for above stay on their way
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // this lane's four tokens (those of the tile's upper half repeat the lower): their RMSNorm factors
    const int tk0 = (4 * kb) & (kRowsTok - 1);
    float scale[4] = {1.f, 1.f, 1.f, 1.f};
    if constexpr (PRO == SHV_PRO_RMSNORM) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float4 *r4 = reinterpret_cast<const float4 *>(red + (tk0 + j) * kRowsWaves);
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < kRowsWaves / 4; w++) {
                const float4 r = r4[w];
                tot += (r.x + r.y) + (r.z + r.w);
            }
            scale[j] = __builtin_amdgcn_rsqf(tot * (1.f / static_cast<float>(K)) + a.eps);
        }
    }
    const char *my_frag = frags + (kb * kRowsTok + (n & (kRowsTok - 1))) * 16;
    const float *my_sx = sxs + tk0;
    uint32_t m0 = 0x000F000Fu, o0 = 0x64006400u, m4 = 0x00F000F0u, o4 = 0x54005400u;
    asm volatile("" : "+s"(m0), "+s"(m4));
    asm volatile("" : "+v"(o0), "+v"(o4));
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

    float4_t y = {0.f, 0.f, 0.f, 0.f};
    for (int base = 0; base < total; base += RD) {
#pragma unroll
        for (int d = 0; d < RD; d++) {
            const int idx = base + d;
            if (idx >= total) break;
            const SbLoads cur = ld[d];
            if (idx + RD < total) ld[d].load(sb_of(idx + RD), kb);
            const int sb = (part << steps_log2) + (idx & (steps - 1));
            const float dd = f16_bits_to_f32(cur.hdr.x), dmin = f16_bits_to_f32(cur.hdr.x >> 16);
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint32_t sc, mn;
                q4k_group_scale_min(cur.hdr, g, sc, mn);
                const uint32_t q0 = cur.q[g].x, q1 = cur.q[g].y;
#pragma unroll
                for (int hi = 0; hi < 2; hi++) {
                    const int sub = sb * 8 + g * 2 + hi;
                    // (C + n) * sc - C * sc = n * sc, a whole number up to 945: bits 0..3 of a half read as
                    // 1024 + n under 1024's exponent, bits 4..7 as 64 + n under 64's
                    const _Float16 s1 = static_cast<_Float16>(static_cast<float>(hi ? sc >> 8 : sc & 0xFFu));
                    const half2_t s2 = {s1, s1};
                    half2_t w[4], c[4];
                    if (hi == 0) {
                        w[0] = __builtin_bit_cast(half2_t, (q0 & m0) | o0); w[1] = __builtin_bit_cast(half2_t, ((q0 >> 4) & m4) | o4);
                        w[2] = __builtin_bit_cast(half2_t, (q1 & m0) | o0); w[3] = __builtin_bit_cast(half2_t, ((q1 >> 4) & m4) | o4);
                        c[0] = c[2] = s2 * static_cast<half2_t>(static_cast<_Float16>(-1024.f));
                        c[1] = c[3] = s2 * static_cast<half2_t>(static_cast<_Float16>(-64.f));
                    } else {
                        w[0] = __builtin_bit_cast(half2_t, (q0 & m4) | o4); w[1] = __builtin_bit_cast(half2_t, ((q0 >> 8) & m4) | o4);
                        w[2] = __builtin_bit_cast(half2_t, (q1 & m4) | o4); w[3] = __builtin_bit_cast(half2_t, ((q1 >> 8) & m4) | o4);
                        c[0] = c[1] = c[2] = c[3] = s2 * static_cast<half2_t>(static_cast<_Float16>(-64.f));
                    }
                    half8_t b;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const half2_t p = __builtin_elementwise_fma(w[i], s2, c[i]);
                        b[2 * i] = p[0];
                        b[2 * i + 1] = p[1];
                    }
                    const char *f = my_frag + static_cast<size_t>(sub) * 2 * kRowsFrag;
                    const half8_t xh = *reinterpret_cast<const half8_t *>(f);
                    const half8_t xl = *reinterpret_cast<const half8_t *>(f + kRowsFrag);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, b, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, b, acc, 0, 0, 0);
                    const float e = dmin * static_cast<float>(hi ? mn >> 8 : mn & 0xFFu);
                    const float4 sx = *reinterpret_cast<const float4 *>(my_sx + sub * kRowsTok);
                    y[0] = fmaf(-e, sx.x, y[0]); y[1] = fmaf(-e, sx.y, y[1]);
                    y[2] = fmaf(-e, sx.z, y[2]); y[3] = fmaf(-e, sx.w, y[3]);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; j++) y[j] = fmaf(dd, acc[j], y[j]);
            if ((idx & (steps - 1)) != steps - 1) continue;
            // ---- the tile's last super-block: the column parts meet in LDS, then C[4 kb + j][n] goes out ----
            const int tile = tl0 + (idx >> steps_log2) * stride, r = tile * kTileRows + n;
            if (ks > 1) {
                *reinterpret_cast<float4_t *>(ytile + (wave * 64 + lane) * 4) = y;
                __syncthreads();
                if (part == 0) {
                    for (int p = 1; p < ks; p++) y += *reinterpret_cast<const float4_t *>(ytile + ((wave + p) * 64 + lane) * 4);
                }
            }
            if (part == 0 && tile < n_tiles && r < a.n && kb < kRowsTok / 4) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int tok = 4 * kb + j;
                    if (tok < nt) {
                        float v = y[j] * scale[j];
                        if (a.residual) v += a.residual[static_cast<size_t>(t0 + tok) * a.y_stride + r];
                        a.y[yoffs[tok] + r] = v;
                    }
                }
            }
            if (ks > 1) __syncthreads();
            y = float4_t{0.f, 0.f, 0.f, 0.f};
        }
    }
}

// ---------------------------------------------------------------- passes of 17 to 64 rows -------
// A prompt chunk has more rows than one block can keep in LDS for the whole width of the matrix,
// so its operands stream: the activations of 64 rows are made once into `staged` as slabs of 128
// columns (four sub-blocks), each slab in the order the products read it, and every block of the
// product walks the slabs through two LDS buffers while its waves stream their own weight rows.
// A wave owns 32 weight rows (two tiles) and all 64 activation rows (four tiles): one
// v_mfma_f32_16x16x32_f16 per (tile, tile, half of x) covers a whole 32-column sub-block, whose
// eight levels a lane already holds in the 8 payload bytes it loaded.  A matrix with few rows is
// also split along its columns over blockIdx.y; the parts meet in a second small launch.
constexpr int kWideTok = 64;                                 // activation rows of a launch
constexpr int kWideFrag = 64 * 16;                           // one operand: a lane's eight halves
constexpr int kWideSlabA = 4 * 4 * 2 * kWideFrag;            // [sub-block 4][token tile 4][hi, lo]
constexpr int kWideSlab = kWideSlabA + 4 * kWideTok * 4;     // + the sub-blocks' sums of x

// After a group's slabs, the same sums as operands of the min term: for every 1024 columns (four
// super-blocks) a fragment per (token tile, part): lane = token in the tile + 16 * (super-block of
// the four), the super-block's eight sums' binary16 values (part 0) and what those leave (part 1).
constexpr int kWideSumFrags = 4 * 2 * kWideFrag;
__host__ __device__ constexpr size_t wide_sums_offset(int k) { return static_cast<size_t>(k / 128) * kWideSlab; }
__host__ __device__ constexpr size_t wide_region(int k) { return wide_sums_offset(k) + static_cast<size_t>((k + 1023) / 1024) * kWideSumFrags; }

// Where activation row t of the pass writes its outputs: the DeltaNet projection ring, or plain rows.
__device__ __forceinline__ size_t out_offset(const shv_gemv_q4k_args &a, int t) {
    if (a.ring_slots > 0 && !a.z_ring) {
        const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
        const int s = t / sl, i = t % sl;
        const int p = a.pos ? a.pos[s] : 0;
        const int slot = a.slot ? a.slot[s] : s;
        return (static_cast<size_t>(slot) * a.ring_slots + (p + i) % a.ring_slots) * a.ring_stride;
    }
    return static_cast<size_t>(t) * a.y_stride;
}

// The same for a pass of up to 64 rows a group, in the slab order gemm_wide_kernel streams.
// grid: (parts of the k/256 column blocks, 16 quartets of rows, groups of 64 rows), 256 threads: a wave takes one row's 64
// quads of one super-block's columns at a time; rows a group does not have are written as zeros.
__global__ __launch_bounds__(256) void gemm_wide_stage_kernel(shv_gemv_q4k_args a, char *staged, float *x_out) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = a.k, grp = blockIdx.z;
    const int t0 = grp * kWideTok;
    const int nt = a.n_tok - t0 < kWideTok ? a.n_tok - t0 : kWideTok;
    const int tl = blockIdx.y * 4 + wave;
    char *region = staged + static_cast<size_t>(grp) * wide_region(K);
    float scale = 1.f;
    if (a.prologue == SHV_PRO_RMSNORM && tl < nt) {
        // the row's factor needs the whole row: every wave adds up its own, in a fixed order
        const float *x = a.x + static_cast<size_t>(t0 + tl) * a.x_stride;
        float ss = 0.f;
        for (int q = lane; q < K / 4; q += 64) {
            const float4 v = *reinterpret_cast<const float4 *>(x + 4 * q);
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
        }
        ss = wave_sum_all(ss);
        scale = 1.f / sqrtf(ss / static_cast<float>(K) + a.eps);
    }
    // the block's waves take their rows' column blocks of 256 in turn, blockIdx.x first: a row's factor is formed once for all of them
    for (int kp = blockIdx.x; kp < K / 256; kp += gridDim.x) {
        const int c = kp * 256 + 4 * lane;
        // the quad's place: slab of 128 columns, sub-block of it, k block of 8 columns, which half of those
        char *slab = region + static_cast<size_t>(c >> 7) * kWideSlab;
        const int sub = (c & 127) >> 5, kb = (c & 31) >> 3, qh = (c & 7) >> 2;
        float x[4] = {0.f, 0.f, 0.f, 0.f};
        if (tl < nt) pro_quad(a, t0 + tl, c, scale, x);
        // the transformed row itself, for a caller that also needs it as plain float32 (the router's xn)
        if (x_out && tl < nt) *reinterpret_cast<float4 *>(x_out + static_cast<size_t>(t0 + tl) * K + c) = float4{x[0], x[1], x[2], x[3]};
        float sum = (x[0] + x[1]) + (x[2] + x[3]);
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        sum += __shfl_xor(sum, 4, 64);
        if ((c & 31) == 0) {
            reinterpret_cast<float *>(slab + kWideSlabA)[sub * kWideTok + tl] = sum;
            const _Float16 hi = static_cast<_Float16>(sum);
            _Float16 *sp = reinterpret_cast<_Float16 *>(region + wide_sums_offset(K) + static_cast<size_t>(((c >> 10) * 4 + (tl >> 4)) * 2) * kWideFrag +
                                                        (((c >> 8) & 3) * 16 + (tl & 15)) * 16) + ((c >> 5) & 7);
            sp[0] = hi;
            sp[kWideFrag / 2] = static_cast<_Float16>(sum - static_cast<float>(hi));
        }
        // slot order of a lane's eight columns: [0, 2, 1, 3, 4, 6, 5, 7]
        const float o[4] = {x[0], x[2], x[1], x[3]};
        half4_t h, l;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const _Float16 hi = static_cast<_Float16>(o[j]);
            h[j] = hi;
            l[j] = static_cast<_Float16>(o[j] - static_cast<float>(hi));
        }
        char *e = slab + static_cast<size_t>((sub * 4 + (tl >> 4)) * 2) * kWideFrag + (kb * 16 + (tl & 15)) * 16 + qh * 8;
        *reinterpret_cast<half4_t *>(e) = h;
        *reinterpret_cast<half4_t *>(e + kWideFrag) = l;
    }
}

// How many blocks share a row's column blocks: under the RMSNorm prologue every one of them reads the whole row for
// its factor, so as few as still fill the chip.
static inline int stage_parts(const shv_gemv_q4k_args &a, int groups) {
    const int all = a.k / 256;
    if (a.prologue != SHV_PRO_RMSNORM) return all;
    int parts = 1;
    while (parts < all && parts * (kWideTok / 4) * groups < 1024) parts *= 2;
    return parts;
}

struct WideLoads {
    uint4 hdr;
    uint2 q[2];
    // step: which 128 columns of the row; the two 64-weight groups of that half of a super-block
    __device__ __forceinline__ void load(const char *row, int step, int kb) {
        const char *sb = row + static_cast<size_t>(step >> 1) * SHV_Q4K_BYTES;
        hdr = *reinterpret_cast<const uint4 *>(sb);
#pragma unroll
        for (int g = 0; g < 2; g++) q[g] = *reinterpret_cast<const uint2 *>(sb + 16 + ((step & 1) * 2 + g) * 32 + kb * 8);
    }
};

// grid: (row groups of NW * R * 16 rows, column parts); NW waves, each owning R row tiles.
// part: [parts][64][n] partial products when the columns are split, else unused.
template <int NW, int kWideR>
__global__ __launch_bounds__(NW * 64) void gemm_wide_kernel(shv_gemv_q4k_args a, int t0, int nt, const char *staged, float *part, int steps_per, int groups) {
    extern __shared__ __align__(16) char smem[];
    size_t *yoffs = reinterpret_cast<size_t *>(smem + 2 * kWideSlab);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int sbs = a.k / SHV_Q4K_BLOCK;
    const size_t row_bytes = static_cast<size_t>(sbs) * SHV_Q4K_BYTES;
    const int s0 = blockIdx.y * steps_per, s1 = s0 + steps_per;
    constexpr int NTHR = NW * 64;
    // A pass of many groups of 64 rows in one launch: neighbouring blocks take the same weight rows
    // for different groups, so that a row block's weights come from HBM once and from L2 after.
    int xb = blockIdx.x;
    if (groups > 1) {
        const int grp = xb % groups;
        xb /= groups;
        t0 = grp * kWideTok;
        nt = a.n_tok - t0 < kWideTok ? a.n_tok - t0 : kWideTok;
        staged += static_cast<size_t>(grp) * wide_region(a.k);
    }
    const int row0 = (xb * NW + wave) * (kWideR * kTileRows);
    const int ntt = (nt + kTileRows - 1) / kTileRows;

    const char *rp[kWideR];
    WideLoads w[kWideR];
#pragma unroll
    for (int r = 0; r < kWideR; r++) {
        const int row = row0 + r * kTileRows + n;
        rp[r] = static_cast<const char *>(a.w) + static_cast<size_t>(row < a.n ? row : a.n - 1) * row_bytes;
        w[r].load(rp[r], s0, kb);
    }
    if (tid < nt) yoffs[tid] = out_offset(a, t0 + tid);
    constexpr int kVec = kWideSlab / 16;  // 16-byte pieces of a slab
    {
        const uint4 *src = reinterpret_cast<const uint4 *>(staged + static_cast<size_t>(s0) * kWideSlab);
        uint4 *dst = reinterpret_cast<uint4 *>(smem);
        for (int i = tid; i < kVec; i += NTHR) dst[i] = src[i];
    }
    __syncthreads();

    const NibbleConsts nc = nibble_consts();
    float4_t y[kWideR][4];
#pragma unroll
    for (int r = 0; r < kWideR; r++)
#pragma unroll
        for (int tt = 0; tt < 4; tt++) y[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int s = s0; s < s1; s++) {
        const int cur = (s - s0) & 1;
        const bool more = s + 1 < s1;
        // the next slab and the next weights are requested before this step's products
        // a slab is kPer pieces of 16 bytes a thread, and the sums one more for the first 64 threads
        constexpr int kPer = kWideSlabA / 16 / NTHR;
        static_assert(kPer * NTHR * 16 == kWideSlabA && kVec - kPer * NTHR == 64, "slab copy layout");
        // (the last step asks for its own slab again, so that the loads are unconditional)
        uint4 an[kPer], asx;
        WideLoads wn[kWideR];
        {
            const int sn = more ? s + 1 : s;
            const uint4 *src = reinterpret_cast<const uint4 *>(staged + static_cast<size_t>(sn) * kWideSlab);
#pragma unroll
            for (int i = 0; i < kPer; i++) an[i] = src[tid + i * NTHR];
            asx = src[kPer * NTHR + (tid & 63)];
#pragma unroll
            for (int r = 0; r < kWideR; r++) wn[r].load(rp[r], sn, kb);
        }
        const char *A = smem + cur * kWideSlab;
        const float *sxs = reinterpret_cast<const float *>(A + kWideSlabA);
        float dd[kWideR], dmin[kWideR];
#pragma unroll
        for (int r = 0; r < kWideR; r++) {
            dd[r] = f16_bits_to_f32(w[r].hdr.x);
            dmin[r] = f16_bits_to_f32(w[r].hdr.x >> 16);
        }
#pragma unroll
        for (int sub = 0; sub < 4; sub++) {
            const int g = sub >> 1, hi = sub & 1;
            half8_t b[kWideR];
            float ds[kWideR], e[kWideR];
#pragma unroll
            for (int r = 0; r < kWideR; r++) {
                uint32_t sc, mn;
                q4k_group_scale_min(w[r].hdr, (s & 1) * 2 + g, sc, mn);
                const uint32_t q0 = w[r].q[g].x, q1 = w[r].q[g].y;
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                u32x4 v;
                // slot order of the eight columns: bytes [0, 2, 1, 3, 4, 6, 5, 7]
                if (hi == 0) {
                    v.x = ((q0 << 4) & nc.mask) | nc.one; v.y = ((q0 >> 4) & nc.mask) | nc.one;
                    v.z = ((q1 << 4) & nc.mask) | nc.one; v.w = ((q1 >> 4) & nc.mask) | nc.one;
                } else {
                    v.x = (q0 & nc.mask) | nc.one; v.y = ((q0 >> 8) & nc.mask) | nc.one;
                    v.z = (q1 & nc.mask) | nc.one; v.w = ((q1 >> 8) & nc.mask) | nc.one;
                }
                b[r] = __builtin_bit_cast(half8_t, v);
                ds[r] = dd[r] * static_cast<float>(hi ? sc >> 8 : sc & 0xFFu);
                e[r] = fmaf(64.f, ds[r], dmin[r] * static_cast<float>(hi ? mn >> 8 : mn & 0xFFu));
            }
#pragma unroll
            for (int tt = 0; tt < 4; tt++) {
                if (tt < ntt) {
                    const char *f = A + static_cast<size_t>((sub * 4 + tt) * 2) * kWideFrag + lane * 16;
                    const half8_t xh = *reinterpret_cast<const half8_t *>(f);
                    const half8_t xl = *reinterpret_cast<const half8_t *>(f + kWideFrag);
                    const float4 sx = *reinterpret_cast<const float4 *>(sxs + sub * kWideTok + tt * kTileRows + 4 * kb);
                    const float sxv[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
                    for (int r = 0; r < kWideR; r++) {
                        float4_t acc = {0.f, 0.f, 0.f, 0.f};
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, b[r], acc, 0, 0, 0);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, b[r], acc, 0, 0, 0);
#pragma unroll
                        for (int j = 0; j < 4; j++) y[r][tt][j] = fmaf(-e[r], sxv[j], fmaf(ds[r], acc[j], y[r][tt][j]));
                    }
                }
            }
        }
        if (more) {
            // the other buffer was last read a step ago, before the barrier that ended that step
            uint4 *dst = reinterpret_cast<uint4 *>(smem + (cur ^ 1) * kWideSlab);
#pragma unroll
            for (int i = 0; i < kPer; i++) dst[tid + i * NTHR] = an[i];
            if (tid < 64) dst[kPer * NTHR + tid] = asx;
#pragma unroll
            for (int r = 0; r < kWideR; r++) w[r] = wn[r];
        }
        __syncthreads();
    }

    // C[token 16 tt + 4 kb + j][row n] of each tile
#pragma unroll
    for (int r = 0; r < kWideR; r++) {
        const int row = row0 + r * kTileRows + n;
        if (row >= a.n) continue;
#pragma unroll
        for (int tt = 0; tt < 4; tt++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int tok = tt * kTileRows + 4 * kb + j;
                if (tok >= nt) continue;
                float v = y[r][tt][j];
                if (gridDim.y > 1) {
                    part[(static_cast<size_t>(blockIdx.y) * kWideTok + tok) * a.n + row] = v;
                } else {
                    if (a.residual) v += a.residual[static_cast<size_t>(t0 + tok) * a.y_stride + row];
                    a.y[yoffs[tok] + row] = v;
                }
            }
        }
    }
}

// The same product for a pass of many groups, every group in one launch, with the second operand
// formed as the experts' grouped kernels form theirs: a sub-block's eight weights a lane become the
// whole numbers n * sc (exact in binary16), one matrix accumulator runs over a super-block and takes
// its d at the end, and the min term is the only per-sub-block vector work: half the vector
// instructions per matrix instruction of the kernel above, and no branch inside a step.
// grid: (row blocks of NW*R*16 rows) x groups; all four token tiles are multiplied whatever the
// group holds (rows it does not have were staged as zeros).
template <int NW, int R>
__global__ __launch_bounds__(NW * 64) void gemm_pass_kernel(shv_gemv_q4k_args a, const char *staged_all, int groups) {
    extern __shared__ __align__(16) char smem[];
    char *sumf = smem + 2 * kWideSlab;   // the sums of the quarter of the columns in hand, as operands
    size_t *yoffs = reinterpret_cast<size_t *>(sumf + kWideSumFrags);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int sbs = a.k / SHV_Q4K_BLOCK;
    const size_t row_bytes = static_cast<size_t>(sbs) * SHV_Q4K_BYTES;
    const int grp = blockIdx.x % groups, xb = blockIdx.x / groups;
    const int t0 = grp * kWideTok;
    const int nt = a.n_tok - t0 < kWideTok ? a.n_tok - t0 : kWideTok;
    const char *staged = staged_all + static_cast<size_t>(grp) * wide_region(a.k);
    const int row0 = (xb * NW + wave) * (R * kTileRows);
    const int steps = a.k / 128;

    const char *rp[R];
    uint4 hdr[R], hdrn[R];
    uint2 q[R][2], qn[R][2];
    // step s: the 128 columns s*128.. of the row = groups 2(s&1), 2(s&1)+1 of super-block s>>1
    auto load_q = [&](int s, uint2 (&dst)[R][2]) {
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int g = 0; g < 2; g++)
                dst[r][g] = *reinterpret_cast<const uint2 *>(rp[r] + static_cast<size_t>(s >> 1) * SHV_Q4K_BYTES + 16 + ((s & 1) * 2 + g) * 32 + kb * 8);
    };
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = row0 + r * kTileRows + n;
        rp[r] = static_cast<const char *>(a.w) + static_cast<size_t>(row < a.n ? row : a.n - 1) * row_bytes;
        hdr[r] = *reinterpret_cast<const uint4 *>(rp[r]);
    }
    load_q(0, q);
    if (tid < nt) yoffs[tid] = out_offset(a, t0 + tid);
    // A slab is 33 pieces of 1 KB that lie in `staged` as they will in LDS: the loads place them
    // there themselves (lane l's 16 bytes at 16 l of the piece), through no register.
    constexpr int kPieces = kWideSlab / 1024;
    static_assert(kPieces * 1024 == kWideSlab, "whole pieces");
    auto ask_slab = [&](int s, char *buf) {
        const char *src = staged + static_cast<size_t>(s) * kWideSlab + lane * 16;
        for (int c = wave; c < kPieces; c += NW)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + c * 1024), (__attribute__((address_space(3))) void *)(buf + c * 1024), 16, 0, 0);
    };
    // the min term of columns [1024 qt, 1024 qt + 1024): the tokens' sums (wave w asks for fragment w of eight) and this lane's
    // rows' headers of super-block 4 qt + kb, both a step ahead of their use
    static_assert(NW >= 8, "a fragment of sums a wave");
    uint4 hq[R];
    auto ask_quarter = [&](int qt) {
        if (wave < 8)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(staged + wide_sums_offset(a.k) + static_cast<size_t>(qt * 8 + wave) * kWideFrag + lane * 16),
                                             (__attribute__((address_space(3))) void *)(sumf + wave * kWideFrag), 16, 0, 0);
        const int sb = 4 * qt + kb < sbs ? 4 * qt + kb : 0;
#pragma unroll
        for (int r = 0; r < R; r++) hq[r] = *reinterpret_cast<const uint4 *>(rp[r] + static_cast<size_t>(sb) * SHV_Q4K_BYTES);
    };
    ask_slab(0, smem);
    ask_quarter(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    const NibbleConsts nc = nibble_consts();
    uint32_t m0 = 0x000F000Fu, o0 = 0x64006400u;   // bits 0..3 of both halves under the exponent of 1024
    asm volatile("" : "+s"(m0));
    asm volatile("" : "+v"(o0));
    float4_t y[R][4], acc[R][4];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int tt = 0; tt < 4; tt++) y[r][tt] = acc[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int s = 0; s < steps; s++) {
        const int cur = s & 1;
        const bool more = s + 1 < steps;
        {
            const int sn = more ? s + 1 : s;
            if (more) ask_slab(sn, smem + (cur ^ 1) * kWideSlab);   // the other buffer was read to its end before the barrier that ended the last step
            if (more && (sn & 7) == 0) {
                // the sums in LDS were read at this quarter's first step, steps ago; every wave is past that
                ask_quarter(sn >> 3);
            }
            load_q(sn, qn);
            if (s & 1) {
#pragma unroll
                for (int r = 0; r < R; r++) hdrn[r] = *reinterpret_cast<const uint4 *>(rp[r] + static_cast<size_t>(sn >> 1) * SHV_Q4K_BYTES);
            }
        }
        const char *A = smem + cur * kWideSlab;
        if ((s & 7) == 0) {
            // y -= sum over the quarter's sub-blocks of dmin * m * sum(x), as three matrix products a token tile:
            // -dmin * m has 17 significant bits and goes as two halves, the sums come as two halves too
            // (the small halves' product is below float32's last bit)
            const bool on = 4 * (s >> 3) + kb < sbs;
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float nd = on ? -f16_bits_to_f32(hq[r].x >> 16) : 0.f;
                const uint32_t m03 = hq[r].z & 0x3F3F3F3Fu, m47 = ((hq[r].w >> 4) & 0x0F0F0F0Fu) | ((hq[r].z >> 2) & 0x30303030u);
                half8_t bh, bl;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float p = nd * static_cast<float>(((j < 4 ? m03 : m47) >> (8 * (j & 3))) & 0xFFu);
                    const _Float16 hi = static_cast<_Float16>(p);
                    bh[j] = hi;
                    bl[j] = static_cast<_Float16>(p - static_cast<float>(hi));
                }
#pragma unroll
                for (int tt = 0; tt < 4; tt++) {
                    half8_t sh = *reinterpret_cast<const half8_t *>(sumf + (tt * 2) * kWideFrag + lane * 16);
                    half8_t sl = *reinterpret_cast<const half8_t *>(sumf + (tt * 2 + 1) * kWideFrag + lane * 16);
                    if (!on) sh = sl = static_cast<half8_t>(static_cast<_Float16>(0.f));   // a super-block past the row: nothing was staged there
                    y[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sh, bh, y[r][tt], 0, 0, 0);
                    y[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sl, bh, y[r][tt], 0, 0, 0);
                    y[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sh, bl, y[r][tt], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int g = 0; g < 2; g++) {
            uint32_t sc[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                uint32_t mn;
                q4k_group_scale_min(hdr[r], (s & 1) * 2 + g, sc[r], mn);
            }
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {
                const int sub = g * 2 + hi;
                half8_t b[R];
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const uint32_t q0 = q[r][g].x, q1 = q[r][g].y;
                    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                    // A nibble in the low bits of a half's mantissa reads, under the right exponent, as
                    // C + n: bits 0..3 under 1024's, bits 4..7 under 64's (the odd bytes' nibbles take
                    // one shift down there).  One fused multiply-add then makes (C + n) * sc - C * sc =
                    // n * sc: a whole number up to 15 * 63, exact in binary16, as are C * sc.
                    // slot order of the eight columns: bytes [0, 2, 1, 3, 4, 6, 5, 7]
                    const _Float16 s1 = static_cast<_Float16>(static_cast<float>(hi ? sc[r] >> 8 : sc[r] & 0xFFu));
                    const half2_t s2 = {s1, s1};
                    half2_t w[4], c[4];
                    if (hi == 0) {
                        w[0] = __builtin_bit_cast(half2_t, (q0 & m0) | o0); w[1] = __builtin_bit_cast(half2_t, ((q0 >> 4) & nc.mask) | nc.one);
                        w[2] = __builtin_bit_cast(half2_t, (q1 & m0) | o0); w[3] = __builtin_bit_cast(half2_t, ((q1 >> 4) & nc.mask) | nc.one);
                        c[0] = c[2] = s2 * static_cast<half2_t>(static_cast<_Float16>(-1024.f));
                        c[1] = c[3] = s2 * static_cast<half2_t>(static_cast<_Float16>(-64.f));
                    } else {
                        w[0] = __builtin_bit_cast(half2_t, (q0 & nc.mask) | nc.one); w[1] = __builtin_bit_cast(half2_t, ((q0 >> 8) & nc.mask) | nc.one);
                        w[2] = __builtin_bit_cast(half2_t, (q1 & nc.mask) | nc.one); w[3] = __builtin_bit_cast(half2_t, ((q1 >> 8) & nc.mask) | nc.one);
                        c[0] = c[1] = c[2] = c[3] = s2 * static_cast<half2_t>(static_cast<_Float16>(-64.f));
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const half2_t p = __builtin_elementwise_fma(w[i], s2, c[i]);
                        b[r][2 * i] = p[0];
                        b[r][2 * i + 1] = p[1];
                    }
                }
#pragma unroll
                for (int tt = 0; tt < 4; tt++) {
                    const char *f = A + static_cast<size_t>((sub * 4 + tt) * 2) * kWideFrag + lane * 16;
                    const half8_t xh = *reinterpret_cast<const half8_t *>(f);
                    const half8_t xl = *reinterpret_cast<const half8_t *>(f + kWideFrag);
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        acc[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, b[r], acc[r][tt], 0, 0, 0);
                        acc[r][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, b[r], acc[r][tt], 0, 0, 0);
                    }
                }
            }
        }
        if (s & 1) {
            // the super-block ends: its sums take its d, the next one's header moves in
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float dd = f16_bits_to_f32(hdr[r].x);
#pragma unroll
                for (int tt = 0; tt < 4; tt++) {
#pragma unroll
                    for (int j = 0; j < 4; j++) y[r][tt][j] = fmaf(dd, acc[r][tt][j], y[r][tt][j]);
                    acc[r][tt] = float4_t{0.f, 0.f, 0.f, 0.f};
                }
                hdr[r] = hdrn[r];
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int g = 0; g < 2; g++) q[r][g] = qn[r][g];
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's pieces of the next slab have landed, then everybody's
        __syncthreads();
    }

    // C[token 16 tt + 4 kb + j][row n] of each tile
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = row0 + r * kTileRows + n;
        if (row >= a.n) continue;
#pragma unroll
        for (int tt = 0; tt < 4; tt++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int tok = tt * kTileRows + 4 * kb + j;
                if (tok >= nt) continue;
                float v = y[r][tt][j];
                if (a.residual) v += a.residual[static_cast<size_t>(t0 + tok) * a.y_stride + row];
                a.y[yoffs[tok] + row] = v;
            }
        }
    }
}

// ------------------------------------------------------------ the router of a long pass -------
// logits[t][e] = xn[t] . W[e] for float32 rows W (the router's experts and, as one more row, the
// shared expert's gate) against the staged rows of a pass: the same streaming of slabs as above,
// the second operand formed from 32 bytes of float32 a lane instead of from nibbles.  A float32
// weight enters as two binary16 values (hi, and the remainder scaled by 2^11 so that it stays a
// normal number); x_hi*w_hi + x_lo*w_hi run in one accumulator, x_hi*w_lo in a second one that
// carries the 2^11: about 22 bits of either operand, float32 sums.
// grid: (row blocks of NW*16 rows) x groups, NW waves; wave w owns one tile of 16 rows.
template <int NW>
__global__ __launch_bounds__(NW * 64) void router_wide_kernel(const float *W, const float *extra_row, int n_rows, int K, int n_tok, const char *staged_all,
                                                              float *logits, int logits_stride, int groups) {
    extern __shared__ __align__(16) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;
    constexpr int NTHR = NW * 64;
    const int grp = blockIdx.x % groups, xb = blockIdx.x / groups;
    const int t0 = grp * kWideTok;
    const int nt = n_tok - t0 < kWideTok ? n_tok - t0 : kWideTok;
    const char *staged = staged_all + static_cast<size_t>(grp) * wide_region(K);
    const int row = (xb * NW + wave) * kTileRows + n;
    // rows past the end read the last row (their results are dropped); row n_rows - 1 may live apart
    const int rr = row < n_rows ? row : n_rows - 1;
    const float *wp = (extra_row && rr == n_rows - 1) ? extra_row : W + static_cast<size_t>(rr) * K;
    const int steps = K / 128;
    constexpr int kVec = kWideSlab / 16;
    constexpr int kPer = kWideSlabA / 16 / NTHR;
    static_assert(kPer * NTHR * 16 == kWideSlabA && kVec - kPer * NTHR == 64, "slab copy layout");
    float4 w[4][2], wn[4][2];
    auto load_w = [&](int s, float4 (&dst)[4][2]) {
#pragma unroll
        for (int sub = 0; sub < 4; sub++) {
            const float *p = wp + s * 128 + sub * 32 + kb * 8;
            dst[sub][0] = *reinterpret_cast<const float4 *>(p);
            dst[sub][1] = *reinterpret_cast<const float4 *>(p + 4);
        }
    };
    load_w(0, w);
    {
        const uint4 *src = reinterpret_cast<const uint4 *>(staged);
        uint4 *dst = reinterpret_cast<uint4 *>(smem);
        for (int i = tid; i < kVec; i += NTHR) dst[i] = src[i];
    }
    __syncthreads();
    float4_t ym[4], yl[4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++) ym[tt] = yl[tt] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < steps; s++) {
        const int cur = s & 1;
        const bool more = s + 1 < steps;
        uint4 an[kPer], asx;
        {
            const int sn = more ? s + 1 : s;
            const uint4 *src = reinterpret_cast<const uint4 *>(staged + static_cast<size_t>(sn) * kWideSlab);
#pragma unroll
            for (int i = 0; i < kPer; i++) an[i] = src[tid + i * NTHR];
            asx = src[kPer * NTHR + (tid & 63)];
            load_w(sn, wn);
        }
        const char *A = smem + cur * kWideSlab;
#pragma unroll
        for (int sub = 0; sub < 4; sub++) {
            // slot order of the eight columns, as the rows were staged: [0, 2, 1, 3, 4, 6, 5, 7]
            const float o[8] = {w[sub][0].x, w[sub][0].z, w[sub][0].y, w[sub][0].w, w[sub][1].x, w[sub][1].z, w[sub][1].y, w[sub][1].w};
            half8_t bh, bl;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const _Float16 hi = static_cast<_Float16>(o[j]);
                bh[j] = hi;
                bl[j] = static_cast<_Float16>((o[j] - static_cast<float>(hi)) * 2048.f);
            }
            // all four token tiles, whatever the group holds: rows it does not have were staged as zeros
#pragma unroll
            for (int tt = 0; tt < 4; tt++) {
                const char *f = A + static_cast<size_t>((sub * 4 + tt) * 2) * kWideFrag + lane * 16;
                const half8_t xh = *reinterpret_cast<const half8_t *>(f);
                const half8_t xl = *reinterpret_cast<const half8_t *>(f + kWideFrag);
                ym[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, bh, ym[tt], 0, 0, 0);
                ym[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl, bh, ym[tt], 0, 0, 0);
                yl[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh, bl, yl[tt], 0, 0, 0);
            }
        }
        if (more) {
            uint4 *dst = reinterpret_cast<uint4 *>(smem + (cur ^ 1) * kWideSlab);
#pragma unroll
            for (int i = 0; i < kPer; i++) dst[tid + i * NTHR] = an[i];
            if (tid < 64) dst[kPer * NTHR + tid] = asx;
#pragma unroll
            for (int sub = 0; sub < 4; sub++) {
                w[sub][0] = wn[sub][0];
                w[sub][1] = wn[sub][1];
            }
        }
        __syncthreads();
    }
    if (row >= n_rows) return;
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int tok = tt * kTileRows + 4 * kb + j;
            if (tok < nt) logits[static_cast<size_t>(t0 + tok) * logits_stride + row] = fmaf(yl[tt][j], 1.f / 2048.f, ym[tt][j]);
        }
}

// The column parts of a split product added up in a fixed order.  grid: (ceil(n/256), nt), one
// wave a block; a thread takes four neighbouring outputs, with 16-byte moves when the row count
// and the addresses allow them.
__global__ __launch_bounds__(64) void gemm_wide_join_kernel(shv_gemv_q4k_args a, int t0, const float *part, int parts, int vec) {
    const int tok = blockIdx.y;
    const size_t yo = out_offset(a, t0 + tok);
    const int row = (blockIdx.x * 64 + threadIdx.x) * 4;
    if (row >= a.n) return;
    if (vec) {
        float4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int p = 0; p < parts; p++) {
            const float4 o = *reinterpret_cast<const float4 *>(part + (static_cast<size_t>(p) * kWideTok + tok) * a.n + row);
            v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
        }
        if (a.residual) {
            const float4 r = *reinterpret_cast<const float4 *>(a.residual + static_cast<size_t>(t0 + tok) * a.y_stride + row);
            v.x += r.x; v.y += r.y; v.z += r.z; v.w += r.w;
        }
        *reinterpret_cast<float4 *>(a.y + yo + row) = v;
        return;
    }
    for (int i = 0; i < 4 && row + i < a.n; i++) {
        float v = 0.f;
        for (int p = 0; p < parts; p++) v += part[(static_cast<size_t>(p) * kWideTok + tok) * a.n + row + i];
        if (a.residual) v += a.residual[static_cast<size_t>(t0 + tok) * a.y_stride + row + i];
        a.y[yo + row + i] = v;
    }
}

template <int TT, int NTHR, int MAXQ>
int launch_tt(shv_ctx *ctx, const shv_gemv_q4k_args &a, int t0, int nt, const char *staged) {
    constexpr int NW = NTHR / 64;
    SHV_REQUIRE(nt * (a.k / 4) <= MAXQ * NTHR, "gemm_q4k: %d rows of %d columns are more than one block stages", nt, a.k);
    const int n_tiles = (a.n + kTileRows - 1) / kTileRows;
    const size_t lds = Lds<TT>::total(a.k, NW);
    static std::atomic<size_t> raised{0};
    if (lds > 48 * 1024 && lds > raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_kernel<TT, NTHR, MAXQ>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised.store(lds, std::memory_order_release);
    }
    int per_cu = 0;
    SHV_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(&gemm_q4k_kernel<TT, NTHR, MAXQ>), NTHR, lds));
    SHV_REQUIRE(per_cu >= 1, "gemm_q4k: a block of %d threads with %zu bytes of LDS does not fit a compute unit", NTHR, lds);
    // One round of resident blocks, so that the activations are staged once per block.  A matrix
    // with too few row tiles to occupy the waves is also split along its columns.
    const int slots = ctx->prop.multiProcessorCount * per_cu * NW;
    const int sbs = a.k / SHV_Q4K_BLOCK;
    int ks = 1;
    while (ks * 2 <= NW && sbs % (ks * 2) == 0 && n_tiles * ks * 2 <= slots) ks *= 2;
    const int tiles_per_block = NW / ks;
    int blocks = ctx->prop.multiProcessorCount * per_cu;
    const int need = (n_tiles + tiles_per_block - 1) / tiles_per_block;
    if (blocks > need) blocks = need;
    const int rounds = (need + blocks - 1) / blocks;
    blocks = (need + rounds - 1) / rounds;
    SHV_LAUNCH(ctx, (gemm_q4k_kernel<TT, NTHR, MAXQ>), dim3(blocks), dim3(NTHR), lds, a, t0, nt, n_tiles, ks, staged);
    return SHV_OK;
}

// Every group of `cap` rows of the pass transformed once into ctx->gemm_stage.
template <int TT>
int launch_stage(shv_ctx *ctx, const shv_gemv_q4k_args &a, int cap) {
    const int groups = (a.n_tok + cap - 1) / cap;
    SHV_REQUIRE(groups * Lds<TT>::region(a.k) <= static_cast<size_t>(shv_ctx::kGemmStageBytes), "gemm_q4k: %d rows of %d columns do not fit the staging buffer", a.n_tok, a.k);
    SHV_LAUNCH(ctx, (gemm_stage_kernel<TT>), dim3(a.k / 256, groups), dim3(256), 0, a, ctx->gemm_stage, cap);
    return SHV_OK;
}

// One group of up to 64 rows whose operands are already in `staged`.
template <int NW, int R>
int launch_wide(shv_ctx *ctx, const shv_gemv_q4k_args &a, int t0, int nt, const char *staged) {
    constexpr int kRows = NW * R * kTileRows;
    const int bx = (a.n + kRows - 1) / kRows;
    const int steps = a.k / 128;
    // few row groups: the columns are split too, as far as every part keeps two steps, the launch
    // stays within one round of the chip (a block a compute unit, see below), and the parts fit
    int ks = 1;
    const int cus = ctx->prop.multiProcessorCount;
    while (steps % (ks * 2) == 0 && steps / (ks * 2) >= 2 && bx * ks * 2 <= cus &&
           static_cast<size_t>(ks * 2) * kWideTok * a.n * 4 <= static_cast<size_t>(shv_ctx::kGemmPartBytes))
        ks *= 2;
    SHV_REQUIRE(ks == 1 || ctx->gemm_part, "gemm_q4k: no buffer for the parts of a split product");
    // More than half a compute unit's LDS, so that two blocks never share one: a launch of fewer
    // blocks than compute units would otherwise double up on some and leave others idle.
    const size_t lds = std::max<size_t>(2 * kWideSlab + kWideTok * sizeof(size_t), 84 * 1024);
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_wide_kernel<NW, R>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised.store(true, std::memory_order_release);
    }
    SHV_LAUNCH(ctx, (gemm_wide_kernel<NW, R>), dim3(bx, ks), dim3(NW * 64), lds, a, t0, nt, staged, ctx->gemm_part, steps / ks, 1);
    if (ks > 1) {
        // 16-byte moves need whole quads of outputs at 16-byte addresses in every row
        const bool ring = a.ring_slots > 0 && !a.z_ring;
        const int vec = a.n % 4 == 0 && shv_aligned16(a.y) && (ring ? a.ring_stride % 4 == 0 : a.y_stride % 4 == 0) &&
                        (!a.residual || (shv_aligned16(a.residual) && a.y_stride % 4 == 0));
        SHV_LAUNCH(ctx, gemm_wide_join_kernel, dim3((a.n + 255) / 256, nt), dim3(64), 0, a, t0, ctx->gemm_part, ks, vec);
    }
    return SHV_OK;
}

// Eight rows a launch on the sixteen-wave kernel: a matrix of few row tiles is split along its
// columns over the waves of a block as far as that fills the chip's wave slots.
template <int K, int PRO, int RD>
int launch_rows_kp(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    constexpr int SBS = K / SHV_Q4K_BLOCK;
    const int n_tiles = (a.n + kTileRows - 1) / kTileRows;
    const long long slots = static_cast<long long>(ctx->prop.multiProcessorCount) * kRowsWaves;
    int ks_log2 = 0;
    while ((2 << ks_log2) <= kRowsWaves && (2 << ks_log2) <= SBS && static_cast<long long>(n_tiles) * (2 << ks_log2) <= slots) ks_log2++;
    const int tpb = kRowsWaves >> ks_log2;
    int blocks = (n_tiles + tpb - 1) / tpb;
    if (blocks > ctx->prop.multiProcessorCount) blocks = ctx->prop.multiProcessorCount;
    constexpr size_t lds = RowsLds<K>::total;
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_rows_kernel<K, PRO, RD>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised.store(true, std::memory_order_release);
    }
    for (int t0 = 0; t0 < a.n_tok; t0 += kRowsTok) {
        const int nt = a.n_tok - t0 < kRowsTok ? a.n_tok - t0 : kRowsTok;
        SHV_LAUNCH(ctx, (gemm_rows_kernel<K, PRO, RD>), dim3(blocks), dim3(kRowsThreads), lds, a, t0, nt, n_tiles, ks_log2);
    }
    return SHV_OK;
}

template <int K, int RD>
int launch_rows_k(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    switch (a.prologue) {
        case SHV_PRO_NONE: return launch_rows_kp<K, SHV_PRO_NONE, RD>(ctx, a);
        case SHV_PRO_RMSNORM: return launch_rows_kp<K, SHV_PRO_RMSNORM, RD>(ctx, a);
        case SHV_PRO_GATED_NORM: return launch_rows_kp<K, SHV_PRO_GATED_NORM, RD>(ctx, a);
        default: return launch_rows_kp<K, SHV_PRO_MUL_SIGMOID, RD>(ctx, a);
    }
}

// Which passes the sixteen-wave kernel takes (the arguments have passed shv_gemm_q4k_covers).
bool rows_kernel_covers(const shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (ctx->gemm_rows_min <= 0 || a.n_tok < ctx->gemm_rows_min) return false;
    if (a.k != 2048 && a.k != 4096) return false;
    if (a.n_tok > kRowsTok) return false;  // more rows would read the weights once per eight
    if (a.prologue == SHV_PRO_GATED_NORM && a.head_dim != 128) return false;  // a head is four staging steps of a lane
    if (a.prologue == SHV_PRO_MUL_SIGMOID && a.head_dim != 0 && (a.head_dim < 4 || (a.head_dim & (a.head_dim - 1)) != 0)) return false;
    return true;
}

// Every group of 64 rows of a long pass in one launch (the operands of all of them are in
// ctx->gemm_stage): no split along the columns, the groups themselves fill the chip.
template <int NW, int R>
int launch_wide_all(shv_ctx *ctx, const shv_gemv_q4k_args &a, int groups) {
    constexpr int kRows = NW * R * kTileRows;
    const int bx = (a.n + kRows - 1) / kRows;
    const size_t lds = 2 * kWideSlab + kWideSumFrags + kWideTok * sizeof(size_t);
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_pass_kernel<NW, R>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised.store(true, std::memory_order_release);
    }
    SHV_REQUIRE(static_cast<long long>(bx) * groups <= 0x7fffffffll, "gemm_q4k: %d row blocks of %d groups", bx, groups);
    SHV_LAUNCH(ctx, (gemm_pass_kernel<NW, R>), dim3(bx * groups), dim3(NW * 64), lds, a, static_cast<const char *>(ctx->gemm_stage), groups);
    return SHV_OK;
}

}  // namespace

// The router of a pass of many rows: xn = rmsnorm(h) * gamma staged (and written out as float32),
// then every token's n_expert (+ 1, the shared expert's gate) logits on the matrix cores.
bool shv_router_wide_covers(const shv_ctx *ctx, const shv_moe_router_args &a) {
    if (!ctx->gemm_stage || a.n_tok < 128 || !a.gamma || !a.xn) return false;
    if (a.n_embd % 256 != 0 || a.n_embd < 256 || a.h_stride % 4 != 0) return false;
    if (!shv_aligned16(a.h) || !shv_aligned16(a.gamma) || !shv_aligned16(a.xn) || !shv_aligned16(a.router) || (a.shared_gate && !shv_aligned16(a.shared_gate))) return false;
    const int groups = (a.n_tok + kWideTok - 1) / kWideTok;
    return groups * wide_region(a.n_embd) <= static_cast<size_t>(shv_ctx::kGemmStageBytes);
}

int shv_launch_router_wide(shv_ctx *ctx, const shv_moe_router_args &a) {
    shv_gemv_q4k_args g{};
    g.x = a.h;
    g.gamma = a.gamma;
    g.k = a.n_embd;
    g.n_tok = a.n_tok;
    g.prologue = SHV_PRO_RMSNORM;
    g.eps = a.eps;
    g.x_stride = a.h_stride;
    const int groups = (a.n_tok + kWideTok - 1) / kWideTok;
    SHV_LAUNCH(ctx, gemm_wide_stage_kernel, dim3(stage_parts(g, groups), kWideTok / 4, groups), dim3(256), 0, g, ctx->gemm_stage, a.xn);
    const int n_rows = a.n_expert + (a.shared_gate ? 1 : 0);
    const size_t lds = 2 * kWideSlab;
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&router_wide_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&router_wide_kernel<8>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised.store(true, std::memory_order_release);
    }
    // Every block reads its group's slabs whole: blocks of eight waves (128 router rows) halve that traffic, and from 64 groups
    // on there are still blocks enough for the chip (4096 rows, 513 router rows: 320 blocks; the 2048-row pass is 1.7 % faster
    // with four waves a block and 288 of them)
    if (groups >= 64) {
        constexpr int NW = 8;
        const int bx = (n_rows + NW * kTileRows - 1) / (NW * kTileRows);
        SHV_LAUNCH(ctx, (router_wide_kernel<NW>), dim3(bx * groups), dim3(NW * 64), lds, a.router, a.shared_gate, n_rows, a.n_embd, a.n_tok,
                   static_cast<const char *>(ctx->gemm_stage), a.logits, a.n_expert + 1, groups);
    } else {
        constexpr int NW = 4;
        const int bx = (n_rows + NW * kTileRows - 1) / (NW * kTileRows);
        SHV_LAUNCH(ctx, (router_wide_kernel<NW>), dim3(bx * groups), dim3(NW * 64), lds, a.router, a.shared_gate, n_rows, a.n_embd, a.n_tok,
                   static_cast<const char *>(ctx->gemm_stage), a.logits, a.n_expert + 1, groups);
    }
    return SHV_OK;
}

// Whether the matrix-core kernel takes this call: arguments are already validated by the GEMV's
// launcher, which falls back to its own multi-row kernel otherwise.
bool shv_gemm_q4k_covers(const shv_gemv_q4k_args &a) {
    if (a.k != 256 && a.k != 512 && a.k != 1024 && a.k != 2048 && a.k != 4096) return false;
    if (a.prologue == SHV_PRO_RMSNORM_PAIR) return false;
    if (a.prologue == SHV_PRO_GATED_NORM) {
        const int span = a.head_dim / 4;
        if (a.head_dim % 4 != 0 || span < 1 || span > 64 || (span & (span - 1)) != 0 || !shv_aligned16(a.gamma)) return false;
    }
    if (a.prologue == SHV_PRO_MUL_SIGMOID && a.head_dim % 4 != 0) return false;
    // 16-byte loads of the activation rows, their gates and the norm's gamma
    if (a.x_stride % 4 != 0 || !shv_aligned16(a.x)) return false;
    if (a.prologue == SHV_PRO_RMSNORM && !shv_aligned16(a.gamma)) return false;
    if ((a.prologue == SHV_PRO_GATED_NORM || a.prologue == SHV_PRO_MUL_SIGMOID) &&
        (!shv_aligned16(a.z) || a.z_stride % 4 != 0 || (a.z_ring && a.ring_stride % 4 != 0)))
        return false;
    return true;
}

int shv_launch_gemm_q4k(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (rows_kernel_covers(ctx, a)) return a.k == 2048 ? launch_rows_k<2048, 3>(ctx, a) : launch_rows_k<4096, 1>(ctx, a);
    // the fragments of 16 rows of 4096 columns do not fit LDS: such a pass goes 8 rows at a time
    const int cap = a.k > 2048 ? 8 : 16;
    // more rows than one block keeps in LDS: groups of 64 stream their operands
    if (a.n_tok > cap && ctx->gemm_stage && (a.prologue != SHV_PRO_GATED_NORM || 256 % a.head_dim == 0)) {
        const int groups = (a.n_tok + kWideTok - 1) / kWideTok;
        SHV_REQUIRE(groups * wide_region(a.k) <= static_cast<size_t>(shv_ctx::kGemmStageBytes), "gemm_q4k: %d rows of %d columns do not fit the staging buffer", a.n_tok, a.k);
        SHV_LAUNCH(ctx, gemm_wide_stage_kernel, dim3(stage_parts(a, groups), kWideTok / 4, groups), dim3(256), 0, a, ctx->gemm_stage, static_cast<float *>(nullptr));
        if (groups >= 4) return launch_wide_all<8, 1>(ctx, a, groups);
        for (int g = 0; g < groups; g++) {
            const int t0 = g * kWideTok;
            const int nt = a.n_tok - t0 < kWideTok ? a.n_tok - t0 : kWideTok;
            const char *st = ctx->gemm_stage + static_cast<size_t>(g) * wide_region(a.k);
            // many rows: sixteen waves a block keep a compute unit's matrix cores and vector units
            // both busy; a matrix of few rows needs smaller blocks to spread over the chip
            const int rc = a.n >= 8192 ? launch_wide<16, 1>(ctx, a, t0, nt, st) : launch_wide<8, 1>(ctx, a, t0, nt, st);
            if (rc != SHV_OK) return rc;
        }
        return SHV_OK;
    }
    // A pass of several groups of rows, or of wide rows, has its activations transformed once, by
    // a launch of its own, instead of by every block of the products (hundreds of them): the
    // groups of `cap` rows are staged with the tile size their product will use.  One group of
    // narrow rows is cheaper staged by the blocks themselves, under their first weight loads.
    const bool pre = ctx->gemm_stage && a.n_tok > 4 && (a.n_tok > cap || a.k > 2048) &&
                     (a.prologue != SHV_PRO_GATED_NORM || 256 % a.head_dim == 0);
    if (pre) {
        int rc;
        if (cap == 8 || a.n_tok <= 8) rc = launch_stage<8>(ctx, a, a.n_tok <= 8 ? 8 : cap);
        else rc = launch_stage<16>(ctx, a, cap);
        if (rc != SHV_OK) return rc;
    }
    const int gcap = pre && a.n_tok <= 8 ? 8 : cap;
    for (int t0 = 0; t0 < a.n_tok; t0 += gcap) {
        const int nt = a.n_tok - t0 < gcap ? a.n_tok - t0 : gcap;
        int rc;
        if (!pre) {
            if (nt <= 4) rc = launch_tt<4, 1024, 4>(ctx, a, t0, nt, nullptr);
            else if (nt <= 8) rc = launch_tt<8, 512, 16>(ctx, a, t0, nt, nullptr);
            else rc = launch_tt<16, 1024, 8>(ctx, a, t0, nt, nullptr);
        } else if (gcap == 8) {
            rc = launch_tt<8, 512, 16>(ctx, a, t0, nt, ctx->gemm_stage + static_cast<size_t>(t0 / gcap) * Lds<8>::region(a.k));
        } else {
            rc = launch_tt<16, 1024, 8>(ctx, a, t0, nt, ctx->gemm_stage + static_cast<size_t>(t0 / gcap) * Lds<16>::region(a.k));
        }
        if (rc != SHV_OK) return rc;
    }
    return SHV_OK;
}
