// Q4_K dequant-fused GEMM for passes of 2..16 rows: Y[t] = W * pro(X[t]) (+ residual[t]) on the
// matrix cores, with the GEMV's arguments and results (verification passes, batched decode rows,
// prompt chunks: llm/graph.go:1383-1429,1527-1666; the reference's form is llm_gemv.comp's
// multi-row arm).
//
// Still HBM-bound on the weights, which are read once for all rows of the pass.  A 64-lane wave
// multiplies a tile of 16 weight rows by up to 16 activation rows with v_mfma_f32_16x16x16_f16:
//   A (tokens x k)  the activations, split into two halves hi + lo (lo = x - hi) so that the
//                   product keeps float32 accuracy; a wave keeps the fragments of its 256 columns
//                   in registers for the whole kernel
//   B (k x rows)    the 4-bit levels as exact halves 64+n (a level sits in mantissa bits 4..7 of
//                   64.0); lane (row = lane%16, kb = lane/16) reads 8 payload bytes of each
//                   64-weight group, whose low nibbles feed the group's first 32 columns and whose
//                   high nibbles feed the other 32
//   C (tokens x rows) one 32-column sub-block at a time, because each has its own scale and min;
//                   the lane that loaded row n also holds C[.][n], so d*sc and dmin*m apply without
//                   any exchange:  y += d*sc*(acc - 64*sum(x)) - dmin*m*sum(x).
// The waves of a block share a row tile, each over its own super-block column, and add their tiles
// through LDS.  Activation rows are staged four at a time through LDS, where the prologue runs.
// A block covers up to 2048 columns at a time; a wider matrix is taken as column ranges one after
// the other, each adding to what the one before left in y.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;
constexpr int kMaxRows = 16;   // activation rows one launch covers
constexpr int kStage = 4;      // activation rows staged together
constexpr int kSlice = 256;    // columns per wave: one super-block of each row
constexpr int kSubs = kSlice / 32;

__host__ __device__ constexpr int xs_stride(int k) { return k + 8; }

// One wave's loads for one row tile: the 16-byte header of the lane's row in the wave's
// super-block column and 8 payload bytes of each of its four 64-weight groups.
struct TileLoads {
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

// K here is the width of the column range one launch covers (a.k, or a part of it).
template <int K>
struct Gemm {
    static constexpr int NW = K / kSlice;
    static constexpr int NTHR = NW * 64;
    static constexpr int PER = 4;  // columns a thread stages per row: K / NTHR
    static constexpr int XS = xs_stride(K);
    static constexpr size_t lds_bytes() { return (static_cast<size_t>(kStage) * XS + K / 32 * 16 + NW * 256 + kStage * NW) * sizeof(float); }
};

// Columns col0..col0+K of pro(x[t]) for gn <= 4 consecutive rows t_first.. into LDS rows of xs, by
// all threads of the block; same prologues as the GEMV.  Every row's loads are issued before any
// is used, so the rows cost one memory round trip together.  The RMSNorm needs the whole row and
// runs only when the column range is the whole row.
template <int K>
__device__ __forceinline__ void stage_rows(const shv_gemv_q4k_args &a, int t_first, int gn, int col0, float *xs, float *red, int tid) {
    using G = Gemm<K>;
    const int lane = tid & 63, wave = tid >> 6;
    // the gated norm reduces over a head, so its threads own consecutive columns; the others
    // take columns NTHR apart, which coalesces better
    const bool consec = a.prologue == SHV_PRO_GATED_NORM;
    int col[G::PER];
#pragma unroll
    for (int i = 0; i < G::PER; i++) col[i] = consec ? tid * G::PER + i : tid + i * G::NTHR;
    float v[kStage][G::PER], zv[kStage][G::PER];
    const bool has_z = a.prologue == SHV_PRO_GATED_NORM || a.prologue == SHV_PRO_MUL_SIGMOID;
    // every row's gate pointer first: the positions they depend on are then fetched together
    const float *zp[kStage];
#pragma unroll
    for (int r = 0; r < kStage; r++) {
        const int t = t_first + (r < gn ? r : 0);
        zp[r] = a.z + static_cast<size_t>(t) * a.z_stride;
        if (has_z && a.z_ring) {
            const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
            const int s = t / sl, k = t % sl;
            const int p = a.pos ? a.pos[s] : 0;
            const int slot = a.slot ? a.slot[s] : s;
            zp[r] = a.z + (static_cast<size_t>(slot) * a.ring_slots + (p + k) % a.ring_slots) * a.ring_stride;
        }
    }
#pragma unroll
    for (int r = 0; r < kStage; r++) {
        if (r >= gn) continue;
        const float *x = a.x + static_cast<size_t>(t_first + r) * a.x_stride + col0;
#pragma unroll
        for (int i = 0; i < G::PER; i++) v[r][i] = x[col[i]];
        if (has_z) {
#pragma unroll
            for (int i = 0; i < G::PER; i++) {
                const int cg = col0 + col[i];
                // sigmoid gate with head_dim: z rows are [q | gate] per head and the gate half is wanted
                const int zi = a.prologue == SHV_PRO_MUL_SIGMOID && a.head_dim > 0
                                   ? (cg / a.head_dim) * 2 * a.head_dim + a.head_dim + cg % a.head_dim : cg;
                zv[r][i] = zp[r][zi];
            }
        }
    }
    if (a.prologue == SHV_PRO_RMSNORM) {
#pragma unroll
        for (int r = 0; r < kStage; r++) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < G::PER; i++) ss = r < gn ? fmaf(v[r][i], v[r][i], ss) : ss;
            ss = wave_sum_all(ss);
            if (lane == 0) red[r * G::NW + wave] = ss;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kStage; r++) {
            if (r >= gn) continue;
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < G::NW; w++) tot += red[r * G::NW + w];
            const float scale = 1.f / sqrtf(tot / static_cast<float>(K) + a.eps);
#pragma unroll
            for (int i = 0; i < G::PER; i++) xs[r * G::XS + col[i]] = v[r][i] * scale * a.gamma[col[i]];
        }
    } else if (a.prologue == SHV_PRO_GATED_NORM) {
        const int span = a.head_dim / G::PER;  // lanes a head spans
#pragma unroll
        for (int r = 0; r < kStage; r++) {
            if (r >= gn) continue;
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < G::PER; i++) ss = fmaf(v[r][i], v[r][i], ss);
            for (int off = 1; off < span; off <<= 1) ss += __shfl_xor(ss, off, 64);
            const float scale = 1.f / sqrtf(ss / static_cast<float>(a.head_dim) + a.eps);
#pragma unroll
            for (int i = 0; i < G::PER; i++) {
                const float g = 1.f / (1.f + expf(-zv[r][i]));
                xs[r * G::XS + col[i]] = v[r][i] * scale * a.gamma[(col0 + col[i]) % a.head_dim] * g;
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < kStage; r++) {
            if (r >= gn) continue;
#pragma unroll
            for (int i = 0; i < G::PER; i++) {
                const float g = a.prologue == SHV_PRO_MUL_SIGMOID ? 1.f / (1.f + expf(-zv[r][i])) : 1.f;
                xs[r * G::XS + col[i]] = v[r][i] * g;
            }
        }
    }
}

// grid: blocks take row tiles round-robin.  t0: first activation row of this launch, nt: how many.
// A matrix wider than K runs as n_ranges column ranges one after the other; from the second on a
// thread adds to the outputs it stored itself in the range before.
template <int K>
__global__ __launch_bounds__(Gemm<K>::NTHR) void gemm_q4k_kernel(shv_gemv_q4k_args a, int t0, int nt, int n_tiles, int n_ranges) {
    using G = Gemm<K>;
    extern __shared__ float smem[];
    float *xs = smem;                             // [kStage][XS]
    float *sxs = xs + kStage * G::XS;             // [K/32][16] sum of x per 32-column sub-block and row
    float *tile = sxs + K / 32 * 16;              // [NW][256] the waves' partial tiles
    float *red = tile + G::NW * 256;              // [kStage][NW]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, kb = lane >> 4;      // B: weight row of the tile, k block; A: token n
    const size_t row_bytes = static_cast<size_t>(a.k / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES;

    // where each activation row's outputs go (the DeltaNet projection ring, or plain rows)
    const int o_tok = tid >> 4;  // the activation row of the output this thread adds up and stores, when tid < 256
    size_t y_off = 0;
    if (o_tok < nt) {
        const int t = t0 + o_tok;
        if (a.ring_slots > 0 && !a.z_ring) {
            const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
            const int s = t / sl, i = t % sl;
            const int p = a.pos ? a.pos[s] : 0;
            const int slot = a.slot ? a.slot[s] : s;
            y_off = (static_cast<size_t>(slot) * a.ring_slots + (p + i) % a.ring_slots) * a.ring_stride;
        } else {
            y_off = static_cast<size_t>(t) * a.y_stride;
        }
    }
    const NibbleConsts nc = nibble_consts();
    const float4 *sx4 = reinterpret_cast<const float4 *>(sxs) + wave * kSubs * 4 + kb;  // rows 4kb..4kb+3 of C

    for (int rg = 0; rg < n_ranges; rg++) {
    const int col0 = rg * K;
    const float *residual = rg == 0 ? a.residual : a.y;
    const char *wslice = static_cast<const char *>(a.w) + static_cast<size_t>(col0 / SHV_Q4K_BLOCK + wave) * SHV_Q4K_BYTES;

    // the first tile's weights do not depend on the activations
    TileLoads cur, nxt;
    int tl = blockIdx.x;
    {
        const int r = tl * kTileRows + n;
        cur.load(wslice + static_cast<size_t>(r < a.n ? r : a.n - 1) * row_bytes, kb);
    }

    // ---- activations: this lane's token is n; its fragments cover the wave's 256 columns ----
    half4_t xh[kSubs][2], xl[kSubs][2];
#pragma unroll
    for (int s = 0; s < kSubs; s++)
#pragma unroll
        for (int c = 0; c < 2; c++) {
            xh[s][c] = half4_t{0, 0, 0, 0};
            xl[s][c] = half4_t{0, 0, 0, 0};
        }
    for (int g0 = 0; g0 < nt; g0 += kStage) {
        const int gn = nt - g0 < kStage ? nt - g0 : kStage;
        stage_rows<K>(a, t0 + g0, gn, col0, xs, red, tid);
        __syncthreads();
        if (n >= g0 && n < g0 + gn) {
            const float *row = xs + (n - g0) * G::XS + wave * kSlice;
#pragma unroll
            for (int s = 0; s < kSubs; s++) {
                // sub-block s of the slice: 64-weight group s/2, low (s even) or high nibbles
                float sum = 0.f;
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const float4 f = *reinterpret_cast<const float4 *>(row + s * 32 + kb * 8 + c * 4);
                    const float v[4] = {f.x, f.z, f.y, f.w};  // the k order of levels()
                    half4_t h, l;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const _Float16 hi = static_cast<_Float16>(v[j]);
                        h[j] = hi;
                        l[j] = static_cast<_Float16>(v[j] - static_cast<float>(hi));
                    }
                    xh[s][c] = h;
                    xl[s][c] = l;
                    sum += (f.x + f.y) + (f.z + f.w);
                }
                sum += __shfl_xor(sum, 16, 64);
                sum += __shfl_xor(sum, 32, 64);
                if (kb == 0) sxs[(wave * kSubs + s) * 16 + n] = sum;
                __builtin_amdgcn_sched_barrier(0);  // one sub-block at a time: keeps the live set small
            }
        }
        __syncthreads();
    }
    // rows of the pass beyond nt contribute nothing; their sums are never read

    for (; tl < n_tiles; tl += gridDim.x) {
        const int tn = tl + gridDim.x;
        if (tn < n_tiles) {
            const int r = tn * kTileRows + n;
            nxt.load(wslice + static_cast<size_t>(r < a.n ? r : a.n - 1) * row_bytes, kb);
        }
        float4_t y = {0.f, 0.f, 0.f, 0.f};
        const float d = f16_bits_to_f32(cur.hdr.x), dmin = f16_bits_to_f32(cur.hdr.x >> 16);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            uint32_t sc, mn;
            q4k_group_scale_min(cur.hdr, g, sc, mn);
            const uint32_t q0 = cur.q[g].x, q1 = cur.q[g].y;
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {
                const int sub = g * 2 + hi;
                half4_t b0, b1;
                if (hi == 0) {
                    b0 = levels(((q0 << 4) & nc.mask) | nc.one, ((q0 >> 4) & nc.mask) | nc.one);
                    b1 = levels(((q1 << 4) & nc.mask) | nc.one, ((q1 >> 4) & nc.mask) | nc.one);
                } else {
                    b0 = levels((q0 & nc.mask) | nc.one, ((q0 >> 8) & nc.mask) | nc.one);
                    b1 = levels((q1 & nc.mask) | nc.one, ((q1 >> 8) & nc.mask) | nc.one);
                }
                float4_t acc = {0.f, 0.f, 0.f, 0.f};
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xh[sub][0], b0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xh[sub][1], b1, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xl[sub][0], b0, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x16f16(xl[sub][1], b1, acc, 0, 0, 0);
                const float ds = d * static_cast<float>(hi ? sc >> 8 : sc & 0xFFu);
                const float dm = dmin * static_cast<float>(hi ? mn >> 8 : mn & 0xFFu);
                const float4 sx = sx4[sub * 4];
                const float sxv[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
                for (int j = 0; j < 4; j++) y[j] += ds * fmaf(-64.f, sxv[j], acc[j]) - dm * sxv[j];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- add the waves' tiles and store: lane holds C[4kb+j][n] ----
        float *mine = tile + wave * 256;
#pragma unroll
        for (int j = 0; j < 4; j++) mine[(4 * kb + j) * 16 + n] = y[j];
        __syncthreads();
        for (int o = tid; o < 256; o += G::NTHR) {
            const int orow = o & 15, otok = o >> 4;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < G::NW; w++) v += tile[w * 256 + o];
            const int r = tl * kTileRows + orow;
            if (otok < nt && r < a.n) {
                // NTHR >= 256: o == tid and y_off is this thread's; smaller blocks recompute it
                size_t off = y_off;
                if (G::NTHR < 256) {
                    const int t = t0 + otok;
                    if (a.ring_slots > 0 && !a.z_ring) {
                        const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
                        const int s = t / sl, i = t % sl;
                        const int p = a.pos ? a.pos[s] : 0;
                        const int slot = a.slot ? a.slot[s] : s;
                        off = (static_cast<size_t>(slot) * a.ring_slots + (p + i) % a.ring_slots) * a.ring_stride;
                    } else {
                        off = static_cast<size_t>(t) * a.y_stride;
                    }
                }
                if (residual) v += residual[static_cast<size_t>(t0 + otok) * a.y_stride + r];
                a.y[off + r] = v;
            }
        }
        __syncthreads();
        cur = nxt;
    }
    }  // column ranges
}

template <int K>
int launch_gemm(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    using G = Gemm<K>;
    const int n_tiles = (a.n + kTileRows - 1) / kTileRows;
    const size_t lds = G::lds_bytes();
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_kernel<K>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        raised = true;
    }
    // one round of resident blocks, so that the activations are staged once per block; the tiles
    // are dealt evenly among them
    static int per_cu = 0;
    if (per_cu == 0) {
        SHV_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(&gemm_q4k_kernel<K>), G::NTHR, lds));
        if (per_cu < 1) per_cu = 1;
    }
    int blocks = ctx->prop.multiProcessorCount * per_cu;
    if (blocks > n_tiles) blocks = n_tiles;
    const int rounds = (n_tiles + blocks - 1) / blocks;
    blocks = (n_tiles + rounds - 1) / rounds;
    for (int t0 = 0; t0 < a.n_tok; t0 += kMaxRows) {
        const int nt = a.n_tok - t0 < kMaxRows ? a.n_tok - t0 : kMaxRows;
        SHV_LAUNCH(ctx, (gemm_q4k_kernel<K>), dim3(blocks), dim3(G::NTHR), lds, a, t0, nt, n_tiles, a.k / K);
    }
    return SHV_OK;
}

}  // namespace

// Whether the matrix-core kernel takes this call: arguments are already validated by the GEMV's
// launcher, which falls back to its own multi-row kernel otherwise.
bool shv_gemm_q4k_covers(const shv_gemv_q4k_args &a) {
    if (a.k != 256 && a.k != 512 && a.k != 1024 && a.k != 2048 && a.k != 4096) return false;
    if (a.prologue == SHV_PRO_RMSNORM_PAIR) return false;
    if (a.k > 2048) {
        // column ranges: no whole-row statistic, and plain rows to add into
        if (a.prologue == SHV_PRO_RMSNORM || (a.ring_slots > 0 && !a.z_ring) || a.y_stride < a.n) return false;
    }
    if (a.prologue == SHV_PRO_GATED_NORM) {
        const int span = a.head_dim / 4;
        if (a.head_dim % 4 != 0 || span < 1 || span > 64 || (span & (span - 1)) != 0 || 2048 % a.head_dim != 0) return false;
    }
    // 8-byte loads of the payload and 16-byte loads of the staged rows
    return a.x_stride % 4 == 0 && shv_aligned16(a.x);
}

int shv_launch_gemm_q4k(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    switch (a.k) {
        case 256: return launch_gemm<256>(ctx, a);
        case 512: return launch_gemm<512>(ctx, a);
        case 1024: return launch_gemm<1024>(ctx, a);
        default: return launch_gemm<2048>(ctx, a);  // 2048, and 4096 as two column ranges
    }
}
