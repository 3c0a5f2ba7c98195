// Gated full-attention decode over an fp16 KV cache, GQA with 8 query heads per KV head, one or
// two consecutive rows of a sequence per launch, on the matrix cores.
//
// HBM-bound on the cache: a block owns one KV head and one slice of the cells and serves all the
// query heads of that KV head, for both rows, from a single pass over K and a single pass over V.
// The 8 heads x 2 rows are the 16 rows of a v_mfma_f32_16x16x16_f16 tile:
//   S^T = K Q^T   A = 16 cells x 16 dims of K straight from the cache (it is binary16 already),
//                 B = the queries as hi + lo halves (so the product keeps float32 accuracy), kept
//                 in LDS in operand order.  Computing the transpose leaves each lane with the
//                 scores of one query row and four consecutive cells, which is exactly the A
//                 operand of the second product: the probabilities never move between lanes
//   O += P V      A = P as hi + lo halves, B = 16 cells x 16 dims of V.  V is cached transposed in
//                 tiles of 32 cells, [cell/32][kv head][dim][cell%32], so that a lane's four cells of
//                 one dim are 8 contiguous bytes and a wave's tile is 16 contiguous KB
//   softmax       running max and sum per query row in the four lanes that share the row; the
//                 accumulators are rescaled only when some row's maximum moved
//   prologue      the wave's first tile of K and V is requested before anything else; per-head RMS
//                 norm + rotary of the queries; the block whose slice holds a new cell normalises /
//                 rotates K, rounds K and V to binary16 and appends them
//   epilogue      the four waves' (max, sum, accumulator) are merged through LDS and go to scratch
// A second, small kernel merges the slices: one wave a (row, head, 64 dims), every slice's value
// requested at once.  (Merging in the last block to arrive instead costs more than the launch: that
// block walks all the records alone, a few dependent round trips to memory.)
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kBlock = 256;
constexpr int kD = 256;        // head dimension the kernel is built for
constexpr int kRep = 8;        // query heads per KV head
constexpr int kTile = 32;         // cells a wave takes at a time
constexpr int kSliceCells = 128;  // cells a slice gets while there are slices to spare: one tile a wave
constexpr int kMaxSplits = 512;
constexpr int kRec = kRep * (kD + 2);  // floats of one (slice, row) record: per head d values, max, sum

// RMS norm over the 256 dims of one head by one wave (4 dims per lane: lane l holds dims 4l..4l+3),
// then NeoX rotary on the first rope_dims dims, all in registers: dims i and i + rope_dims/2 turn
// together and sit rope_dims/8 lanes apart, which the launcher requires to be a power of two, so
// the partner is lane ^ (rope_dims/8).  cs4 / sn4: the rotary factors of this lane's four dims,
// i.e. entries 4*(lane mod rope_dims/8) .. +3 of the position's cos and sin rows.
__device__ __forceinline__ float rope_turn(float x, float o, float c, float sn, bool first, bool turns) {
    // first of the pair: x0' = x0*cos - x1*sin ; second: x1' = x0*sin + x1*cos  (o is the partner's value)
    const float r = first ? x * c - o * sn : o * sn + x * c;
    return turns ? r : x;
}

__device__ __forceinline__ void norm_rope_regs(const float4 v, const float4 g, const float4 cs4, const float4 sn4, int rope_dims, float eps, int lane,
                                               float &x0, float &x1, float &x2, float &x3) {
    const float ss = wave_sum_all(fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w))));
    const float sc = __builtin_amdgcn_rsqf(ss / static_cast<float>(kD) + eps);
    x0 = v.x * sc * g.x;
    x1 = v.y * sc * g.y;
    x2 = v.z * sc * g.z;
    x3 = v.w * sc * g.w;
    const int step = rope_dims >> 3;  // lanes between the two dims of a pair
    if (step > 0) {
        const float o0 = __shfl_xor(x0, step, 64), o1 = __shfl_xor(x1, step, 64), o2 = __shfl_xor(x2, step, 64), o3 = __shfl_xor(x3, step, 64);
        const bool first = (lane & step) == 0;  // holds the pair's first dim
        const bool turns = lane < 2 * step;     // inside the rotated dims
        x0 = rope_turn(x0, o0, cs4.x, sn4.x, first, turns);
        x1 = rope_turn(x1, o1, cs4.y, sn4.y, first, turns);
        x2 = rope_turn(x2, o2, cs4.z, sn4.z, first, turns);
        x3 = rope_turn(x3, o3, cs4.w, sn4.w, first, turns);
    }
}

// The same through LDS, for the kernel that only appends cells (dst is 256 floats of LDS).
__device__ __forceinline__ void norm_rope_loaded(const float4 v, const float4 g, float cs, float sn, int rope_dims, float eps,
                                                 float *dst, int lane) {
    const float ss = wave_sum_all(fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w))));
    const float sc = 1.f / sqrtf(ss / static_cast<float>(kD) + eps);
    *reinterpret_cast<float4 *>(dst + 4 * lane) = make_float4(v.x * sc * g.x, v.y * sc * g.y, v.z * sc * g.z, v.w * sc * g.w);
    __builtin_amdgcn_wave_barrier();
    const int half = rope_dims / 2;
    if (lane < half) {
        const float x0 = dst[lane], x1 = dst[lane + half];
        dst[lane] = x0 * cs - x1 * sn;
        dst[lane + half] = x0 * sn + x1 * cs;
    }
    __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ void norm_rope_head(const float *src, const float *gamma, const float *rope_row, int rope_dims,
                                               float eps, float *dst, int lane) {
    const int half = rope_dims / 2;
    const float cs = lane < half ? rope_row[lane] : 0.f, sn = lane < half ? rope_row[half + lane] : 0.f;
    norm_rope_loaded(*reinterpret_cast<const float4 *>(src + 4 * lane), *reinterpret_cast<const float4 *>(gamma + 4 * lane), cs, sn, rope_dims, eps, dst, lane);
}

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half4_t as_half4(uint32_t a, uint32_t b) {
    u32x2_t v;
    v.x = a;
    v.y = b;
    return __builtin_bit_cast(half4_t, v);
}

// x -> (hi, lo) halves with hi + lo = x to about 2^-22
__device__ __forceinline__ void split4(const float *x, half4_t &h, half4_t &l) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const _Float16 hi = static_cast<_Float16>(x[t]);
        h[t] = hi;
        l[t] = static_cast<_Float16>(x[t] - static_cast<float>(hi));
    }
}

__device__ __forceinline__ void split1(float x, half4_t &h, half4_t &l, int t) {
    const _Float16 hi = static_cast<_Float16>(x);
    h[t] = hi;
    l[t] = static_cast<_Float16>(x - static_cast<float>(hi));
}

// LDS of one block.  The queries are kept as matrix-core operands: entry [i][h][part][lane] is the
// four dims 8*(kb + 4*i) + 4*h .. +3 of query row lane%16 (kb = lane/16), as hi or lo halves.
struct Smem {
    half4_t qf[8][2][2][64];       // 16 KB
    float big[4][kRep][kD];        // 32 KB: queries in float32 first; later the waves' accumulators of one row
    float al[4][16];               // per wave: the factor each query row's running sums shrink by
    float wm[4][16], wl[4][16];    // per wave: running max and sum of each query row
};

// grid: (n_splits, n_head_kv, n_seq * n_groups); group g of a sequence is its rows row0 + R*g ..
// row0 + R*g + R-1.  With append the launch also writes its rows' cells; without, the cells are there
// already and any number of groups go in one launch, each masked to its own positions.  A later group
// reads the cells of the rows before it, which another block may still be writing: append 1 is for
// one group; with append 2 (two groups: three or four rows) a block of the second group writes the
// first group's cells in its slice as well, the same bytes the first group's block writes there, so
// that it reads only what it has written itself.  Query row r of the
// tile is head r%8 of sequence row r/8; with R = 1 rows 8..15 are padding.
// QSA: a.mask names, a bit a cell, the cells each row may read (the block-sparse indexer's
// selection, llm/attn.go:423-443); a tile none of the wave's rows may read is not loaded at all.
template <int R, bool QSA = false>
__global__ __launch_bounds__(kBlock, 1) void attn_decode_kernel(shv_attn_decode_args a, int row00, int n_groups, int append, int slice_cells) {
    __shared__ Smem sm;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the groups of a pass run over blockIdx.x, the fastest-varying index: the blocks that read one
    // slice of the cache for different row pairs are dispatched next to one another (and so land
    // a few on each die), and all but the first of a die find the slice in its L2
    const int gz = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
    const int seq = gz / n_groups, row0 = row00 + R * (gz % n_groups);
    // The sequence's slot and position come from device memory.  Asked for first; what does not
    // depend on them (the rows' q heads of this wave, the new cells' k and v, the norms' gammas) is
    // asked for right behind, before either is waited for: loads come back in the order they
    // were issued, and a chain of dependent round trips is what this kernel's prologue costs.
    const int slot = a.slot ? a.slot[seq] : seq;
    const int pos_first = a.pos ? a.pos[seq] : 0;
    const int tid_ = threadIdx.x, lane_ = tid_ & 63, wave_ = tid_ >> 6;
    const int valid_ = a.seq_len - row0 < R ? a.seq_len - row0 : R;
    const float *qkv0 = a.qkv + static_cast<size_t>(seq * a.seq_len + row0) * a.qkv_stride;
    // Which of the KV head's 8 query heads this wave prepares.  A slice of one tile (a decode
    // step: slices are made small so that many compute units pull the cache, each at the rate one
    // unit issues loads) is loaded by the first wave alone, which prepares nothing; the other
    // three share the heads 3, 3 and 2 and the last appends.  Otherwise every wave takes two heads
    // and its own tiles.
    const bool single = slice_cells <= kTile;
    const int h0 = single ? 3 * (wave_ - 1) : 2 * wave_;
    const int nh = single ? (wave_ == 0 ? 0 : wave_ == 3 ? 2 : 3) : 2;
    float4 qv[R][3], kv[R];
    float vv[R];
#pragma unroll
    for (int j = 0; j < R; j++) {
        const int jr = j < valid_ ? j : valid_ - 1;
        const float *qkv = qkv0 + static_cast<size_t>(jr) * a.qkv_stride;
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const int hh = min(max(h0 + i, 0), kRep - 1);  // a head it will not use is asked for all the same: no branch around loads
            qv[j][i] = *reinterpret_cast<const float4 *>(qkv + static_cast<size_t>(kvh * kRep + hh) * 2 * kD + 4 * lane_);
        }
        kv[j] = *reinterpret_cast<const float4 *>(qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvh * kD + 4 * lane_);
        vv[j] = qkv[static_cast<size_t>(a.n_head) * 2 * kD + a.n_head_kv * kD + kvh * kD + tid_];
    }
    // append 2: the rows of the pass before this group's (at most kForeign), whose cells this block writes too
    constexpr int kForeign = 2;
    const int n_foreign = append == 2 ? row0 - row00 : 0;
    float4 kvf[kForeign];
    float vvf[kForeign];
#pragma unroll
    for (int f = 0; f < kForeign; f++) {
        const float *qkv = a.qkv + static_cast<size_t>(seq * a.seq_len + row00 + (f < n_foreign ? f : 0)) * a.qkv_stride;
        kvf[f] = *reinterpret_cast<const float4 *>(qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvh * kD + 4 * lane_);
        vvf[f] = qkv[static_cast<size_t>(a.n_head) * 2 * kD + a.n_head_kv * kD + kvh * kD + tid_];
    }
    const float4 gq = *reinterpret_cast<const float4 *>(a.q_norm + 4 * lane_), gk = *reinterpret_cast<const float4 *>(a.k_norm + 4 * lane_);
    const int p_first = pos_first + row0;  // position of the group's first row
    // the last group of a sequence with an odd number of rows holds one: its second row repeats
    // the first and is thrown away
    const int valid = a.seq_len - row0 < R ? a.seq_len - row0 : R;
    const int n_cells = p_first + valid;                   // cells the last row sees
    // The grid is sized for the cache's capacity; how many of its slices take part depends on how
    // many cells the sequence holds now: about kSliceCells a slice while there are slices to spare.
    int n_active = (n_cells + slice_cells - 1) / slice_cells;
    if (n_active > a.n_splits) n_active = a.n_splits;
    if (split >= n_active) return;
    int cps = (n_cells + n_active - 1) / n_active;
    cps = (cps + kTile - 1) & ~(kTile - 1);  // slices start on a tile of V
    const int c0 = split * cps;
    const int c1 = c0 + cps < n_cells ? c0 + cps : n_cells;

    const int kvw = a.n_head_kv * kD;
    // K is [cell][kv head][dim]; V is kept transposed in tiles of 32 cells,
    // [cell/32][kv head][dim][cell%32], so that four cells of one dim are 8 contiguous bytes and a
    // tile of one KV head is 16 contiguous KB
    uint16_t *kc = static_cast<uint16_t *>(a.kcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;
    uint16_t *vt = static_cast<uint16_t *>(a.vcache) + static_cast<size_t>(slot) * a.max_cells * kvw + static_cast<size_t>(kvh) * kD * kTile;
    const size_t vtile = static_cast<size_t>(kvw) * kTile;  // halves from one tile of V to the next
    const int n = lane & 15, q = lane >> 4;

    // One tile = 32 cells of this wave.  Score tile T (0,1), slot s (= lane%16 as the A row) is cell
    // t0 + 8*(s/4) + 4*T + s%4, so that after the first product lane (row n, q) holds the scores of
    // cells t0 + 8q + 4T + 0..3: the four consecutive cells its V operand covers.
    struct Tile {
        uint4 k[2][8], v[16];
    };
    Tile ta;
    auto load_tile = [&](Tile &tl, int t0) {
        uint4(&kreg)[2][8] = tl.k;
        uint4(&vreg)[16] = tl.v;
#pragma unroll
        for (int T = 0; T < 2; T++) {
            int c = t0 + 8 * (n >> 2) + 4 * T + (n & 3);
            c = c < c1 ? c : c1 - 1;
            const uint16_t *row = kc + static_cast<size_t>(c) * kvw + 8 * q;
#pragma unroll
            for (int i = 0; i < 8; i++) kreg[T][i] = *reinterpret_cast<const uint4 *>(row + 32 * i);
        }
        // this lane's eight cells of V.  The cache is whole tiles, so the cells of the last tile
        // past the sequence's end exist; they hold finite values and get weight 0.
#pragma unroll
        for (int db = 0; db < 16; db++)
            vreg[db] = *reinterpret_cast<const uint4 *>(vt + static_cast<size_t>(t0 / kTile) * vtile + (16 * db + n) * kTile + 8 * q);
    };
    // ---- prologue: queries, new cells.  The rows' values were asked for at the top; the rotary
    //      factors (whose row the position names) and the wave's first tile of the cache go out
    //      together now.  Norms and rotation stay in registers and every wave writes its heads'
    //      queries straight into the operand table, so there is one block-wide wait ----
    const int rstep = a.rope_dims >> 3;
    float4 cs4[R], sn4[R];
    bool app[R];
#pragma unroll
    for (int j = 0; j < R; j++) {
        const int jr = j < valid ? j : valid - 1;
        const int p = p_first + jr;
        const float *rope_row = a.rope_dims > 0 ? a.rope + static_cast<size_t>(p) * a.rope_dims : a.q_norm;  // no rotary: any readable words
        app[j] = append && p >= c0 && p < c1;  // the new cell of row j lies in this slice
        const int rl = rstep > 0 ? 4 * (lane & (rstep - 1)) : 0;
        cs4[j] = *reinterpret_cast<const float4 *>(rope_row + rl);
        sn4[j] = *reinterpret_cast<const float4 *>(rope_row + (a.rope_dims >> 1) + rl);
    }
    // the wave's first tile, unless this launch is about to append cells inside it.  (After this
    // branch the compiler no longer knows how many loads are in flight and waits for all of them
    // where it needs an earlier one: a wave that has both a tile and heads to prepare waits for
    // the tile before it prepares them.  In a slice of one tile no wave has both.)
    float4 csf[kForeign], snf[kForeign];
    bool appf[kForeign];
#pragma unroll
    for (int f = 0; f < kForeign; f++) {
        const int p = pos_first + row00 + (f < n_foreign ? f : 0);
        const float *rope_row = a.rope_dims > 0 ? a.rope + static_cast<size_t>(p) * a.rope_dims : a.q_norm;
        appf[f] = f < n_foreign && p >= c0 && p < c1;
        const int rl = rstep > 0 ? 4 * (lane & (rstep - 1)) : 0;
        csf[f] = *reinterpret_cast<const float4 *>(rope_row + rl);
        snf[f] = *reinterpret_cast<const float4 *>(rope_row + (a.rope_dims >> 1) + rl);
    }
    const int t_first = c0 + kTile * wave;
    // (the first position any block of this pass may be writing is the pass's first row's)
    const bool early = !QSA && t_first < c1 && t_first + kTile <= p_first - n_foreign;
    if (early) load_tile(ta, t_first);
    // the lane's query row is sequence row n / 8: its mask words
    const uint32_t *mrow = nullptr;
    if constexpr (QSA) {
        const int jr = (n >> 3) < valid ? (n >> 3) : valid - 1;
        mrow = a.mask + static_cast<size_t>(seq * a.seq_len + row0 + jr) * a.mask_stride;
    }

    // operand table entry [i][h][part][16*kb + row] holds dims 8*(kb + 4*i) + 4*h .. +3 of query row
    // `row`: lane l's four dims 4l..4l+3 are h = l&1, kb = (l>>1)&3, i = l>>3
    const float scale = 1.f / sqrtf(static_cast<float>(kD));
    const int op_h = lane & 1, op_kb = (lane >> 1) & 3, op_i = lane >> 3;
#pragma unroll
    for (int j = 0; j < R; j++) {
        const int jr = j < valid ? j : valid - 1;
        const int p = p_first + jr;
#pragma unroll
        for (int i = 0; i < 3; i++) {
            if (i >= nh) break;
            float q0, q1, q2, q3;
            norm_rope_regs(qv[j][i], gq, cs4[j], sn4[j], a.rope_dims, a.eps, lane, q0, q1, q2, q3);
            half4_t hi, lo;
            split1(q0 * scale, hi, lo, 0);
            split1(q1 * scale, hi, lo, 1);
            split1(q2 * scale, hi, lo, 2);
            split1(q3 * scale, hi, lo, 3);
            const int row = 8 * j + h0 + i;
            sm.qf[op_i][op_h][0][16 * op_kb + row] = hi;
            sm.qf[op_i][op_h][1][16 * op_kb + row] = lo;
        }
        if (app[j]) {
            // one wave appends the new cell's K, all threads its V
            if (wave == (single ? 3 : ((2 * j) & 3))) {
                float k0, k1, k2, k3;
                norm_rope_regs(kv[j], gk, cs4[j], sn4[j], a.rope_dims, a.eps, lane, k0, k1, k2, k3);
                const __half2 k01 = __floats2half2_rn(k0, k1), k23 = __floats2half2_rn(k2, k3);
                uint2 packed;
                packed.x = *reinterpret_cast<const uint32_t *>(&k01);
                packed.y = *reinterpret_cast<const uint32_t *>(&k23);
                *reinterpret_cast<uint2 *>(kc + static_cast<size_t>(p) * kvw + 4 * lane) = packed;
            }
            vt[static_cast<size_t>(p / kTile) * vtile + tid * kTile + p % kTile] = __half_as_ushort(__float2half_rn(vv[j]));
        }
    }
#pragma unroll
    for (int f = 0; f < kForeign; f++) {
        if (appf[f]) {
            const int p = pos_first + row00 + f;
            if (wave == ((2 * f + 1) & 3)) {
                float k0, k1, k2, k3;
                norm_rope_regs(kvf[f], gk, csf[f], snf[f], a.rope_dims, a.eps, lane, k0, k1, k2, k3);
                const __half2 k01 = __floats2half2_rn(k0, k1), k23 = __floats2half2_rn(k2, k3);
                uint2 packed;
                packed.x = *reinterpret_cast<const uint32_t *>(&k01);
                packed.y = *reinterpret_cast<const uint32_t *>(&k23);
                *reinterpret_cast<uint2 *>(kc + static_cast<size_t>(p) * kvw + 4 * lane) = packed;
            }
            vt[static_cast<size_t>(p / kTile) * vtile + tid * kTile + p % kTile] = __half_as_ushort(__float2half_rn(vvf[f]));
        }
    }
    if (R == 1) {
        // rows 8..15 of the tile are padding: zero operands (entries of lane ln with ln%16 >= 8)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int idx = tid + e * kBlock;  // [i][h][ln]
            const int ln = idx & 63, h = (idx >> 6) & 1, i = idx >> 7;
            if ((ln & 15) >= 8) {
                sm.qf[i][h][0][ln] = half4_t{0, 0, 0, 0};
                sm.qf[i][h][1][ln] = half4_t{0, 0, 0, 0};
            }
        }
    }
    // Only a block that appended cells reads its own stores back (its waves' tiles are asked for
    // again after the wait).  The fence would also wait for every load in flight, i.e. for the
    // first tile, before the block-wide wait instead of after it: the other blocks skip it.
    bool appended = false;
#pragma unroll
    for (int j = 0; j < R; j++) appended = appended || app[j];
#pragma unroll
    for (int f = 0; f < kForeign; f++) appended = appended || appf[f];
    if (appended) __threadfence_block();
    __syncthreads();

    // per lane: O[row 4q+i][dim 16*db + n] for the 16 dim blocks; the running max and sum of query
    // row n (the same in the four lanes that share it)
    float4_t o[16];
#pragma unroll
    for (int db = 0; db < 16; db++) o[db] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    const int my_row_pos = p_first + (n >> 3);  // the last cell query row n may see

    auto compute = [&](const Tile &tl, int t0, uint32_t mw) {
        const uint4(&kreg)[2][8] = tl.k;
        const uint4(&vreg)[16] = tl.v;
        // ---- S^T = K Q^T: A = K (cells x dims), B = Q^T (dims x rows); four independent chains
        //      of products (two score tiles, even and odd dim groups) keep the matrix pipe busy ----
        float4_t st[2];
        {
            float4_t acc[2][2];
#pragma unroll
            for (int T = 0; T < 2; T++)
#pragma unroll
                for (int e = 0; e < 2; e++) acc[T][e] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                // the query operands come from LDS as they are used: held in registers for the
                // whole loop they would push the tiles out to scratch
                const half4_t qh0 = sm.qf[i][0][0][lane], qh1 = sm.qf[i][1][0][lane];
                const half4_t ql0 = sm.qf[i][0][1][lane], ql1 = sm.qf[i][1][1][lane];
#pragma unroll
                for (int T = 0; T < 2; T++) {
                    const half4_t k0 = as_half4(kreg[T][i].x, kreg[T][i].y), k1 = as_half4(kreg[T][i].z, kreg[T][i].w);
                    float4_t c = acc[T][i & 1];
                    c = __builtin_amdgcn_mfma_f32_16x16x16f16(k0, qh0, c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_16x16x16f16(k1, qh1, c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_16x16x16f16(k0, ql0, c, 0, 0, 0);
                    c = __builtin_amdgcn_mfma_f32_16x16x16f16(k1, ql1, c, 0, 0, 0);
                    acc[T][i & 1] = c;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            st[0] = acc[0][0] + acc[0][1];
            st[1] = acc[1][0] + acc[1][1];
        }
        // ---- running softmax of query row n over this tile's 32 cells (8 here, 24 in the three
        //      other lanes of the row); causal: row n sees cells up to its own position ----
        float mx = -INFINITY;
#pragma unroll
        for (int T = 0; T < 2; T++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = t0 + 8 * q + 4 * T + i;
                bool ok = c < c1 && c <= my_row_pos;
                if constexpr (QSA) ok = ok && ((mw >> (8 * q + 4 * T + i)) & 1u) != 0u;
                st[T][i] = ok ? st[T][i] : -INFINITY;
                mx = fmaxf(mx, st[T][i]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;  // nothing visible yet: all weights 0
        float sum = 0.f;
        half4_t ph[2], pl[2];
#pragma unroll
        for (int T = 0; T < 2; T++) {
            float pv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                pv[i] = __expf(st[T][i] - m_use);
                sum += pv[i];
            }
            split4(pv, ph[T], pl[T]);
        }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        const float alpha = __expf(m_run - m_use);  // 0 while the old max is -inf
        l_run = l_run * alpha + sum;
        m_run = m_new;
        // the accumulators hold other rows than this lane's: the factors go through LDS, and are
        // applied only when some row's maximum moved
        if (__ballot(alpha != 1.f) != 0ull) {
            if (q == 0) sm.al[wave][n] = alpha;
            __builtin_amdgcn_wave_barrier();
            const float4 af = *reinterpret_cast<const float4 *>(&sm.al[wave][4 * q]);
            const float av[4] = {af.x, af.y, af.z, af.w};
#pragma unroll
            for (int db = 0; db < 16; db++)
#pragma unroll
                for (int i = 0; i < 4; i++) o[db][i] *= av[i];
            __builtin_amdgcn_wave_barrier();
        }
        // ---- O += P V: A = P (rows x cells), B = V (cells x dims) ----
#pragma unroll
        for (int db = 0; db < 16; db++) {
            const uint4 v = vreg[db];
            const half4_t v0 = as_half4(v.x, v.y), v1 = as_half4(v.z, v.w);
            float4_t acc = o[db];
            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(ph[0], v0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(pl[0], v0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(ph[1], v1, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x16f16(pl[1], v1, acc, 0, 0, 0);
            o[db] = acc;
        }
    };
    // the wave's tiles are 4*kTile cells apart; two blocks share a compute unit, one's loads
    // overlap the other's products
    constexpr int kStep = 4 * kTile;
    for (int t0 = t_first; t0 < c1; t0 += kStep) {
        uint32_t mw = 0xFFFFFFFFu;
        if constexpr (QSA) {
            mw = mrow[t0 >> 5];  // tiles start on multiples of 32 cells: one word a tile and row
            if (__ballot(mw != 0u) == 0ull) continue;
        }
        if (!early || t0 != t_first) load_tile(ta, t0);
        compute(ta, t0, mw);
    }
    // ---- the four waves' results of each sequence row are merged and go to scratch ----
    if (q == 0) {
        sm.wm[wave][n] = m_run;
        sm.wl[wave][n] = l_run;
    }
    __syncthreads();  // everyone is done with the queries in sm.qf / sm.big
    float *part_base = a.partial + ((static_cast<size_t>(gz) * a.n_head_kv + kvh) * a.n_splits + split) * R * kRec;
#pragma unroll
    for (int j = 0; j < R; j++) {
        // this lane's rows 4q..4q+3 belong to sequence row j when q/2 == j
        if ((q >> 1) == j) {
#pragma unroll
            for (int db = 0; db < 16; db++)
#pragma unroll
                for (int i = 0; i < 4; i++) sm.big[wave][(4 * q + i) & 7][16 * db + n] = o[db][i];
        }
        __syncthreads();
        {
            // thread = (head, 8 dims)
            const int hh = tid >> 5, d0 = (tid & 31) * 8, r = 8 * j + hh;
            float M = fmaxf(fmaxf(sm.wm[0][r], sm.wm[1][r]), fmaxf(sm.wm[2][r], sm.wm[3][r]));
            float w[4], L = 0.f;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                w[k] = sm.wm[k][r] == -INFINITY ? 0.f : __expf(sm.wm[k][r] - M);
                L = fmaf(w[k], sm.wl[k][r], L);
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

// grid: (n_head * 4, R, n_seq * n_groups), one block = 64 dims of one head; its waves share the slices'
// records of that (row, head), each folds its share with a running max (all of a batch's loads in
// flight together), and the first wave folds their results.
// NW waves a block: eight for a decode step, whose one row pair has a slice per 128 cells of context to fold;
// one for a pass of many row pairs, which takes few slices a pair and would launch eight times the waves for nothing.
constexpr int kMergeWaves = 8;
template <int R, int NW>
__global__ __launch_bounds__(64 * NW) void attn_merge_kernel(shv_attn_decode_args a, int row00, int n_groups, int slice_cells) {
    __shared__ float red[3][NW][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int head = blockIdx.x >> 2, d = (blockIdx.x & 3) * 64 + lane, j = blockIdx.y;
    const int seq = blockIdx.z / n_groups, row0 = row00 + R * (blockIdx.z % n_groups);
    const int kvh = head / kRep, hh = head % kRep;
    if (row0 + j >= a.seq_len) return;  // the thrown-away second row of a last group of one
    const int valid = a.seq_len - row0 < R ? a.seq_len - row0 : R;
    const int n_cells = (a.pos ? a.pos[seq] : 0) + row0 + valid;
    int n_active = (n_cells + slice_cells - 1) / slice_cells;
    if (n_active > a.n_splits) n_active = a.n_splits;
    const float *pin = a.partial + (static_cast<size_t>(blockIdx.z) * a.n_head_kv + kvh) * a.n_splits * R * kRec + j * kRec + hh * (kD + 2);
    constexpr int MB = 16;
    float num = 0.f, den = 0.f, M = -INFINITY;
    for (int s0 = wave; s0 < n_active; s0 += NW * MB) {
        float v[MB];
        float2 ml[MB];
#pragma unroll
        for (int u = 0; u < MB; u++) {
            const int sidx = s0 + NW * u < n_active ? s0 + NW * u : s0;
            const float *rec = pin + static_cast<size_t>(sidx) * R * kRec;
            v[u] = rec[d];
            ml[u] = *reinterpret_cast<const float2 *>(rec + kD);
        }
#pragma unroll
        for (int u = 0; u < MB; u++) {
            if (s0 + NW * u >= n_active || ml[u].x == -INFINITY) continue;
            const float Mn = fmaxf(M, ml[u].x);
            const float shrink = __expf(M - Mn), w = __expf(ml[u].x - Mn);  // shrink is 0 while M is -inf
            den = fmaf(den, shrink, w * ml[u].y);
            num = fmaf(num, shrink, w * v[u]);
            M = Mn;
        }
    }
    red[0][wave][lane] = M;
    red[1][wave][lane] = den;
    red[2][wave][lane] = num;
    __syncthreads();
    if (wave != 0) return;
    float Mt = red[0][0][lane];
#pragma unroll
    for (int k = 1; k < NW; k++) Mt = fmaxf(Mt, red[0][k][lane]);
    float nt = 0.f, dt = 0.f;
#pragma unroll
    for (int k = 0; k < NW; k++) {
        const float mk = red[0][k][lane];
        const float w = mk == -INFINITY ? 0.f : __expf(mk - Mt);
        dt = fmaf(w, red[1][k][lane], dt);
        nt = fmaf(w, red[2][k][lane], nt);
    }
    a.out[static_cast<size_t>(seq * a.seq_len + row0 + j) * a.n_head * kD + static_cast<size_t>(head) * kD + d] = nt / dt;
}

// grid: (n_head_kv, seq_len, n_seq): the cells of every row of a pass, written before any of
// them is read: K normed and rotated by the first wave, V transposed into its tile by all threads.
__global__ __launch_bounds__(kBlock) void attn_append_kernel(shv_attn_decode_args a) {
    __shared__ float ktmp[kD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kvh = blockIdx.x, row = blockIdx.y, seq = blockIdx.z;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int p = (a.pos ? a.pos[seq] : 0) + row;
    const int kvw = a.n_head_kv * kD;
    uint16_t *kc = static_cast<uint16_t *>(a.kcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;
    uint16_t *vt = static_cast<uint16_t *>(a.vcache) + static_cast<size_t>(slot) * a.max_cells * kvw + static_cast<size_t>(kvh) * kD * kTile;
    const size_t vtile = static_cast<size_t>(kvw) * kTile;
    const float *qkv = a.qkv + static_cast<size_t>(seq * a.seq_len + row) * a.qkv_stride;
    if (wave == 0) {
        const float *ksrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvh * kD;
        norm_rope_head(ksrc, a.k_norm, a.rope + static_cast<size_t>(p) * a.rope_dims, a.rope_dims, a.eps, ktmp, lane);
        uint16_t *dst = kc + static_cast<size_t>(p) * kvw;
#pragma unroll
        for (int i = 0; i < 4; i++) dst[4 * lane + i] = __half_as_ushort(__float2half_rn(ktmp[4 * lane + i]));
    }
    const float *vsrc = qkv + static_cast<size_t>(a.n_head) * 2 * kD + kvw + kvh * kD;
    vt[static_cast<size_t>(p / kTile) * vtile + tid * kTile + p % kTile] = __half_as_ushort(__float2half_rn(vsrc[tid]));
}

// ---- prompt passes: eight row pairs a block, every tile of the cache through LDS once ---------
// The kernel above lets each row pair pull the whole cache for itself, which a pass of a thousand
// pairs pays in L2 bandwidth.  Here a block is eight pairs (128 query rows of one KV head), one a
// wave.  A 32-cell tile of K and V is 32 chunks of 1 KB, each exactly what one LDS read of a wave
// takes (64 lanes x 16 bytes, in lane order: no bank is asked twice), and the loads put them
// there themselves: a lane names the 16 bytes of the cache that belong at its place in the chunk
// and the load writes LDS, so a tile passes through no register and costs no vector work.  Four
// tiles are in the ring: three on their way while one is multiplied.  Every wave forms its
// products from there, as v_mfma_f32_16x16x32_f16 (eight dims or eight cells a lane), slices the
// cache and writes its records exactly as a block of the kernel above would for that pair, so the
// same merge follows.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef const __attribute__((address_space(1))) void *global_ptr_t;
typedef __attribute__((address_space(3))) void *lds_ptr_t;
constexpr int kPfWaves = 8;
constexpr int kPfThreads = kPfWaves * 64;
constexpr int kPfStages = 4;
constexpr int kChunk = 64 * 16;
constexpr int kTileBytes = 32 * kChunk;   // K: chunk 8 T + i (score tile T, 32-dim step i); V: chunk 16 + db (16 dims)
struct PrefillSmem {
    // the queries pass through here once, on their way from the lanes that normalised them to the
    // lanes that hold them as operands (per wave: [32-dim step][hi, lo][16 * (dim group) + query
    // row]); after that the same bytes are the ring of tiles
    union {
        half8_t qf[kPfWaves][8][2][64];
        char ring[kPfStages][kTileBytes];
    } u;
};

// The barrier between two tiles.  A wave's loads complete in order, so "at most eight of mine still
// out" says that all but its two youngest tiles' loads have written LDS; the LDS reads of the tile
// just multiplied have returned (their values were used); then the workgroup meets.  Written out
// because __syncthreads() would first wait for every load in flight, the tiles ahead included.
__device__ __forceinline__ void tile_barrier() {
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// The same for the kernel that also loads mask words between the tiles' loads, which the count above
// does not know of: it waits for everything (the tiles ahead included; that build gives up their
// head start).
__device__ __forceinline__ void tile_barrier_all() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// grid: (n_seq * ceil(n_groups / 8), n_head_kv, n_splits); the cells of the pass are in the cache already.
template <bool QSA>
__global__ __launch_bounds__(kPfThreads) void attn_prefill_kernel(shv_attn_decode_args a, int n_groups, int slice_cells, int direct) {
    extern __shared__ __align__(16) char praw[];
    PrefillSmem &sm = *reinterpret_cast<PrefillSmem *>(praw);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, q = lane >> 4;
    // Workgroups are handed to the chip's eight dies in turn (workgroup i to die i % 8), and each die has its
    // own L2: the blocks of one die all take the same KV head, so that a die's L2 holds one head's K and V
    // (half the cells' bytes) and the blocks that walk it side by side find each other's tiles there.
    int kvh = blockIdx.y, bx = blockIdx.x;
    {
        const int per = 8 / a.n_head_kv;  // dies a KV head gets
        if (a.n_head_kv <= 8 && per * a.n_head_kv == 8 && gridDim.x % per == 0) {
            const int id = blockIdx.x + gridDim.x * blockIdx.y, die = id & 7;
            kvh = die % a.n_head_kv;
            bx = (id >> 3) * per + die / a.n_head_kv;
        }
    }
    const int split = blockIdx.z;
    const int bps = (n_groups + kPfWaves - 1) / kPfWaves;
    const int seq = bx / bps, g0 = (bx % bps) * kPfWaves;
    const int slot = a.slot ? a.slot[seq] : seq;
    const int pos_first = a.pos ? a.pos[seq] : 0;
    // pair gg of the sequence: its rows, what it sees, its slice of that
    struct Slice { int c0, c1, p_first, valid; bool mine, empty; };
    auto slice_of = [&](int gg) {
        Slice s;
        const bool live = gg < n_groups;
        const int g = live ? gg : n_groups - 1;
        const int row0 = 2 * g;
        s.valid = a.seq_len - row0 < 2 ? a.seq_len - row0 : 2;
        s.p_first = pos_first + row0;
        const int n_cells = s.p_first + s.valid;
        int n_active = (n_cells + slice_cells - 1) / slice_cells;
        if (n_active > a.n_splits) n_active = a.n_splits;
        int cps = (n_cells + n_active - 1) / n_active;
        cps = (cps + kTile - 1) & ~(kTile - 1);
        s.c0 = split * cps;
        s.c1 = s.c0 + cps < n_cells ? s.c0 + cps : n_cells;
        s.mine = live && split < n_active && s.c1 > s.c0;
        // slices start on a tile of V: rounded up, the last of a pair's slices can start past its cells
        s.empty = live && split < n_active && s.c1 <= s.c0;
        return s;
    };
    const Slice me = slice_of(g0 + wave);
    if (me.empty && lane < 2 * kRep) {
        // the merge reads every slice the pair counts as taking part: this one says it holds nothing
        const int gz = seq * n_groups + g0 + wave;
        float *rec = a.partial + ((static_cast<size_t>(gz) * a.n_head_kv + kvh) * a.n_splits + split) * 2 * kRec;
        *reinterpret_cast<float2 *>(rec + (lane >> 3) * kRec + (lane & 7) * (kD + 2) + kD) = make_float2(-INFINITY, 0.f);
    }
    int lo = 0x7fffffff, hi = 0;
#pragma unroll
    for (int w = 0; w < kPfWaves; w++) {
        const Slice o = slice_of(g0 + w);
        if (o.mine) {
            lo = o.c0 < lo ? o.c0 : lo;
            hi = o.c1 > hi ? o.c1 : hi;
        }
    }
    if (hi <= lo) return;  // no pair of the block has cells in this slice (the same for every wave)
    const int g = g0 + wave < n_groups ? g0 + wave : n_groups - 1;
    const int row0 = 2 * g, gz = seq * n_groups + g;

    const int kvw = a.n_head_kv * kD;
    const uint16_t *kc = static_cast<const uint16_t *>(a.kcache) + static_cast<size_t>(slot) * a.max_cells * kvw + kvh * kD;
    const uint16_t *vtg = static_cast<const uint16_t *>(a.vcache) + static_cast<size_t>(slot) * a.max_cells * kvw + static_cast<size_t>(kvh) * kD * kTile;
    const size_t vtile = static_cast<size_t>(kvw) * kTile;

    // ---- the tile copy: four chunks a wave, waves 0..3 the keys, 4..7 the values ----
    // K chunk (T, i): lane (n, q) stands for score-tile slot n = cell 8 (n / 4) + 4 T + n % 4 of the tile, dims 32 i + 8 q ..;
    // V chunk db: lane (n, q) stands for dim 16 db + n, cells 8 q .. of the tile.  A tile past the last repeats it.
    const int last_tile = (hi - 1) / kTile;
    auto ask_tile = [&](int t0, int stage) {
        char *ring = sm.u.ring[stage];
        const int tile = t0 / kTile < last_tile ? t0 / kTile : last_tile;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int ch = 4 * wave + u;
            const uint16_t *g;
            if (wave < 4) {
                const int T = ch >> 3, i = ch & 7;
                int c = tile * kTile + 8 * (n >> 2) + 4 * T + (n & 3);
                c = c < hi ? c : hi - 1;
                g = kc + static_cast<size_t>(c) * kvw + 32 * i + 8 * q;
            } else {
                const int db = ch - 16;
                g = vtg + static_cast<size_t>(tile) * vtile + (16 * db + n) * kTile + 8 * q;
            }
            __builtin_amdgcn_global_load_lds((global_ptr_t)(g), (lds_ptr_t)(ring + ch * kChunk), 16, 0, 0);
        }
    };

    // ---- the wave's 16 query rows: norm, rotation, scale, operand order ----
    {
        const float4 gq = *reinterpret_cast<const float4 *>(a.q_norm + 4 * lane);
        const int rstep = a.rope_dims >> 3;
        const float scale = 1.f / sqrtf(static_cast<float>(kD));
        const int op_h = lane & 1, op_kb = (lane >> 1) & 3, op_i = lane >> 3;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int jr = j < me.valid ? j : me.valid - 1;
            const int p = me.p_first + jr;
            const float *rope_row = a.rope_dims > 0 ? a.rope + static_cast<size_t>(p) * a.rope_dims : a.q_norm;
            const int rl = rstep > 0 ? 4 * (lane & (rstep - 1)) : 0;
            const float4 cs4 = *reinterpret_cast<const float4 *>(rope_row + rl);
            const float4 sn4 = *reinterpret_cast<const float4 *>(rope_row + (a.rope_dims >> 1) + rl);
            const float *qkv = a.qkv + static_cast<size_t>(seq * a.seq_len + row0 + jr) * a.qkv_stride;
            float4 qv[kRep];
#pragma unroll
            for (int hh = 0; hh < kRep; hh++) qv[hh] = *reinterpret_cast<const float4 *>(qkv + static_cast<size_t>(kvh * kRep + hh) * 2 * kD + 4 * lane);
#pragma unroll
            for (int hh = 0; hh < kRep; hh++) {
                float q0, q1, q2, q3;
                norm_rope_regs(qv[hh], gq, cs4, sn4, a.rope_dims, a.eps, lane, q0, q1, q2, q3);
                half4_t h4, l4;
                split1(q0 * scale, h4, l4, 0);
                split1(q1 * scale, h4, l4, 1);
                split1(q2 * scale, h4, l4, 2);
                split1(q3 * scale, h4, l4, 3);
                const int row = 8 * j + hh;
                half4_t *dh = reinterpret_cast<half4_t *>(&sm.u.qf[wave][op_i][0][16 * op_kb + row]) + op_h;
                half4_t *dl = reinterpret_cast<half4_t *>(&sm.u.qf[wave][op_i][1][16 * op_kb + row]) + op_h;
                *dh = h4;
                *dl = l4;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();   // a wave reads back only what it wrote itself
    half8_t qh[8], ql[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        qh[i] = sm.u.qf[wave][i][0][lane];
        ql[i] = sm.u.qf[wave][i][1][lane];
    }
    __syncthreads();   // every wave holds its queries: the bytes become the ring of tiles
    ask_tile(lo, 0);
    ask_tile(lo + kTile, 1);
    ask_tile(lo + 2 * kTile, 2);
    if constexpr (QSA) tile_barrier_all();
    else tile_barrier();   // the first tile has landed: all but the two youngest tiles' loads of every wave
    const uint32_t *mrow = nullptr;
    if constexpr (QSA) {
        const int jr = (n >> 3) < me.valid ? (n >> 3) : me.valid - 1;
        mrow = a.mask + static_cast<size_t>(seq * a.seq_len + row0 + jr) * a.mask_stride;
    }

    float4_t o[16];
#pragma unroll
    for (int db = 0; db < 16; db++) o[db] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    const int my_row_pos = me.p_first + (n >> 3);

    int b = 0;
    for (int t0 = lo; t0 < hi; t0 += kTile, b = (b + 1) & (kPfStages - 1)) {
        // three tiles on: into the stage read a tile ago (every wave has passed the barrier that ended that tile)
        ask_tile(t0 + 3 * kTile, (b + 3) & (kPfStages - 1));
        uint32_t mw = 0xFFFFFFFFu;
        if constexpr (QSA) mw = mrow[t0 >> 5];
        // tiles wholly outside the wave's slice or beyond what its rows see are skipped
        if (me.mine && t0 < me.c1 && t0 + kTile > me.c0 && t0 <= me.p_first + 1 && (!QSA || __ballot(mw != 0u) != 0ull)) {
            const char *kt = sm.u.ring[b], *vt = sm.u.ring[b] + 16 * kChunk;
            // operands come from LDS four reads ahead of the products that use them: a read's
            // latency is about what eight products take, and asked for one at a time it is paid 32 times a tile
            float4_t st[2];
            half8_t vb[2][4];
            {
                float4_t acc[2][2];
#pragma unroll
                for (int T = 0; T < 2; T++)
#pragma unroll
                    for (int e = 0; e < 2; e++) acc[T][e] = float4_t{0.f, 0.f, 0.f, 0.f};
                half8_t kb[2][4];
                auto read_k = [&](half8_t (&dst)[4], int g4) {   // batch g4: dim steps 2 g4, 2 g4 + 1 of both score tiles
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int i = 2 * g4 + (e >> 1), T = e & 1;
                        dst[e] = *reinterpret_cast<const half8_t *>(kt + (8 * T + i) * kChunk + lane * 16);
                    }
                };
                read_k(kb[0], 0);
#pragma unroll
                for (int g4 = 0; g4 < 4; g4++) {
                    if (g4 + 1 < 4) read_k(kb[(g4 + 1) & 1], g4 + 1);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int i = 2 * g4 + (e >> 1), T = e & 1;
                        acc[T][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb[g4 & 1][e], qh[i], acc[T][0], 0, 0, 0);
                        acc[T][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb[g4 & 1][e], ql[i], acc[T][1], 0, 0, 0);
                    }
                }
                // the first values go out now, under the softmax arithmetic
#pragma unroll
                for (int e = 0; e < 4; e++) vb[0][e] = *reinterpret_cast<const half8_t *>(vt + e * kChunk + lane * 16);
                st[0] = acc[0][0] + acc[0][1];
                st[1] = acc[1][0] + acc[1][1];
            }
            float mx = -INFINITY;
#pragma unroll
            for (int T = 0; T < 2; T++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int c = t0 + 8 * q + 4 * T + i;
                    bool ok = c >= me.c0 && c < me.c1 && c <= my_row_pos;
                    if constexpr (QSA) ok = ok && ((mw >> (8 * q + 4 * T + i)) & 1u) != 0u;
                    st[T][i] = ok ? st[T][i] : -INFINITY;
                    mx = fmaxf(mx, st[T][i]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run, mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            float sum = 0.f;
            half8_t ph, pl;
#pragma unroll
            for (int T = 0; T < 2; T++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float pv = __expf(st[T][i] - m_use);
                    sum += pv;
                    const _Float16 hi16 = static_cast<_Float16>(pv);
                    ph[4 * T + i] = hi16;
                    pl[4 * T + i] = static_cast<_Float16>(pv - static_cast<float>(hi16));
                }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            const float alpha = __expf(m_run - m_use);
            l_run = l_run * alpha + sum;
            m_run = m_new;
            if (__ballot(alpha != 1.f) != 0ull) {
                // a lane's four accumulator rows are query rows 4 q + i: their factors sit in lanes 4 q + i
                float av[4];
#pragma unroll
                for (int i = 0; i < 4; i++) av[i] = __shfl(alpha, 4 * q + i, 64);
#pragma unroll
                for (int db = 0; db < 16; db++)
#pragma unroll
                    for (int i = 0; i < 4; i++) o[db][i] *= av[i];
            }
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                if (g4 + 1 < 4) {
#pragma unroll
                    for (int e = 0; e < 4; e++) vb[(g4 + 1) & 1][e] = *reinterpret_cast<const half8_t *>(vt + (4 * (g4 + 1) + e) * kChunk + lane * 16);
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int db = 4 * g4 + e;
                    float4_t acc = o[db];
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph, vb[g4 & 1][e], acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(pl, vb[g4 & 1][e], acc, 0, 0, 0);
                    o[db] = acc;
                }
            }
        }
        if constexpr (QSA) tile_barrier_all();
        else tile_barrier();   // the next tile has landed, this one has been read
    }
    // the loads asked for past the last tile still write LDS: none may be out when the wave ends and its LDS goes to another workgroup
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (!me.mine) return;
    if (direct) {
        // one slice a pair: what the merge would make of its single record, sums / sum, goes straight out
        float lr[4];
#pragma unroll
        for (int i = 0; i < 4; i++) lr[i] = __shfl(l_run, 4 * q + i, 64);   // query row 4 q + i keeps its sum in lane 4 q + i
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int r = 4 * q + i;  // query row: sequence row r / 8, head r % 8
            if ((r >> 3) >= me.valid) continue;
            float *dst = a.out + (static_cast<size_t>(seq * a.seq_len + row0 + (r >> 3)) * a.n_head + kvh * kRep + (r & 7)) * kD;
#pragma unroll
            for (int db = 0; db < 16; db++) dst[16 * db + n] = o[db][i] / lr[i];
        }
        return;
    }
    // the wave's record of this slice: per row and head the unnormalised sums, then (max, sum)
    float *rec = a.partial + ((static_cast<size_t>(gz) * a.n_head_kv + kvh) * a.n_splits + split) * 2 * kRec;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = 4 * q + i;  // query row: sequence row r / 8, head r % 8
        float *dst = rec + (r >> 3) * kRec + (r & 7) * (kD + 2);
#pragma unroll
        for (int db = 0; db < 16; db++) dst[16 * db + n] = o[db][i];
    }
    if (q == 0) *reinterpret_cast<float2 *>(rec + (n >> 3) * kRec + (n & 7) * (kD + 2) + kD) = make_float2(m_run, l_run);
}

template <int R>
int launch_rows(shv_ctx *ctx, const shv_attn_decode_args &a, int row0, int n_groups, int append) {
    // The slices are there to spread ONE row pair's cache over the chip.  A pass of many pairs (or
    // of many sequences) brings its own parallelism, and every block pays the query prologue
    // (norms and rotation of its 16 rows) whatever its slice holds: such a pass takes as many
    // slices as make two blocks a compute unit, no more (64 rows at 32 768 cells: 359 to 214 us).
    shv_attn_decode_args b = a;
    const int lanes = a.n_seq * n_groups * a.n_head_kv;
    const int want = (2 * ctx->prop.multiProcessorCount + lanes - 1) / lanes;
    if (b.n_splits > want) b.n_splits = want < 1 ? 1 : want;
    // one row pair: slices of one tile while there are slices to spare, so that as many compute
    // units as possible pull the cache (a unit issues a wave's 16-byte loads at about 25 B a clock;
    // 36 units over 2 300 cells took 2.2 us to ask for them, 144 take a quarter of that)
    const int slice_cells = a.n_seq * n_groups == 1 ? kTile : kSliceCells;
    if (R == 2 && !append && row0 == 0 && n_groups >= 8) {
        // a prompt pass: eight pairs a block share the cache's tiles
        static std::atomic<bool> raised{false};
        if (!raised.load(std::memory_order_acquire)) {
            SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_prefill_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(sizeof(PrefillSmem))));
            SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_prefill_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(sizeof(PrefillSmem))));
            raised.store(true, std::memory_order_release);
        }
        // with one slice a pair there is nothing to merge: the kernel writes the rows themselves
        const int direct = b.n_splits == 1 ? 1 : 0;
        const dim3 grid(a.n_seq * ((n_groups + kPfWaves - 1) / kPfWaves), a.n_head_kv, b.n_splits);
        if (a.mask) SHV_LAUNCH(ctx, attn_prefill_kernel<true>, grid, dim3(kPfThreads), sizeof(PrefillSmem), b, n_groups, slice_cells, direct);
        else SHV_LAUNCH(ctx, attn_prefill_kernel<false>, grid, dim3(kPfThreads), sizeof(PrefillSmem), b, n_groups, slice_cells, direct);
        if (direct) return SHV_OK;
    } else {
        dim3 grid(a.n_seq * n_groups, a.n_head_kv, b.n_splits);
        if (a.mask) SHV_LAUNCH(ctx, (attn_decode_kernel<R, true>), grid, dim3(kBlock), 0, b, row0, n_groups, append, slice_cells);
        else SHV_LAUNCH(ctx, (attn_decode_kernel<R>), grid, dim3(kBlock), 0, b, row0, n_groups, append, slice_cells);
    }
    if (a.n_seq * n_groups >= 8 && b.n_splits <= 16) SHV_LAUNCH(ctx, (attn_merge_kernel<R, 1>), dim3(a.n_head * 4, R, a.n_seq * n_groups), dim3(64), 0, b, row0, n_groups, slice_cells);
    else SHV_LAUNCH(ctx, (attn_merge_kernel<R, kMergeWaves>), dim3(a.n_head * 4, R, a.n_seq * n_groups), dim3(64 * kMergeWaves), 0, b, row0, n_groups, slice_cells);
    return SHV_OK;
}

}  // namespace

int shv_launch_attn_decode(shv_ctx *ctx, const shv_attn_decode_args *pa) {
    const shv_attn_decode_args &a = *pa;
    SHV_REQUIRE(a.qkv && a.q_norm && a.k_norm && a.rope && a.kcache && a.vcache && a.partial && a.out, "attn_decode: NULL argument");
    SHV_REQUIRE(a.head_dim == kD, "attn_decode: head_dim %d; built for %d", a.head_dim, kD);
    SHV_REQUIRE(a.n_head_kv >= 1 && a.n_head == a.n_head_kv * kRep, "attn_decode: %d query heads over %d KV heads; built for %d per KV head",
                a.n_head, a.n_head_kv, kRep);
    SHV_REQUIRE(a.rope_dims >= 0 && a.rope_dims <= 128 && (a.rope_dims == 0 || (a.rope_dims >= 8 && (a.rope_dims & (a.rope_dims - 1)) == 0)),
                "attn_decode: rope_dims %d; 0 or a power of two from 8 to 128 (the rotation pairs dims rope_dims/8 lanes apart)", a.rope_dims);
    SHV_REQUIRE(shv_aligned16(a.rope), "attn_decode: the rotary table must be 16-byte aligned");
    SHV_REQUIRE(a.n_seq >= 1 && a.seq_len >= 1, "attn_decode: %d sequences of %d rows", a.n_seq, a.seq_len);
    SHV_REQUIRE(a.n_seq <= 65535, "attn_decode: %d sequences", a.n_seq);
    SHV_REQUIRE(a.n_splits >= 1 && a.n_splits <= kMaxSplits, "attn_decode: %d slices; 1..%d", a.n_splits, kMaxSplits);
    SHV_REQUIRE(a.qkv_stride >= a.n_head * 2 * kD + 2 * a.n_head_kv * kD, "attn_decode: qkv_stride %d", a.qkv_stride);
    SHV_REQUIRE(a.max_cells >= kTile && a.max_cells % kTile == 0, "attn_decode: max_cells %d; a multiple of %d", a.max_cells, kTile);
    SHV_REQUIRE(!a.mask || a.mask_stride >= a.max_cells / 32, "attn_decode: mask_stride %d words for %d cells", a.mask_stride, a.max_cells);
    SHV_REQUIRE(shv_aligned16(a.qkv) && shv_aligned16(a.kcache) && shv_aligned16(a.vcache) && shv_aligned16(a.q_norm) &&
                    shv_aligned16(a.k_norm) && shv_aligned16(a.out) && shv_aligned16(a.partial) && a.qkv_stride % 4 == 0,
                "attn_decode: qkv, caches, norms, partial and out must be 16-byte aligned");
    // The rows of a sequence go two at a time: both see one pass over the cache.  One or two rows
    // write their own cells on the way; more rows have all their cells written first and then go
    // through as pairs of one launch (a last pair of one row repeats it and drops the copy).
    if (a.seq_len <= 2) return a.seq_len == 2 ? launch_rows<2>(ctx, a, 0, 1, 1) : launch_rows<1>(ctx, a, 0, 1, 1);
    const int pairs = (a.seq_len + 1) / 2;
    SHV_REQUIRE(static_cast<long long>(a.n_seq) * pairs <= 65535, "attn_decode: %d sequences of %d rows in one call", a.n_seq, a.seq_len);
    // three or four rows (a verification pass): the second pair's blocks write the first pair's cells too, no launch for them
    if (pairs == 2 && !ctx->attn_append_launch) return launch_rows<2>(ctx, a, 0, pairs, 2);
    SHV_LAUNCH(ctx, attn_append_kernel, dim3(a.n_head_kv, a.seq_len, a.n_seq), dim3(kBlock), 0, a);
    return launch_rows<2>(ctx, a, 0, pairs, 0);
}
