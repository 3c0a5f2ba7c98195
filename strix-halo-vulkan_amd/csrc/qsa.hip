// The block-sparse indexer beside a full-attention layer (llm/attn.go:221-443, 588-682; the
// reference's kernels are llm_attn_idx / score / select / selblk.comp): which cells of the cache
// each row of a pass may read.
//
//   project   float32 [heads*dim + dim][n_embd] rows against RMSNorm(x): four query heads and one key
//   keys      the raw key goes to a binary16 cache; every block of `ratio` cells the pass completes
//             is pooled (mean), normed, turned at its first cell's position and kept in a table;
//             a block that does not exist pools cell 0 (the reference's zero fill) and its key is
//             made again by every pass (it is what the unpooled tail of the sequence is scored by)
//   queries   per head: norm and rotation at the row's own position
//   scores    per (row, whole block): the sum over heads of the rectified dot products
//   select    per row: a cell's value is its block's score, plus 1e9 for the blocks at and after the
//             row's own incomplete block and for the unpooled tail; the (top_k + ratio - 1) largest
//             among the visible cells by a radix select (four 8-bit passes over an order-preserving
//             integer key), everything strictly above the threshold, then cells equal to it in
//             ascending index.  The result is a bit mask a row, which the attention kernels apply.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

constexpr int kProjTokens = 4;

// grid (ceil(rows/4), ceil(n_tok/kProjTokens)), 256 threads: a wave a row of w, kProjTokens rows of x
template <int H>
__global__ __launch_bounds__(256) void qsa_project_kernel(shv_qsa_index_args a, int rows) {
    __shared__ __align__(16) float xs[kProjTokens][H];
    __shared__ float red[kProjTokens][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.x * 4 + wave, t0 = blockIdx.y * kProjTokens, n_tok = a.n_seq * a.seq_len;
    const int nt = n_tok - t0 < kProjTokens ? n_tok - t0 : kProjTokens;
    float v[kProjTokens][H / 256], gm[H / 256];
#pragma unroll
    for (int i = 0; i < H / 256; i++) gm[i] = a.gamma[tid + i * 256];
#pragma unroll
    for (int g = 0; g < kProjTokens; g++)
#pragma unroll
        for (int i = 0; i < H / 256; i++) v[g][i] = g < nt ? a.x[static_cast<size_t>(t0 + g) * a.n_embd + tid + i * 256] : 0.f;
    float4 wr[H / 256];
    const float *w = a.w + static_cast<size_t>(row < rows ? row : 0) * H;
#pragma unroll
    for (int i = 0; i < H / 256; i++) wr[i] = *reinterpret_cast<const float4 *>(w + (i * 64 + lane) * 4);
#pragma unroll
    for (int g = 0; g < kProjTokens; g++) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < H / 256; i++) ss = fmaf(v[g][i], v[g][i], ss);
        ss = wave_sum_all(ss);
        if (lane == 0) red[g][wave] = ss;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < kProjTokens; g++) {
        const float scale = 1.f / sqrtf(((red[g][0] + red[g][1]) + (red[g][2] + red[g][3])) / static_cast<float>(H) + a.eps);
#pragma unroll
        for (int i = 0; i < H / 256; i++) xs[g][tid + i * 256] = v[g][i] * scale * gm[i];
    }
    __syncthreads();
    if (row >= rows) return;
    for (int g = 0; g < nt; g++) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < H / 256; i++) {
            const float4 xv = *reinterpret_cast<const float4 *>(&xs[g][(i * 64 + lane) * 4]);
            acc = fmaf(wr[i].x, xv.x, fmaf(wr[i].y, xv.y, fmaf(wr[i].z, xv.z, fmaf(wr[i].w, xv.w, acc))));
        }
        acc = wave_sum_all(acc);
        if (lane == 0) a.work[static_cast<size_t>(t0 + g) * rows + row] = acc;
    }
}

__device__ __forceinline__ float half_round(float v) { return __half2float(__float2half_rn(v)); }

// Sum over the block's idx_dim threads (idx_dim a multiple of 64, at most 256); red: 4 floats.
__device__ __forceinline__ float dim_sum(float v, float *red, int n_waves) {
    v = wave_sum_all(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.f;
    for (int w = 0; w < n_waves; w++) r += red[w];
    __syncthreads();
    return r;
}

// x (one value a thread, dim threads) -> RMS norm * gamma -> NeoX rotation of the first rope_dims
// dims with the table row of `position`; the result of this thread's dim.  buf: dim floats of LDS.
__device__ __forceinline__ float norm_rope_dim(float x, const float *gamma, const float *rope_row, int rope_dims, int dim, float eps,
                                               float *buf, float *red) {
    const int j = threadIdx.x;
    const float ss = dim_sum(x * x, red, dim / 64);
    const float y = x * (1.f / sqrtf(ss / static_cast<float>(dim) + eps)) * gamma[j];
    buf[j] = y;
    __syncthreads();
    const int half = rope_dims / 2;
    float out = y;
    if (j < half) {
        const float cs = rope_row[j], sn = rope_row[half + j];
        out = buf[j] * cs - buf[j + half] * sn;
    } else if (j < rope_dims) {
        const float cs = rope_row[j - half], sn = rope_row[j];
        out = buf[j - half] * sn + buf[j] * cs;
    }
    __syncthreads();
    return out;
}

// grid (seq_len + seq_len/ratio + 2, n_seq), idx_dim threads.  Blocks [0, seq_len): row i's raw key
// into the cache.  Blocks after them: one pooled block each that this pass may have completed, and
// the last one the key of the block that does not exist.
__global__ void qsa_keys_kernel(shv_qsa_index_args a, int rows) {
    __shared__ float buf[256];
    __shared__ float red[4];
    const int s = blockIdx.y, j = threadIdx.x, D = a.idx_dim, R = a.ratio;
    const int slot = a.slot ? a.slot[s] : s, past = a.pos ? a.pos[s] : 0;
    const int N = past + a.seq_len;
    const int key_col = a.idx_heads * D;
    uint16_t *cache = a.idxcache + static_cast<size_t>(slot) * a.max_cells * D;
    const int n_blocks_max = a.max_cells / R;
    float *pooled = a.pooled + static_cast<size_t>(slot) * (n_blocks_max + 1) * D;
    const float *work = a.work + static_cast<size_t>(s) * a.seq_len * rows;
    const int bx = blockIdx.x;
    if (bx < a.seq_len) {
        cache[static_cast<size_t>(past + bx) * D + j] = __half_as_ushort(__float2half_rn(work[static_cast<size_t>(bx) * rows + key_col + j]));
        return;
    }
    const int n_new = a.seq_len / R + 1;            // blocks a pass of seq_len rows can complete
    const bool dead = bx == a.seq_len + n_new;      // the block that does not exist
    const int b = past / R + (bx - a.seq_len);
    if (!dead && (b + 1) * R > N) return;           // not whole yet
    // cell values as the cache holds them: rows of this pass straight from the projection (rounded
    // as the cache rounds them; another block of this launch is writing them), older ones read back
    float sum = 0.f;
    for (int c = 0; c < R; c++) {
        const int cell = dead ? 0 : b * R + c;
        float v;
        if (cell >= past) v = half_round(work[static_cast<size_t>(cell - past) * rows + key_col + j]);
        else v = __half2float(__ushort_as_half(cache[static_cast<size_t>(cell) * D + j]));
        sum += v;
    }
    sum *= 1.f / static_cast<float>(R);
    const int position = dead ? 0 : b * R;          // a block's position is its first cell's
    const float out = norm_rope_dim(sum, a.k_norm, a.rope + static_cast<size_t>(position) * a.rope_dims, a.rope_dims, D, a.eps, buf, red);
    pooled[static_cast<size_t>(dead ? n_blocks_max : b) * D + j] = out;
}

// grid (idx_heads, seq_len, n_seq), idx_dim threads: the queries normed and turned in place
__global__ void qsa_query_kernel(shv_qsa_index_args a, int rows) {
    __shared__ float buf[256];
    __shared__ float red[4];
    const int h = blockIdx.x, i = blockIdx.y, s = blockIdx.z, j = threadIdx.x, D = a.idx_dim;
    const int past = a.pos ? a.pos[s] : 0;
    float *q = a.work + (static_cast<size_t>(s) * a.seq_len + i) * rows + h * D;
    const float out = norm_rope_dim(q[j], a.q_norm, a.rope + static_cast<size_t>(past + i) * a.rope_dims, a.rope_dims, D, a.eps, buf, red);
    q[j] = out;
}

// Whether any row of sequence s has more visible cells than the selection holds: otherwise every
// visible cell is selected and no score is needed.
__device__ __forceinline__ int qsa_width(const shv_qsa_index_args &a) {
    const int w = a.top_k + a.ratio - 1;
    return w < a.max_cells ? w : a.max_cells;
}

// grid (ceil((max_cells/ratio + 1)/256), seq_len, n_seq), 256 threads: thread = one pooled block
__global__ __launch_bounds__(256) void qsa_score_kernel(shv_qsa_index_args a, int rows) {
    extern __shared__ float qs[];  // [idx_heads][idx_dim]
    const int i = blockIdx.y, s = blockIdx.z, D = a.idx_dim, R = a.ratio;
    const int slot = a.slot ? a.slot[s] : s, past = a.pos ? a.pos[s] : 0;
    const int N = past + a.seq_len, n_bid = N / R, n_blocks_max = a.max_cells / R;
    if (N <= qsa_width(a)) return;
    const float *q = a.work + (static_cast<size_t>(s) * a.seq_len + i) * rows;
    for (int k = threadIdx.x; k < a.idx_heads * D; k += 256) qs[k] = q[k];
    __syncthreads();
    const int b = blockIdx.x * 256 + threadIdx.x;   // n_blocks_max is the block that does not exist
    if (b > n_blocks_max || (b >= n_bid && b < n_blocks_max)) return;
    const float *k = a.pooled + (static_cast<size_t>(slot) * (n_blocks_max + 1) + b) * D;
    float total = 0.f;
    for (int h = 0; h < a.idx_heads; h++) {
        float d = 0.f;
        for (int jj = 0; jj < D; jj += 4) {
            const float4 kv = *reinterpret_cast<const float4 *>(k + jj);
            const float *qq = qs + h * D + jj;
            d = fmaf(qq[0], kv.x, d);
            d = fmaf(qq[1], kv.y, d);
            d = fmaf(qq[2], kv.z, d);
            d = fmaf(qq[3], kv.w, d);
        }
        if (d > 0.f) total += d;
    }
    a.score[(static_cast<size_t>(s) * a.seq_len + i) * (n_blocks_max + 1) + b] = total;
}

__device__ __forceinline__ uint32_t f2ui(float v) {
    const uint32_t y = __float_as_uint(v);
    return (y & 0x80000000u) ? ~y : (y | 0x80000000u);
}

// grid (seq_len, n_seq), 1024 threads: one row's selection
constexpr int kSelThreads = 1024;
__global__ __launch_bounds__(kSelThreads) void qsa_select_kernel(shv_qsa_index_args a) {
    __shared__ uint32_t histo[256];
    __shared__ uint32_t s_prefix, s_desired;
    __shared__ int scan[kSelThreads];
    const int i = blockIdx.x, s = blockIdx.y, tid = threadIdx.x, R = a.ratio;
    const int past = a.pos ? a.pos[s] : 0;
    const int N = past + a.seq_len, p = past + i, vis = p + 1;
    const int n_bid = N / R, n_blocks_max = a.max_cells / R, width = qsa_width(a);
    uint32_t *mask = a.mask + (static_cast<size_t>(s) * a.seq_len + i) * a.mask_stride;
    const int wpt = (a.mask_stride + kSelThreads - 1) / kSelThreads;  // mask words a thread writes
    const int w0 = tid * wpt;
    if (vis <= width) {  // every visible cell
        for (int w = w0; w < w0 + wpt && w < a.mask_stride; w++) {
            const int c0 = w * 32;
            mask[w] = c0 + 32 <= vis ? 0xFFFFFFFFu : c0 >= vis ? 0u : ((1u << (vis - c0)) - 1u);
        }
        return;
    }
    const float *score = a.score + (static_cast<size_t>(s) * a.seq_len + i) * (n_blocks_max + 1);
    const int tail_start = (p + 1) / R * R;
    const float dead = score[n_blocks_max] + 1e9f;
    auto key_of = [&](int j) -> uint32_t {
        float v;
        if (j < n_bid * R) {
            const int b = j / R;
            v = score[b] + (b * R >= tail_start ? 1e9f : 0.f);
        } else {
            v = dead;
        }
        return f2ui(v);
    };
    // the threshold: four 8-bit passes, each over the keys that match the bits fixed so far
    if (tid == 0) { s_prefix = 0u; s_desired = static_cast<uint32_t>(width); }
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) histo[tid] = 0u;
        __syncthreads();
        const uint32_t hi_mask = shift + 8 < 32 ? 0xFFFFFFFFu << (shift + 8) : 0u;
        const uint32_t prefix_hi = s_prefix & hi_mask;
        for (int j = tid; j < vis; j += kSelThreads) {
            const uint32_t key = key_of(j);
            if ((key & hi_mask) == prefix_hi) atomicAdd(&histo[(key >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t acc = 0u, b = 0u;
            const uint32_t desired = s_desired;
            for (int bb = 255; bb >= 0; bb--) {
                const uint32_t c = histo[bb];
                if (acc + c >= desired) { b = static_cast<uint32_t>(bb); break; }
                acc += c;
            }
            s_prefix |= b << shift;
            s_desired = desired - acc;
        }
        __syncthreads();
    }
    const uint32_t thr = s_prefix;
    const int need = static_cast<int>(s_desired);  // cells equal to the threshold still to take, in index order
    // every thread owns a run of whole mask words; how many cells equal to the threshold lie before it
    int eq = 0;
    for (int w = w0; w < w0 + wpt && w < a.mask_stride; w++)
        for (int bit = 0; bit < 32; bit++) {
            const int j = w * 32 + bit;
            if (j < vis && key_of(j) == thr) eq++;
        }
    scan[tid] = eq;
    __syncthreads();
    for (int off = 1; off < kSelThreads; off <<= 1) {
        const int v = tid >= off ? scan[tid - off] : 0;
        __syncthreads();
        scan[tid] += v;
        __syncthreads();
    }
    int before = scan[tid] - eq;
    for (int w = w0; w < w0 + wpt && w < a.mask_stride; w++) {
        uint32_t bits = 0u;
        for (int bit = 0; bit < 32; bit++) {
            const int j = w * 32 + bit;
            if (j >= vis) break;
            const uint32_t key = key_of(j);
            if (key > thr) bits |= 1u << bit;
            else if (key == thr) {
                if (before < need) bits |= 1u << bit;
                before++;
            }
        }
        mask[w] = bits;
    }
}

}  // namespace

int shv_launch_qsa_index(shv_ctx *ctx, const shv_qsa_index_args *pa) {
    const shv_qsa_index_args &a = *pa;
    SHV_REQUIRE(a.x && a.gamma && a.w && a.q_norm && a.k_norm && a.rope && a.idxcache && a.pooled && a.work && a.score && a.mask,
                "qsa_index: NULL argument");
    SHV_REQUIRE(a.n_seq >= 1 && a.seq_len >= 1 && a.n_seq * a.seq_len <= 4096 && a.n_seq <= 65535, "qsa_index: %d sequences of %d rows", a.n_seq, a.seq_len);
    SHV_REQUIRE(a.n_embd == 2048, "qsa_index: n_embd = %d; built for 2048", a.n_embd);
    SHV_REQUIRE(a.idx_heads >= 1 && a.idx_heads <= 8 && a.idx_dim >= 64 && a.idx_dim <= 256 && a.idx_dim % 64 == 0,
                "qsa_index: %d heads of %d dims; 1..8 heads of 64, 128, 192 or 256", a.idx_heads, a.idx_dim);
    SHV_REQUIRE(a.ratio >= 1 && a.top_k >= 1 && a.max_cells >= a.ratio && a.max_cells % a.ratio == 0 && a.max_cells % 32 == 0,
                "qsa_index: ratio %d, top_k %d over %d cells (whole blocks, whole mask words)", a.ratio, a.top_k, a.max_cells);
    SHV_REQUIRE(a.rope_dims >= 0 && a.rope_dims <= a.idx_dim && a.rope_dims % 2 == 0, "qsa_index: %d of %d dims turn", a.rope_dims, a.idx_dim);
    SHV_REQUIRE(a.mask_stride >= a.max_cells / 32, "qsa_index: mask_stride %d words for %d cells", a.mask_stride, a.max_cells);
    SHV_REQUIRE(shv_aligned16(a.w) && shv_aligned16(a.pooled), "qsa_index: w and pooled must be 16-byte aligned");
    const int rows = a.idx_heads * a.idx_dim + a.idx_dim, n_tok = a.n_seq * a.seq_len;
    SHV_LAUNCH(ctx, qsa_project_kernel<2048>, dim3((rows + 3) / 4, (n_tok + kProjTokens - 1) / kProjTokens), dim3(256), 0, a, rows);
    SHV_LAUNCH(ctx, qsa_keys_kernel, dim3(a.seq_len + a.seq_len / a.ratio + 2, a.n_seq), dim3(a.idx_dim), 0, a, rows);
    SHV_LAUNCH(ctx, qsa_query_kernel, dim3(a.idx_heads, a.seq_len, a.n_seq), dim3(a.idx_dim), 0, a, rows);
    const int n_blocks_max = a.max_cells / a.ratio;
    SHV_LAUNCH(ctx, qsa_score_kernel, dim3((n_blocks_max + 1 + 255) / 256, a.seq_len, a.n_seq), dim3(256), static_cast<size_t>(a.idx_heads) * a.idx_dim * sizeof(float), a, rows);
    SHV_LAUNCH(ctx, qsa_select_kernel, dim3(a.seq_len, a.n_seq), dim3(kSelThreads), 0, a);
    return SHV_OK;
}
