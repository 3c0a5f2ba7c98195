// Format-level kernels: bit-exact Q4_K dequantisation and on-device synthetic fill.
#include <mutex>

#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

// One thread per 64-weight group: 32 payload bytes -> 64 floats, written as the reference's
// dequantQ4_K orders them (32 low nibbles, then 32 high nibbles).  d*sc and dmin*m are formed
// first and the product and difference are rounded separately, so the bits are the reference's.
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t *w, float *dst, long long n_groups) {
    const long long gid = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (gid >= n_groups) return;
    const long long blk = gid >> 2;
    const int g = static_cast<int>(gid & 3);
    const uint8_t *bp = w + blk * SHV_Q4K_BYTES;
    const uint4 hdr = *reinterpret_cast<const uint4 *>(bp);
    uint32_t sc, mn;
    q4k_group_scale_min(hdr, g, sc, mn);
    const float d = f16_bits_to_f32(hdr.x), dmin = f16_bits_to_f32(hdr.x >> 16);
    const float d1 = __fmul_rn(d, static_cast<float>(sc & 0xFFu)), m1 = __fmul_rn(dmin, static_cast<float>(mn & 0xFFu));
    const float d2 = __fmul_rn(d, static_cast<float>(sc >> 8)), m2 = __fmul_rn(dmin, static_cast<float>(mn >> 8));
    const uint4 q0 = *reinterpret_cast<const uint4 *>(bp + 16 + g * 32);
    const uint4 q1 = *reinterpret_cast<const uint4 *>(bp + 32 + g * 32);
    const uint32_t q[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    float *o = dst + blk * SHV_Q4K_BLOCK + g * 64;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t byte = (q[i] >> (8 * b)) & 0xFFu;
            o[4 * i + b] = __fsub_rn(__fmul_rn(d1, static_cast<float>(byte & 0xFu)), m1);
            o[32 + 4 * i + b] = __fsub_rn(__fmul_rn(d2, static_cast<float>(byte >> 4)), m2);
        }
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// dst[i] = mean + std * z_i, z_i from Box-Muller on the two halves of splitmix64(seed, i).
__global__ __launch_bounds__(256) void fill_normal_kernel(void *dstv, long long n, uint64_t seed, float mean, float std, int half) {
    float *dst = static_cast<float *>(dstv);
    uint16_t *dsth = static_cast<uint16_t *>(dstv);
    const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
    for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + static_cast<uint64_t>(i));
        const float u1 = (static_cast<float>(static_cast<uint32_t>(r >> 40)) + 1.0f) * (1.0f / 16777216.0f);
        const float u2 = static_cast<float>(static_cast<uint32_t>(r) >> 8) * (1.0f / 16777216.0f);
        const float rad = sqrtf(-2.0f * logf(u1));
        const float v = mean + std * rad * cosf(6.28318530717958647692f * u2);
        if (half) dsth[i] = __half_as_ushort(__float2half_rn(v)); else dst[i] = v;
    }
}

}  // namespace

int shv_launch_dequant_q4k(shv_ctx *ctx, const shv_dequant_q4k_args *a) {
    SHV_REQUIRE(a->w && a->dst, "dequant_q4k: NULL w or dst");
    SHV_REQUIRE(a->rows > 0 && a->k > 0 && a->k % SHV_Q4K_BLOCK == 0, "dequant_q4k: rows %lld, k %d", static_cast<long long>(a->rows), a->k);
    SHV_REQUIRE(shv_aligned16(a->w), "dequant_q4k: w must be 16-byte aligned");
    const long long groups = a->rows * (a->k / 64);
    const long long blocks = (groups + 255) / 256;
    SHV_REQUIRE(blocks < (1ll << 31), "dequant_q4k: %lld groups is too many for one launch", groups);
    SHV_LAUNCH(ctx, dequant_q4k_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<const uint8_t *>(a->w), a->dst, groups);
    return SHV_OK;
}

int shv_launch_fill_normal(shv_ctx *ctx, const shv_fill_normal_args *a) {
    SHV_REQUIRE(a->dst && a->n > 0, "fill_normal: NULL dst or n = %lld", static_cast<long long>(a->n));
    long long blocks = (a->n + 255) / 256;
    const long long cap = static_cast<long long>(ctx->prop.multiProcessorCount) * 32;
    if (blocks > cap) blocks = cap;
    SHV_LAUNCH(ctx, fill_normal_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, a->dst,
                       static_cast<long long>(a->n), a->seed, a->mean, a->std, a->half);
    return SHV_OK;
}

// ---- token-loop glue: embedding gather, greedy arg-max, position advance ------------------------

namespace {

__global__ __launch_bounds__(256) void embed_kernel(shv_embed_args a) {
    const int t = blockIdx.y;
    const int id = a.ids[(a.pos ? a.pos[0] : 0) + t];
    const bool ok = id >= 0 && id < a.vocab;
    const uint16_t *row = static_cast<const uint16_t *>(a.table) + static_cast<size_t>(ok ? id : 0) * a.n_embd;
    float *x = a.x + static_cast<size_t>(t) * a.x_stride;
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < a.n_embd; c += gridDim.x * blockDim.x)
        x[c] = ok ? __half2float(__ushort_as_half(row[c])) : __int_as_float(0x7fc00000);
}

// (value, index) ordered so that the larger value wins and, between equal values, the lower index.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__device__ __forceinline__ void wave_best(float &v, int &i) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(i, off, 64);
        if (better(ov, oi, v, i)) { v = ov; i = oi; }
    }
}

// grid: (blocks, n_rows).  Each block scans a contiguous chunk of one row; the last block of the
// row to arrive reduces the per-block winners.
__global__ __launch_bounds__(256) void argmax_kernel(shv_argmax_args a, float *pval, int32_t *pidx, int32_t *counters) {
    __shared__ float sv[4];
    __shared__ int si[4];
    __shared__ int is_last;
    const int r = blockIdx.y, nb = gridDim.x;
    const float *lg = a.logits + static_cast<size_t>(r) * a.logits_stride;
    const int chunk = (a.n + nb - 1) / nb;
    const int lo = blockIdx.x * chunk, hi = lo + chunk < a.n ? lo + chunk : a.n;
    // "no candidate" is (-inf, n): any real element beats it, including -inf at a lower index
    float bv = -INFINITY;
    int bi = a.n;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const float v = lg[i];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    wave_best(bv, bi);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++)
            if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        shv::store_agent(pval + r * nb + blockIdx.x, bv);
        shv::store_agent(pidx + r * nb + blockIdx.x, bi);
    }
    if (!shv::arrive_last(counters + r, nb, &is_last)) return;
    bv = -INFINITY;
    bi = a.n;
    for (int b = threadIdx.x; b < nb; b += blockDim.x) {
        const float v = shv::load_agent(pval + r * nb + b);
        const int i = shv::load_agent(pidx + r * nb + b);
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    wave_best(bv, bi);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++)
            if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        // a row of NaN (or -inf only at the top) has no element that is `>` -inf: the reference
        // returns 0 there
        if (bi >= a.n) bi = 0;
        a.best[r] = bi;
        if (a.ids && a.pos) {
            const int p = a.pos[0] + (a.advance > 0 ? a.advance : 1);
            a.ids[p] = bi;
            a.pos[0] = p;
        }
    }
}

__global__ void advance_kernel(shv_advance_args a) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s < a.n_seq) a.pos[s] += a.delta;
}

// grid: (column chunks of 1024 floats, count); one block a piece of a row
__global__ __launch_bounds__(256) void ring_rows_kernel(shv_ring_rows_args a) {
    const int p = (a.pos ? a.pos[0] : 0) + a.first + static_cast<int>(blockIdx.y);
    if (p < 0) return;
    const float *src = a.src + static_cast<size_t>(p % a.src_slots) * a.stride;
    float *dst = a.dst + static_cast<size_t>(p % a.dst_slots) * a.stride;
    const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c + 4 <= a.n) *reinterpret_cast<float4 *>(dst + c) = *reinterpret_cast<const float4 *>(src + c);
    else for (int i = c; i < a.n; i++) dst[i] = src[i];
}

// ---- the arg-max that allocates nothing ------------------------------------------------------
// Its per-block winners and arrival counters live in this array instead of in memory the context
// allocated: kArgmaxBlocks values, kArgmaxBlocks indices, then kStaticCounters arrival counters.
// Every GPU holds its own copy until the process ends; in host code the name is only a handle, the
// device address comes from hipGetSymbolAddress (shv_static_scratch_bind, once per device).
constexpr int kStaticCounters = 16;
constexpr size_t kStaticScratchBytes = shv_ctx::kArgmaxBlocks * (sizeof(float) + sizeof(int32_t)) + kStaticCounters * sizeof(int32_t);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;  // shv_init may run on several threads at once

__global__ void clear_counters_kernel(int32_t *c, int n) {
    if (static_cast<int>(threadIdx.x) < n) c[threadIdx.x] = 0;
}

}  // namespace

int shv_launch_ring_rows(shv_ctx *ctx, const shv_ring_rows_args *pa) {
    const shv_ring_rows_args &a = *pa;
    SHV_REQUIRE(a.src && a.dst, "ring_rows: NULL argument");
    SHV_REQUIRE(a.src_slots >= 1 && a.dst_slots >= 1 && a.n >= 1 && a.stride >= a.n && a.count >= 1 && a.count <= 65535,
                "ring_rows: %d rows of %d floats between rings of %d and %d slots", a.count, a.n, a.src_slots, a.dst_slots);
    SHV_REQUIRE(shv_aligned16(a.src) && shv_aligned16(a.dst) && a.stride % 4 == 0, "ring_rows: rings must be 16-byte aligned, rows a multiple of 4 floats apart");
    SHV_LAUNCH(ctx, ring_rows_kernel, dim3((a.n + 1023) / 1024, a.count), dim3(256), 0, a);
    return SHV_OK;
}

int shv_static_scratch_bind(shv_ctx *ctx) {
    SHV_REQUIRE(ctx->device >= 0 && ctx->device < kMaxDevices, "shv_init: device %d; the static scratch table covers %d devices", ctx->device, kMaxDevices);
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (!g_scratch_ptr[ctx->device]) {
        void *p = nullptr;
        SHV_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));  // the calling thread's current device is ctx->device
        g_scratch_ptr[ctx->device] = p;
    }
    ctx->static_scratch = g_scratch_ptr[ctx->device];
    return SHV_OK;
}

int shv_launch_embed(shv_ctx *ctx, const shv_embed_args *a) {
    SHV_REQUIRE(a->table && a->ids && a->x, "embed: NULL argument");
    SHV_REQUIRE(a->n_tok >= 1 && a->n_tok <= 65535 && a->n_embd >= 1 && a->vocab >= 1 && a->x_stride >= a->n_embd,
                "embed: n_tok %d, n_embd %d, vocab %d, x_stride %d", a->n_tok, a->n_embd, a->vocab, a->x_stride);
    if (a->type != SHV_GGML_F16) return shv_launch_embed_typed(ctx, a);
    const int bx = (a->n_embd + 255) / 256;
    SHV_LAUNCH(ctx, embed_kernel, dim3(bx < 8 ? bx : 8, a->n_tok), dim3(256), 0, *a);
    return SHV_OK;
}

static int argmax_blocks(const shv_argmax_args *a) {
    int nb = (a->n + 1023) / 1024;
    const int cap = shv_ctx::kArgmaxBlocks / a->n_rows;
    if (nb > cap) nb = cap;
    return nb > 256 ? 256 : nb;
}

int shv_launch_argmax(shv_ctx *ctx, const shv_argmax_args *a) {
    SHV_REQUIRE(a->logits && a->best, "argmax: NULL logits or best");
    SHV_REQUIRE(a->n_rows >= 1 && a->n >= 1 && a->logits_stride >= a->n, "argmax: %d rows of %d, stride %d", a->n_rows, a->n, a->logits_stride);
    SHV_REQUIRE((a->ids == nullptr) == (a->pos == nullptr), "argmax: ids and pos go together");
    SHV_REQUIRE(!a->ids || a->n_rows == 1, "argmax: storing the next token needs exactly one row");
    SHV_REQUIRE(a->advance >= 0, "argmax: advance %d", a->advance);
    SHV_REQUIRE(a->n_rows <= 14, "argmax: %d rows is more than one launch covers", a->n_rows);
    SHV_LAUNCH(ctx, argmax_kernel, dim3(argmax_blocks(a), a->n_rows), dim3(256), 0, *a, ctx->argmax_val, ctx->argmax_idx,
                       ctx->counters + shv_ctx::kCounterArgmax);
    return SHV_OK;
}

int shv_launch_argmax_static(shv_ctx *ctx, const shv_argmax_args *a) {
    SHV_REQUIRE(a->logits && a->best, "argmax_static: NULL logits or best");
    SHV_REQUIRE(a->n_rows >= 1 && a->n >= 1 && a->logits_stride >= a->n, "argmax_static: %d rows of %d, stride %d", a->n_rows, a->n, a->logits_stride);
    SHV_REQUIRE(a->n_rows <= SHV_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows; the static scratch holds the partial results of at most %d rows a call",
                a->n_rows, SHV_ARGMAX_STATIC_MAX_ROWS);
    SHV_REQUIRE((a->ids == nullptr) == (a->pos == nullptr), "argmax_static: ids and pos go together");
    SHV_REQUIRE(!a->ids || a->n_rows == 1, "argmax_static: storing the next token needs exactly one row");
    SHV_REQUIRE(a->advance >= 0, "argmax_static: advance %d", a->advance);
    SHV_REQUIRE(ctx->static_scratch, "argmax_static: the static scratch of device %d was not bound at shv_init", ctx->device);
    float *pval = static_cast<float *>(ctx->static_scratch);
    int32_t *pidx = reinterpret_cast<int32_t *>(pval + shv_ctx::kArgmaxBlocks);
    int32_t *counters = pidx + shv_ctx::kArgmaxBlocks;
    // the array keeps what the last call left: the arrival counters must start at zero (a fill
    // kernel, not a memset node, so that a caller may record this call into a graph)
    SHV_LAUNCH(ctx, clear_counters_kernel, dim3(1), dim3(64), 0, counters, kStaticCounters);
    SHV_LAUNCH(ctx, argmax_kernel, dim3(argmax_blocks(a), a->n_rows), dim3(256), 0, *a, pval, pidx, counters);
    return SHV_OK;
}

int shv_launch_advance(shv_ctx *ctx, const shv_advance_args *a) {
    SHV_REQUIRE(a->pos && a->n_seq >= 1, "advance: NULL pos or n_seq %d", a->n_seq);
    SHV_LAUNCH(ctx, advance_kernel, dim3((a->n_seq + 63) / 64), dim3(64), 0, *a);
    return SHV_OK;
}
