// Q4_K projections of two to eight activation rows (a verification pass, a few sequences decoded
// together): y[t] = W pro(x[t]) (+ residual[t]) with the weights formed once for all rows.
//
// The row kernels of gemv_q4k.hip pay their ~2.6 vector operations a weight once per activation
// row.  Here a weight is turned into a binary16 operand once (~2 operations) and the matrix cores
// multiply it with every row at no further vector cost:
//   v_mfma_f32_16x16x32_f16   A = 16 weight rows x 32 columns, B = 32 columns x 16, of which
//                             column 2t holds the high part of row t's activations (cut to eleven
//                             bits) and 2t+1 the remainder, so y[t] = C[.][2t] + C[.][2t+1]; a wave
//                             first scales its part of a row by a power of two that brings the
//                             largest magnitude to [512, 1024), so that the parts are normal numbers
//   a weight as an operand    n * sc, a whole number below 946 and exact in binary16: the nibble is
//                             masked into the mantissa of 1024.0 (low nibbles) or 64.0 (high
//                             nibbles) and one packed fma takes off 1024 * sc or 64 * sc again;
//                             one accumulator a super-block, scaled by the row's d afterwards
//   the min term              -dmin * m * sum(x over the sub-block): one v_mfma_f32_16x16x16_f16 a
//                             super-block, the sub-blocks' mins (whole numbers) against their sums
//                             of x as halves, scaled by the row's dmin afterwards
// A block is 16 weight rows and four waves; a wave takes a quarter of the columns (its own
// super-blocks of each row), stages only that quarter of the activation rows, in operand order,
// and the four partial tiles meet in LDS.  Nothing is re-read: a lane's 16 payload bytes of a
// row feed four products.
#include "shv_device.hpp"
#include "shv_internal.hpp"

namespace {

using namespace shv;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// x -> a high part that binary16 holds exactly (x cut to eleven significant bits: one mask) and the exact remainder.
// For the rows this kernel stages, scaled so that their largest magnitude is in [512, 1024), a remainder too small
// for a normal binary16 belongs to an entry below 0.125, and what is lost of it is below 2^-33 of the largest.
__device__ __forceinline__ void split_cut(float x, float &hi, float &lo) {
    hi = __uint_as_float(__float_as_uint(x) & 0xFFFFE000u);
    lo = x - hi;
}
// two floats to one dword of two halves, rounded toward zero (exact for split_cut's high parts)
__device__ __forceinline__ uint32_t pack_halves(float a, float b) { return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b)); }

// the largest of a wave's values, none of them negative, in every lane
__device__ __forceinline__ float wave_max_nonneg(float v) {
    v = fmaxf(v, dpp_f32<kDppXor1>(v));
    v = fmaxf(v, dpp_f32<kDppXor2>(v));
    v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f32<kDppMirror>(v));
    v = fmaxf(v, dpp_f32<kDppBcast15, 0xA>(v));  // rows the mask leaves out read 0
    v = fmaxf(v, dpp_f32<kDppBcast31, 0xC>(v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Eight weights of two payload dwords (bytes 0..7 of the lane's 16 or bytes 8..15) as n * sc:
// HI false: the low nibbles, HI true: the high nibbles.  sc2 = (sc, sc), off2 = -(1024 or 64) * sc.
template <bool HI>
__device__ __forceinline__ half8_t weights8(uint32_t d0, uint32_t d1, half2_t sc2, half2_t off2) {
    constexpr uint32_t mask = HI ? 0x00F000F0u : 0x000F000Fu, one = HI ? 0x54005400u : 0x64006400u;
    const half2_t a0 = __builtin_elementwise_fma(as_half2((d0 & mask) | one), sc2, off2);         // bytes 0, 2
    const half2_t a1 = __builtin_elementwise_fma(as_half2(((d0 >> 8) & mask) | one), sc2, off2);  // bytes 1, 3
    const half2_t a2 = __builtin_elementwise_fma(as_half2((d1 & mask) | one), sc2, off2);         // bytes 4, 6
    const half2_t a3 = __builtin_elementwise_fma(as_half2(((d1 >> 8) & mask) | one), sc2, off2);  // bytes 5, 7
    half8_t r;
    r[0] = a0[0]; r[1] = a0[1]; r[2] = a1[0]; r[3] = a1[1];
    r[4] = a2[0]; r[5] = a2[1]; r[6] = a3[0]; r[7] = a3[1];
    return r;
}

// the largest of the values, none negative, of the lane's half of the wave (lanes 0..31, 32..63), in every lane of the half
__device__ __forceinline__ float half_max_nonneg(float v, int lane) {
    v = fmaxf(v, dpp_f32<kDppXor1>(v));
    v = fmaxf(v, dpp_f32<kDppXor2>(v));
    v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f32<kDppMirror>(v));
    v = fmaxf(v, dpp_f32<kDppBcast15, 0xA>(v));
    const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 31)), hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    return lane < 32 ? lo : hi;
}
__device__ __forceinline__ float half_sum(float v, int lane) {
    v = group_sum<32>(v);
    const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 31)), hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    return lane < 32 ? lo : hi;
}

// K columns, NT activation rows, prologue PRO, W waves a block.  grid: n / (16 TILES) blocks of 64 W threads.
// Fragment f of a wave's part (KW = K/W columns, NF = KW/8 fragments) is eight consecutive
// columns: f = ((s * 2 + L) * 4 + m) * 4 + jj  with s the super-block within the part, L the
// half of the super-block (64-weight groups 2L, 2L+1), m the product within a lane's 16 payload
// bytes (0, 1: low nibbles of bytes 0..7 / 8..15; 2, 3: the high nibbles) and jj the operand's
// column group (lane / 16): columns  256 s' + 64 (2L + jj/2) + 32 (m/2) + 16 (jj%2) + 8 (m%2) ..+7.
// What a block pays per activation row is the staging, which every block repeats: W says over how many waves a row's
// columns are spread.  Four waves suit two to four rows; with sixteen waves over 4096 columns (eight over 2048) a wave
// stages one super-block of each row, 32 fragments, and two rows share the wave's lanes; the launcher says where that pays.
template <int K, int PRO, int NT, int TILES, int W>
__global__ __launch_bounds__(64 * W) void gemv_mrows_kernel(shv_gemv_q4k_args a) {
    constexpr int KW = K / W, NSB = KW / 256, NF = KW / 8, NC = 2 * NT, FS = NC | 1;
    constexpr bool HALF = NF < 64;                 // two activation rows side by side in a wave's lanes
    constexpr int FPL = HALF ? 1 : NF / 64;        // fragments of one row a lane stages
    constexpr int PPL = HALF ? (NT + 1) / 2 : NT * FPL;  // (row, fragment) pairs a lane stages
    constexpr int ROWB = K / SHV_Q4K_BLOCK * SHV_Q4K_BYTES;
    static_assert(NSB >= 1 && (NF == 32 || NF % 64 == 0) && NT >= 2 && NT <= 8, "shape");
    extern __shared__ __align__(16) char smem[];
    // a fragment's columns lie FS entries of 16 bytes apart, an odd number: sixteen lanes that store one column of
    // sixteen consecutive fragments then hit sixteen different groups of four banks
    half8_t *bf_all = reinterpret_cast<half8_t *>(smem);                                  // [W waves][NF][FS]
    half4_t *sf_all = reinterpret_cast<half4_t *>(smem + sizeof(half8_t) * W * NF * FS);  // [W waves][NSB][4][NC]
    float *red = reinterpret_cast<float *>(smem + sizeof(half8_t) * W * NF * FS + sizeof(half4_t) * W * NSB * 4 * NC);  // [NT][W]
    float *uns = red + NT * W;                                                            // [W][NT]
    // the waves' partial tiles: behind everything with four waves, over the operands (read to their end by then) with
    // more, where they fit there
    constexpr bool ALIAS = W != 4 && sizeof(half8_t) * W * NF * FS >= sizeof(float) * TILES * W * 64 * 4;
    float *cpart = ALIAS ? reinterpret_cast<float *>(smem) : uns + W * NT;                // [TILES][W][64][4]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, j = lane >> 4;
    half8_t *bf = bf_all + wave * NF * FS;
    half4_t *sf = sf_all + wave * NSB * 4 * NC;

    // where each activation row goes (ring output) or comes from (the gate's ring): asked for first
    const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
    int ring_row[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        ring_row[t] = 0;
        if (a.ring_slots > 0) {
            const int s = t / sl, i = t % sl;
            const int p = a.pos ? a.pos[s] : 0;
            const int slot = a.slot ? a.slot[s] : s;
            ring_row[t] = slot * a.ring_slots + (p + i) % a.ring_slots;
        }
    }
    // ---- the wave's part of every activation row: pair u of a lane is (row pt[u], fragment pf[u]) ----
    float4 xv[PPL][2], zv[PPL][2], gv[PPL][2];
    int pt[PPL], pf[PPL];
    bool pv[PPL];
#pragma unroll
    for (int u = 0; u < PPL; u++) {
        const int t_raw = HALF ? 2 * u + (lane >> 5) : u / FPL;
        pv[u] = t_raw < NT;
        pt[u] = pv[u] ? t_raw : NT - 1;
        pf[u] = HALF ? (lane & 31) : lane + 64 * (u % FPL);
        const int f = pf[u], t = pt[u];
        const int jj = f & 3, m = (f >> 2) & 3, L = (f >> 4) & 1, s = f >> 5;
        const int c = wave * KW + 256 * s + 64 * (2 * L + (jj >> 1)) + 32 * (m >> 1) + 16 * (jj & 1) + 8 * (m & 1);
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            gv[u][0] = *reinterpret_cast<const float4 *>(a.gamma + c);
            gv[u][1] = *reinterpret_cast<const float4 *>(a.gamma + c + 4);
        } else if constexpr (PRO == SHV_PRO_GATED_NORM) {
            gv[u][0] = *reinterpret_cast<const float4 *>(a.gamma + (c & (a.head_dim - 1)));
            gv[u][1] = *reinterpret_cast<const float4 *>(a.gamma + (c & (a.head_dim - 1)) + 4);
        }
        const float *x = a.x + static_cast<size_t>(t) * a.x_stride + c;
        xv[u][0] = *reinterpret_cast<const float4 *>(x);
        xv[u][1] = *reinterpret_cast<const float4 *>(x + 4);
        if constexpr (PRO == SHV_PRO_GATED_NORM) {
            // the lane's row of the ring, picked without indexing the register array by a variable
            int rr = 0;
#pragma unroll
            for (int tt = 0; tt < NT; tt++) rr = tt == t ? ring_row[tt] : rr;
            const float *z = a.z_ring ? a.z + static_cast<size_t>(rr) * a.ring_stride : a.z + static_cast<size_t>(t) * a.z_stride;
            zv[u][0] = *reinterpret_cast<const float4 *>(z + c);
            zv[u][1] = *reinterpret_cast<const float4 *>(z + c + 4);
        } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
            const HeadSplit hs(a.head_dim > 0 ? a.head_dim : 1);
            const int zi = a.head_dim > 0 ? hs.head(c) * 2 * a.head_dim + a.head_dim + hs.dim(c) : c;
            const float *z = a.z + static_cast<size_t>(t) * a.z_stride + zi;
            zv[u][0] = *reinterpret_cast<const float4 *>(z);
            zv[u][1] = *reinterpret_cast<const float4 *>(z + 4);
        }
    }
    // ---- the wave's weights, of every tile of the block: per super-block the row's header and this lane's 2 x 16
    // payload bytes ----
    uint4 hdr[TILES][NSB], pl[TILES][NSB][2];
#pragma unroll
    for (int ti = 0; ti < TILES; ti++) {
        const int row = (static_cast<int>(blockIdx.x) * TILES + ti) * 16 + r;
        const char *wrow = static_cast<const char *>(a.w) + static_cast<size_t>(row < a.n ? row : 0) * ROWB + static_cast<size_t>(wave) * NSB * SHV_Q4K_BYTES;
#pragma unroll
        for (int s = 0; s < NSB; s++) {
            const char *sb = wrow + s * SHV_Q4K_BYTES;
            hdr[ti][s] = load_stream16(sb);
#pragma unroll
            for (int L = 0; L < 2; L++) pl[ti][s][L] = load_stream16(sb + 16 + (2 * L + (j >> 1)) * 32 + (j & 1) * 16);
        }
    }
    // the residual of the values this thread stores at the end: thread = (row tid % 16, activation row tid / 16) of each tile
    const int out_r = tid & 15, out_t = tid >> 4;
    float res[TILES];
#pragma unroll
    for (int ti = 0; ti < TILES; ti++) {
        const int out_row = (static_cast<int>(blockIdx.x) * TILES + ti) * 16 + out_r;
        res[ti] = (a.residual && out_t < NT && out_row < a.n) ? a.residual[static_cast<size_t>(out_t) * a.y_stride + out_row] : 0.f;
    }

    // ---- stage: prologue, a power of two that brings the wave's part of the row into binary16's range, operand
    // order, the sub-blocks' sums ----
    float v[PPL][8], ssq[PPL], mxp[PPL];
#pragma unroll
    for (int u = 0; u < PPL; u++) {
        const float x8[8] = {xv[u][0].x, xv[u][0].y, xv[u][0].z, xv[u][0].w, xv[u][1].x, xv[u][1].y, xv[u][1].z, xv[u][1].w};
#pragma unroll
        for (int i = 0; i < 8; i++) v[u][i] = x8[i];
        ssq[u] = 0.f;
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            const float g[8] = {gv[u][0].x, gv[u][0].y, gv[u][0].z, gv[u][0].w, gv[u][1].x, gv[u][1].y, gv[u][1].z, gv[u][1].w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                ssq[u] = fmaf(v[u][i], v[u][i], ssq[u]);
                v[u][i] *= g[i];
            }
        } else if constexpr (PRO == SHV_PRO_GATED_NORM) {
            // a head of 128 columns is sixteen consecutive fragments: the sixteen lanes of a row of the wave
            const float g[8] = {gv[u][0].x, gv[u][0].y, gv[u][0].z, gv[u][0].w, gv[u][1].x, gv[u][1].y, gv[u][1].z, gv[u][1].w};
            const float z[8] = {zv[u][0].x, zv[u][0].y, zv[u][0].z, zv[u][0].w, zv[u][1].x, zv[u][1].y, zv[u][1].z, zv[u][1].w};
            float hs = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) hs = fmaf(v[u][i], v[u][i], hs);
            hs = group_sum<16>(hs);
            const float sc = __builtin_amdgcn_rsqf(hs / 128.f + a.eps);
#pragma unroll
            for (int i = 0; i < 8; i++) v[u][i] = v[u][i] * sc * g[i] * sigmoid_fast(z[i]);
        } else if constexpr (PRO == SHV_PRO_MUL_SIGMOID) {
            const float z[8] = {zv[u][0].x, zv[u][0].y, zv[u][0].z, zv[u][0].w, zv[u][1].x, zv[u][1].y, zv[u][1].z, zv[u][1].w};
#pragma unroll
            for (int i = 0; i < 8; i++) v[u][i] *= sigmoid_fast(z[i]);
        }
        mxp[u] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) mxp[u] = fmaxf(mxp[u], fabsf(v[u][i]));
    }
    // per activation row: the largest magnitude of the wave's part goes to [512, 1024): a sub-block's sum stays below
    // binary16's limit, and what is smaller than the largest by 2^-23 and more loses bits that the sum would not show
    float up[PPL];
#pragma unroll
    for (int g0 = 0; g0 < PPL; g0 += FPL) {
        // the pairs g0 .. g0 + FPL - 1 are one row's (of each half of the wave, when two rows share it)
        float mx = 0.f, ss = 0.f;
#pragma unroll
        for (int u = g0; u < g0 + FPL; u++) {
            mx = fmaxf(mx, mxp[u]);
            ss += ssq[u];
        }
        mx = HALF ? half_max_nonneg(mx, lane) : wave_max_nonneg(mx);
        int ex = static_cast<int>((__float_as_uint(mx) >> 23) & 0xFFu);
        ex = ex < 9 ? 9 : ex > 254 ? 254 : ex;
        const float upv = __uint_as_float(static_cast<uint32_t>(263 - ex) << 23);      // 2^(136 - ex)
        const float unscale = __uint_as_float(static_cast<uint32_t>(ex - 9) << 23);    // its inverse (0 below 2^-118)
#pragma unroll
        for (int u = g0; u < g0 + FPL; u++) up[u] = upv;
        const bool writer = (lane & (HALF ? 31 : 63)) == 0 && pv[g0];
        if (writer) uns[wave * NT + pt[g0]] = unscale;
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            ss = HALF ? half_sum(ss, lane) : wave_sum_all(ss);
            if (writer) red[pt[g0] * W + wave] = ss;
        }
    }
#pragma unroll
    for (int u = 0; u < PPL; u++) {
        const int f = pf[u], t = pt[u];
        float h8[8], l8[8], s8 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float vs = v[u][i] * up[u];
            split_cut(vs, h8[i], l8[i]);
            s8 += vs;
        }
        // operand order within a fragment: the order a payload dword's nibbles come out of the masks (bytes 0, 2, 1, 3)
        const uint4 hw = make_uint4(pack_halves(h8[0], h8[2]), pack_halves(h8[1], h8[3]), pack_halves(h8[4], h8[6]), pack_halves(h8[5], h8[7]));
        const uint4 lw = make_uint4(pack_halves(l8[0], l8[2]), pack_halves(l8[1], l8[3]), pack_halves(l8[4], l8[6]), pack_halves(l8[5], l8[7]));
        const half8_t hi = __builtin_bit_cast(half8_t, hw), lo = __builtin_bit_cast(half8_t, lw);
        // the sub-block's 32 columns are the fragments f, f ^ 1 (jj % 2) and f ^ 4, f ^ 5 (m % 2): lanes of one half
        float s32 = s8 + dpp_f32<kDppXor1>(s8);
        s32 += __shfl_xor(s32, 4, 64);
        if (pv[u]) {
            bf[f * FS + 2 * t] = hi;
            bf[f * FS + 2 * t + 1] = lo;
            if ((f & 5) == 0) {
                const int jj = f & 3, m = (f >> 2) & 3, L = (f >> 4) & 1, s = f >> 5;
                const int grp = 2 * L + (jj >> 1), odd = m >> 1;  // sub-block 2 grp + odd of the super-block
                float sh, sl;
                split_cut(s32, sh, sl);
                // operand (column group grp, column 2t / 2t+1), halves (sub 2 grp, 0, sub 2 grp + 1, 0)
                uint32_t *dst_hi = reinterpret_cast<uint32_t *>(&sf[(s * 4 + grp) * NC + 2 * t]) + odd;
                uint32_t *dst_lo = reinterpret_cast<uint32_t *>(&sf[(s * 4 + grp) * NC + 2 * t + 1]) + odd;
                *dst_hi = pack_halves(sh, 0.f);
                *dst_lo = pack_halves(sl, 0.f);
            }
        }
    }
    __builtin_amdgcn_wave_barrier();  // a wave reads back only what it staged itself; its LDS operations complete in order

    // ---- products ----
    const int bc = r < NC ? r : NC - 1;  // columns past the rows' hold whatever: their results are never read
    // a lane's column: activation row r / 2 (its high parts in the even column, the remainders in the odd one)
    const float back = (r >> 1) < NT ? uns[wave * NT + (r >> 1)] : 0.f;
    float4_t ytile[TILES];
#pragma unroll
    for (int ti = 0; ti < TILES; ti++) {
    float4_t yacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NSB; s++) {
        float4_t cacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int L = 0; L < 2; L++) {
            uint32_t sc, mn;
            q4k_group_scale_min(hdr[ti][s], 2 * L + (j >> 1), sc, mn);
            const _Float16 sc_lo = static_cast<_Float16>(static_cast<float>(sc & 0xFFu)), sc_hi = static_cast<_Float16>(static_cast<float>(sc >> 8));
            half2_t s2lo, s2hi, o2lo, o2hi;
            s2lo[0] = sc_lo; s2lo[1] = sc_lo;
            s2hi[0] = sc_hi; s2hi[1] = sc_hi;
            const _Float16 olo = static_cast<_Float16>(-1024.f * static_cast<float>(sc & 0xFFu)), ohi = static_cast<_Float16>(-64.f * static_cast<float>(sc >> 8));
            o2lo[0] = olo; o2lo[1] = olo;
            o2hi[0] = ohi; o2hi[1] = ohi;
            const uint4 q = pl[ti][s][L];
            const half8_t *b = bf + ((s * 2 + L) * 16 + j) * FS + bc;  // product m: + 4 m FS
            cacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(weights8<false>(q.x, q.y, s2lo, o2lo), b[0 * 4 * FS], cacc, 0, 0, 0);
            cacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(weights8<false>(q.z, q.w, s2lo, o2lo), b[1 * 4 * FS], cacc, 0, 0, 0);
            cacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(weights8<true>(q.x, q.y, s2hi, o2hi), b[2 * 4 * FS], cacc, 0, 0, 0);
            cacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(weights8<true>(q.z, q.w, s2hi, o2hi), b[3 * 4 * FS], cacc, 0, 0, 0);
        }
        // the min term: this lane holds (row r, sub-blocks 2j and 2j+1 of the super-block); the mins are whole
        // numbers below 64, the sums come as halves in the columns the activations use
        float4_t cmin = {0.f, 0.f, 0.f, 0.f};
        {
            uint32_t sc, mn;
            q4k_group_scale_min(hdr[ti][s], j, sc, mn);
            half4_t am;
            am[0] = static_cast<_Float16>(static_cast<float>(mn & 0xFFu));
            am[1] = static_cast<_Float16>(0.f);
            am[2] = static_cast<_Float16>(static_cast<float>(mn >> 8));
            am[3] = static_cast<_Float16>(0.f);
            cmin = __builtin_amdgcn_mfma_f32_16x16x16f16(am, sf[(s * 4 + j) * NC + bc], cmin, 0, 0, 0);
        }
        // y += d * (the super-block's products) - dmin * (its mins' products): the tile's rows 4 j + i are the rows
        // whose headers the lanes 4 j + i hold
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t dd = static_cast<uint32_t>(__shfl(static_cast<int>(hdr[ti][s].x), 4 * j + i, 64));
            yacc[i] = fmaf(f16_bits_to_f32(dd), cacc[i], yacc[i]);
            yacc[i] = fmaf(-f16_bits_to_f32(dd >> 16), cmin[i], yacc[i]);
        }
    }
    ytile[ti] = yacc * back;
    }
    if constexpr (ALIAS) __syncthreads();  // every wave has read its operands to the end: the partial tiles take their place
#pragma unroll
    for (int ti = 0; ti < TILES; ti++)
#pragma unroll
        for (int i = 0; i < 4; i++) cpart[((ti * W + wave) * 64 + lane) * 4 + i] = ytile[ti][i];
    // ---- the waves' tiles meet; thread (row, activation row) adds its two columns of each ----
    __syncthreads();
    if (out_t < NT) {
        float scale = 1.f;
        if constexpr (PRO == SHV_PRO_RMSNORM) {
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < W; w++) tot += red[out_t * W + w];
            scale = __builtin_amdgcn_rsqf(tot / static_cast<float>(K) + a.eps);
        }
        // ring_row of this thread's activation row: picked without indexing the register array by a variable
        int rr = 0;
#pragma unroll
        for (int t = 0; t < NT; t++) rr = t == out_t ? ring_row[t] : rr;
        float *dst = (a.ring_slots > 0 && !a.z_ring) ? a.y + static_cast<size_t>(rr) * a.ring_stride : a.y + static_cast<size_t>(out_t) * a.y_stride;
#pragma unroll
        for (int ti = 0; ti < TILES; ti++) {
            const int out_row = (static_cast<int>(blockIdx.x) * TILES + ti) * 16 + out_r;
            float y = 0.f;
#pragma unroll
            for (int w = 0; w < W; w++) {
                const float *cp = cpart + ((ti * W + w) * 64 + 16 * (out_r >> 2)) * 4 + (out_r & 3);
                y += cp[(2 * out_t) * 4] + cp[(2 * out_t + 1) * 4];
            }
            if (out_row < a.n) dst[out_row] = fmaf(y, scale, res[ti]);
        }
    }
}

template <int K, int NT, int TILES, int W>
size_t mrows_lds() {
    constexpr int KW = K / W, NSB = KW / 256, NF = KW / 8, NC = 2 * NT, FS = NC | 1;
    constexpr bool ALIAS = W != 4 && sizeof(half8_t) * W * NF * FS >= sizeof(float) * TILES * W * 64 * 4;
    return sizeof(half8_t) * W * NF * FS + sizeof(half4_t) * W * NSB * 4 * NC + sizeof(float) * (2 * NT * W + (ALIAS ? 0 : TILES * W * 64 * 4));
}

template <int K, int PRO, int NT, int TILES, int W = 4>
int launch_tiles(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    const size_t lds = mrows_lds<K, NT, TILES, W>();
    if (lds > 48 * 1024) {
        static std::atomic<bool> raised{false};  // above the default allowance the limit is raised once per kernel
        if (!raised.load(std::memory_order_acquire)) {
            SHV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_mrows_kernel<K, PRO, NT, TILES, W>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            raised.store(true, std::memory_order_release);
        }
    }
    SHV_LAUNCH(ctx, (gemv_mrows_kernel<K, PRO, NT, TILES, W>), dim3((a.n + 16 * TILES - 1) / (16 * TILES)), dim3(64 * W), lds, a);
    return SHV_OK;
}

// Every block stages the activation rows anew, which is what a row more costs, and a block of several row
// tiles does so once for all of them; but its waves then work through the tiles one after another.  Measured
// over chains of distinct matrices (us a launch, tiles a block 1 / 2 / 4):
//   12352 x 2048, 772 tiles   3 rows 9.2 / 9.3 / 10.1    6 rows 13.0 / 11.2 / 11.9    8 rows 15.5 / 16.0 / 12.8
//   151936 x 2048, 9496 tiles 2 rows 56 / 48 / 52        3 rows 74 / 59 / 59          4 rows 81 / 63 / 60
// From five rows on the staging is what a launch takes, and a row's columns go over more waves (SHV_MROWS_WAVES=4
// keeps four).
template <int K, int PRO, int NT>
int launch_pro(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    const int tiles = (a.n + 15) / 16, cus = ctx->prop.multiProcessorCount;
    if constexpr (NT >= 5 && K == 4096) {
        // 2048 x 4096 at eight rows: 13.7 us on four waves, 10.2 on sixteen (a gated norm in front), 12.5 and 9.2 (a sigmoid
        // gate).
        if (!ctx->mrows_four_waves && tiles < 8 * cus) return launch_tiles<K, PRO, NT, 1, 16>(ctx, a);
    }
    if constexpr (K == 2048 && NT >= 4) {
        // 2048 columns over eight waves (a super-block of every row a wave) and several tiles a block, us a launch
        // against the blocks of four waves below: 12352 rows at 8 / 5 / 4 rows 10.2 / 9.5 / 8.5 against 12.3 / 11.3 / 9.8,
        // 9216 rows at 8 rows 10.0 against 11.6; at two and three rows nothing either way (8.0 and 8.5-8.9 against 8.1
        // and 8.8) and four waves stay.
        if (!ctx->mrows_four_waves && tiles < 8 * cus && (NT >= 5 || tiles >= 3 * cus)) {
            if (tiles >= 2 * cus) return launch_tiles<K, PRO, NT, 4, 8>(ctx, a);
            if (tiles >= cus) return launch_tiles<K, PRO, NT, 2, 8>(ctx, a);
            return launch_tiles<K, PRO, NT, 1, 8>(ctx, a);
        }
    }
    if constexpr (K == 2048) {
        if (tiles >= 8 * cus) return NT >= 4 ? launch_tiles<K, PRO, NT, 4>(ctx, a) : launch_tiles<K, PRO, NT, 2>(ctx, a);
        if (NT >= 6 && tiles >= 2 * cus) return launch_tiles<K, PRO, NT, 4>(ctx, a);
    }
    return launch_tiles<K, PRO, NT, 1>(ctx, a);
}

template <int K, int NT>
int launch_nt(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    switch (a.prologue) {
        case SHV_PRO_NONE: return launch_pro<K, SHV_PRO_NONE, NT>(ctx, a);
        case SHV_PRO_RMSNORM: return launch_pro<K, SHV_PRO_RMSNORM, NT>(ctx, a);
        case SHV_PRO_GATED_NORM: return launch_pro<K, SHV_PRO_GATED_NORM, NT>(ctx, a);
        default: return launch_pro<K, SHV_PRO_MUL_SIGMOID, NT>(ctx, a);
    }
}

template <int K>
int launch_k(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    switch (a.n_tok) {
        case 2: return launch_nt<K, 2>(ctx, a);
        case 3: return launch_nt<K, 3>(ctx, a);
        case 4: return launch_nt<K, 4>(ctx, a);
        case 5: return launch_nt<K, 5>(ctx, a);
        case 6: return launch_nt<K, 6>(ctx, a);
        case 7: return launch_nt<K, 7>(ctx, a);
        default: return launch_nt<K, 8>(ctx, a);
    }
}

}  // namespace

// Which calls this kernel takes: two to eight rows of 2048 or 4096 columns, whole float4s everywhere,
// a gated norm over heads of 128, no router rows and no arg-max riding along.
bool shv_gemv_mrows_covers(const shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    if (ctx->mrows_off || a.n_tok < 2 || a.n_tok > 8 || (a.k != 2048 && a.k != 4096)) return false;
    if (a.fold || a.amax_best || a.y_flat || a.prologue == SHV_PRO_RMSNORM_PAIR) return false;
    if (!shv_aligned16(a.x) || a.x_stride % 4 != 0 || (a.gamma && !shv_aligned16(a.gamma))) return false;
    if (a.prologue == SHV_PRO_GATED_NORM && (a.head_dim != 128 || !shv_aligned16(a.z) || (a.z_ring ? a.ring_stride % 4 != 0 : a.z_stride % 4 != 0))) return false;
    if (a.prologue == SHV_PRO_MUL_SIGMOID && (!shv_aligned16(a.z) || a.z_stride % 4 != 0 || (a.head_dim != 0 && a.head_dim < 8))) return false;
    const int sl = a.seq_len > 0 ? a.seq_len : a.n_tok;
    if (a.n_tok % sl != 0) return false;
    // a matrix of many rounds of the chip (the vocabulary projection) is a stream: from five rows on the tiled
    // kernel, which walks it with every wave resident, is ahead (76 against 110 us at eight rows)
    if (a.n_tok >= 5 && (a.n + 15) / 16 >= 8 * ctx->prop.multiProcessorCount) return false;
    return true;
}

int shv_launch_gemv_mrows(shv_ctx *ctx, const shv_gemv_q4k_args &a) {
    return a.k == 2048 ? launch_k<2048>(ctx, a) : launch_k<4096>(ctx, a);
}
