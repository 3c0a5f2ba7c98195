// Device-side helpers shared by the kernels: wave64 reductions over DPP, Q4_K header decode,
// nibble unpacking.  Written for gfx950 (CDNA4, 64-wide wavefronts) only.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace shv {

constexpr int kWave = 64;

// ---- DPP lane exchange ----------------------------------------------------------------------
// update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl): lanes of disabled rows keep `old`.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f32(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
    return __int_as_float(r);
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i within 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i within 16
constexpr int kDppBcast15 = 0x142;    // lane 15 of each row of 16 -> the next row
constexpr int kDppBcast31 = 0x143;    // lane 31 -> lanes 32..63

// Sum over aligned groups of W consecutive lanes.  For W <= 16 every lane of the group ends up
// with the group's sum; for W = 32 and 64 only the LAST 16 lanes of the group hold it.
template <int W>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(W == 1 || W == 2 || W == 4 || W == 8 || W == 16 || W == 32 || W == 64, "group width");
    if (W >= 2) v += dpp_f32<kDppXor1>(v);
    if (W >= 4) v += dpp_f32<kDppXor2>(v);
    if (W >= 8) v += dpp_f32<kDppHalfMirror>(v);
    if (W >= 16) v += dpp_f32<kDppMirror>(v);
    if (W >= 32) v += dpp_f32<kDppBcast15, 0xA>(v);
    if (W >= 64) v += dpp_f32<kDppBcast31, 0xC>(v);
    return v;
}

// The lane of a W-group that is guaranteed to hold group_sum's result.
template <int W>
__device__ __forceinline__ bool group_sum_owner(int lane) {
    return (lane & (W - 1)) == (W - 1);
}

// Sum over the whole wave, delivered to every lane.
__device__ __forceinline__ float wave_sum_all(float v) {
    v = group_sum<64>(v);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float wave_max_all(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Sum over a 256-thread block; `red` is 4 floats of LDS.  Every thread gets the result.
__device__ __forceinline__ float block_sum_256(float v, float *red) {
    v = wave_sum_all(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0] + red[1] + red[2] + red[3];
    __syncthreads();
    return r;
}

// ---- Q4_K -----------------------------------------------------------------------------------
// Super-block: f16 d @0, f16 dmin @2, 12 bytes of packed 6-bit (scale, min) pairs @4, 128 bytes of
// nibbles @16.  Within each group of 64 weights the low nibbles of 32 bytes come first, then the
// high nibbles.  The header is read as one 16-byte word: x = d | dmin<<16, y,z,w = scale bytes.

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(h & 0xffffu)));
}

// Scales and mins of sub-blocks 2g and 2g+1 (the two halves of 64-weight group g), as packed
// bytes sc = sc0 | sc1<<8, mn = m0 | m1<<8.  Integer-exact get_scale_min_k4.
__device__ __forceinline__ void q4k_group_scale_min(const uint4 &hdr, int g, uint32_t &sc, uint32_t &mn) {
    const uint32_t sh = (g & 1) * 16;
    const uint32_t a = hdr.y >> sh, b = hdr.z >> sh, c = hdr.w >> sh;
    const uint32_t sc_lo = a & 0x3F3Fu, mn_lo = b & 0x3F3Fu;
    const uint32_t sc_hi = (c & 0x0F0Fu) | ((a >> 2) & 0x3030u);
    const uint32_t mn_hi = ((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);
    sc = g >= 2 ? sc_hi : sc_lo;
    mn = g >= 2 ? mn_hi : mn_lo;
}

typedef _Float16 f16x2_native __attribute__((ext_vector_type(2)));

// Constants of the nibble-to-half trick, made opaque to the optimiser so that they live in
// registers and (q & mask) | one becomes a single v_and_or_b32.
struct NibbleConsts {
    uint32_t mask;  // 0x00F000F0: bits 4..7 of both halves
    uint32_t one;   // 0x54005400: the half 64.0 in both halves
};
__device__ __forceinline__ NibbleConsts nibble_consts() {
    NibbleConsts c;
    c.mask = 0x00F000F0u;
    c.one = 0x54005400u;
    asm volatile("" : "+s"(c.mask));
    asm volatile("" : "+v"(c.one));
    return c;
}

// A 4-bit level n placed in mantissa bits 4..7 of the half 64.0 reads as exactly 64 + n, and
// v_fma_mix_f32 widens a half operand for free, so each weight costs one FMA and half of a
// bit-field op.  The accumulators therefore carry 64*sum(x) on top of sum(n*x); the caller
// takes it off again with the same sums of x it needs for the Q4_K min term.
//
// One payload dword holds 8 weights: the low nibbles of its four bytes meet xlo[0..3] and the
// high nibbles meet xhi[0..3].
__device__ __forceinline__ void q4k_dot8(uint32_t q, const NibbleConsts &c, const float *xlo, const float *xhi,
                                         float &acc_lo, float &acc_hi) {
    const f16x2_native t1 = __builtin_bit_cast(f16x2_native, (q & c.mask) | c.one);         // high nibbles of bytes 0,2
    const f16x2_native t3 = __builtin_bit_cast(f16x2_native, ((q >> 8) & c.mask) | c.one);  // high nibbles of bytes 1,3
    const f16x2_native t0 = __builtin_bit_cast(f16x2_native, ((q << 4) & c.mask) | c.one);  // low nibbles of bytes 0,2
    const f16x2_native t2 = __builtin_bit_cast(f16x2_native, ((q >> 4) & c.mask) | c.one);  // low nibbles of bytes 1,3
    acc_lo = fmaf(static_cast<float>(t0.x), xlo[0], acc_lo);
    acc_lo = fmaf(static_cast<float>(t2.x), xlo[1], acc_lo);
    acc_lo = fmaf(static_cast<float>(t0.y), xlo[2], acc_lo);
    acc_lo = fmaf(static_cast<float>(t2.y), xlo[3], acc_lo);
    acc_hi = fmaf(static_cast<float>(t1.x), xhi[0], acc_hi);
    acc_hi = fmaf(static_cast<float>(t3.x), xhi[1], acc_hi);
    acc_hi = fmaf(static_cast<float>(t1.y), xhi[2], acc_hi);
    acc_hi = fmaf(static_cast<float>(t3.y), xhi[3], acc_hi);
}

// One lane's share of one row: a 64-weight group (32 payload bytes in p0,p1) against the 64
// activations xr[0..63] of the same columns.  xs_lo / xs_hi are the sums of xr[0..31] / xr[32..63].
__device__ __forceinline__ float q4k_group_dot(const uint4 &hdr, const uint4 &p0, const uint4 &p1, int g,
                                               const NibbleConsts &c, const float *xr, float xs_lo, float xs_hi) {
    uint32_t sc, mn;
    q4k_group_scale_min(hdr, g, sc, mn);
    const float d = f16_bits_to_f32(hdr.x), dmin = f16_bits_to_f32(hdr.x >> 16);
    float lo = 0.f, hi = 0.f;
    q4k_dot8(p0.x, c, xr + 0, xr + 32, lo, hi);
    q4k_dot8(p0.y, c, xr + 4, xr + 36, lo, hi);
    q4k_dot8(p0.z, c, xr + 8, xr + 40, lo, hi);
    q4k_dot8(p0.w, c, xr + 12, xr + 44, lo, hi);
    q4k_dot8(p1.x, c, xr + 16, xr + 48, lo, hi);
    q4k_dot8(p1.y, c, xr + 20, xr + 52, lo, hi);
    q4k_dot8(p1.z, c, xr + 24, xr + 56, lo, hi);
    q4k_dot8(p1.w, c, xr + 28, xr + 60, lo, hi);
    lo = fmaf(-64.f, xs_lo, lo);
    hi = fmaf(-64.f, xs_hi, hi);
    const float ds0 = d * static_cast<float>(sc & 0xFFu), ds1 = d * static_cast<float>(sc >> 8);
    const float dm0 = dmin * static_cast<float>(mn & 0xFFu), dm1 = dmin * static_cast<float>(mn >> 8);
    return ds0 * lo - dm0 * xs_lo + ds1 * hi - dm1 * xs_hi;
}

// The same with the group's scales already multiplied out: sc = (d*sc_lo, d*sc_hi, dmin*m_lo, dmin*m_hi).
__device__ __forceinline__ float q4k_group_dot_scaled(const uint4 &p0, const uint4 &p1, const float4 sc, const NibbleConsts &c,
                                                      const float *xr, float xs_lo, float xs_hi) {
    float lo = 0.f, hi = 0.f;
    q4k_dot8(p0.x, c, xr + 0, xr + 32, lo, hi);
    q4k_dot8(p0.y, c, xr + 4, xr + 36, lo, hi);
    q4k_dot8(p0.z, c, xr + 8, xr + 40, lo, hi);
    q4k_dot8(p0.w, c, xr + 12, xr + 44, lo, hi);
    q4k_dot8(p1.x, c, xr + 16, xr + 48, lo, hi);
    q4k_dot8(p1.y, c, xr + 20, xr + 52, lo, hi);
    q4k_dot8(p1.z, c, xr + 24, xr + 56, lo, hi);
    q4k_dot8(p1.w, c, xr + 28, xr + 60, lo, hi);
    lo = fmaf(-64.f, xs_lo, lo);
    hi = fmaf(-64.f, xs_hi, hi);
    return sc.x * lo - sc.z * xs_lo + sc.y * hi - sc.w * xs_hi;
}

typedef uint32_t u32x4_native __attribute__((ext_vector_type(4)));

// 128-bit load of weight bytes.  A plain load on purpose: the lanes of a super-block share its
// header and the two halves of a payload line are fetched by different instructions, and with the
// nontemporal hint those repeats went back to L2 (a streaming read of 175 MB measured 40 us with
// the hint and 29 us without).
__device__ __forceinline__ uint4 load_stream16(const void *p) {
    const u32x4_native v = *reinterpret_cast<const u32x4_native *>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// ---- staging an activation vector for the Q4_K row kernels -----------------------------------
// LDS layout: each 64-float slice is followed by 4 floats of padding so that the lanes of a wave,
// which read slices 256 bytes apart, fall on different banks.
__device__ __forceinline__ int lds_slot(int i) { return i + (i >> 6) * 4; }
__host__ __device__ constexpr int lds_padded(int k) { return k + (k >> 6) * 4; }

// The 64 activations of 64-weight group `gi`, from a vector staged with lds_slot(), plus the sums
// of their first and second 32 (the columns the low and the high nibbles of the group meet).
__device__ __forceinline__ void load_x_slice(const float *xs, int gi, float *xr, float &xs_lo, float &xs_hi) {
    const float4 *src = reinterpret_cast<const float4 *>(xs + gi * 68);
    float lo = 0.f, hi = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float4 f = src[i];
        xr[4 * i + 0] = f.x;
        xr[4 * i + 1] = f.y;
        xr[4 * i + 2] = f.z;
        xr[4 * i + 3] = f.w;
        const float s = (f.x + f.y) + (f.z + f.w);
        if (i < 8) lo += s; else hi += s;
    }
    xs_lo = lo;
    xs_hi = hi;
}

// The same 64 activations when the staging threads have already left the sums of every 32 columns
// in `sums` (sums[2*gi], sums[2*gi+1] are this group's): 64 additions a lane saved per visit.
__device__ __forceinline__ void load_x_slice_presummed(const float *xs, const float *sums, int gi, float *xr, float &xs_lo, float &xs_hi) {
    const float4 *src = reinterpret_cast<const float4 *>(xs + gi * 68);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float4 f = src[i];
        xr[4 * i + 0] = f.x;
        xr[4 * i + 1] = f.y;
        xr[4 * i + 2] = f.z;
        xr[4 * i + 3] = f.w;
    }
    const float2 sm = *reinterpret_cast<const float2 *>(sums + 2 * gi);
    xs_lo = sm.x;
    xs_hi = sm.y;
}

// Sum over aligned groups of 8 lanes (in every lane of the group), for the staging threads that
// hold four consecutive columns each: eight of them cover one 32-column sub-block.
__device__ __forceinline__ float sum8_all(float v) {
    v += dpp_f32<kDppXor1>(v);
    v += dpp_f32<kDppXor2>(v);
    v += dpp_f32<kDppHalfMirror>(v);
    return v;
}

// One lane's loads for one row: the super-block header and the 32 payload bytes of its group.
struct Q4kLane {
    uint4 hdr, q0, q1;
    __device__ __forceinline__ void load(const char *row_sb, int g) {
        hdr = load_stream16(row_sb);
        q0 = load_stream16(row_sb + 16 + g * 32);
        q1 = load_stream16(row_sb + 32 + g * 32);
    }
    __device__ __forceinline__ float dot(int g, const NibbleConsts &c, const float *xr, float xs_lo, float xs_hi) const {
        return q4k_group_dot(hdr, q0, q1, g, c, xr, xs_lo, xs_hi);
    }
};

// ---- handing results from many blocks to the last one to finish ---------------------------------
// The L2 caches of the chip's eight dies are not coherent with one another, and a device-scope
// release or acquire fence pays for that by writing back and invalidating a whole L2 — tens of
// microseconds when every block of a grid does it.  Instead, the few values that cross between
// blocks inside one kernel are written and read with device-scope atomic accesses, which go
// through to the coherence point on their own; the arrival counter is a relaxed device-scope
// atomic, ordered after the block's stores by waiting for them to complete.
__device__ __forceinline__ void store_agent(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_agent(int32_t *p, int32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float load_agent(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int32_t load_agent(const int32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_agent2(float *p, float a, float b) {
    const unsigned long long v = static_cast<unsigned long long>(__float_as_uint(a)) | (static_cast<unsigned long long>(__float_as_uint(b)) << 32);
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 load_agent2(const float *p) {
    const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__uint_as_float(static_cast<unsigned int>(v)), __uint_as_float(static_cast<unsigned int>(v >> 32)));
}

// Block-wide: every thread's earlier device-scope stores have completed, then one thread counts
// the block in.  Returns true in every thread of the block that arrived last; that block also
// re-arms the counter for the next launch.
__device__ __forceinline__ bool arrive_last(int32_t *counter, int expected, int *lds_flag) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const int prev = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev == expected - 1;
        if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *lds_flag = last;
    }
    __syncthreads();
    return *lds_flag != 0;
}

// ---- greedy arg-max: (value, index) pairs ordered so that the larger value wins and, between
// equal values, the lower index; NaN never wins (Argmax, llm/sample.go:359-367) ------------------
__device__ __forceinline__ bool amax_better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }
__device__ __forceinline__ void amax_wave(float &v, int &i) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(i, off, 64);
        if (amax_better(ov, oi, v, i)) { v = ov; i = oi; }
    }
}

__device__ __forceinline__ float sigmoid_exact(float x) { return 1.f / (1.f + expf(-x)); }

// Sigmoid through the hardware exp2 and reciprocal, a few units in the last place from the exact
// one: for the gates every workgroup of a projection applies to a whole activation vector, where
// sixteen exact ones a thread were a visible part of the kernel.
__device__ __forceinline__ float sigmoid_fast(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }

// i / d and i % d for a head width d that is a power of two (the launchers check): a shift and a
// mask, and no branch to keep the loads around them from being merged.
struct HeadSplit {
    int mask, shift;
    __device__ __forceinline__ explicit HeadSplit(int head_dim) : mask(head_dim - 1), shift(__ffs(head_dim) - 1) {}
    __device__ __forceinline__ int head(int i) const { return i >> shift; }
    __device__ __forceinline__ int dim(int i) const { return i & mask; }
};

__device__ __forceinline__ float sigmoidf_dev(float x) { return 1.f / (1.f + __expf(-x)); }
__device__ __forceinline__ float siluf_dev(float x) { return x * sigmoidf_dev(x); }

}  // namespace shv
