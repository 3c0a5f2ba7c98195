// Internal declarations shared by the C-ABI layer and the kernel launchers.
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "shv_hip.h"

struct shv_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop{};
    uint64_t submits = 0;
    bool capturing = false;
    // Q4_K projections of at least this many rows run on the matrix cores: from 3 rows where the
    // rows are up to 2048 columns, from 5 where they are wider (a 2048x4096 output projection is a
    // few short launches' worth of bytes, and the row kernel's four rows cost less than staging
    // operands).  SHV_MFMA_MIN_ROWS in the environment sets both; a large value keeps every pass
    // on the row kernel.
    int mfma_min_rows = 3, mfma_min_rows_wide = 5;
    bool mfma_rows_forced = false;  // SHV_MFMA_MIN_ROWS was given: the few-rows GEMV steps aside for the caller's threshold
    // SHV_GEMV_SCALES=lds: the one-row GEMV hands each super-block's eight (d*sc, dmin*m) pairs from one lane to
    // the four that use them through LDS instead of letting every lane decode its own (for comparison; slower)
    bool gemv_scales_lds = false;
    // passes of this many rows up to 16 (8 where rows are 4096 wide) take the sixteen-wave matrix-core kernel that
    // stages its rows under the weight loads (SHV_GEMM_ROWS_MIN; 0: never)
    int gemm_rows_min = 5;
    // SHV_MROWS=0: projections of two to eight rows go the ways they went before the kernel that forms each weight
    // once for all rows (the side-by-side row kernel up to four rows, the tiled matrix-core kernels above)
    bool mrows_off = false;
    bool mrows_four_waves = false;  // SHV_MROWS_WAVES=4: five to eight rows stay on blocks of four waves
    // SHV_ATTN_APPEND=launch: passes of three and four rows write their new cells in a launch of their own, as longer ones do
    bool attn_append_launch = false;
    int moe_group_min = 128;  // rows from which a MoE pass with a workspace is grouped by expert on the matrix cores (SHV_MOE_GROUP_MIN)
    bool dn_chunk_no_recs = false;  // SHV_DN_RECS=0: the chunked delta rule forms every chunk's state-independent part inside the walk, whatever the workspace holds
    bool moe_group_one_block = false;  // SHV_MOE_GROUP_BLOCKS=1: the per-expert lists of a long pass by one block in one launch
    int moe_tall_min = 16;  // tokens from which the MoE kernels' blocks make several passes over their staged rows (SHV_MOE_TALL_MIN)
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    hipEvent_t stamps[SHV_STAMPS] = {};  // shv_stamp's, made when first used
    // shv_upload_async copies up to kUpSlotBytes into the next slot of a ring of pinned host memory and hands them
    // to the stream from there: the call returns without waiting for the device (a pass's control words, a few
    // token ids).  up_pending counts the slots written since the stream was last waited for; a full ring waits.
    // SHV_UPLOAD_SYNC=1 leaves the ring out: every upload blocks.
    char *up_ring = nullptr;
    enum { kUpSlots = 128, kUpSlotBytes = SHV_UPLOAD_ASYNC_MAX };
    int up_next = 0, up_pending = 0;
    hipError_t wait_stream() {
        const hipError_t e = hipStreamSynchronize(stream);
        if (e == hipSuccess) up_pending = 0;
        return e;
    }
    // scratch the library's own kernels need (arrival counters for last-block epilogues)
    int32_t *counters = nullptr;
    int n_counters = 0;
    // activations of a many-row projection, transformed once into matrix-core operand order and
    // copied from here by every block (kGemmStageBytes covers 4096 rows of 4096 columns)
    char *gemm_stage = nullptr;
    enum { kGemmStageBytes = 72 << 20 };
    // partial products of a pass whose columns are split over blocks: [parts][64 rows][n] floats
    float *gemm_part = nullptr;
    enum { kGemmPartBytes = 16 << 20 };
    // per-block partial results of the arg-max reduction: (value, index) pairs
    float *argmax_val = nullptr;
    int32_t *argmax_idx = nullptr;
    enum { kArgmaxBlocks = 512 };
    // the same for the arg-max a vocabulary projection makes in its own launch: one pair a block
    float *gemv_amax_val = nullptr;
    int32_t *gemv_amax_idx = nullptr;
    enum { kGemvAmaxBlocks = 2048 };
    // device address of this GPU's copy of the library's static scratch array (misc.hip), for the
    // entry point that allocates nothing
    void *static_scratch = nullptr;
    // Per-kernel GPU timestamps for a marked dispatch: while `marking` is set every launch is
    // bracketed by a pair of events taken from the dispatch packet itself, so an op's time is the
    // time its kernels ran and holds no launch gap.
    bool marking = false;
    int mark_op = 0;
    std::vector<hipEvent_t> mark_pool;
    struct Mark { int op, start, stop; };
    std::vector<Mark> marks;
    hipError_t next_marks(hipEvent_t *s, hipEvent_t *e) {
        const size_t need = marks.size() * 2 + 2;
        while (mark_pool.size() < need) {
            hipEvent_t ev;
            const hipError_t rc = hipEventCreate(&ev);
            if (rc != hipSuccess) return rc;
            mark_pool.push_back(ev);
        }
        const int i = static_cast<int>(marks.size()) * 2;
        marks.push_back({mark_op, i, i + 1});
        *s = mark_pool[i];
        *e = mark_pool[i + 1];
        return hipSuccess;
    }
    enum { kCounterRouter = 0, kCounterArgmax = 1, kCounterAttn = 16, kCounterGemvAmax = 15 };
    // What the last shv_moe_up on this context left behind for the shv_moe_down that follows it:
    // the pass its per-expert lists in `group` belong to, and whether act holds matrix-core
    // operands instead of floats.  shv_moe_down believes its group_ready / act_packed flags only
    // when they agree with this.
    struct MoeStamp {
        const void *topk = nullptr, *group = nullptr, *act = nullptr;
        int n_tok = 0, n_used = 0;
        bool grouped = false, packed = false;
    } moe_stamp;
};

struct shv_prerecorded {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int count = 0;
};

int shv_set_error(int code, const char *fmt, ...);

#define SHV_HIP_CHECK(expr)                                                                    \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess)                                                                  \
            return shv_set_error(SHV_E_HIP, "%s: %s (%s:%d)", #expr, hipGetErrorString(e_),    \
                                 __FILE__, __LINE__);                                          \
    } while (0)

#define SHV_REQUIRE(cond, ...)                                                                 \
    do {                                                                                       \
        if (!(cond)) return shv_set_error(SHV_E_INVALID, __VA_ARGS__);                         \
    } while (0)

// Every kernel launch of the library goes through here.
#define SHV_LAUNCH(ctx, kern, grid, block, lds, ...)                                           \
    do {                                                                                       \
        if ((ctx)->marking) {                                                                  \
            hipEvent_t ms_, me_;                                                               \
            SHV_HIP_CHECK((ctx)->next_marks(&ms_, &me_));                                      \
            hipExtLaunchKernelGGL(kern, grid, block, lds, (ctx)->stream, ms_, me_, 0, __VA_ARGS__); \
        } else {                                                                               \
            hipLaunchKernelGGL(kern, grid, block, lds, (ctx)->stream, __VA_ARGS__);            \
        }                                                                                      \
        SHV_HIP_CHECK(hipGetLastError());                                                      \
    } while (0)

static inline bool shv_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// one launcher per op kind; each validates its argument block on the host before launching
int shv_launch_gemv_q4k(shv_ctx *ctx, const shv_gemv_q4k_args *a);
// the matrix-core kernel for passes of two rows and more (gemm_q4k.hip)
bool shv_gemm_q4k_covers(const shv_gemv_q4k_args &a);
bool shv_gemv_mrows_covers(const shv_ctx *ctx, const shv_gemv_q4k_args &a);
int shv_launch_gemv_mrows(shv_ctx *ctx, const shv_gemv_q4k_args &a);
int shv_launch_gemm_q4k(shv_ctx *ctx, const shv_gemv_q4k_args &a);
bool shv_router_wide_covers(const shv_ctx *ctx, const shv_moe_router_args &a);
int shv_launch_router_wide(shv_ctx *ctx, const shv_moe_router_args &a);
int shv_launch_dequant_q4k(shv_ctx *ctx, const shv_dequant_q4k_args *a);
int shv_launch_dequant(shv_ctx *ctx, const shv_dequant_args *a);
int shv_launch_gemv(shv_ctx *ctx, const shv_gemv_args *a);
int shv_launch_quantize_q4k(shv_ctx *ctx, const shv_quantize_q4k_args *a);
int shv_launch_fill_normal(shv_ctx *ctx, const shv_fill_normal_args *a);
int shv_launch_moe_router(shv_ctx *ctx, const shv_moe_router_args *a);
int shv_launch_moe_up(shv_ctx *ctx, const shv_moe_up_args *a);
int shv_launch_moe_down(shv_ctx *ctx, const shv_moe_down_args *a);
// passes of many rows grouped by expert on the matrix cores (moe_grouped.hip)
bool shv_moe_up_grouped_covers(const shv_ctx *ctx, const shv_moe_up_args &a);
int shv_launch_moe_up_grouped(shv_ctx *ctx, const shv_moe_up_args &a);
bool shv_moe_down_grouped_covers(const shv_ctx *ctx, const shv_moe_down_args &a);
int shv_launch_moe_down_grouped(shv_ctx *ctx, const shv_moe_down_args &a);
int shv_launch_dn_step(shv_ctx *ctx, const shv_dn_step_args *a);
int shv_launch_attn_decode(shv_ctx *ctx, const shv_attn_decode_args *a);
// expert banks in other types than Q4_K: slots [slot0, slot0 + slots) of the up projection; slots
// [s_lo, s_hi) of the down projection, added to out when `add` (another launch wrote the rest)
int shv_launch_moe_up_any(shv_ctx *ctx, const shv_moe_up_args *a, int slot0, int slots);
int shv_launch_moe_down_any(shv_ctx *ctx, const shv_moe_down_args *a, int s_lo, int s_hi, int add);
int shv_launch_embed(shv_ctx *ctx, const shv_embed_args *a);
int shv_launch_embed_typed(shv_ctx *ctx, const shv_embed_args *a);  // a table in a type other than binary16
long long shv_type_bytes(int type, long long n);                    // bytes of n elements of a ggml type, -1 if refused
int shv_launch_argmax(shv_ctx *ctx, const shv_argmax_args *a);
int shv_launch_advance(shv_ctx *ctx, const shv_advance_args *a);
int shv_launch_ring_rows(shv_ctx *ctx, const shv_ring_rows_args *a);
int shv_launch_router_fold(shv_ctx *ctx, const shv_router_fold_args *a);
int shv_launch_qsa_index(shv_ctx *ctx, const shv_qsa_index_args *a);
bool shv_dn_chunk_covers(const shv_dn_step_args &a);
int shv_launch_dn_chunk(shv_ctx *ctx, const shv_dn_step_args &a);
int shv_static_scratch_bind(shv_ctx *ctx);  // at shv_init, with ctx->device current
int shv_launch_argmax_static(shv_ctx *ctx, const shv_argmax_args *a);
