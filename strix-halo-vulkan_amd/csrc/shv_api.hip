// C-ABI layer: context, buffers, op dispatch, timed sequences and prerecorded (HIP graph) replay.
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "shv_internal.hpp"

static thread_local char g_err[512] = "";

int shv_set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" {

const char *shv_last_error(void) { return g_err; }

int shv_device_count(int *out) {
    SHV_REQUIRE(out != nullptr, "shv_device_count: out is NULL");
    int n = 0;
    SHV_HIP_CHECK(hipGetDeviceCount(&n));
    *out = n;
    return SHV_OK;
}

int shv_init(int device, shv_ctx **out) {
    SHV_REQUIRE(out != nullptr, "shv_init: out is NULL");
    *out = nullptr;
    int n = 0;
    SHV_HIP_CHECK(hipGetDeviceCount(&n));
    SHV_REQUIRE(device >= 0 && device < n, "shv_init: device %d of %d", device, n);
    SHV_HIP_CHECK(hipSetDevice(device));
    shv_ctx *ctx = new (std::nothrow) shv_ctx();
    if (!ctx) return shv_set_error(SHV_E_NOMEM, "shv_init: out of host memory");
    ctx->device = device;
    if (const char *e = std::getenv("SHV_MFMA_MIN_ROWS")) {
        const int v = std::atoi(e);
        if (v >= 2) {
            ctx->mfma_min_rows = ctx->mfma_min_rows_wide = v;
            ctx->mfma_rows_forced = true;
        }
    }
    if (const char *e = std::getenv("SHV_GEMV_SCALES")) ctx->gemv_scales_lds = std::strcmp(e, "lds") == 0;
    if (const char *e = std::getenv("SHV_GEMM_ROWS_MIN")) {
        const int v = std::atoi(e);
        if (v >= 0) ctx->gemm_rows_min = v;
    }
    if (const char *e = std::getenv("SHV_MROWS")) ctx->mrows_off = std::atoi(e) == 0;
    if (const char *e = std::getenv("SHV_MROWS_WAVES")) ctx->mrows_four_waves = std::atoi(e) == 4;
    if (const char *e = std::getenv("SHV_ATTN_APPEND")) ctx->attn_append_launch = std::strcmp(e, "launch") == 0;
    if (const char *e = std::getenv("SHV_MOE_GROUP_MIN")) {
        const int v = std::atoi(e);
        if (v >= 1) ctx->moe_group_min = v;
    }
    if (const char *e = std::getenv("SHV_DN_RECS")) ctx->dn_chunk_no_recs = std::atoi(e) == 0;
    if (const char *e = std::getenv("SHV_MOE_GROUP_BLOCKS")) ctx->moe_group_one_block = std::atoi(e) == 1;
    if (const char *e = std::getenv("SHV_MOE_TALL_MIN")) {
        const int v = std::atoi(e);
        if (v >= 1) ctx->moe_tall_min = v;
    }
    hipError_t e = hipGetDeviceProperties(&ctx->prop, device);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev_begin);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev_end);
    const char *up_sync = std::getenv("SHV_UPLOAD_SYNC");
    if (e == hipSuccess && !(up_sync && std::atoi(up_sync) != 0))
        e = hipHostMalloc(reinterpret_cast<void **>(&ctx->up_ring), static_cast<size_t>(shv_ctx::kUpSlots) * shv_ctx::kUpSlotBytes, hipHostMallocDefault);
    ctx->n_counters = 4096;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->counters), ctx->n_counters * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemset(ctx->counters, 0, ctx->n_counters * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->gemm_stage), shv_ctx::kGemmStageBytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->gemm_part), shv_ctx::kGemmPartBytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->argmax_val), shv_ctx::kArgmaxBlocks * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->argmax_idx), shv_ctx::kArgmaxBlocks * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->gemv_amax_val), shv_ctx::kGemvAmaxBlocks * sizeof(float));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->gemv_amax_idx), shv_ctx::kGemvAmaxBlocks * sizeof(int32_t));
    if (e != hipSuccess) {
        shv_destroy(ctx);
        return shv_set_error(SHV_E_HIP, "shv_init: %s", hipGetErrorString(e));
    }
    if (std::strncmp(ctx->prop.gcnArchName, "gfx950", 6) == 0) {
        const int rc = shv_static_scratch_bind(ctx);
        if (rc != SHV_OK) {
            shv_destroy(ctx);
            return rc;
        }
    }
    if (std::strncmp(ctx->prop.gcnArchName, "gfx950", 6) != 0) {
        char arch[64];
        std::snprintf(arch, sizeof(arch), "%s", ctx->prop.gcnArchName);
        shv_destroy(ctx);
        return shv_set_error(SHV_E_INVALID, "shv_init: device %d is %s; this library holds gfx950 code only", device, arch);
    }
    *out = ctx;
    return SHV_OK;
}

void shv_destroy(shv_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->counters) (void)hipFree(ctx->counters);
    if (ctx->gemm_stage) (void)hipFree(ctx->gemm_stage);
    if (ctx->gemm_part) (void)hipFree(ctx->gemm_part);
    if (ctx->argmax_val) (void)hipFree(ctx->argmax_val);
    if (ctx->argmax_idx) (void)hipFree(ctx->argmax_idx);
    if (ctx->gemv_amax_val) (void)hipFree(ctx->gemv_amax_val);
    if (ctx->gemv_amax_idx) (void)hipFree(ctx->gemv_amax_idx);
    if (ctx->up_ring) (void)hipHostFree(ctx->up_ring);
    for (hipEvent_t ev : ctx->mark_pool) (void)hipEventDestroy(ev);
    for (hipEvent_t ev : ctx->stamps)
        if (ev) (void)hipEventDestroy(ev);
    if (ctx->ev_begin) (void)hipEventDestroy(ctx->ev_begin);
    if (ctx->ev_end) (void)hipEventDestroy(ctx->ev_end);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

int shv_device_props(shv_ctx *ctx, shv_props *out) {
    SHV_REQUIRE(ctx && out, "shv_device_props: NULL argument");
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", ctx->prop.name);
    std::snprintf(out->arch, sizeof(out->arch), "%s", ctx->prop.gcnArchName);
    out->compute_units = ctx->prop.multiProcessorCount;
    out->wave_size = ctx->prop.warpSize;
    out->lds_bytes_per_cu = static_cast<int32_t>(ctx->prop.maxSharedMemoryPerMultiProcessor);
    out->clock_mhz = ctx->prop.clockRate / 1000;
    out->hbm_bytes = ctx->prop.totalGlobalMem;
    return SHV_OK;
}

int shv_sync(shv_ctx *ctx) {
    SHV_REQUIRE(ctx, "shv_sync: NULL context");
    SHV_HIP_CHECK(ctx->wait_stream());
    return SHV_OK;
}

int shv_submits(shv_ctx *ctx, uint64_t *out) {
    SHV_REQUIRE(ctx && out, "shv_submits: NULL argument");
    *out = ctx->submits;
    return SHV_OK;
}

int shv_alloc(shv_ctx *ctx, size_t bytes, void **dptr) {
    SHV_REQUIRE(ctx && dptr, "shv_alloc: NULL argument");
    SHV_REQUIRE(bytes > 0, "shv_alloc: zero bytes");
    *dptr = nullptr;
    hipError_t e = hipMalloc(dptr, bytes);
    if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        return shv_set_error(SHV_E_NOMEM, "shv_alloc: %zu bytes do not fit in device memory", bytes);
    }
    SHV_HIP_CHECK(e);
    return SHV_OK;
}

int shv_free(shv_ctx *ctx, void *dptr) {
    SHV_REQUIRE(ctx, "shv_free: NULL context");
    if (!dptr) return SHV_OK;
    SHV_HIP_CHECK(ctx->wait_stream());
    SHV_HIP_CHECK(hipFree(dptr));
    return SHV_OK;
}

int shv_upload(shv_ctx *ctx, void *dst, const void *src, size_t bytes) {
    SHV_REQUIRE(ctx && dst && src, "shv_upload: NULL argument");
    SHV_REQUIRE(!ctx->capturing, "shv_upload: not valid while recording");
    if (bytes == 0) return SHV_OK;
    SHV_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    SHV_HIP_CHECK(ctx->wait_stream());
    return SHV_OK;
}

int shv_upload_async(shv_ctx *ctx, void *dst, const void *src, size_t bytes) {
    SHV_REQUIRE(ctx && dst && src, "shv_upload_async: NULL argument");
    SHV_REQUIRE(!ctx->capturing, "shv_upload_async: not valid while recording");
    if (bytes == 0) return SHV_OK;
    if (!ctx->up_ring || bytes > shv_ctx::kUpSlotBytes) return shv_upload(ctx, dst, src, bytes);
    // a slot is free again once the stream has been waited for after the copy that read it
    if (ctx->up_pending == shv_ctx::kUpSlots) SHV_HIP_CHECK(ctx->wait_stream());
    char *slot = ctx->up_ring + static_cast<size_t>(ctx->up_next) * shv_ctx::kUpSlotBytes;
    std::memcpy(slot, src, bytes);
    SHV_HIP_CHECK(hipMemcpyAsync(dst, slot, bytes, hipMemcpyHostToDevice, ctx->stream));
    ctx->up_next = (ctx->up_next + 1) % shv_ctx::kUpSlots;
    ctx->up_pending++;
    return SHV_OK;
}

int shv_download(shv_ctx *ctx, void *dst, const void *src, size_t bytes) {
    SHV_REQUIRE(ctx && dst && src, "shv_download: NULL argument");
    SHV_REQUIRE(!ctx->capturing, "shv_download: not valid while recording");
    if (bytes == 0) return SHV_OK;
    SHV_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    SHV_HIP_CHECK(ctx->wait_stream());
    return SHV_OK;
}

int shv_copy(shv_ctx *ctx, void *dst, const void *src, size_t bytes) {
    SHV_REQUIRE(ctx && dst && src, "shv_copy: NULL argument");
    if (bytes == 0) return SHV_OK;
    SHV_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return SHV_OK;
}

int shv_host_alloc(shv_ctx *ctx, size_t bytes, void **hptr) {
    SHV_REQUIRE(ctx && hptr && bytes > 0, "shv_host_alloc: bad argument");
    SHV_HIP_CHECK(hipHostMalloc(hptr, bytes, hipHostMallocDefault));
    return SHV_OK;
}

int shv_host_free(shv_ctx *ctx, void *hptr) {
    SHV_REQUIRE(ctx, "shv_host_free: NULL context");
    if (hptr) SHV_HIP_CHECK(hipHostFree(hptr));
    return SHV_OK;
}

}  // extern "C"

// ---- op dispatch ----------------------------------------------------------------------------

template <typename T>
static int run_as(shv_ctx *ctx, const void *args, size_t bytes, int (*fn)(shv_ctx *, const T *), const char *name) {
    static_assert(sizeof(T) <= sizeof(shv_op::args), "argument block exceeds the op record");
    SHV_REQUIRE(bytes >= sizeof(T), "%s: argument block is %zu bytes, need %zu", name, bytes, sizeof(T));
    T a;
    std::memcpy(&a, args, sizeof(T));
    return fn(ctx, &a);
}

static int dispatch_one(shv_ctx *ctx, uint32_t kind, const void *args, size_t bytes) {
    SHV_REQUIRE(ctx && args, "shv_enqueue: NULL argument");
    switch (kind) {
        case SHV_OP_GEMV_Q4K: return run_as<shv_gemv_q4k_args>(ctx, args, bytes, shv_launch_gemv_q4k, "gemv_q4k");
        case SHV_OP_DEQUANT_Q4K: return run_as<shv_dequant_q4k_args>(ctx, args, bytes, shv_launch_dequant_q4k, "dequant_q4k");
        case SHV_OP_QUANTIZE_Q4K: return run_as<shv_quantize_q4k_args>(ctx, args, bytes, shv_launch_quantize_q4k, "quantize_q4k");
        case SHV_OP_FILL_NORMAL: return run_as<shv_fill_normal_args>(ctx, args, bytes, shv_launch_fill_normal, "fill_normal");
        case SHV_OP_MOE_ROUTER: return run_as<shv_moe_router_args>(ctx, args, bytes, shv_launch_moe_router, "moe_router");
        case SHV_OP_MOE_UP: return run_as<shv_moe_up_args>(ctx, args, bytes, shv_launch_moe_up, "moe_up");
        case SHV_OP_MOE_DOWN: return run_as<shv_moe_down_args>(ctx, args, bytes, shv_launch_moe_down, "moe_down");
        case SHV_OP_DN_STEP: return run_as<shv_dn_step_args>(ctx, args, bytes, shv_launch_dn_step, "dn_step");
        case SHV_OP_ATTN_DECODE: return run_as<shv_attn_decode_args>(ctx, args, bytes, shv_launch_attn_decode, "attn_decode");
        case SHV_OP_EMBED: return run_as<shv_embed_args>(ctx, args, bytes, shv_launch_embed, "embed");
        case SHV_OP_ARGMAX: return run_as<shv_argmax_args>(ctx, args, bytes, shv_launch_argmax, "argmax");
        case SHV_OP_ADVANCE: return run_as<shv_advance_args>(ctx, args, bytes, shv_launch_advance, "advance");
        case SHV_OP_DEQUANT: return run_as<shv_dequant_args>(ctx, args, bytes, shv_launch_dequant, "dequant");
        case SHV_OP_GEMV: return run_as<shv_gemv_args>(ctx, args, bytes, shv_launch_gemv, "gemv");
        case SHV_OP_RING_ROWS: return run_as<shv_ring_rows_args>(ctx, args, bytes, shv_launch_ring_rows, "ring_rows");
        case SHV_OP_ROUTER_FOLD: return run_as<shv_router_fold_args>(ctx, args, bytes, shv_launch_router_fold, "router_fold");
        case SHV_OP_QSA_INDEX: return run_as<shv_qsa_index_args>(ctx, args, bytes, shv_launch_qsa_index, "qsa_index");
        case SHV_OP_ARGMAX_STATIC: return run_as<shv_argmax_args>(ctx, args, bytes, shv_launch_argmax_static, "argmax_static");
        default: return shv_set_error(SHV_E_INVALID, "shv_enqueue: unknown op kind %u", kind);
    }
}

extern "C" {

int shv_enqueue(shv_ctx *ctx, uint32_t kind, const void *args, size_t args_bytes) {
    return dispatch_one(ctx, kind, args, args_bytes);
}

int shv_zero(shv_ctx *ctx, void *dst, size_t bytes) {
    SHV_REQUIRE(ctx && dst, "shv_zero: NULL argument");
    SHV_REQUIRE(!ctx->capturing, "shv_zero: not valid while recording");
    if (bytes == 0) return SHV_OK;
    SHV_HIP_CHECK(hipMemsetAsync(dst, 0, bytes, ctx->stream));
    return SHV_OK;
}

int shv_dispatch_multi(shv_ctx *ctx, const shv_op *ops, int n_ops, int iters, uint64_t *total_ns,
                       uint64_t *per_op_ns) {
    SHV_REQUIRE(ctx && ops, "shv_dispatch_multi: NULL argument");
    SHV_REQUIRE(n_ops > 0, "shv_dispatch_multi: empty op sequence");
    SHV_REQUIRE(iters >= 1, "shv_dispatch_multi: iters %d", iters);
    SHV_REQUIRE(!ctx->capturing, "shv_dispatch_multi: not valid while recording");
    SHV_REQUIRE(per_op_ns == nullptr || iters == 1, "shv_dispatch_multi: per-op times need iters == 1");
    // per-op times come from timestamps on the kernels themselves, so they hold no launch gap
    ctx->marks.clear();
    ctx->marking = per_op_ns != nullptr;
    int rc = SHV_OK;
    hipError_t e = hipEventRecord(ctx->ev_begin, ctx->stream);
    for (int it = 0; it < iters && rc == SHV_OK && e == hipSuccess; it++)
        for (int i = 0; i < n_ops && rc == SHV_OK; i++) {
            ctx->mark_op = i;
            rc = dispatch_one(ctx, ops[i].kind, ops[i].args, sizeof(ops[i].args));
        }
    ctx->marking = false;
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_end, ctx->stream);
    const hipError_t es = ctx->wait_stream();
    if (e == hipSuccess) e = es;
    ctx->submits++;
    if (rc == SHV_OK && e == hipSuccess) {
        float ms = 0;
        e = hipEventElapsedTime(&ms, ctx->ev_begin, ctx->ev_end);
        if (total_ns) *total_ns = static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
        if (per_op_ns) {
            for (int i = 0; i < n_ops; i++) per_op_ns[i] = 0;
            for (const auto &m : ctx->marks) {
                if (e != hipSuccess) break;
                e = hipEventElapsedTime(&ms, ctx->mark_pool[m.start], ctx->mark_pool[m.stop]);
                per_op_ns[m.op] += static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
            }
        }
    }
    ctx->marks.clear();
    if (rc != SHV_OK) return rc;
    if (e != hipSuccess) return shv_set_error(SHV_E_HIP, "shv_dispatch_multi: %s", hipGetErrorString(e));
    return SHV_OK;
}

int shv_prerecord(shv_ctx *ctx, const shv_op *ops, int n_ops, shv_prerecorded **out) {
    SHV_REQUIRE(ctx && ops && out, "shv_prerecord: NULL argument");
    SHV_REQUIRE(n_ops > 0, "shv_prerecord: empty op sequence");
    SHV_REQUIRE(!ctx->capturing, "shv_prerecord: already recording");
    *out = nullptr;
    SHV_HIP_CHECK(ctx->wait_stream());
    SHV_HIP_CHECK(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    int rc = SHV_OK;
    for (int i = 0; i < n_ops && rc == SHV_OK; i++)
        rc = dispatch_one(ctx, ops[i].kind, ops[i].args, sizeof(ops[i].args));
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    ctx->capturing = false;
    if (rc != SHV_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e != hipSuccess) return shv_set_error(SHV_E_HIP, "shv_prerecord: end capture: %s", hipGetErrorString(e));
    shv_prerecorded *p = new (std::nothrow) shv_prerecorded();
    if (!p) {
        (void)hipGraphDestroy(graph);
        return shv_set_error(SHV_E_NOMEM, "shv_prerecord: out of host memory");
    }
    p->graph = graph;
    p->count = n_ops;
    e = hipGraphInstantiate(&p->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        delete p;
        return shv_set_error(SHV_E_HIP, "shv_prerecord: instantiate: %s", hipGetErrorString(e));
    }
    *out = p;
    return SHV_OK;
}

int shv_prerecorded_launch(shv_ctx *ctx, shv_prerecorded *p) {
    SHV_REQUIRE(ctx && p && p->exec, "shv_prerecorded_launch: NULL argument");
    SHV_HIP_CHECK(hipGraphLaunch(p->exec, ctx->stream));
    ctx->submits++;
    return SHV_OK;
}

int shv_stamp(shv_ctx *ctx, int i) {
    SHV_REQUIRE(ctx && i >= 0 && i < SHV_STAMPS, "shv_stamp: stamp %d of %d", i, SHV_STAMPS);
    SHV_REQUIRE(!ctx->capturing, "shv_stamp: not valid while recording");
    if (!ctx->stamps[i]) SHV_HIP_CHECK(hipEventCreate(&ctx->stamps[i]));
    SHV_HIP_CHECK(hipEventRecord(ctx->stamps[i], ctx->stream));
    return SHV_OK;
}

int shv_stamp_elapsed(shv_ctx *ctx, int from, int to, uint64_t *ns) {
    SHV_REQUIRE(ctx && ns && from >= 0 && from < SHV_STAMPS && to >= 0 && to < SHV_STAMPS, "shv_stamp_elapsed: bad argument");
    SHV_REQUIRE(ctx->stamps[from] && ctx->stamps[to], "shv_stamp_elapsed: a stamp that was never made");
    float ms = 0;
    const hipError_t e = hipEventElapsedTime(&ms, ctx->stamps[from], ctx->stamps[to]);
    if (e == hipErrorNotReady) {
        (void)hipGetLastError();
        return shv_set_error(SHV_E_STATE, "shv_stamp_elapsed: the stream has not reached the stamps yet; wait for it first");
    }
    SHV_HIP_CHECK(e);
    *ns = static_cast<uint64_t>(static_cast<double>(ms < 0 ? 0 : ms) * 1e6);
    return SHV_OK;
}

int shv_prerecorded_submit(shv_ctx *ctx, shv_prerecorded *p, int iters, uint64_t *total_ns) {
    SHV_REQUIRE(ctx && p && p->exec, "shv_prerecorded_submit: NULL argument");
    SHV_REQUIRE(iters >= 1, "shv_prerecorded_submit: iters %d", iters);
    SHV_HIP_CHECK(hipEventRecord(ctx->ev_begin, ctx->stream));
    for (int i = 0; i < iters; i++) SHV_HIP_CHECK(hipGraphLaunch(p->exec, ctx->stream));
    SHV_HIP_CHECK(hipEventRecord(ctx->ev_end, ctx->stream));
    SHV_HIP_CHECK(ctx->wait_stream());
    ctx->submits += static_cast<uint64_t>(iters);
    float ms = 0;
    SHV_HIP_CHECK(hipEventElapsedTime(&ms, ctx->ev_begin, ctx->ev_end));
    if (total_ns) *total_ns = static_cast<uint64_t>(static_cast<double>(ms) * 1e6);
    return SHV_OK;
}

int shv_prerecorded_count(const shv_prerecorded *p) { return p ? p->count : 0; }

void shv_prerecorded_destroy(shv_ctx *ctx, shv_prerecorded *p) {
    if (!p) return;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (p->exec) (void)hipGraphExecDestroy(p->exec);
    if (p->graph) (void)hipGraphDestroy(p->graph);
    delete p;
}

int shv_gemv_q4k(shv_ctx *ctx, const shv_gemv_q4k_args *a) { return dispatch_one(ctx, SHV_OP_GEMV_Q4K, a, sizeof(*a)); }
int shv_dequant_q4k(shv_ctx *ctx, const shv_dequant_q4k_args *a) { return dispatch_one(ctx, SHV_OP_DEQUANT_Q4K, a, sizeof(*a)); }
int shv_dequant(shv_ctx *ctx, const shv_dequant_args *a) { return dispatch_one(ctx, SHV_OP_DEQUANT, a, sizeof(*a)); }
int shv_gemv(shv_ctx *ctx, const shv_gemv_args *a) { return dispatch_one(ctx, SHV_OP_GEMV, a, sizeof(*a)); }
int shv_quantize_q4k(shv_ctx *ctx, const shv_quantize_q4k_args *a) { return dispatch_one(ctx, SHV_OP_QUANTIZE_Q4K, a, sizeof(*a)); }
int shv_fill_normal(shv_ctx *ctx, const shv_fill_normal_args *a) { return dispatch_one(ctx, SHV_OP_FILL_NORMAL, a, sizeof(*a)); }
int shv_moe_router(shv_ctx *ctx, const shv_moe_router_args *a) { return dispatch_one(ctx, SHV_OP_MOE_ROUTER, a, sizeof(*a)); }
int shv_moe_up(shv_ctx *ctx, const shv_moe_up_args *a) { return dispatch_one(ctx, SHV_OP_MOE_UP, a, sizeof(*a)); }
int shv_moe_down(shv_ctx *ctx, const shv_moe_down_args *a) { return dispatch_one(ctx, SHV_OP_MOE_DOWN, a, sizeof(*a)); }
int shv_dn_step(shv_ctx *ctx, const shv_dn_step_args *a) { return dispatch_one(ctx, SHV_OP_DN_STEP, a, sizeof(*a)); }
int shv_attn_decode(shv_ctx *ctx, const shv_attn_decode_args *a) { return dispatch_one(ctx, SHV_OP_ATTN_DECODE, a, sizeof(*a)); }
int shv_embed(shv_ctx *ctx, const shv_embed_args *a) { return dispatch_one(ctx, SHV_OP_EMBED, a, sizeof(*a)); }
int shv_argmax(shv_ctx *ctx, const shv_argmax_args *a) { return dispatch_one(ctx, SHV_OP_ARGMAX, a, sizeof(*a)); }
int shv_advance(shv_ctx *ctx, const shv_advance_args *a) { return dispatch_one(ctx, SHV_OP_ADVANCE, a, sizeof(*a)); }
int shv_ring_rows(shv_ctx *ctx, const shv_ring_rows_args *a) { return dispatch_one(ctx, SHV_OP_RING_ROWS, a, sizeof(*a)); }
int shv_router_fold(shv_ctx *ctx, const shv_router_fold_args *a) { return dispatch_one(ctx, SHV_OP_ROUTER_FOLD, a, sizeof(*a)); }
int shv_qsa_index(shv_ctx *ctx, const shv_qsa_index_args *a) { return dispatch_one(ctx, SHV_OP_QSA_INDEX, a, sizeof(*a)); }

int shv_argmax_static(shv_ctx *ctx, const shv_argmax_args *a) {
    SHV_REQUIRE(ctx && a, "shv_argmax_static: NULL argument");
    return shv_launch_argmax_static(ctx, a);
}

}  // extern "C"
