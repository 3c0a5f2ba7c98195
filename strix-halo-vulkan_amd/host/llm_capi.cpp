// Flat C entry points over llm::Graph for ctypes callers: see shv_llm.h.
#include "shv_llm.h"

#include <cstdio>
#include <cstring>
#include <memory>

#include "llm.hpp"

struct shvllm {
    std::unique_ptr<llm::Device> dev;
    std::unique_ptr<llm::Model> model;
    std::unique_ptr<llm::Graph> graph;
    llm::GraphOpts opts;
    std::vector<std::string> names;
};

static thread_local char g_err[512] = "";

template <typename F>
static int guard(F &&f) {
    try {
        f();
        return 0;
    } catch (const std::exception &e) {
        std::snprintf(g_err, sizeof(g_err), "%s", e.what());
        return -1;
    }
}

static llm::Graph &graph_of(shvllm *h) {
    if (!h || !h->graph) throw llm::Error("llm: the graph has not been staged");
    return *h->graph;
}

extern "C" {

const char *shvllm_last_error(void) { return g_err; }

int shvllm_open(int device, const shvllm_config *c, shvllm **out) {
    return guard([&] {
        if (!c || !out) throw llm::Error("llm: shvllm_open: NULL argument");
        auto h = std::make_unique<shvllm>();
        h->dev = std::make_unique<llm::Device>(device);
        llm::Config cfg;
        cfg.NLayer = c->n_layer;
        cfg.NEmbd = c->n_embd;
        cfg.NHead = c->n_head;
        cfg.NHeadKV = c->n_head_kv;
        cfg.HeadDim = c->head_dim;
        cfg.RopeDims = c->rope_dims;
        cfg.RopeBase = c->rope_base;
        cfg.NExpert = c->n_expert;
        cfg.NExpertUsed = c->n_expert_used;
        cfg.FFNExpert = c->ffn_expert;
        cfg.VocabSize = c->vocab;
        cfg.RMSEps = c->rms_eps;
        cfg.SSMHeadDim = c->ssm_head_dim;
        cfg.SSMHeadK = c->ssm_head_k;
        cfg.SSMHeadV = c->ssm_head_v;
        cfg.SSMConv = c->ssm_conv;
        cfg.AttnEvery = c->attn_every;
        h->opts.NKV = c->nkv;
        h->opts.Layers = c->layers;
        h->opts.NoHead = c->no_head != 0;
        h->opts.AttnSplits = c->attn_splits;
        h->model = std::make_unique<llm::Model>(*h->dev, cfg);
        for (const auto &kv : h->model->Tensors()) h->names.push_back(kv.first);
        *out = h.release();
    });
}

void shvllm_close(shvllm *h) {
    if (!h) return;
    h->graph.reset();
    h->model.reset();
    h->dev.reset();
    delete h;
}

shv_ctx *shvllm_ctx(shvllm *h) { return h && h->dev ? h->dev->ctx() : nullptr; }

int shvllm_init_synthetic(shvllm *h, uint64_t seed) {
    return guard([&] { h->model->InitSynthetic(seed); });
}

int shvllm_tensor_count(shvllm *h) { return h ? static_cast<int>(h->names.size()) : 0; }

int shvllm_tensor_at(shvllm *h, int i, const char **name, void **dptr, uint64_t *bytes, int32_t *kind, int64_t *rows,
                     int64_t *cols, int32_t *is_alias) {
    return guard([&] {
        if (!h || i < 0 || i >= static_cast<int>(h->names.size())) throw llm::Error("llm: tensor index out of range");
        const llm::TensorView &t = h->model->Tensor(h->names[i]);
        if (name) *name = h->names[i].c_str();
        if (dptr) *dptr = t.ptr;
        if (bytes) *bytes = t.bytes;
        if (kind) *kind = static_cast<int32_t>(t.kind);
        if (rows) *rows = t.rows;
        if (cols) *cols = t.cols;
        if (is_alias) *is_alias = t.init_std < 0.f;
    });
}

int shvllm_tensor(shvllm *h, const char *name, void **dptr, uint64_t *bytes) {
    return guard([&] {
        const llm::TensorView &t = h->model->Tensor(name);
        if (dptr) *dptr = t.ptr;
        if (bytes) *bytes = t.bytes;
    });
}

uint64_t shvllm_weight_bytes(shvllm *h) { return h && h->model ? h->model->WeightBytes() : 0; }

int shvllm_stage(shvllm *h) {
    return guard([&] { h->graph = std::make_unique<llm::Graph>(*h->dev, *h->model, h->opts); });
}

int shvllm_reset(shvllm *h) {
    return guard([&] { graph_of(h).Reset(); });
}

int shvllm_extend(shvllm *h, const int32_t *ids, int n, float *logits, float *hidden) {
    return guard([&] {
        if (!ids || n < 1) throw llm::Error("llm: shvllm_extend: no tokens");
        std::vector<int32_t> v(ids, ids + n);
        std::vector<float> lg, hd;
        graph_of(h).Extend(v, logits ? &lg : nullptr, hidden ? &hd : nullptr);
        if (logits) std::memcpy(logits, lg.data(), lg.size() * 4);
        if (hidden) std::memcpy(hidden, hd.data(), hd.size() * 4);
    });
}

int shvllm_generate(shvllm *h, int n, int32_t *out_ids, uint64_t *gpu_nanos) {
    return guard([&] {
        auto ids = graph_of(h).Generate(n, gpu_nanos);
        if (out_ids) std::memcpy(out_ids, ids.data(), ids.size() * 4);
    });
}

int shvllm_past(shvllm *h) { return h && h->graph ? h->graph->Past() : -1; }
int shvllm_dispatches(shvllm *h) { return h && h->graph ? h->graph->Dispatches() : -1; }

int shvllm_profile_step(shvllm *h, char (*labels)[32], uint64_t *nanos, int max, int *n) {
    return guard([&] {
        auto st = graph_of(h).ProfileStep();
        int k = 0;
        for (const auto &s : st) {
            if (k >= max) break;
            std::snprintf(labels[k], 32, "%s", s.Kind.c_str());
            nanos[k] = s.GPUNanos;
            k++;
        }
        if (n) *n = k;
    });
}

int shvllm_dn_state(shvllm *h, int layer, float *dst) {
    return guard([&] {
        auto s = graph_of(h).DeltaNet().State(layer);
        std::memcpy(dst, s.data(), s.size() * 4);
    });
}

int shvllm_kv(shvllm *h, int layer, int cells, uint16_t *k, uint16_t *v) {
    return guard([&] {
        auto kk = graph_of(h).Attn().K(layer, cells);
        auto vv = graph_of(h).Attn().V(layer, cells);
        if (k) std::memcpy(k, kk.data(), kk.size() * 2);
        if (v) std::memcpy(v, vv.data(), vv.size() * 2);
    });
}

uint64_t shvllm_gpu_nanos(shvllm *h) { return h && h->graph ? h->graph->Stats.GPUNanos : 0; }

}  // extern "C"
