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
    std::unique_ptr<llm::MTPHead> mtp;
    std::unique_ptr<llm::Speculator> spec;
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
        cfg.NextN = c->nextn;
        h->opts.NKV = c->nkv;
        h->opts.Layers = c->layers;
        h->opts.NoHead = c->no_head != 0;
        h->opts.AttnSplits = c->attn_splits;
        h->opts.MaxTokens = c->max_tokens > 0 ? c->max_tokens : 1;
        h->opts.Slots = c->slots > 0 ? c->slots : 1;
        h->opts.HeadRows = c->head_rows;
        h->opts.Speculative = c->speculative != 0;
        if (c->spec_rows > 0) h->opts.SpecRows = c->spec_rows;
        h->model = std::make_unique<llm::Model>(*h->dev, cfg);
        for (const auto &kv : h->model->Tensors()) h->names.push_back(kv.first);
        *out = h.release();
    });
}

void shvllm_close(shvllm *h) {
    if (!h) return;
    h->spec.reset();
    h->mtp.reset();
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
    return guard([&] {
        h->spec.reset();
        h->mtp.reset();
        h->graph = std::make_unique<llm::Graph>(*h->dev, *h->model, h->opts);
    });
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

static void stages_out(const std::vector<llm::Stage> &st, char (*labels)[32], uint64_t *nanos, int max, int *n) {
    int k = 0;
    for (const auto &s : st) {
        if (k >= max) break;
        std::snprintf(labels[k], 32, "%s", s.Kind.c_str());
        nanos[k] = s.GPUNanos;
        k++;
    }
    if (n) *n = k;
}

int shvllm_extend_rows(shvllm *h, const int32_t *ids, int n, float *logits, float *res, int32_t *best) {
    return guard([&] {
        if (!ids || n < 1) throw llm::Error("llm: shvllm_extend_rows: no tokens");
        std::vector<float> lg, rs;
        graph_of(h).ExtendRows(std::vector<int32_t>(ids, ids + n), logits ? &lg : nullptr, res ? &rs : nullptr);
        if (logits) std::memcpy(logits, lg.data(), lg.size() * 4);
        if (res) std::memcpy(res, rs.data(), rs.size() * 4);
        if (best) {
            auto b = graph_of(h).Argmaxes();
            std::memcpy(best, b.data(), b.size() * 4);
        }
    });
}

int shvllm_decode_rows(shvllm *h, const int32_t *slots, const int32_t *ids, int n, float *logits, int32_t *best) {
    return guard([&] {
        if (!ids || !slots || n < 1) throw llm::Error("llm: shvllm_decode_rows: no rows");
        std::vector<float> lg;
        const bool single = n == 1;
        graph_of(h).DecodeRows(std::vector<int>(slots, slots + n), std::vector<int32_t>(ids, ids + n), logits ? &lg : nullptr);
        if (logits) std::memcpy(logits, lg.data(), lg.size() * 4);
        if (best) {
            auto b = graph_of(h).Argmaxes();
            std::memcpy(best, b.data(), (single ? 1 : b.size()) * 4);
        }
    });
}

int shvllm_use_slot(shvllm *h, int slot) {
    return guard([&] { graph_of(h).UseSlot(slot); });
}
int shvllm_speculate(shvllm *h, int on) {
    return guard([&] { graph_of(h).Speculate(on != 0); });
}
int shvllm_speculate_first(shvllm *h, int on) {
    return guard([&] { graph_of(h).SpeculateFirst(on != 0); });
}
int shvllm_keep(shvllm *h, int k) {
    return guard([&] { graph_of(h).Keep(k); });
}
int shvllm_commit(shvllm *h) {
    return guard([&] { graph_of(h).Commit(); });
}
int shvllm_checkpoint(shvllm *h, shvllm_checkpoint_t **out) {
    return guard([&] {
        auto c = std::make_unique<llm::Checkpoint>();
        graph_of(h).Checkpoint(*c);
        *out = reinterpret_cast<shvllm_checkpoint_t *>(c.release());
    });
}

int shvllm_restore(shvllm *h, const shvllm_checkpoint_t *c) {
    return guard([&] {
        if (!c) throw llm::Error("llm: no checkpoint");
        graph_of(h).Restore(*reinterpret_cast<const llm::Checkpoint *>(c));
    });
}

void shvllm_checkpoint_free(shvllm_checkpoint_t *c) { delete reinterpret_cast<llm::Checkpoint *>(c); }

int shvllm_rewind(shvllm *h) {
    return guard([&] { graph_of(h).Rewind(); });
}
int shvllm_plane(shvllm *h) { return h && h->graph ? h->graph->Plane() : -1; }

int shvllm_ids(shvllm *h, int32_t *dst, int max, int *n) {
    return guard([&] {
        auto v = graph_of(h).Ids();
        const int k = static_cast<int>(v.size()) < max ? static_cast<int>(v.size()) : max;
        if (dst && k > 0) std::memcpy(dst, v.data(), static_cast<size_t>(k) * 4);
        if (n) *n = static_cast<int>(v.size());
    });
}

int shvllm_dn_state_at(shvllm *h, int layer, int slot, int plane, float *dst) {
    return guard([&] {
        auto s = graph_of(h).DeltaNet().State(layer, slot, plane);
        std::memcpy(dst, s.data(), s.size() * 4);
    });
}

int shvllm_kv_at(shvllm *h, int layer, int slot, int cells, uint16_t *k, uint16_t *v) {
    return guard([&] {
        auto kk = graph_of(h).Attn().K(layer, cells, slot);
        auto vv = graph_of(h).Attn().V(layer, cells, slot);
        if (k) std::memcpy(k, kk.data(), kk.size() * 2);
        if (v) std::memcpy(v, vv.data(), vv.size() * 2);
    });
}

int shvllm_profile_rows(shvllm *h, int rows, char (*labels)[32], uint64_t *nanos, int max, int *n) {
    return guard([&] { stages_out(graph_of(h).ProfileRows(rows), labels, nanos, max, n); });
}

int shvllm_profile_chunk(shvllm *h, const int32_t *ids, int rows, char (*labels)[32], uint64_t *nanos, int max, int *n) {
    return guard([&] { stages_out(graph_of(h).ProfileChunk(std::vector<int32_t>(ids, ids + rows)), labels, nanos, max, n); });
}

static llm::MTPHead &mtp_of(shvllm *h) {
    if (!h || !h->mtp) throw llm::Error("llm: the draft head has not been staged");
    return *h->mtp;
}

static llm::Speculator &spec_of(shvllm *h) {
    if (!h || !h->spec) throw llm::Error("llm: no speculator has been opened");
    return *h->spec;
}

int shvllm_mtp_stage(shvllm *h, int max_tok, int vocab_prefix) {
    return guard([&] {
        llm::Graph &g = graph_of(h);
        h->spec.reset();
        h->mtp = std::make_unique<llm::MTPHead>(*h->dev, *h->model, g.Head(), max_tok, g.NKV(), g.Slots());
        h->mtp->SetVocab(vocab_prefix);
    });
}

int shvllm_mtp_rows(shvllm *h, const float *hs, const int32_t *ids, int n, int pos, int head, float *logits, float *res) {
    return guard([&] {
        if (!hs || !ids || n < 1) throw llm::Error("llm: shvllm_mtp_rows: no rows");
        const size_t E = h->model->config().NEmbd;
        std::vector<float> lg, rs;
        mtp_of(h).RowsHost(std::vector<float>(hs, hs + n * E), std::vector<int32_t>(ids, ids + n), pos, head != 0,
                           logits ? &lg : nullptr, res ? &rs : nullptr);
        if (logits && !lg.empty()) std::memcpy(logits, lg.data(), lg.size() * 4);
        if (res) std::memcpy(res, rs.data(), rs.size() * 4);
    });
}

int shvllm_mtp_rewind(shvllm *h, int n) {
    return guard([&] { mtp_of(h).Rewind(n); });
}
int shvllm_mtp_past(shvllm *h) { return h && h->mtp ? h->mtp->Past() : -1; }

int shvllm_spec_open(shvllm *h, int depth) {
    return guard([&] { h->spec = std::make_unique<llm::Speculator>(graph_of(h), mtp_of(h), depth); });
}

int shvllm_spec_start(shvllm *h, const int32_t *prompt, int n, int32_t *first) {
    return guard([&] {
        if (!prompt || n < 1) throw llm::Error("llm: shvllm_spec_start: no prompt");
        const int32_t t = spec_of(h).Start(std::vector<int32_t>(prompt, prompt + n));
        if (first) *first = t;
    });
}

int shvllm_spec_round(shvllm *h, const int32_t *forced, int n_forced, int32_t *out, int max, int *n_out) {
    return guard([&] {
        std::vector<int32_t> f;
        if (forced && n_forced > 0) f.assign(forced, forced + n_forced);
        auto v = spec_of(h).Round(f);
        if (static_cast<int>(v.size()) > max) throw llm::Error("llm: shvllm_spec_round: the round emitted more tokens than the caller has room for");
        if (out) std::memcpy(out, v.data(), v.size() * 4);
        if (n_out) *n_out = static_cast<int>(v.size());
    });
}

int shvllm_spec_stats(shvllm *h, int32_t *counts, uint64_t *nanos) {
    return guard([&] {
        const llm::SpecStats &s = spec_of(h).Stats;
        if (counts) {
            int k = 0;
            counts[k++] = s.Rounds;
            counts[k++] = s.Drafted;
            counts[k++] = s.Accepted;
            counts[k++] = s.Tokens;
            for (int i = 0; i < 5; i++) counts[k++] = s.Passes[i];
            for (int i = 0; i < 4; i++) counts[k++] = s.DraftedAt[i];
            for (int i = 0; i < 4; i++) counts[k++] = s.AcceptedAt[i];
        }
        if (nanos) {
            nanos[0] = s.DraftNanos;
            nanos[1] = s.VerifyNanos;
        }
    });
}

}  // extern "C"
