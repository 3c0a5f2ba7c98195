// Flat C entry points over llm::Graph for ctypes callers: see shv_llm.h.
#include "shv_llm.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <set>

#include "llm.hpp"
#include "sampler_handle.hpp"
#include "sched.hpp"
#include "text.hpp"

struct shvllm {
    std::unique_ptr<llm::Device> dev;
    std::unique_ptr<llm::Model> model;
    std::unique_ptr<llm::Graph> graph;
    std::unique_ptr<llm::MTPHead> mtp;
    std::unique_ptr<llm::Speculator> spec;
    std::unique_ptr<llm::Sampler> sampler;
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

static void graph_opts(shvllm &hh, const shvllm_config &cc) {
    shvllm *h = &hh;
    const shvllm_config *c = &cc;
    h->opts.NKV = c->nkv;
    h->opts.Layers = c->layers;
    h->opts.NoHead = c->no_head != 0;
    h->opts.AttnSplits = c->attn_splits;
    h->opts.MaxTokens = c->max_tokens > 0 ? c->max_tokens : 1;
    h->opts.Slots = c->slots > 0 ? c->slots : 1;
    h->opts.HeadRows = c->head_rows;
    h->opts.Speculative = c->speculative != 0;
    if (c->spec_rows > 0) h->opts.SpecRows = c->spec_rows;
}

template <typename T>
static int copy_out(const std::vector<T> *v, T *dst, uint64_t max) {
    if (!v || !dst) return 0;
    std::copy(v->begin(), v->begin() + std::min<uint64_t>(max, v->size()), dst);
    return 1;
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
        cfg.IdxHeads = c->idx_heads, cfg.IdxDim = c->idx_dim, cfg.IdxTopK = c->idx_top_k, cfg.IdxRatio = c->idx_ratio;
        graph_opts(*h, *c);
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

int shvllm_open_gguf(int device, const char *path, const shvllm_config *c, shvllm **out) {
    return guard([&] {
        if (!path || !c || !out) throw llm::Error("llm: shvllm_open_gguf: NULL argument");
        std::unique_ptr<gguf::Set> set = gguf::Set::Open(path);
        auto h = std::make_unique<shvllm>();
        h->dev = std::make_unique<llm::Device>(device);
        graph_opts(*h, *c);
        h->model = std::make_unique<llm::Model>(*h->dev, llm::Model::ConfigFromGGUF(*set));
        const char *tc = std::getenv("LLM_TRANSCODE");  // 0: refuse a matrix that is not Q4_K instead of fitting it again
        llm::Model::LoadOpts lo;
        lo.transcode = !(tc && tc[0] == '0');
        if (const char *ht = std::getenv("LLM_HEAD_TYPE")) {  // q4_k: the vocabulary projection refitted like every other dense matrix
            if (std::strcmp(ht, "q4_k") == 0) lo.head_native = false;
            else if (std::strcmp(ht, "own") != 0) throw llm::Error(std::string("llm: LLM_HEAD_TYPE=") + ht + "; own (the checkpoint's type, the default) or q4_k");
        }
        if (const char *plan = std::getenv("LLM_MOE_BANK")) lo.moe_plan = plan;  // family=q4_k,...: expert banks refitted instead of read natively
        if (const char *mode = std::getenv("LLM_MOE_BANK_QUANT"))
            if (std::strcmp(mode, "rtn") != 0) throw llm::Error(std::string("llm: LLM_MOE_BANK_QUANT=") + mode + "; banks are refitted round-to-nearest here (rtn), no importance matrix is read");
        h->model->LoadGGUF(*set, lo);
        for (const auto &kv : h->model->Tensors()) h->names.push_back(kv.first);
        *out = h.release();
    });
}

int shvllm_get_config(shvllm *h, shvllm_config *o) {
    return guard([&] {
        if (!h || !h->model || !o) throw llm::Error("llm: shvllm_get_config: NULL argument");
        const llm::Config &c = h->model->config();
        o->n_layer = c.NLayer, o->n_embd = c.NEmbd, o->n_head = c.NHead, o->n_head_kv = c.NHeadKV, o->head_dim = c.HeadDim;
        o->rope_dims = c.RopeDims, o->rope_base = c.RopeBase, o->n_expert = c.NExpert, o->n_expert_used = c.NExpertUsed;
        o->ffn_expert = c.FFNExpert, o->vocab = c.VocabSize, o->rms_eps = c.RMSEps, o->ssm_head_dim = c.SSMHeadDim;
        o->ssm_head_k = c.SSMHeadK, o->ssm_head_v = c.SSMHeadV, o->ssm_conv = c.SSMConv, o->attn_every = c.AttnEvery, o->nextn = c.NextN;
        o->nkv = h->opts.NKV, o->layers = h->opts.Layers, o->no_head = h->opts.NoHead, o->attn_splits = h->opts.AttnSplits;
        o->max_tokens = h->opts.MaxTokens, o->slots = h->opts.Slots, o->head_rows = h->opts.HeadRows;
        o->speculative = h->opts.Speculative, o->spec_rows = h->opts.SpecRows;
        o->idx_heads = c.IdxHeads, o->idx_dim = c.IdxDim, o->idx_top_k = c.IdxTopK, o->idx_ratio = c.IdxRatio;
    });
}

int shvllm_save_gguf(shvllm *h, const char *path) {
    return guard([&] {
        if (!h || !h->model || !path) throw llm::Error("llm: shvllm_save_gguf: NULL argument");
        h->model->SaveGGUF(path);
    });
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

int shvllm_tensor_type(shvllm *h, const char *name, int32_t *ggml_type) {
    return guard([&] {
        if (!h || !h->model || !name || !ggml_type) throw llm::Error("llm: shvllm_tensor_type: NULL argument");
        *ggml_type = static_cast<int32_t>(h->model->Tensor(name).ggml);
    });
}

int shvllm_transcoded(shvllm *h, char *buf, size_t cap) {
    if (!h || !h->model) return 0;
    const std::vector<std::string> &v = h->model->Transcoded();
    size_t at = 0;
    for (const std::string &n : v)
        for (size_t i = 0; i <= n.size() && buf && at + 1 < cap; i++) buf[at++] = i < n.size() ? n[i] : '\n';
    if (buf && cap) buf[at] = 0;
    return static_cast<int>(v.size());
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

int shvllm_spec_sampler(shvllm *h, float temp, int top_k, float top_p, float min_p, float repeat_penalty, float presence_penalty,
                        int64_t seed, int64_t draft_seed) {
    return guard([&] {
        llm::Speculator &sp = spec_of(h);
        h->sampler = std::make_unique<llm::Sampler>(temp, top_k, top_p, seed);
        h->sampler->MinP = min_p;
        h->sampler->RepeatPenalty = repeat_penalty;
        h->sampler->PresencePenalty = presence_penalty;
        sp.UseSampler(h->sampler.get(), draft_seed);
    });
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

// ---- the scheduler ------------------------------------------------------------------------------

struct shvllm_sched {
    std::unique_ptr<llm::Sched> s;
    llm::SchedPass last;  // what shvllm_sched_next handed out and shvllm_sched_finish books
};

static llm::Sched &sched_of(shvllm_sched *s) {
    if (!s || !s->s) throw llm::Error("llm: NULL scheduler");
    return *s->s;
}

static void pass_out(const llm::SchedPass &p, shvllm_sched_pass *o) {
    if (!o) return;
    std::memset(o, 0, sizeof(*o));
    o->kind = p.kind, o->unit = p.unit, o->slot = p.slot, o->pos = p.pos, o->n = p.n;
    o->fresh = p.fresh, o->restore = p.restore, o->take = p.take, o->step = p.step;
    o->wait_ms = p.wait_ms;
    o->prime = p.prime, o->tracked = p.tracked;
    o->n_units = static_cast<int32_t>(std::min<size_t>(p.units.size(), SHVLLM_SCHED_MAX_ROWS));
    for (int i = 0; i < o->n_units; i++) o->units[i] = p.units[i], o->slots[i] = p.slots[i];
}

int shvllm_sched_open(shvllm *h, int slots, const shvllm_sched_opts *opts, shvllm_sched **out) {
    return guard([&] {
        if (!out) throw llm::Error("llm: shvllm_sched_open: NULL argument");
        llm::SchedOpts o;
        if (opts) {
            if (opts->batch > 0) o.Batch = opts->batch;
            o.PreemptChunk = opts->preempt_chunk;
            o.Reserve = opts->reserve;
            o.NoBatchDecode = opts->no_batch_decode != 0;
            if (opts->coalesce_ms >= 0) o.CoalesceMs = opts->coalesce_ms;
            o.SpecDepth = opts->spec_depth;
        }
        llm::Graph *g = h ? &graph_of(h) : nullptr;
        if ((g ? g->Slots() : slots) > SHVLLM_SCHED_MAX_ROWS) throw llm::Error("llm: a scheduler covers at most " + std::to_string(SHVLLM_SCHED_MAX_ROWS) + " slots");
        auto s = std::make_unique<shvllm_sched>();
        s->s = std::make_unique<llm::Sched>(g, slots, o, h && o.SpecDepth > 0 ? &mtp_of(h) : nullptr);
        *out = s.release();
    });
}

void shvllm_sched_close(shvllm_sched *s) { delete s; }

int shvllm_sched_acquire(shvllm_sched *s, int cls, const int32_t *prompt, int n, int mark, double now_ms, int *job) {
    return guard([&] {
        if (!prompt || n < 1 || !job) throw llm::Error("llm: shvllm_sched_acquire: an empty prompt or NULL argument");
        *job = sched_of(s).Acquire(cls, std::vector<int32_t>(prompt, prompt + n), mark, now_ms);
    });
}

int shvllm_sched_release(shvllm_sched *s, int job, double now_ms) {
    return guard([&] { sched_of(s).Release(job, now_ms); });
}

int shvllm_sched_job_info(shvllm_sched *s, int job, shvllm_sched_job *out) {
    return guard([&] {
        if (!out) throw llm::Error("llm: shvllm_sched_job_info: NULL argument");
        const llm::SchedJobInfo j = sched_of(s).Job(job);
        out->cls = j.cls, out->slot = j.slot, out->reused = j.reused, out->restored = j.restored, out->stepping = j.stepping;
        out->served_ms = j.served_ms, out->arrival = j.arrival;
    });
}

int shvllm_sched_run(shvllm_sched *s, int job, const int32_t *ids, int n, int fresh, int *unit) {
    return guard([&] {
        if (!ids || n < 1 || !unit) throw llm::Error("llm: shvllm_sched_run: no ids or NULL argument");
        *unit = sched_of(s).Run(job, std::vector<int32_t>(ids, ids + n), fresh != 0);
    });
}

int shvllm_sched_step(shvllm_sched *s, int job, int32_t id, int *unit) {
    return guard([&] {
        if (!unit) throw llm::Error("llm: shvllm_sched_step: NULL argument");
        *unit = sched_of(s).Step(job, id);
    });
}

int shvllm_sched_decode(shvllm_sched *s, int job, int32_t id, int room, int *unit) {
    return guard([&] {
        if (!unit) throw llm::Error("llm: shvllm_sched_decode: NULL argument");
        *unit = sched_of(s).Decode(job, id, room);
    });
}

int shvllm_sched_decode_sampled(shvllm_sched *s, int job, int32_t id, int room, shvsampler *sampler, int exact, int64_t draft_seed, int *unit) {
    return guard([&] {
        if (!unit) throw llm::Error("llm: shvllm_sched_decode_sampled: NULL argument");
        *unit = sched_of(s).Decode(job, id, room, sampler ? &sampler->s : nullptr, exact != 0, draft_seed);
    });
}

int shvllm_sched_withdraw(shvllm_sched *s, int unit) {
    return guard([&] { sched_of(s).Withdraw(unit); });
}

int shvllm_sched_next(shvllm_sched *s, double now_ms, shvllm_sched_pass *out) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        if (s->last.kind != llm::SchedPass::kNone) throw llm::Error("llm: the last pass has not been finished");
        s->last = sc.Next(now_ms);
        pass_out(s->last, out);
    });
}

int shvllm_sched_finish(shvllm_sched *s, double took_ms, int ok, double now_ms) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        if (s->last.kind == llm::SchedPass::kNone) throw llm::Error("llm: no pass is out");
        if (s->last.kind == llm::SchedPass::kRound && ok) throw llm::Error("llm: a round is finished with its tokens (shvllm_sched_finish_round)");
        const llm::SchedPass p = s->last;
        s->last = llm::SchedPass();
        sc.Finish(p, took_ms, ok != 0, now_ms, nullptr, ok ? "" : "the caller's pass failed");
    });
}

int shvllm_sched_finish_round(shvllm_sched *s, double took_ms, int ok, double now_ms, const int32_t *toks, int n) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        if (s->last.kind != llm::SchedPass::kRound) throw llm::Error("llm: no round is out");
        if (ok && (!toks || n < 1)) throw llm::Error("llm: a finished round names its tokens");
        const llm::SchedPass p = s->last;
        s->last = llm::SchedPass();
        const std::vector<int32_t> t(toks, toks + (ok ? n : 0));
        sc.Finish(p, took_ms, ok != 0, now_ms, nullptr, ok ? "" : "the caller's round failed", &t);
    });
}

int shvllm_sched_pump(shvllm_sched *s, shvllm_sched_pass *out) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        if (s->last.kind != llm::SchedPass::kNone) throw llm::Error("llm: the last pass has not been finished");
        pass_out(sc.Pump(), out);
    });
}

int shvllm_sched_unit(shvllm_sched *s, int unit, int *state, int *left, double *busy_ms, float *logits, int max) {
    return guard([&] {
        const llm::Sched::UnitState u = sched_of(s).Unit(unit);
        if (!u.known) throw llm::Error("llm: no such unit " + std::to_string(unit));
        if (state) *state = !u.done ? 0 : (u.failed ? 2 : 1);
        if (left) *left = u.left;
        if (busy_ms) *busy_ms = u.busy_ms;
        if (u.failed) std::snprintf(g_err, sizeof(g_err), "%s", u.err.c_str());
        if (logits && u.done && !u.failed) std::copy(u.logits.begin(), u.logits.begin() + std::min<size_t>(max, u.logits.size()), logits);
    });
}

int shvllm_sched_unit_tokens(shvllm_sched *s, int unit, int32_t *dst, int max, int *n) {
    return guard([&] {
        const llm::Sched::UnitState u = sched_of(s).Unit(unit);
        if (!u.known) throw llm::Error("llm: no such unit " + std::to_string(unit));
        if (n) *n = static_cast<int>(u.toks.size());
        if (dst) std::copy(u.toks.begin(), u.toks.begin() + std::min<size_t>(max, u.toks.size()), dst);
    });
}

int shvllm_sched_forget(shvllm_sched *s, int unit) {
    return guard([&] { sched_of(s).Forget(unit); });
}

int shvllm_sched_counts(shvllm_sched *s, int32_t counts[6]) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        const llm::SchedCounts c = sc.Counts();
        counts[0] = c.restores, counts[1] = c.batches, counts[2] = c.batch_rows, counts[3] = c.passes;
        counts[4] = sc.Waiting(), counts[5] = sc.Pending();
    });
}

int shvllm_sched_held(shvllm_sched *s, int slot, int32_t *dst, int max, int *n, int *ckpt_len) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        if (slot < 0 || slot >= sc.Slots()) throw llm::Error("llm: slot " + std::to_string(slot));
        const std::vector<int32_t> &h = sc.Held(slot);
        if (n) *n = static_cast<int>(h.size());
        if (dst) std::copy(h.begin(), h.begin() + std::min<size_t>(max, h.size()), dst);
        if (ckpt_len) *ckpt_len = sc.CheckpointLen(slot);
    });
}

int shvllm_sched_round_counts(shvllm_sched *s, int32_t counts[2]) {
    return guard([&] {
        const llm::SchedCounts c = sched_of(s).Counts();
        counts[0] = c.rounds, counts[1] = c.round_tokens;
    });
}

int shvllm_sched_tracked(shvllm_sched *s, int slot, int *tracked) {
    return guard([&] {
        llm::Sched &sc = sched_of(s);
        if (slot < 0 || slot >= sc.Slots() || !tracked) throw llm::Error("llm: slot " + std::to_string(slot));
        *tracked = sc.Tracked(slot) ? 1 : 0;
    });
}

// ---- the GGUF container by itself ---------------------------------------------------------------

struct shvgguf {
    std::unique_ptr<gguf::Set> set;    // OpenSet
    std::unique_ptr<gguf::File> file;  // Open: one file, shards not joined
    std::vector<const gguf::Tensor *> tensors;
    const gguf::KV *kv = nullptr;
    const std::vector<std::string> *keys = nullptr;
};

static shvgguf &gg(shvgguf *g) {
    if (!g) throw gguf::Error("gguf: NULL handle");
    return *g;
}
static const gguf::Value *value_of(shvgguf *g, const char *key) { return g && key ? g->kv->Find(key) : nullptr; }

int shvgguf_open(const char *path, shvgguf **out) {
    return guard([&] {
        if (!path || !out) throw gguf::Error("gguf: NULL argument");
        auto g = std::make_unique<shvgguf>();
        g->set = gguf::Set::Open(path);
        g->tensors = g->set->Tensors;
        g->kv = g->set.get();
        g->keys = &g->set->Keys();
        *out = g.release();
    });
}

int shvgguf_open_file(const char *path, shvgguf **out) {
    return guard([&] {
        if (!path || !out) throw gguf::Error("gguf: NULL argument");
        auto g = std::make_unique<shvgguf>();
        g->file = gguf::File::Open(path);
        for (const gguf::Tensor &t : g->file->Tensors) g->tensors.push_back(&t);
        g->kv = g->file.get();
        g->keys = &g->file->Keys();
        *out = g.release();
    });
}

void shvgguf_close(shvgguf *g) { delete g; }
int shvgguf_files(shvgguf *g) { return !g ? 0 : g->set ? static_cast<int>(g->set->Files.size()) : 1; }

int shvgguf_file_info(shvgguf *g, int i, const char **path, uint32_t *version, uint64_t *alignment, int64_t *data_start) {
    return guard([&] {
        if (i < 0 || i >= shvgguf_files(g)) throw gguf::Error("gguf: file index out of range");
        const gguf::File &f = gg(g).set ? *g->set->Files[i] : *g->file;
        if (path) *path = f.Path.c_str();
        if (version) *version = f.Version;
        if (alignment) *alignment = f.Alignment;
        if (data_start) *data_start = f.DataStart;
    });
}

int shvgguf_len(shvgguf *g) { return g ? static_cast<int>(g->tensors.size()) : 0; }
int64_t shvgguf_params(shvgguf *g) {
    int64_t n = 0;
    if (g)
        for (const gguf::Tensor *t : g->tensors) n += t->Elems();
    return n;
}
int64_t shvgguf_bytes(shvgguf *g) {
    int64_t n = 0;
    if (g)
        for (const gguf::Tensor *t : g->tensors) n += static_cast<int64_t>(t->Bytes);
    return n;
}
const char *shvgguf_arch(shvgguf *g) {
    const gguf::Value *v = value_of(g, gguf::kKeyArchitecture);
    return v && v->kind == gguf::Value::Str ? v->s.c_str() : "";
}

int shvgguf_tensor_at(shvgguf *g, int i, const char **name, uint32_t *type, int32_t *n_dims, int64_t *dims, const void **data,
                      uint64_t *bytes, int32_t *shard, int64_t *rows, int64_t *row_bytes) {
    return guard([&] {
        if (i < 0 || i >= shvgguf_len(g)) throw gguf::Error("gguf: tensor index out of range");
        const gguf::Tensor &t = *gg(g).tensors[i];
        if (name) *name = t.Name.c_str();
        if (type) *type = t.Type;
        if (n_dims) *n_dims = static_cast<int32_t>(t.Dims.size());
        if (dims)
            for (size_t j = 0; j < t.Dims.size(); j++) dims[j] = t.Dims[j];
        if (data) *data = t.Data;
        if (bytes) *bytes = t.Bytes;
        if (shard) *shard = t.Shard;
        if (rows) *rows = t.Rows();
        if (row_bytes) *row_bytes = t.RowBytes();
    });
}

int shvgguf_find(shvgguf *g, const char *name) {
    if (!g || !name) return -1;
    for (size_t i = 0; i < g->tensors.size(); i++)
        if (g->tensors[i]->Name == name) return static_cast<int>(i);
    return -1;
}

int shvgguf_advise_random(shvgguf *g, int i) {
    return guard([&] {
        if (i < 0 || i >= shvgguf_len(g)) throw gguf::Error("gguf: tensor index out of range");
        gg(g).tensors[i]->AdviseRandom();
    });
}

int shvgguf_key_count(shvgguf *g) { return g ? static_cast<int>(g->keys->size()) : 0; }
const char *shvgguf_key_at(shvgguf *g, int i) { return g && i >= 0 && i < shvgguf_key_count(g) ? (*g->keys)[i].c_str() : nullptr; }
int shvgguf_kind(shvgguf *g, const char *key) {
    const gguf::Value *v = value_of(g, key);
    return v ? static_cast<int>(v->kind) : 0;
}
int shvgguf_uint(shvgguf *g, const char *key, uint64_t *out) { return g && key && out && g->kv->Uint(key, out); }
int shvgguf_int(shvgguf *g, const char *key, int64_t *out) { return g && key && out && g->kv->Int(key, out); }
int shvgguf_float(shvgguf *g, const char *key, double *out) { return g && key && out && g->kv->Float(key, out); }
int shvgguf_bool(shvgguf *g, const char *key, int32_t *out) {
    bool b = false;
    if (!g || !key || !out || !g->kv->Bool(key, &b)) return 0;
    *out = b;
    return 1;
}
int shvgguf_str(shvgguf *g, const char *key, const char **out, uint64_t *len) {
    const gguf::Value *v = value_of(g, key);
    if (!v || v->kind != gguf::Value::Str) return 0;
    if (out) *out = v->s.data();
    if (len) *len = v->s.size();
    return 1;
}
int shvgguf_array_len(shvgguf *g, const char *key, uint64_t *n) {
    const gguf::Value *v = value_of(g, key);
    if (!v || v->kind < gguf::Value::Uints) return 0;
    if (n) *n = v->Len();
    return 1;
}
int shvgguf_uints(shvgguf *g, const char *key, uint64_t *dst, uint64_t max) { return g && key ? copy_out(g->kv->Uints(key), dst, max) : 0; }
int shvgguf_ints(shvgguf *g, const char *key, int64_t *dst, uint64_t max) { return g && key ? copy_out(g->kv->Ints(key), dst, max) : 0; }
int shvgguf_floats(shvgguf *g, const char *key, double *dst, uint64_t max) { return g && key ? copy_out(g->kv->Floats(key), dst, max) : 0; }
int shvgguf_string_at(shvgguf *g, const char *key, uint64_t i, const char **out, uint64_t *len) {
    const std::vector<std::string> *v = g && key ? g->kv->Strings(key) : nullptr;
    if (!v || i >= v->size()) return 0;
    if (out) *out = (*v)[i].data();
    if (len) *len = (*v)[i].size();
    return 1;
}

const char *shvgguf_type_name(uint32_t type) {
    static thread_local std::string name;
    name = gguf::TypeName(type);
    return name.c_str();
}
int shvgguf_type_block(uint32_t type, int32_t *elems, int32_t *nbytes) {
    const gguf::TypeInfo *i = gguf::Info(type);
    if (!i) return 0;
    if (elems) *elems = i->elems;
    if (nbytes) *nbytes = i->nbytes;
    return 1;
}
int64_t shvgguf_size_of(uint32_t type, int64_t n) {
    int64_t out = -1;
    guard([&] { out = gguf::SizeOf(type, n); });
    return out;
}


// ---- text: tokenizer, stop set, chat template, completion reader ---------------------------------

struct shvtext_tokenizer {
    llm::text::Tokenizer tok;
};
struct shvtext_decoder {
    llm::text::ChatDecoder dec;
    std::string stopped;
};

static char *dup_bytes(const std::string &s, uint64_t *len) {
    char *p = static_cast<char *>(std::malloc(s.size() + 1));
    if (!p) throw std::bad_alloc();
    std::memcpy(p, s.data(), s.size());
    p[s.size()] = 0;
    if (len) *len = s.size();
    return p;
}
static std::string bytes_of(const char *p, uint64_t len) { return p ? std::string(p, static_cast<size_t>(len)) : std::string(); }
static std::vector<std::string> tools_of(const char *tools_json) {
    std::vector<std::string> tools;
    if (tools_json && *tools_json) {
        const llm::text::JValue v = llm::text::ParseJSON(tools_json);
        if (v.kind != llm::text::JValue::Array) throw llm::text::Error("llm: tools is not a JSON array");
        for (const auto &t : v.items) tools.push_back(t.raw);
    }
    return tools;
}

void shvtext_free(void *p) { std::free(p); }

int shvtext_tokenizer_from_vocab(const char *const *tokens, const uint64_t *token_len, int n_tokens, const char *const *merges,
                                 const uint64_t *merge_len, int n_merges, const int32_t *types, const char *const *specials,
                                 int n_specials, const char *pre, shvtext_tokenizer **out) {
    return guard([&] {
        if (!out || (n_tokens > 0 && (!tokens || !token_len)) || (n_merges > 0 && (!merges || !merge_len))) throw llm::text::Error("tokenizer: NULL argument");
        llm::text::Vocab v;
        for (int i = 0; i < n_tokens; i++) v.Tokens.emplace_back(tokens[i], static_cast<size_t>(token_len[i]));
        for (int i = 0; i < n_merges; i++) v.Merges.emplace_back(merges[i], static_cast<size_t>(merge_len[i]));
        if (types) v.Types.assign(types, types + n_tokens);
        for (int i = 0; i < n_specials; i++) v.Specials.emplace_back(specials[i]);
        if (pre) v.Pre = pre;
        *out = new shvtext_tokenizer{llm::text::Tokenizer::FromVocab(v)};
    });
}

int shvtext_tokenizer_from_gguf(shvgguf *g, shvtext_tokenizer **out, int32_t *eog, int eog_max, int *n_eog) {
    return guard([&] {
        if (!out) throw llm::text::Error("tokenizer: NULL argument");
        auto t = std::make_unique<shvtext_tokenizer>(shvtext_tokenizer{llm::text::Tokenizer::FromGGUF(*gg(g).kv)});
        const std::set<int32_t> stop = llm::text::EndOfGeneration(*gg(g).kv, t->tok);
        if (n_eog) *n_eog = static_cast<int>(stop.size());
        int k = 0;
        for (int32_t id : stop)
            if (eog && k < eog_max) eog[k++] = id;
        *out = t.release();
    });
}

void shvtext_tokenizer_free(shvtext_tokenizer *t) { delete t; }
int shvtext_tokenizer_size(shvtext_tokenizer *t) { return t ? t->tok.Size() : 0; }
int shvtext_tokenizer_id(shvtext_tokenizer *t, const char *token, int32_t *id) {
    int32_t v = -1;
    const bool ok = t && token && t->tok.ID(token, &v);
    if (id) *id = v;
    return ok ? 1 : 0;
}

int shvtext_encode(shvtext_tokenizer *t, const char *text, uint64_t len, int32_t **ids, int *n) {
    return guard([&] {
        if (!t || !ids || !n) throw llm::text::Error("tokenizer: NULL argument");
        const std::vector<int32_t> v = t->tok.Encode(bytes_of(text, len));
        int32_t *p = static_cast<int32_t *>(std::malloc((v.size() + 1) * sizeof(int32_t)));
        if (!p) throw std::bad_alloc();
        std::copy(v.begin(), v.end(), p);
        *ids = p;
        *n = static_cast<int>(v.size());
    });
}

int shvtext_decode(shvtext_tokenizer *t, const int32_t *ids, int n, char **out, uint64_t *len) {
    return guard([&] {
        if (!t || !out || (n > 0 && !ids)) throw llm::text::Error("tokenizer: NULL argument");
        *out = dup_bytes(t->tok.Decode(std::vector<int32_t>(ids, ids + n)), len);
    });
}

int shvtext_split(const char *text, uint64_t len, int marks, char **out, uint64_t *out_len, int32_t **piece_len, int *n) {
    return guard([&] {
        if (!out || !piece_len || !n) throw llm::text::Error("tokenizer: NULL argument");
        const std::vector<std::string> pieces = llm::text::Split(bytes_of(text, len), marks != 0);
        std::string all;
        int32_t *lens = static_cast<int32_t *>(std::malloc((pieces.size() + 1) * sizeof(int32_t)));
        if (!lens) throw std::bad_alloc();
        for (size_t i = 0; i < pieces.size(); i++) {
            all += pieces[i];
            lens[i] = static_cast<int32_t>(pieces[i].size());
        }
        *out = dup_bytes(all, out_len);
        *piece_len = lens;
        *n = static_cast<int>(pieces.size());
    });
}

int shvtext_pyjson(const char *raw, char **out) {
    return guard([&] {
        if (!raw || !out) throw llm::text::Error("llm: NULL argument");
        *out = dup_bytes(llm::text::PyJSON(raw), nullptr);
    });
}

int shvtext_parse_tool_arguments(const char *s, char **out_json) {
    return guard([&] {
        if (!s || !out_json) throw llm::text::Error("llm: NULL argument");
        std::string j = "[";
        bool first = true;
        for (const llm::text::ChatArg &a : llm::text::ParseToolArguments(s)) {
            if (!first) j += ',';
            first = false;
            j += "{\"name\":" + llm::text::GoJSONString(a.Name) + ",\"value\":" + a.Value + "}";
        }
        j += ']';
        *out_json = dup_bytes(j, nullptr);
    });
}

int shvtext_render_chat(const char *request_json, char **out) {
    return guard([&] {
        using llm::text::JValue;
        if (!request_json || !out) throw llm::text::Error("llm: NULL argument");
        const JValue req = llm::text::ParseJSON(request_json);
        const auto str = [](const JValue *v) { return v && v->kind == JValue::String ? v->str : std::string(); };
        const auto flag = [](const JValue *v) { return v && v->kind == JValue::Bool && v->b; };
        std::vector<llm::text::ChatMessage> msgs;
        if (const JValue *ms = req.Get("messages"))
            for (const JValue &m : ms->items) {
                llm::text::ChatMessage msg;
                msg.Role = str(m.Get("role"));
                msg.Content = str(m.Get("content"));
                msg.Reasoning = str(m.Get("reasoning"));
                if (const JValue *parts = m.Get("parts"))
                    if (parts->kind == JValue::Array) {
                        msg.HasParts = true;
                        for (const JValue &p : parts->items) msg.Parts.push_back({str(p.Get("text")), flag(p.Get("image"))});
                    }
                if (const JValue *calls = m.Get("tool_calls"))
                    for (const JValue &c : calls->items) {
                        llm::text::ChatToolCall call;
                        call.Name = str(c.Get("name"));
                        if (const JValue *args = c.Get("args"))
                            for (const JValue &a : args->items) {
                                const JValue *val = a.Get("value");
                                call.Args.push_back({str(a.Get("name")), val ? val->raw : std::string()});
                            }
                        msg.ToolCalls.push_back(call);
                    }
                msgs.push_back(msg);
            }
        llm::text::ChatOpts opt;
        if (const JValue *tools = req.Get("tools"))
            for (const JValue &t : tools->items) opt.Tools.push_back(t.raw);
        if (const JValue *o = req.Get("opts")) {
            opt.Effort = str(o->Get("effort"));
            opt.NoThinking = flag(o->Get("no_thinking"));
            opt.DropThinking = flag(o->Get("drop_thinking"));
            opt.NoGenerationPrompt = flag(o->Get("no_generation_prompt"));
            opt.AddVisionID = flag(o->Get("add_vision_id"));
        }
        *out = dup_bytes(llm::text::RenderChat(msgs, opt), nullptr);
    });
}

int shvtext_decoder_new(const char *tools_json, int thinking, shvtext_decoder **out) {
    return guard([&] {
        if (!out) throw llm::text::Error("llm: NULL argument");
        *out = new shvtext_decoder{llm::text::ChatDecoder(tools_of(tools_json), thinking != 0), std::string()};
    });
}
void shvtext_decoder_free(shvtext_decoder *d) { delete d; }
int shvtext_decoder_stop_at(shvtext_decoder *d, const char *const *seqs, const uint64_t *lens, int n) {
    return guard([&] {
        if (!d || (n > 0 && (!seqs || !lens))) throw llm::text::Error("llm: NULL argument");
        std::vector<std::string> v;
        for (int i = 0; i < n; i++) v.emplace_back(seqs[i], static_cast<size_t>(lens[i]));
        d->dec.StopAt(v);
    });
}
const char *shvtext_decoder_stopped(shvtext_decoder *d, uint64_t *len) {
    if (!d) return "";
    d->stopped = d->dec.Stopped();
    if (len) *len = d->stopped.size();
    return d->stopped.c_str();
}
int shvtext_decoder_write(shvtext_decoder *d, const char *piece, uint64_t len, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len) {
    return guard([&] {
        if (!d || !reasoning || !content) throw llm::text::Error("llm: NULL argument");
        std::string r, c;
        d->dec.Write(bytes_of(piece, len), &r, &c);
        *reasoning = dup_bytes(r, r_len);
        *content = dup_bytes(c, c_len);
    });
}
int shvtext_decoder_close(shvtext_decoder *d, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len, char **calls_json) {
    return guard([&] {
        if (!d || !reasoning || !content || !calls_json) throw llm::text::Error("llm: NULL argument");
        std::string r, c;
        std::vector<llm::text::ChatCall> calls;
        d->dec.Close(&r, &c, &calls);
        std::string j = "[";
        for (size_t i = 0; i < calls.size(); i++) {
            if (i) j += ',';
            j += "{\"name\":" + llm::text::GoJSONString(calls[i].Name) + ",\"arguments\":" + llm::text::GoJSONString(calls[i].Arguments) + "}";
        }
        j += ']';
        *reasoning = dup_bytes(r, r_len);
        *content = dup_bytes(c, c_len);
        *calls_json = dup_bytes(j, nullptr);
    });
}

struct shvtext_stream {
    llm::text::ChatStream st;
    std::string stopped;
};

int shvtext_stream_new(shvtext_tokenizer *t, const int32_t *eog, int n_eog, const char *tools_json, int thinking, shvtext_stream **out) {
    return guard([&] {
        if (!t || !out || (n_eog > 0 && !eog)) throw llm::text::Error("llm: NULL argument");
        *out = new shvtext_stream{llm::text::ChatStream(&t->tok, std::set<int32_t>(eog, eog + n_eog), tools_of(tools_json), thinking != 0), std::string()};
    });
}
void shvtext_stream_free(shvtext_stream *s) { delete s; }
int shvtext_stream_stop_at(shvtext_stream *s, const char *const *seqs, const uint64_t *lens, int n) {
    return guard([&] {
        if (!s || (n > 0 && (!seqs || !lens))) throw llm::text::Error("llm: NULL argument");
        std::vector<std::string> v;
        for (int i = 0; i < n; i++) v.emplace_back(seqs[i], static_cast<size_t>(lens[i]));
        s->st.StopAt(v);
    });
}
int shvtext_stream_push(shvtext_stream *s, int32_t id, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len, int *finish) {
    return guard([&] {
        if (!s || !reasoning || !content || !finish) throw llm::text::Error("llm: NULL argument");
        std::string r, c;
        *finish = static_cast<int>(s->st.Push(id, &r, &c));
        *reasoning = dup_bytes(r, r_len);
        *content = dup_bytes(c, c_len);
    });
}
const char *shvtext_stream_stopped(shvtext_stream *s, uint64_t *len) {
    if (!s) return "";
    s->stopped = s->st.Stopped();
    if (len) *len = s->stopped.size();
    return s->stopped.c_str();
}
int shvtext_stream_close(shvtext_stream *s, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len, char **calls_json) {
    return guard([&] {
        if (!s || !reasoning || !content || !calls_json) throw llm::text::Error("llm: NULL argument");
        std::string r, c;
        std::vector<llm::text::ChatCall> calls;
        s->st.Close(&r, &c, &calls);
        std::string j = "[";
        for (size_t i = 0; i < calls.size(); i++) {
            if (i) j += ',';
            j += "{\"name\":" + llm::text::GoJSONString(calls[i].Name) + ",\"arguments\":" + llm::text::GoJSONString(calls[i].Arguments) + "}";
        }
        j += ']';
        *reasoning = dup_bytes(r, r_len);
        *content = dup_bytes(c, c_len);
        *calls_json = dup_bytes(j, nullptr);
    });
}

}  // extern "C"
