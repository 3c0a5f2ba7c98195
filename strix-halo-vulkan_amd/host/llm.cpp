// Host side of the token loop above the C ABI: see llm.hpp.
#include "llm.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>

namespace llm {

void check(int rc, const char *what) {
    if (rc != SHV_OK) throw Error(std::string("llm: ") + what + ": " + shv_last_error());
}

static uint64_t q4k_bytes(int64_t rows, int64_t cols) { return rows * (cols / SHV_Q4K_BLOCK) * SHV_Q4K_BYTES; }

// ------------------------------------------------------------------------------- Device -------

Device::Device(int index) { check(shv_init(index, &ctx_), "NewDevice"); }

Device::~Device() {
    if (!ctx_) return;
    shv_sync(ctx_);
    for (void *p : owned_) shv_free(ctx_, p);
    for (void *p : host_owned_) shv_host_free(ctx_, p);
    shv_destroy(ctx_);
}

void *Device::host_alloc(size_t bytes) {
    void *p = nullptr;
    check(shv_host_alloc(ctx_, bytes, &p), "host_alloc");
    std::memset(p, 0, bytes);
    host_owned_.push_back(p);
    return p;
}

void *Device::alloc(size_t bytes) {
    void *p = nullptr;
    check(shv_alloc(ctx_, bytes < 256 ? 256 : bytes, &p), "alloc");
    owned_.push_back(p);
    allocated_ += bytes;
    return p;
}

void Device::release(void *p, size_t bytes) {
    auto it = std::find(owned_.begin(), owned_.end(), p);
    if (it == owned_.end()) throw Error("llm: release of memory this device did not hand out");
    sync();
    check(shv_free(ctx_, p), "free");
    owned_.erase(it);
    allocated_ -= bytes;
}

void *Device::alloc_zero(size_t bytes) {
    void *p = alloc(bytes);
    zero(p, bytes < 256 ? 256 : bytes);
    return p;
}

// small transfers (a pass's control words and ids) do not wait for the device; everything here runs on this
// device's one stream, which orders them
void Device::upload(void *dst, const void *src, size_t bytes) { check(shv_upload_async(ctx_, dst, src, bytes), "upload"); }
void Device::download(void *dst, const void *src, size_t bytes) { check(shv_download(ctx_, dst, src, bytes), "download"); }
void Device::zero(void *dst, size_t bytes) { check(shv_zero(ctx_, dst, bytes), "zero"); }
void Device::sync() { check(shv_sync(ctx_), "sync"); }

void Device::run(const std::vector<shv_op> &ops) {
    uint64_t ns = 0;
    check(shv_dispatch_multi(ctx_, ops.data(), static_cast<int>(ops.size()), 1, &ns, nullptr), "dispatch");
}

// -------------------------------------------------------------------------------- Model -------

std::string Model::Blk(int layer, const char *name) {
    char buf[96];
    std::snprintf(buf, sizeof(buf), "blk.%d.%s.weight", layer, name);
    return buf;
}

void Model::add(const std::string &name, TensorView::Kind kind, int64_t rows, int64_t cols, float mean, float std) {
    TensorView t;
    t.kind = kind;
    t.rows = rows;
    t.cols = cols;
    t.init_mean = mean;
    t.init_std = std;
    if (kind == TensorView::Q4K) {
        if (cols % SHV_Q4K_BLOCK != 0) throw Error("llm: " + name + ": a Q4_K row of " + std::to_string(cols) + " is not whole super-blocks");
        t.bytes = q4k_bytes(rows, cols);
    } else {
        t.bytes = static_cast<uint64_t>(rows) * cols * (kind == TensorView::F16 ? 2 : 4);
    }
    t.ggml = kind == TensorView::Q4K ? gguf::Q4_K : kind == TensorView::F16 ? gguf::F16 : gguf::F32;
    t.ptr = dev_.alloc(t.bytes);
    tensors_[name] = t;
}

// A named window of rows inside a fused tensor: the projection the GEMV streams is one matrix,
// and its GGUF constituents stay addressable by their own names.
void Model::alias(const std::string &name, const std::string &of, int64_t row0, int64_t rows) {
    const TensorView &base = tensors_.at(of);
    TensorView t = base;
    const uint64_t row_bytes = base.bytes / base.rows;
    t.ptr = static_cast<char *>(base.ptr) + row0 * row_bytes;
    t.rows = rows;
    t.bytes = rows * row_bytes;
    t.init_std = -1.f;  // initialised through the fused tensor
    tensors_[name] = t;
}

Model::Model(Device &dev, const Config &cfg) : dev_(dev), cfg_(cfg) {
    const Config &c = cfg_;
    if (c.NEmbd % SHV_Q4K_BLOCK || c.FFNExpert % SHV_Q4K_BLOCK || c.VWidth() % SHV_Q4K_BLOCK || (c.NHead * c.HeadDim) % SHV_Q4K_BLOCK)
        throw Error("llm: every Q4_K row length must be a multiple of 256");
    if (c.NHead % c.NHeadKV || c.SSMHeadV % c.SSMHeadK) throw Error("llm: head counts do not divide");
    add("token_embd.weight", TensorView::F16, c.VocabSize, c.NEmbd, 0.f, 1.f);
    add("output_norm.weight", TensorView::F32, 1, c.NEmbd, 1.f, 0.1f);
    add("output.weight", TensorView::Q4K, c.VocabSize, c.NEmbd, 0.f, 0.02f);
    if (c.NextN < 0 || c.NextN > 1) throw Error("llm: nextn_predict_layers " + std::to_string(c.NextN) + "; one draft block at most");
    if (c.IdxRatio < 0 || (c.IdxRatio > 0 && (c.IdxHeads < 1 || c.IdxHeads > 8 || c.IdxDim < 64 || c.IdxDim > 256 || c.IdxDim % 64 || c.IdxTopK < 1 || 32 % c.IdxRatio)))
        throw Error("llm: indexer of " + std::to_string(c.IdxHeads) + " heads x " + std::to_string(c.IdxDim) + ", top " + std::to_string(c.IdxTopK) + ", ratio " +
                    std::to_string(c.IdxRatio) + "; 1..8 heads of 64..256 dims, a ratio that divides 32");
    for (int l = 0; l < c.Blocks(); l++) {
        if (l >= c.NLayer) {
            // the draft block's own tensors (llm/mtp.go:36-53): the two input norms side by side
            // so that one projection prologue reads them, eh_proj [NEmbd][2*NEmbd], the head norm
            add(Blk(l, "nextn.ehnorm_fused"), TensorView::F32, 2, c.NEmbd, 1.f, 0.1f);
            alias(Blk(l, "nextn.enorm"), Blk(l, "nextn.ehnorm_fused"), 0, 1);
            alias(Blk(l, "nextn.hnorm"), Blk(l, "nextn.ehnorm_fused"), 1, 1);
            add(Blk(l, "nextn.eh_proj"), TensorView::Q4K, c.NEmbd, 2 * c.NEmbd, 0.f, 0.02f);
            add(Blk(l, "nextn.shared_head_norm"), TensorView::F32, 1, c.NEmbd, 1.f, 0.1f);
        }
        add(Blk(l, "attn_norm"), TensorView::F32, 1, c.NEmbd, 1.f, 0.1f);
        add(Blk(l, "post_attention_norm"), TensorView::F32, 1, c.NEmbd, 1.f, 0.1f);
        if (c.IsAttn(l)) {
            // fused rows: q|gate per head, then k, then v (llm/attn.go:77-94)
            add(Blk(l, "attn_qkv_fused"), TensorView::Q4K, c.AttnFusedRows(), c.NEmbd, 0.f, 0.02f);
            const int qrows = c.NHead * 2 * c.HeadDim, kvrows = c.NHeadKV * c.HeadDim;
            alias(Blk(l, "attn_q"), Blk(l, "attn_qkv_fused"), 0, qrows);
            alias(Blk(l, "attn_k"), Blk(l, "attn_qkv_fused"), qrows, kvrows);
            alias(Blk(l, "attn_v"), Blk(l, "attn_qkv_fused"), qrows + kvrows, kvrows);
            add(Blk(l, "attn_output"), TensorView::Q4K, c.NEmbd, c.NHead * c.HeadDim, 0.f, 0.02f);
            add(Blk(l, "attn_q_norm"), TensorView::F32, 1, c.HeadDim, 1.f, 0.1f);
            add(Blk(l, "attn_k_norm"), TensorView::F32, 1, c.HeadDim, 1.f, 0.1f);
            if (c.QSA(l)) {
                // the indexer's projections (llm/model.go:409-424), float32 and one matrix: four
                // query heads, then the key
                add(Blk(l, "indexer.qk_fused"), TensorView::F32, c.IdxRows(), c.NEmbd, 0.f, 0.02f);
                alias(Blk(l, "indexer.q_proj"), Blk(l, "indexer.qk_fused"), 0, c.IdxHeads * c.IdxDim);
                alias(Blk(l, "indexer.k_proj"), Blk(l, "indexer.qk_fused"), c.IdxHeads * c.IdxDim, c.IdxDim);
                add(Blk(l, "indexer.q_norm"), TensorView::F32, 1, c.IdxDim, 1.f, 0.1f);
                add(Blk(l, "indexer.k_norm"), TensorView::F32, 1, c.IdxDim, 1.f, 0.1f);
            }
        } else {
            // fused rows: qkv | z | alpha | beta (llm/deltanet.go:135-154)
            add(Blk(l, "ssm_in_fused"), TensorView::Q4K, c.DNFusedRows(), c.NEmbd, 0.f, 0.02f);
            alias(Blk(l, "attn_qkv"), Blk(l, "ssm_in_fused"), 0, c.ConvWidth());
            alias(Blk(l, "attn_gate"), Blk(l, "ssm_in_fused"), c.ConvWidth(), c.VWidth());
            alias(Blk(l, "ssm_alpha"), Blk(l, "ssm_in_fused"), c.ConvWidth() + c.VWidth(), c.SSMHeadV);
            alias(Blk(l, "ssm_beta"), Blk(l, "ssm_in_fused"), c.ConvWidth() + c.VWidth() + c.SSMHeadV, c.SSMHeadV);
            add(Blk(l, "ssm_out"), TensorView::Q4K, c.NEmbd, c.VWidth(), 0.f, 0.02f);
            add(Blk(l, "ssm_conv1d"), TensorView::F32, c.ConvWidth(), c.SSMConv, 0.f, 0.3f);
            add(Blk(l, "ssm_a"), TensorView::F32, 1, c.SSMHeadV, 0.f, 1.f);  // stored as -exp(.)
            add(Blk(l, "ssm_dt"), TensorView::F32, 1, c.SSMHeadV, 0.f, 1.f);
            add(Blk(l, "ssm_norm"), TensorView::F32, 1, c.SSMHeadDim, 1.f, 0.1f);
        }
        add(Blk(l, "ffn_gate_inp"), TensorView::F32, c.NExpert, c.NEmbd, 0.f, 0.02f);
        add(Blk(l, "ffn_gate_inp_shexp"), TensorView::F32, 1, c.NEmbd, 0.f, 0.02f);
        add(Blk(l, "ffn_gate_exps"), TensorView::Q4K, static_cast<int64_t>(c.NExpert) * c.FFNExpert, c.NEmbd, 0.f, 0.02f);
        add(Blk(l, "ffn_up_exps"), TensorView::Q4K, static_cast<int64_t>(c.NExpert) * c.FFNExpert, c.NEmbd, 0.f, 0.02f);
        add(Blk(l, "ffn_down_exps"), TensorView::Q4K, static_cast<int64_t>(c.NExpert) * c.NEmbd, c.FFNExpert, 0.f, 0.02f);
        add(Blk(l, "ffn_gate_shexp"), TensorView::Q4K, c.FFNExpert, c.NEmbd, 0.f, 0.02f);
        add(Blk(l, "ffn_up_shexp"), TensorView::Q4K, c.FFNExpert, c.NEmbd, 0.f, 0.02f);
        add(Blk(l, "ffn_down_shexp"), TensorView::Q4K, c.NEmbd, c.FFNExpert, 0.f, 0.02f);
    }
}

const TensorView &Model::Tensor(const std::string &name) const {
    auto it = tensors_.find(name);
    if (it == tensors_.end()) throw Error("llm: no tensor " + name);
    return it->second;
}

uint64_t Model::WeightBytes() const {
    uint64_t n = 0;
    for (const auto &kv : tensors_)
        if (kv.second.init_std >= 0.f) n += kv.second.bytes;
    return n;
}

void Model::InitSynthetic(uint64_t seed) {
    // float32 staging for the quantiser, reused: 64 Mi weights at a time
    const int64_t chunk = 64ll << 20;
    float *stage = nullptr;
    check(shv_alloc(dev_.ctx(), chunk * sizeof(float), reinterpret_cast<void **>(&stage)), "staging");
    uint64_t n = 0;
    for (const auto &kv : tensors_) {
        const TensorView &t = kv.second;
        if (t.init_std < 0.f) continue;
        const uint64_t s = seed * 1000003ull + (++n);
        if (t.kind == TensorView::Q4K) {
            const int64_t rows_per = std::max<int64_t>(1, chunk / t.cols);
            for (int64_t r0 = 0; r0 < t.rows; r0 += rows_per) {
                const int64_t rows = std::min(rows_per, t.rows - r0);
                shv_fill_normal_args f{stage, rows * t.cols, s + static_cast<uint64_t>(r0) * 7919ull, t.init_mean, t.init_std, 0};
                check(shv_fill_normal(dev_.ctx(), &f), "fill");
                shv_quantize_q4k_args q{stage, static_cast<char *>(t.ptr) + q4k_bytes(r0, t.cols), rows, static_cast<int32_t>(t.cols)};
                check(shv_quantize_q4k(dev_.ctx(), &q), "quantise");
            }
        } else if (kv.first.find("ssm_a") != std::string::npos) {
            // -exp(N(0,1)): the converter stores ssm_a already negated and exponentiated
            std::mt19937_64 rng(s);
            std::normal_distribution<float> nd(0.f, 1.f);
            std::vector<float> v(t.rows * t.cols);
            for (float &x : v) x = -std::exp(nd(rng));
            dev_.upload(t.ptr, v.data(), t.bytes);
        } else {
            shv_fill_normal_args f{t.ptr, t.rows * t.cols, s, t.init_mean, t.init_std, t.kind == TensorView::F16 ? 1 : 0};
            check(shv_fill_normal(dev_.ctx(), &f), "fill");
        }
    }
    dev_.sync();
    shv_free(dev_.ctx(), stage);
}

// The fused tensor a window of rows belongs to, by address.
const std::string *Model::base_of(const TensorView &alias) const {
    for (const auto &kv : tensors_) {
        const TensorView &b = kv.second;
        if (b.init_std < 0.f) continue;
        const char *p = static_cast<const char *>(alias.ptr), *lo = static_cast<const char *>(b.ptr);
        if (p >= lo && p < lo + b.bytes) return &kv.first;
    }
    return nullptr;
}

Config Model::ConfigFromGGUF(const gguf::Set &s) {
    const std::string arch = s.Arch();
    if (arch.empty()) throw Error("llm: checkpoint states no general.architecture");
    Config c;
    auto want = [&](const char *k, int *dst) {
        uint64_t v;
        if (!s.Uint(arch + "." + k, &v)) throw Error("llm: the checkpoint states no " + arch + "." + k);
        *dst = static_cast<int>(v);
    };
    auto may = [&](const char *k, int *dst) {
        uint64_t v;
        if (s.Uint(arch + "." + k, &v)) *dst = static_cast<int>(v);
    };
    int blocks = 0;
    want("block_count", &blocks);
    want("embedding_length", &c.NEmbd);
    want("attention.head_count", &c.NHead);
    want("attention.head_count_kv", &c.NHeadKV);
    want("attention.key_length", &c.HeadDim);
    want("rope.dimension_count", &c.RopeDims);
    want("expert_count", &c.NExpert);
    want("expert_used_count", &c.NExpertUsed);
    want("expert_feed_forward_length", &c.FFNExpert);
    want("ssm.state_size", &c.SSMHeadDim);
    want("ssm.group_count", &c.SSMHeadK);
    want("ssm.time_step_rank", &c.SSMHeadV);
    want("ssm.conv_kernel", &c.SSMConv);
    may("full_attention_interval", &c.AttnEvery);
    c.NextN = 0;
    may("nextn_predict_layers", &c.NextN);
    c.NLayer = blocks - c.NextN;  // block_count counts the draft block (llm/mtp.go:137)
    // llm/model.go:385-405: the indexer's shape, and one compress ratio for the layers that have one
    // (the per-layer array's non-zero entries must agree; a scalar key is read too)
    may("attention.indexer.head_count", &c.IdxHeads);
    may("attention.indexer.key_length", &c.IdxDim);
    may("attention.indexer.top_k", &c.IdxTopK);
    may("attention.compress_ratio", &c.IdxRatio);
    if (const std::vector<int64_t> *cr = s.Ints(arch + ".attention.compress_ratios")) {
        for (size_t l = 0; l < cr->size(); l++) {
            const int r = static_cast<int>((*cr)[l]);
            if (r == 0) continue;
            if (c.IdxRatio != 0 && c.IdxRatio != r) throw Error("llm: attention.compress_ratios names " + std::to_string(c.IdxRatio) + " and " + std::to_string(r) + "; one ratio for all indexed layers is what is built");
            c.IdxRatio = r;
        }
    }
    if (c.IdxHeads == 0 || c.IdxDim == 0 || c.IdxTopK == 0) c.IdxRatio = 0;
    double f;
    if (s.Float(arch + ".attention.layer_norm_rms_epsilon", &f)) c.RMSEps = static_cast<float>(f);
    if (s.Float(arch + ".rope.freq_base", &f)) c.RopeBase = static_cast<float>(f);
    if (!s.Has("token_embd.weight") || s.Get("token_embd.weight").Dims.size() < 2) throw Error("llm: the checkpoint has no 2-D token_embd.weight to read the vocabulary from");
    c.VocabSize = static_cast<int>(s.Get("token_embd.weight").Dims[1]);
    return c;
}

// The ggml types shv_dequant, shv_gemv and the typed embedding gather read (gguf/dequant.go:52-98).
static bool device_expands(uint32_t t) {
    switch (t) {
        case gguf::F32: case gguf::F16: case gguf::BF16: case gguf::Q8_0: case gguf::Q4_1: case gguf::Q5_0: case gguf::Q5_1:
        case gguf::IQ4_NL: case gguf::Q4_K: case gguf::Q5_K: case gguf::Q6_K: return true;
    }
    return false;
}

// ParseMoEBankPlan (llm/moebank.go:165-215) for the one target this build fits banks to: the
// families a plan narrows to Q4_K, by the tensor suffix each selects.
static std::vector<std::string> moe_plan_families(const std::string &spec) {
    static const char *const fam[6] = {"gate_exps", "up_exps", "down_exps", "gate_shexp", "up_shexp", "down_shexp"};
    std::vector<std::string> out;
    size_t at = 0;
    while (at < spec.size()) {
        size_t end = spec.find(',', at);
        if (end == std::string::npos) end = spec.size();
        const std::string part = spec.substr(at, end - at);
        at = end + 1;
        if (part.empty()) continue;
        const size_t eq = part.find('=');
        if (eq == std::string::npos) throw Error("llm: LLM_MOE_BANK entry \"" + part + "\" is not family=format");
        const std::string f = part.substr(0, eq), to = part.substr(eq + 1);
        if (std::find_if(fam, fam + 6, [&](const char *n) { return f == n; }) == fam + 6)
            throw Error("llm: LLM_MOE_BANK names family \"" + f + "\"; the six are gate_exps, up_exps, down_exps, gate_shexp, up_shexp, down_shexp");
        if (to != "q4_k") throw Error("llm: LLM_MOE_BANK " + f + "=" + to + ": q4_k is the format banks are fitted to here");
        out.push_back("ffn_" + f + ".");
    }
    return out;
}

void Model::LoadGGUF(const gguf::Set &s, const LoadOpts &opts) {
    const bool transcode = opts.transcode;
    const std::vector<std::string> narrowed = moe_plan_families(opts.moe_plan);
    auto is_bank = [](const std::string &n) { return n.find("_exps.") != std::string::npos || n.find("_shexp.") != std::string::npos; };
    auto plan_narrows = [&](const std::string &n) {
        for (const std::string &f : narrowed)
            if (n.find(f) != std::string::npos) return true;
        return false;
    };
    std::map<std::string, int64_t> covered;  // rows of each whole tensor that came from the file
    transcoded_.clear();
    // a tensor's bytes as the file holds them, in HBM for the length of one call
    struct Raw {
        Device &dev;
        void *p = nullptr;
        Raw(Device &d, const gguf::Tensor &t) : dev(d) {
            check(shv_alloc(dev.ctx(), t.Bytes, &p), "staging");
            try {
                dev.upload(p, t.Data, t.Bytes);
            } catch (...) {
                shv_free(dev.ctx(), p);
                throw;
            }
        }
        ~Raw() { shv_free(dev.ctx(), p); }
    };
    for (auto &kv : tensors_) {
        const std::string &name = kv.first;
        TensorView &v = kv.second;
        if (!s.Has(name)) continue;
        const gguf::Tensor &t = s.Get(name);
        const std::string shape = "[" + std::to_string(t.Dims[0]) + " x " + std::to_string(t.Rows()) + "] " + gguf::TypeName(t.Type);
        if (t.Dims[0] != v.cols || t.Rows() != v.rows)
            throw Error("llm: " + name + " is " + shape + " in the checkpoint, the metadata makes it [" + std::to_string(v.cols) + " x " + std::to_string(v.rows) + "]");
        const uint32_t same = v.kind == TensorView::Q4K ? gguf::Q4_K : v.kind == TensorView::F32 ? gguf::F32 : v.ggml;
        if (name == "token_embd.weight" && t.Type != v.ggml) {
            // the table in the checkpoint's own type: the gather expands the rows it reads
            if (!device_expands(t.Type)) throw Error("llm: " + name + " is " + shape + ": not a type the device expands");
            if (t.RowBytes() == 0) throw Error("llm: " + name + " is " + shape + ": rows are not whole blocks of the type");
            dev_.release(v.ptr, v.bytes);
            v.ptr = dev_.alloc(t.Bytes);
            v.bytes = t.Bytes;
            v.kind = t.Type == gguf::F16 ? TensorView::F16 : TensorView::RAW;
            v.ggml = t.Type;
            dev_.upload(v.ptr, t.Data, t.Bytes);
        } else if (v.kind != TensorView::F32 && is_bank(name) && t.Type != gguf::Q4_K && t.Type != gguf::F32 && device_expands(t.Type) &&
                   !(plan_narrows(name) && t.Bytes > v.bytes)) {
            // an expert bank in the checkpoint's own type: the expert kernels read it through that type's arm
            if (t.RowBytes() == 0) throw Error("llm: " + name + " is " + shape + ": rows are not whole blocks of the type");
            if (v.kind == TensorView::Q4K || v.bytes != t.Bytes) {
                dev_.release(v.ptr, v.bytes);
                v.ptr = dev_.alloc(t.Bytes);
                v.bytes = t.Bytes;
            }
            v.kind = TensorView::RAW;
            v.ggml = t.Type;
            dev_.upload(v.ptr, t.Data, t.Bytes);
        } else if (name == "output.weight" && v.kind != TensorView::F32 && t.Type != gguf::Q4_K && opts.head_native && device_expands(t.Type)) {
            // the vocabulary projection in the checkpoint's own type (converters keep it wider than the rest: Q6_K,
            // Q8_0): the head's launch reads it through that type's arm (shv_gemv) instead of a Q4_K refit of it
            if (t.RowBytes() == 0) throw Error("llm: " + name + " is " + shape + ": rows are not whole blocks of the type");
            if (v.bytes != t.Bytes) {
                dev_.release(v.ptr, v.bytes);
                v.ptr = dev_.alloc(t.Bytes);
                v.bytes = t.Bytes;
            }
            v.kind = TensorView::RAW;
            v.ggml = t.Type;
            dev_.upload(v.ptr, t.Data, t.Bytes);
        } else if (t.Type == same) {
            if (t.Bytes != v.bytes) throw Error("llm: " + name + ": " + std::to_string(t.Bytes) + " bytes in the checkpoint, " + std::to_string(v.bytes) + " staged");
            dev_.upload(v.ptr, t.Data, t.Bytes);
        } else if (v.kind == TensorView::F32) {
            // small float tensors (norms, routers, conv taps) in whatever the converter chose: expanded on the device
            Raw raw(dev_, t);
            shv_dequant_args d{raw.p, static_cast<float *>(v.ptr), t.Elems(), static_cast<int32_t>(t.Type)};
            check(shv_dequant(dev_.ctx(), &d), name.c_str());
            dev_.sync();
        } else if (v.kind == TensorView::Q4K && transcode) {
            // expanded and fitted again, a bounded number of rows at a time
            const uint64_t row_in = t.RowBytes(), row_out = v.bytes / v.rows;
            const int64_t step = std::max<int64_t>(1, std::min<int64_t>(v.rows, (64ll << 20) / v.cols));
            Raw raw(dev_, t);
            void *f32 = nullptr;
            check(shv_alloc(dev_.ctx(), static_cast<size_t>(step) * v.cols * 4, &f32), "staging");
            try {
                for (int64_t r0 = 0; r0 < v.rows; r0 += step) {
                    const int64_t nr = std::min<int64_t>(step, v.rows - r0);
                    shv_dequant_args d{static_cast<const char *>(raw.p) + r0 * row_in, static_cast<float *>(f32), nr * v.cols, static_cast<int32_t>(t.Type)};
                    check(shv_dequant(dev_.ctx(), &d), name.c_str());
                    shv_quantize_q4k_args q{static_cast<const float *>(f32), static_cast<char *>(v.ptr) + r0 * row_out, nr, static_cast<int32_t>(v.cols)};
                    check(shv_quantize_q4k(dev_.ctx(), &q), name.c_str());
                }
                dev_.sync();
            } catch (...) {
                shv_free(dev_.ctx(), f32);
                throw;
            }
            shv_free(dev_.ctx(), f32);
            transcoded_.push_back(name);
        } else {
            throw Error("llm: " + name + " is " + gguf::TypeName(t.Type) + " in the checkpoint; the kernels stream it as " + gguf::TypeName(same));
        }
        const std::string *base = v.init_std < 0.f ? base_of(v) : &name;
        if (base) covered[*base] += v.rows;
    }
    for (const auto &kv : tensors_) {
        if (kv.second.init_std < 0.f) continue;
        const int64_t got = covered.count(kv.first) ? covered[kv.first] : 0;
        if (got < kv.second.rows)
            throw Error("llm: the checkpoint fills " + std::to_string(got) + " of " + std::to_string(kv.second.rows) + " rows of " + kv.first + " (the tensor or its constituents are missing)");
    }
    dev_.sync();
}

void Model::SaveGGUF(const std::string &path, const std::string &arch) const {
    const Config &c = cfg_;
    gguf::Writer w;
    w.PutStr(gguf::kKeyArchitecture, arch);
    auto u32 = [&](const char *k, int v) { w.PutU32(arch + "." + k, static_cast<uint32_t>(v)); };
    u32("block_count", c.Blocks());
    u32("embedding_length", c.NEmbd);
    u32("attention.head_count", c.NHead);
    u32("attention.head_count_kv", c.NHeadKV);
    u32("attention.key_length", c.HeadDim);
    u32("rope.dimension_count", c.RopeDims);
    w.PutF32(arch + ".rope.freq_base", c.RopeBase);
    u32("expert_count", c.NExpert);
    u32("expert_used_count", c.NExpertUsed);
    u32("expert_feed_forward_length", c.FFNExpert);
    w.PutF32(arch + ".attention.layer_norm_rms_epsilon", c.RMSEps);
    u32("ssm.state_size", c.SSMHeadDim);
    u32("ssm.group_count", c.SSMHeadK);
    u32("ssm.time_step_rank", c.SSMHeadV);
    u32("ssm.conv_kernel", c.SSMConv);
    u32("full_attention_interval", c.AttnEvery);
    u32("nextn_predict_layers", c.NextN);
    if (c.IdxRatio > 0) {
        u32("attention.indexer.head_count", c.IdxHeads);
        u32("attention.indexer.key_length", c.IdxDim);
        u32("attention.indexer.top_k", c.IdxTopK);
        std::vector<int32_t> ratios(c.Blocks(), 0);
        for (int l = 0; l < c.Blocks(); l++) ratios[l] = c.QSA(l) ? c.IdxRatio : 0;
        w.PutI32s(arch + ".attention.compress_ratios", ratios);
    }

    // constituents stand in for a fused tensor when they tile it
    std::map<std::string, std::vector<std::string>> parts;
    for (const auto &kv : tensors_)
        if (kv.second.init_std < 0.f)
            if (const std::string *b = base_of(kv.second)) parts[*b].push_back(kv.first);
    auto emit = [&](const std::string &name, const TensorView &v) {
        std::vector<int64_t> dims;
        if (v.rows == 1) dims = {v.cols};
        else if (name.find("_exps.") != std::string::npos) dims = {v.cols, v.rows / c.NExpert, c.NExpert};
        else dims = {v.cols, v.rows};
        const uint32_t type = v.ggml;
        Device *dev = &dev_;
        const void *src = v.ptr;
        w.AddTensor(name, type, dims, [dev, src](uint8_t *dst, uint64_t bytes) { dev->download(dst, src, bytes); });
    };
    for (const auto &kv : tensors_) {
        if (kv.second.init_std < 0.f) continue;
        int64_t rows = 0;
        auto it = parts.find(kv.first);
        if (it != parts.end())
            for (const std::string &p : it->second) rows += tensors_.at(p).rows;
        if (rows == kv.second.rows)
            for (const std::string &p : it->second) emit(p, tensors_.at(p));
        else
            emit(kv.first, kv.second);
    }
    dev_.sync();
    w.Write(path);
}

// ---------------------------------------------------------------------------------- MoE -------

MoEGPU::MoEGPU(Device &dev, const Model &m, int maxTokens) : dev_(dev), m_(m), c_(m.config()), max_tok_(maxTokens) {
    if (maxTokens < 1) throw Error("llm: MoEGPU needs room for at least one token");
    if (c_.NExpertUsed > c_.NExpert) throw Error("llm: MoEGPU: more experts used than there are");
    // LLM_MOE_ROUTE=fused|rows|kernel says where the selection runs (rows: fused in one-row passes only)
    if (const char *e = std::getenv("LLM_MOE_ROUTE")) route_mode_ = std::strcmp(e, "fused") == 0 ? 1 : std::strcmp(e, "rows") == 0 ? 2 : 0;
    const size_t T = maxTokens;
    in_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    out_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    xn_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    logits_ = static_cast<float *>(dev.alloc(T * (c_.NExpert + 1) * 4));
    topk_ = static_cast<int32_t *>(dev.alloc(T * c_.NExpertUsed * 4));
    weights_ = static_cast<float *>(dev.alloc(T * (c_.NExpertUsed + 1) * 4));
    act_ = static_cast<float *>(dev.alloc(T * (c_.NExpertUsed + 1) * c_.FFNExpert * 4));
    // passes of many rows go grouped by expert on the matrix cores and need the per-expert lists
    // and every (token, slot)'s down products before they are summed
    if (maxTokens > kBlockRows) {
        group_ = static_cast<int32_t *>(dev.alloc((2 * c_.NExpert + 1 + T * c_.NExpertUsed) * 4));
        pairs_ = static_cast<float *>(dev.alloc(T * (c_.NExpertUsed + 1) * c_.NEmbd * 4));
    }
    act_bytes_ = T * (3ull * c_.NEmbd + c_.NExpert + 1 + 2 * c_.NExpertUsed + 1 + (c_.NExpertUsed + 1ull) * c_.FFNExpert) * 4;
}

void MoEGPU::Resize(int nTok) {
    if (nTok < 1 || nTok > max_tok_) throw Error("llm: MoEGPU: " + std::to_string(nTok) + " tokens, staged for " + std::to_string(max_tok_));
    n_tok_ = nTok;
}

void MoEGPU::Upload(const std::vector<float> &x, int nTok) {
    Resize(nTok);
    if (x.size() != static_cast<size_t>(nTok) * c_.NEmbd) throw Error("llm: MoEGPU.Upload: wrong length");
    dev_.upload(in_, x.data(), x.size() * 4);
}

std::vector<shv_op> MoEGPU::Dispatches(int l, const float *in, float *out, int nTok, std::vector<std::string> *labels) const {
    const TensorView &norm = m_.Tensor(Model::Blk(l, "post_attention_norm"));
    shv_moe_router_args r{};
    r.h = in;
    r.gamma = static_cast<const float *>(norm.ptr);
    r.router = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ffn_gate_inp")).ptr);
    r.shared_gate = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ffn_gate_inp_shexp")).ptr);
    r.xn = xn_;
    r.logits = logits_;
    r.topk = topk_;
    r.weights = weights_;
    r.n_tok = nTok;
    r.n_embd = c_.NEmbd;
    r.n_expert = c_.NExpert;
    r.n_used = c_.NExpertUsed;
    r.eps = c_.RMSEps;
    r.h_stride = c_.NEmbd;
    const TensorView &ge = m_.Tensor(Model::Blk(l, "ffn_gate_exps")), &ue = m_.Tensor(Model::Blk(l, "ffn_up_exps"));
    const TensorView &gs = m_.Tensor(Model::Blk(l, "ffn_gate_shexp")), &us = m_.Tensor(Model::Blk(l, "ffn_up_shexp"));
    const TensorView &de = m_.Tensor(Model::Blk(l, "ffn_down_exps")), &ds = m_.Tensor(Model::Blk(l, "ffn_down_shexp"));
    // banks in another type than Q4_K take the selection from the router kernel
    const bool up_q4k = ge.ggml == gguf::Q4_K && ue.ggml == gguf::Q4_K && gs.ggml == gguf::Q4_K && us.ggml == gguf::Q4_K;
    const bool fused = FusedRouter(nTok) && up_q4k;
    r.defer_route = fused ? 1 : 0;
    shv_moe_up_args u{};
    u.xn = xn_;
    u.topk = topk_;
    u.gate_exps = ge.ptr;
    u.up_exps = ue.ptr;
    u.gate_sh = gs.ptr;
    u.up_sh = us.ptr;
    u.gate_type = static_cast<int32_t>(ge.ggml), u.up_type = static_cast<int32_t>(ue.ggml);
    u.gate_sh_type = static_cast<int32_t>(gs.ggml), u.up_sh_type = static_cast<int32_t>(us.ggml);
    u.act = act_;
    u.n_tok = nTok;
    u.n_embd = c_.NEmbd;
    u.n_used = c_.NExpertUsed;
    u.ffn = c_.FFNExpert;
    u.n_expert = c_.NExpert;
    if (fused) {
        u.logits = logits_;
        u.weights = weights_;
    } else {
        u.group = group_;
    }
    shv_moe_down_args d{};
    d.n_expert = c_.NExpert;
    d.group = group_;
    d.pairs = pairs_;
    d.group_ready = (!fused && up_q4k && group_) ? 1 : 0;  // the up projection of this pass has grouped its rows (or neither takes that road)
    // both projections in Q4_K, one right after the other: when they group their rows, act goes from one to the other as operands
    const bool down_q4k = de.ggml == gguf::Q4_K && ds.ggml == gguf::Q4_K;
    u.act_packed = d.act_packed = (d.group_ready && down_q4k && pairs_) ? 1 : 0;
    d.act = act_;
    d.topk = topk_;
    d.weights = weights_;
    d.down_exps = de.ptr;
    d.down_sh = ds.ptr;
    d.down_type = static_cast<int32_t>(de.ggml), d.down_sh_type = static_cast<int32_t>(ds.ggml);
    d.residual = in;
    d.out = out;
    d.n_tok = nTok;
    d.n_embd = c_.NEmbd;
    d.n_used = c_.NExpertUsed;
    d.ffn = c_.FFNExpert;
    d.res_stride = d.out_stride = c_.NEmbd;
    if (labels) labels->insert(labels->end(), {"moe.router", "moe.up", "moe.down"});
    return {make_op(SHV_OP_MOE_ROUTER, r), make_op(SHV_OP_MOE_UP, u), make_op(SHV_OP_MOE_DOWN, d)};
}

bool MoEGPU::Fold(int l, const TensorView &w_out) {
    if (fold_.empty()) fold_.assign(c_.NLayer + 1, nullptr);
    if (l < 0 || l >= static_cast<int>(fold_.size())) return false;
    const TensorView &ge = m_.Tensor(Model::Blk(l, "ffn_gate_exps")), &ue = m_.Tensor(Model::Blk(l, "ffn_up_exps"));
    const TensorView &gs = m_.Tensor(Model::Blk(l, "ffn_gate_shexp")), &us = m_.Tensor(Model::Blk(l, "ffn_up_shexp"));
    const bool up_q4k = ge.ggml == gguf::Q4_K && ue.ggml == gguf::Q4_K && gs.ggml == gguf::Q4_K && us.ggml == gguf::Q4_K;
    // what the fused launches are built for: a 2048-wide stream, a 4096-wide mixer output, the
    // selection inside the gate/up kernel, everything it touches in the types the kernels stream
    if (!up_q4k || !FusedRouter(1) || c_.NEmbd != 2048 || w_out.rows != c_.NEmbd || w_out.cols != 4096 || w_out.ggml != gguf::Q4_K || c_.NExpert > 512)
        return false;
    const size_t rows = c_.NExpert, width = static_cast<size_t>(w_out.cols) + c_.NEmbd;  // the shared gate's product is formed by gate/up
    if (!fold_[l]) fold_[l] = static_cast<float *>(dev_.alloc(rows * width * 4));
    const size_t scratch_bytes = static_cast<size_t>(c_.NEmbd) * w_out.cols * 4;
    float *scratch = static_cast<float *>(dev_.alloc(scratch_bytes));
    shv_router_fold_args f{};
    f.router = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ffn_gate_inp")).ptr);
    f.shared_gate = nullptr;
    f.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "post_attention_norm")).ptr);
    f.w_out = w_out.ptr;
    f.out = fold_[l];
    f.scratch = scratch;
    f.n_expert = c_.NExpert;
    f.n_embd = c_.NEmbd;
    f.k = static_cast<int32_t>(w_out.cols);
    check(shv_router_fold(dev_.ctx(), &f), "MoEGPU.Fold");
    dev_.sync();
    dev_.release(scratch, scratch_bytes);
    fold_k_ = static_cast<int>(w_out.cols);
    return true;
}

void MoEGPU::FoldInto(int l, PassRows &r) const {
    if (!Folded(l)) throw Error("llm: MoEGPU: layer " + std::to_string(l) + " has no folded router");
    r.fold = fold_[l];
    r.fold_rows = c_.NExpert;  // the shared gate's row stays behind: gate/up forms that product from the row it stages
    r.fold_out = logits_;
    r.fold_stride = c_.NExpert + 1;
}

std::vector<shv_op> MoEGPU::DispatchesFolded(int l, const float *in, float *out, int nTok, std::vector<std::string> *labels) const {
    if (!Folded(l)) throw Error("llm: MoEGPU: layer " + std::to_string(l) + " has no folded router");
    if (nTok < 1 || nTok > kFoldRows || !FusedRouter(nTok)) throw Error("llm: MoEGPU: a pass of " + std::to_string(nTok) + " rows makes its selection in a launch of its own");
    auto ops = Dispatches(l, in, out, nTok, nullptr);
    // the router's launch goes; gate/up takes the row as it is and normalises it itself
    shv_moe_up_args u{};
    std::memcpy(&u, ops[1].args, sizeof u);
    u.xn = in;
    u.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "post_attention_norm")).ptr);
    u.eps = c_.RMSEps;
    u.shared_gate = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ffn_gate_inp_shexp")).ptr);
    if (labels) labels->insert(labels->end(), {"moe.up", "moe.down"});
    return {make_op(SHV_OP_MOE_UP, u), ops[2]};
}

void MoEGPU::Run(int layer) {
    if (n_tok_ < 1) throw Error("llm: MoEGPU.Run before Upload");
    dev_.run(Dispatches(layer, in_, out_, n_tok_, nullptr));
}

static std::vector<Stage> profile_ops(Device &dev, const std::vector<shv_op> &ops, const std::vector<std::string> &labels, int iters) {
    std::vector<uint64_t> per(ops.size()), sum(ops.size(), 0);
    for (int i = 0; i < iters; i++) {
        uint64_t total = 0;
        check(shv_dispatch_multi(dev.ctx(), ops.data(), static_cast<int>(ops.size()), 1, &total, per.data()), "profile");
        for (size_t k = 0; k < ops.size(); k++) sum[k] += per[k];
    }
    std::vector<Stage> out;
    for (size_t k = 0; k < ops.size(); k++) out.push_back({labels[k], sum[k] / static_cast<uint64_t>(iters)});
    return out;
}

std::vector<Stage> MoEGPU::Profile(int layer, int iters) {
    std::vector<std::string> labels;
    auto ops = Dispatches(layer, in_, out_, n_tok_, &labels);
    return profile_ops(dev_, ops, labels, iters < 1 ? 1 : iters);
}

template <typename T>
static std::vector<T> read_back(Device &dev, const void *src, size_t n) {
    std::vector<T> v(n);
    dev.download(v.data(), src, n * sizeof(T));
    return v;
}

std::vector<float> MoEGPU::Logits() const { return read_back<float>(dev_, logits_, static_cast<size_t>(n_tok_) * (c_.NExpert + 1)); }
std::vector<int32_t> MoEGPU::TopK() const { return read_back<int32_t>(dev_, topk_, static_cast<size_t>(n_tok_) * c_.NExpertUsed); }
std::vector<float> MoEGPU::Weights() const { return read_back<float>(dev_, weights_, static_cast<size_t>(n_tok_) * (c_.NExpertUsed + 1)); }
std::vector<float> MoEGPU::Swiglu() const { return read_back<float>(dev_, act_, static_cast<size_t>(n_tok_) * (c_.NExpertUsed + 1) * c_.FFNExpert); }
std::vector<float> MoEGPU::Out() const { return read_back<float>(dev_, out_, static_cast<size_t>(n_tok_) * c_.NEmbd); }

// ----------------------------------------------------------------------------- DeltaNet -------

DeltaNetGPU::DeltaNetGPU(Device &dev, const Model &m, int maxTokens, int slots, int32_t *pos, int planes, int32_t *plane)
    : dev_(dev), m_(m), c_(m.config()), max_tok_(maxTokens), slots_(slots), planes_(planes), pos_(pos), plane_(plane) {
    // refusals at construction, never at run (llm/gpu_deltanet.go:423-447)
    if (c_.SSMHeadDim != 128) throw Error("llm: DeltaNetGPU: head dimension " + std::to_string(c_.SSMHeadDim) + ", the step kernel is built for 128");
    if (c_.SSMConv != 4) throw Error("llm: DeltaNetGPU: conv kernel " + std::to_string(c_.SSMConv) + ", built for 4");
    if (maxTokens < 1 || maxTokens > 4096) throw Error("llm: DeltaNetGPU: a pass of " + std::to_string(maxTokens) + " rows; 1..4096");
    if (slots < 1) throw Error("llm: DeltaNetGPU: no slots");
    if (planes < 1 || planes > 64 || (planes > 1 && !plane)) throw Error("llm: DeltaNetGPU: " + std::to_string(planes) + " state planes");
    // the ring holds a pass's rows and the conv's history behind them
    ring_slots_ = std::max(kRing, std::min(maxTokens, kSmallPass) + c_.SSMConv - 1);
    if (maxTokens > kSmallPass) {
        big_slots_ = maxTokens + c_.SSMConv - 1;
        big_ring_ = static_cast<float *>(dev.alloc_zero(static_cast<size_t>(big_slots_) * c_.DNFusedRows() * 4));
    }
    const size_t T = maxTokens;
    if (maxTokens > 16) {
        // the prepared rows of a pass, and behind them a record of 43 520 bytes per (chunk of 64 rows, value head):
        // with that much room the chunks' state-independent part is formed for all of them at once (shv_dn_step)
        work_floats_ = ((static_cast<int64_t>(T) * (c_.ConvWidth() + 2 * c_.SSMHeadV) + 3) & ~int64_t{3}) +
                       static_cast<int64_t>((T + 63) / 64 + 1) * c_.SSMHeadV * (43520 / 4);
        work_ = static_cast<float *>(dev.alloc(static_cast<size_t>(work_floats_) * 4));
    }
    in_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    out_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    attn_ = static_cast<float *>(dev.alloc(T * c_.VWidth() * 4));
    row_ = static_cast<float *>(dev.alloc(static_cast<size_t>(c_.DNFusedRows()) * 4));
    ring_.assign(c_.NLayer, nullptr);
    state_.assign(c_.NLayer, nullptr);
    const size_t ring_bytes = static_cast<size_t>(slots) * ring_slots_ * c_.DNFusedRows() * 4;
    const size_t st_bytes = static_cast<size_t>(slots) * planes * c_.SSMHeadV * c_.SSMHeadDim * c_.SSMHeadDim * 4;
    for (int l = 0; l < c_.NLayer; l++) {
        if (c_.IsAttn(l)) continue;
        ring_[l] = static_cast<float *>(dev.alloc_zero(ring_bytes));
        state_[l] = static_cast<float *>(dev.alloc_zero(st_bytes));
        state_bytes_ += ring_bytes + st_bytes;
    }
}

void DeltaNetGPU::Resize(int nTok) {
    if (nTok < 1 || nTok > max_tok_) throw Error("llm: DeltaNetGPU: " + std::to_string(nTok) + " tokens, staged for " + std::to_string(max_tok_));
    n_tok_ = nTok;
}

void DeltaNetGPU::Upload(const std::vector<float> &x, int nTok) {
    Resize(nTok);
    if (x.size() != static_cast<size_t>(nTok) * c_.NEmbd) throw Error("llm: DeltaNetGPU.Upload: wrong length");
    dev_.upload(in_, x.data(), x.size() * 4);
}

void DeltaNetGPU::Reset(int l) {
    if (l < 0 || l >= c_.NLayer || !state_[l]) throw Error("llm: DeltaNetGPU.Reset: layer " + std::to_string(l) + " is not a DeltaNet layer");
    dev_.zero(ring_[l], static_cast<size_t>(slots_) * ring_slots_ * c_.DNFusedRows() * 4);
    dev_.zero(state_[l], static_cast<size_t>(slots_) * planes_ * c_.SSMHeadV * c_.SSMHeadDim * c_.SSMHeadDim * 4);
}

void DeltaNetGPU::ResetAll() {
    for (int l = 0; l < c_.NLayer; l++)
        if (state_[l]) Reset(l);
}

// One slot's carried history back to an empty sequence's: every plane of its state and its ring.
void DeltaNetGPU::ResetSlot(int slot) {
    if (slot < 0 || slot >= slots_) throw Error("llm: DeltaNetGPU.ResetSlot: slot " + std::to_string(slot) + " of " + std::to_string(slots_));
    const size_t ring_floats = static_cast<size_t>(ring_slots_) * c_.DNFusedRows();
    const size_t st_floats = static_cast<size_t>(planes_) * c_.SSMHeadV * c_.SSMHeadDim * c_.SSMHeadDim;
    for (int l = 0; l < c_.NLayer; l++) {
        if (!state_[l]) continue;
        dev_.zero(ring_[l] + slot * ring_floats, ring_floats * 4);
        dev_.zero(state_[l] + slot * st_floats, st_floats * 4);
    }
}

std::vector<shv_op> DeltaNetGPU::Dispatches(int l, const float *in, float *out, int nTok, std::vector<std::string> *labels) const {
    PassRows r;
    r.pos = pos_;
    r.seq_len = nTok;
    return Dispatches(l, in, out, r, labels);
}

std::vector<shv_op> DeltaNetGPU::Dispatches(int l, const float *in, float *out, const PassRows &r, std::vector<std::string> *labels) const {
    if (l < 0 || l >= c_.NLayer || !state_[l]) throw Error("llm: DeltaNetGPU: layer " + std::to_string(l) + " is not a DeltaNet layer");
    const int nTok = r.rows();
    if (nTok < 1 || nTok > max_tok_) throw Error("llm: DeltaNetGPU: " + std::to_string(nTok) + " rows, staged for " + std::to_string(max_tok_));
    if (r.n_seq > slots_) throw Error("llm: DeltaNetGPU: this block was staged with " + std::to_string(slots_) + " sequence slot(s) (GraphOpts.Slots)");
    if (r.spec && r.seq_len >= planes_)
        throw Error("llm: DeltaNetGPU: a rewindable pass of " + std::to_string(r.seq_len) + " rows needs " + std::to_string(r.seq_len + 1) +
                    " state planes, " + std::to_string(planes_) + " are staged (GraphOpts.Speculative, SpecRows)");
    const int width = c_.DNFusedRows();
    // A pass of one sequence whose slot is known now: its ring rows, state planes and plane word
    // are addressed here, and the kernels take no slot table (a dependent load less on their way).
    const bool own_slot = r.n_seq == 1 && r.host_slot >= 0 && r.host_slot < slots_;
    const size_t slot_off = own_slot ? static_cast<size_t>(r.host_slot) : 0;
    const int32_t *slot_tab = own_slot ? nullptr : r.slot;
    float *slot_ring = ring_[l] + slot_off * ring_slots_ * width;
    const bool big = nTok > kSmallPass;
    if (big && (!own_slot || r.spec || !big_ring_))
        throw Error("llm: DeltaNetGPU: a pass of " + std::to_string(nTok) + " rows is one sequence's plain prompt chunk (no slot table, not rewindable)");
    float *ring = big ? big_ring_ : slot_ring;
    const int ring_slots = big ? big_slots_ : ring_slots_;
    shv_gemv_q4k_args p{};
    p.w = m_.Tensor(Model::Blk(l, "ssm_in_fused")).ptr;
    p.x = in;
    p.y = ring;
    p.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "attn_norm")).ptr);
    p.pos = r.pos;
    p.slot = slot_tab;
    p.n = width;
    p.k = c_.NEmbd;
    p.n_tok = nTok;
    p.prologue = SHV_PRO_RMSNORM;
    p.eps = c_.RMSEps;
    p.x_stride = c_.NEmbd;
    p.y_stride = width;
    p.seq_len = r.seq_len;
    p.ring_slots = ring_slots;
    p.ring_stride = width;
    // one row: the projection also leaves the row where the out projection finds its gate
    // without waiting for the position word
    const bool flat = nTok == 1;
    if (flat) p.y_flat = row_;
    shv_dn_step_args s{};
    s.ring = ring;
    s.conv1d = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_conv1d")).ptr);
    s.a = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_a")).ptr);
    s.dt_bias = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_dt")).ptr);
    s.state = state_[l] + slot_off * planes_ * c_.SSMHeadV * c_.SSMHeadDim * c_.SSMHeadDim;
    s.out = attn_;
    s.pos = r.pos;
    s.slot = slot_tab;
    s.n_seq = r.n_seq;
    s.seq_len = r.seq_len;
    s.plane = plane_ ? plane_ + slot_off : nullptr;
    s.n_planes = planes_;
    s.spec = r.spec ? 1 : 0;
    s.n_head_k = c_.SSMHeadK;
    s.n_head_v = c_.SSMHeadV;
    s.head_dim = c_.SSMHeadDim;
    s.conv = c_.SSMConv;
    s.ring_slots = ring_slots;
    s.ring_stride = width;
    s.eps = c_.RMSEps;
    s.work = work_;   // passes of more than 16 rows of one or more sequences go chunked
    s.work_floats = work_floats_;
    shv_gemv_q4k_args o{};
    o.w = m_.Tensor(Model::Blk(l, "ssm_out")).ptr;
    o.x = attn_;
    o.y = out;
    o.residual = in;
    o.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_norm")).ptr);
    o.n = c_.NEmbd;
    o.k = c_.VWidth();
    o.n_tok = nTok;
    o.prologue = SHV_PRO_GATED_NORM;
    o.head_dim = c_.SSMHeadDim;
    o.eps = c_.RMSEps;
    o.x_stride = c_.VWidth();
    o.y_stride = c_.NEmbd;
    o.fold = r.fold;
    o.fold_rows = r.fold_rows;
    o.fold_out = r.fold_out;
    o.fold_stride = r.fold_stride;
    if (flat) {
        o.z = row_ + c_.ConvWidth();  // the z columns of the projection row
        o.z_stride = width;
    } else {
        o.z = ring + c_.ConvWidth();
        o.pos = r.pos;
        o.slot = slot_tab;
        o.seq_len = r.seq_len;
        o.ring_slots = ring_slots;
        o.ring_stride = width;
        o.z_ring = 1;
    }
    if (big) {
        // history in, the pass, history out: only the conv's channels (q, k, v) are read back later
        const int hist = c_.SSMConv - 1;
        shv_ring_rows_args hin{slot_ring, big_ring_, r.pos, ring_slots_, big_slots_, width, c_.ConvWidth(), -hist, hist};
        shv_ring_rows_args hout{big_ring_, slot_ring, r.pos, big_slots_, ring_slots_, width, c_.ConvWidth(), nTok - hist, hist};
        if (labels) labels->insert(labels->end(), {"dn.hist", "dn.qkv", "dn.step", "dn.hist", "dn.out"});
        return {make_op(SHV_OP_RING_ROWS, hin), make_op(SHV_OP_GEMV_Q4K, p), make_op(SHV_OP_DN_STEP, s), make_op(SHV_OP_RING_ROWS, hout),
                make_op(SHV_OP_GEMV_Q4K, o)};
    }
    if (labels) labels->insert(labels->end(), {"dn.qkv", "dn.step", "dn.out"});
    return {make_op(SHV_OP_GEMV_Q4K, p), make_op(SHV_OP_DN_STEP, s), make_op(SHV_OP_GEMV_Q4K, o)};
}

void DeltaNetGPU::Run(int layer) {
    if (n_tok_ < 1) throw Error("llm: DeltaNetGPU.Run before Upload");
    dev_.run(Dispatches(layer, in_, out_, n_tok_, nullptr));
}

std::vector<float> DeltaNetGPU::State(int l, int slot, int plane) const {
    if (l < 0 || l >= c_.NLayer || !state_[l] || slot < 0 || slot >= slots_ || plane < 0 || plane >= planes_)
        throw Error("llm: DeltaNetGPU.State: no such layer, slot or plane");
    const size_t n = static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim;
    return read_back<float>(dev_, state_[l] + (static_cast<size_t>(slot) * planes_ + plane) * n, n);
}

void DeltaNetGPU::SetState(int l, const std::vector<float> &s, int slot, int plane) {
    const size_t n = static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim;
    if (l < 0 || l >= c_.NLayer || !state_[l] || slot < 0 || slot >= slots_ || plane < 0 || plane >= planes_ || s.size() != n)
        throw Error("llm: DeltaNetGPU.SetState: no such layer, slot or plane, or wrong length");
    dev_.upload(state_[l] + (static_cast<size_t>(slot) * planes_ + plane) * n, s.data(), n * 4);
}

size_t DeltaNetGPU::CarriedLen() const {
    size_t layers = 0;
    for (int l = 0; l < c_.NLayer; l++) layers += state_[l] ? 1 : 0;
    return layers * (static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim + 3 * static_cast<size_t>(c_.DNFusedRows()));
}

void DeltaNetGPU::SaveCarried(float *dst, int slot, int plane, int past) const {
    if (slot < 0 || slot >= slots_ || plane < 0 || plane >= planes_) throw Error("llm: DeltaNetGPU.SaveCarried: no such slot or plane");
    const size_t n = static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim, row = c_.DNFusedRows();
    for (int l = 0; l < c_.NLayer; l++) {
        if (!state_[l]) continue;
        dev_.download(dst, state_[l] + (static_cast<size_t>(slot) * planes_ + plane) * n, n * 4);
        dst += n;
        for (int j = 3; j >= 1; j--, dst += row) {  // positions past-3, past-2, past-1; zero before the start
            if (past - j < 0) std::fill(dst, dst + row, 0.f);
            else dev_.download(dst, ring_[l] + (static_cast<size_t>(slot) * ring_slots_ + (past - j) % ring_slots_) * row, row * 4);
        }
    }
}

void DeltaNetGPU::RestoreCarried(const float *src, int slot, int plane, int past) {
    if (slot < 0 || slot >= slots_ || plane < 0 || plane >= planes_) throw Error("llm: DeltaNetGPU.RestoreCarried: no such slot or plane");
    const size_t n = static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim, row = c_.DNFusedRows();
    for (int l = 0; l < c_.NLayer; l++) {
        if (!state_[l]) continue;
        dev_.upload(state_[l] + (static_cast<size_t>(slot) * planes_ + plane) * n, src, n * 4);
        src += n;
        for (int j = 3; j >= 1; j--, src += row)
            if (past - j >= 0) dev_.upload(ring_[l] + (static_cast<size_t>(slot) * ring_slots_ + (past - j) % ring_slots_) * row, src, row * 4);
    }
}

std::vector<float> DeltaNetGPU::Result() const { return read_back<float>(dev_, attn_, static_cast<size_t>(n_tok_) * c_.VWidth()); }
std::vector<float> DeltaNetGPU::Out() const { return read_back<float>(dev_, out_, static_cast<size_t>(n_tok_) * c_.NEmbd); }

// ---------------------------------------------------------------------------- Attention -------

// The text rotary table, built once at stage time as the reference builds its own
// (llm/gpu_attn.go:1452-1476) with the CPU function's arithmetic (llm/attn.go:553-584):
// theta_i = pos * s^i, s = base^(-2/n_rot), the power by repeated multiplication in float64.
static std::vector<float> rope_table(int cells, int rope_dims, float base) {
    const int half = rope_dims / 2;
    std::vector<float> t(static_cast<size_t>(cells) * rope_dims);
    const double scale = std::pow(static_cast<double>(base), -2.0 / rope_dims);
    for (int p = 0; p < cells; p++) {
        double theta = p;
        for (int i = 0; i < half; i++) {
            t[static_cast<size_t>(p) * rope_dims + i] = static_cast<float>(std::cos(theta));
            t[static_cast<size_t>(p) * rope_dims + half + i] = static_cast<float>(std::sin(theta));
            theta *= scale;
        }
    }
    return t;
}

AttnGPU::AttnGPU(Device &dev, const Model &m, int maxTokens, int nKV, int slots, int32_t *pos, int only_layer)
    : dev_(dev), m_(m), c_(m.config()), max_tok_(maxTokens), n_kv_(nKV), slots_(slots), pos_(pos) {
    if (c_.HeadDim != 256) throw Error("llm: AttnGPU: head dimension " + std::to_string(c_.HeadDim) + ", the decode kernel is built for 256");
    if (c_.NHead != 8 * c_.NHeadKV) throw Error("llm: AttnGPU: the decode kernel is built for 8 query heads per KV head");
    if (maxTokens < 1 || nKV < maxTokens || slots < 1) throw Error("llm: AttnGPU: bad token, cell or slot count");
    n_kv_ = (nKV + 31) & ~31;  // the decode kernel keeps V in tiles of 32 cells
    nKV = n_kv_;
    SetSplits(0);
    const size_t T = maxTokens;
    in_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    out_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    qkv_ = static_cast<float *>(dev.alloc(T * c_.AttnFusedRows() * 4));
    ctx_ = static_cast<float *>(dev.alloc(T * c_.NHead * c_.HeadDim * 4));
    // one set of slice records per sequence of a batched pass (an ordinary pass is one sequence)
    // Slice records: a pass of P row pairs over all its sequences takes min(splits, ceil(2 CUs / (P kv)))
    // slices a pair, two rows of 8 heads a record.  One pair can take every slice; many pairs
    // take at most 2 CUs + P kv records in all, and P is at most the pass's rows.
    partial_records_ = static_cast<size_t>(c_.NHeadKV) * kMaxSplits + 2 * 512 + (T + 1) * c_.NHeadKV;
    partial_ = static_cast<float *>(dev.alloc(partial_records_ * 2 * 8 * (c_.HeadDim + 2) * 4));
    const std::vector<float> rt = rope_table(nKV, c_.RopeDims, c_.RopeBase);
    rope_ = static_cast<float *>(dev.alloc(rt.size() * 4));
    dev.upload(rope_, rt.data(), rt.size() * 4);
    kc_.assign(c_.Blocks(), nullptr);
    vc_.assign(c_.Blocks(), nullptr);
    if (only_layer >= c_.Blocks()) throw Error("llm: AttnGPU: block " + std::to_string(only_layer) + " of " + std::to_string(c_.Blocks()));
    const size_t cb = static_cast<size_t>(slots) * nKV * c_.NHeadKV * c_.HeadDim * 2;
    for (int l = 0; l < c_.Blocks(); l++) {
        if (only_layer >= 0 ? l != only_layer : (l >= c_.NLayer || !c_.IsAttn(l))) continue;
        // zeroed: cells beyond a sequence's end are read (and weighted by zero) with the last tile
        kc_[l] = dev.alloc_zero(cb);
        vc_[l] = dev.alloc_zero(cb);
        cache_bytes_ += 2 * cb;
    }
    idxc_.assign(c_.Blocks(), nullptr);
    pooled_.assign(c_.Blocks(), nullptr);
    for (int l = 0; l < c_.Blocks(); l++) {
        if (!kc_[l] || !c_.QSA(l)) continue;
        if (nKV % c_.IdxRatio) throw Error("llm: AttnGPU: " + std::to_string(nKV) + " cells are not whole blocks of " + std::to_string(c_.IdxRatio));
        const size_t ib = static_cast<size_t>(slots) * nKV * c_.IdxDim * 2, pb = static_cast<size_t>(slots) * (nKV / c_.IdxRatio + 1) * c_.IdxDim * 4;
        idxc_[l] = static_cast<uint16_t *>(dev.alloc_zero(ib));
        pooled_[l] = static_cast<float *>(dev.alloc_zero(pb));
        cache_bytes_ += ib + pb;
        if (!qsa_work_) {
            mask_stride_ = nKV / 32;
            qsa_work_ = static_cast<float *>(dev.alloc(T * c_.IdxRows() * 4));
            qsa_score_ = static_cast<float *>(dev.alloc(T * (nKV / c_.IdxRatio + 1) * 4));
            qsa_mask_ = static_cast<uint32_t *>(dev.alloc(T * mask_stride_ * 4));
        }
    }
}

void AttnGPU::SetSplits(int n) {
    // slices for the cache's capacity: a tile of 32 cells each while there are slices to spare (the
    // kernel engages only as many as the sequence's current length fills)
    if (n <= 0) n = std::min(kMaxSplits, std::max(8, (n_kv_ + 31) / 32));
    if (n > kMaxSplits) throw Error("llm: AttnGPU.SetSplits: at most " + std::to_string(kMaxSplits) + " slices");
    splits_ = n;
}

void AttnGPU::Resize(int nTok) {
    if (nTok < 1 || nTok > max_tok_) throw Error("llm: AttnGPU: " + std::to_string(nTok) + " tokens, staged for " + std::to_string(max_tok_));
    n_tok_ = nTok;
}

void AttnGPU::Upload(const std::vector<float> &x, int nTok) {
    Resize(nTok);
    if (x.size() != static_cast<size_t>(nTok) * c_.NEmbd) throw Error("llm: AttnGPU.Upload: wrong length");
    dev_.upload(in_, x.data(), x.size() * 4);
}

std::vector<shv_op> AttnGPU::Dispatches(int l, const float *in, float *out, int nTok, std::vector<std::string> *labels) const {
    PassRows r;
    r.pos = pos_;
    r.seq_len = nTok;
    return Dispatches(l, in, out, r, labels);
}

std::vector<shv_op> AttnGPU::Dispatches(int l, const float *in, float *out, const PassRows &r, std::vector<std::string> *labels) const {
    if (l < 0 || l >= c_.Blocks() || !kc_[l]) throw Error("llm: AttnGPU: layer " + std::to_string(l) + " is not an attention layer staged here");
    const int nTok = r.rows();
    if (nTok < 1 || nTok > max_tok_) throw Error("llm: AttnGPU: " + std::to_string(nTok) + " rows, staged for " + std::to_string(max_tok_));
    if (r.n_seq > slots_) throw Error("llm: AttnGPU: this block was staged with " + std::to_string(slots_) + " sequence slot(s) (GraphOpts.Slots)");
    {
        // the slice records this pass writes (the launcher's own arithmetic) against what was staged
        const size_t pairs = static_cast<size_t>(r.n_seq) * ((r.seq_len + 1) / 2);
        const size_t per_pair = std::min<size_t>(splits_, (2 * 512 + pairs * c_.NHeadKV - 1) / (pairs * c_.NHeadKV));
        if (pairs * c_.NHeadKV * per_pair > partial_records_)
            throw Error("llm: AttnGPU: " + std::to_string(r.n_seq) + " sequences of " + std::to_string(r.seq_len) + " rows need more slice records than were staged");
    }
    const int width = c_.AttnFusedRows();
    shv_gemv_q4k_args p{};
    p.w = m_.Tensor(Model::Blk(l, "attn_qkv_fused")).ptr;
    p.x = in;
    p.y = qkv_;
    p.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "attn_norm")).ptr);
    p.n = width;
    p.k = c_.NEmbd;
    p.n_tok = nTok;
    p.prologue = SHV_PRO_RMSNORM;
    p.eps = c_.RMSEps;
    p.x_stride = c_.NEmbd;
    p.y_stride = width;
    shv_attn_decode_args a{};
    a.qkv = qkv_;
    a.q_norm = static_cast<const float *>(m_.Tensor(Model::Blk(l, "attn_q_norm")).ptr);
    a.k_norm = static_cast<const float *>(m_.Tensor(Model::Blk(l, "attn_k_norm")).ptr);
    a.rope = rope_;
    // a pass of one sequence whose slot is known now: its cells are addressed here
    const bool own_slot = r.n_seq == 1 && r.host_slot >= 0 && r.host_slot < slots_;
    const size_t slot_bytes = own_slot ? static_cast<size_t>(r.host_slot) * n_kv_ * c_.NHeadKV * c_.HeadDim * 2 : 0;
    a.kcache = static_cast<char *>(kc_[l]) + slot_bytes;
    a.vcache = static_cast<char *>(vc_[l]) + slot_bytes;
    a.partial = partial_;
    a.out = ctx_;
    a.pos = r.pos;
    a.slot = own_slot ? nullptr : r.slot;
    a.n_seq = r.n_seq;
    a.seq_len = r.seq_len;
    a.n_head = c_.NHead;
    a.n_head_kv = c_.NHeadKV;
    a.head_dim = c_.HeadDim;
    a.rope_dims = c_.RopeDims;
    a.max_cells = n_kv_;
    a.qkv_stride = width;
    a.n_splits = splits_;
    a.eps = c_.RMSEps;
    // a layer with an indexer: which cells each row may read, made beside the projection (both read the block's input)
    shv_qsa_index_args qi{};
    const bool qsa = idxc_[l] != nullptr;
    if (qsa) {
        qi.x = in;
        qi.gamma = p.gamma;
        qi.w = static_cast<const float *>(m_.Tensor(Model::Blk(l, "indexer.qk_fused")).ptr);
        qi.q_norm = static_cast<const float *>(m_.Tensor(Model::Blk(l, "indexer.q_norm")).ptr);
        qi.k_norm = static_cast<const float *>(m_.Tensor(Model::Blk(l, "indexer.k_norm")).ptr);
        qi.rope = rope_;
        const size_t slot_off = own_slot ? static_cast<size_t>(r.host_slot) : 0;
        qi.idxcache = idxc_[l] + slot_off * n_kv_ * c_.IdxDim;
        qi.pooled = pooled_[l] + slot_off * (n_kv_ / c_.IdxRatio + 1) * c_.IdxDim;
        qi.pos = r.pos;
        qi.slot = own_slot ? nullptr : r.slot;
        qi.work = qsa_work_;
        qi.score = qsa_score_;
        qi.mask = qsa_mask_;
        qi.n_seq = r.n_seq;
        qi.seq_len = r.seq_len;
        qi.n_embd = c_.NEmbd;
        qi.idx_heads = c_.IdxHeads;
        qi.idx_dim = c_.IdxDim;
        qi.top_k = c_.IdxTopK;
        qi.ratio = c_.IdxRatio;
        qi.rope_dims = c_.RopeDims;
        qi.max_cells = n_kv_;
        qi.mask_stride = mask_stride_;
        qi.eps = c_.RMSEps;
        a.mask = qsa_mask_;
        a.mask_stride = mask_stride_;
    }
    shv_gemv_q4k_args o{};
    o.w = m_.Tensor(Model::Blk(l, "attn_output")).ptr;
    o.x = ctx_;
    o.y = out;
    o.residual = in;
    o.z = qkv_;
    o.n = c_.NEmbd;
    o.k = c_.NHead * c_.HeadDim;
    o.n_tok = nTok;
    o.prologue = SHV_PRO_MUL_SIGMOID;
    o.head_dim = c_.HeadDim;
    o.x_stride = c_.NHead * c_.HeadDim;
    o.y_stride = c_.NEmbd;
    o.z_stride = width;
    o.fold = r.fold;
    o.fold_rows = r.fold_rows;
    o.fold_out = r.fold_out;
    o.fold_stride = r.fold_stride;
    if (qsa) {
        if (labels) labels->insert(labels->end(), {"attn.qkv", "attn.index", "attn.attn", "attn.out"});
        return {make_op(SHV_OP_GEMV_Q4K, p), make_op(SHV_OP_QSA_INDEX, qi), make_op(SHV_OP_ATTN_DECODE, a), make_op(SHV_OP_GEMV_Q4K, o)};
    }
    if (labels) labels->insert(labels->end(), {"attn.qkv", "attn.attn", "attn.out"});
    return {make_op(SHV_OP_GEMV_Q4K, p), make_op(SHV_OP_ATTN_DECODE, a), make_op(SHV_OP_GEMV_Q4K, o)};
}

void AttnGPU::Run(int layer) {
    if (n_tok_ < 1) throw Error("llm: AttnGPU.Run before Upload");
    dev_.run(Dispatches(layer, in_, out_, n_tok_, nullptr));
}

std::vector<float> AttnGPU::Context() const { return read_back<float>(dev_, ctx_, static_cast<size_t>(n_tok_) * c_.NHead * c_.HeadDim); }
std::vector<float> AttnGPU::Out() const { return read_back<float>(dev_, out_, static_cast<size_t>(n_tok_) * c_.NEmbd); }

std::vector<uint16_t> AttnGPU::K(int l, int cells, int slot) const {
    if (l < 0 || l >= c_.Blocks() || !kc_[l] || cells > n_kv_ || slot < 0 || slot >= slots_) throw Error("llm: AttnGPU.K: no such layer, cell or slot");
    const size_t per = static_cast<size_t>(c_.NHeadKV) * c_.HeadDim;
    return read_back<uint16_t>(dev_, static_cast<uint16_t *>(kc_[l]) + static_cast<size_t>(slot) * n_kv_ * per, cells * per);
}

std::vector<uint16_t> AttnGPU::V(int l, int cells, int slot) const {
    if (l < 0 || l >= c_.Blocks() || !vc_[l] || cells > n_kv_ || slot < 0 || slot >= slots_) throw Error("llm: AttnGPU.V: no such layer, cell or slot");
    // the device keeps V transposed in tiles of 32 cells, [cell/32][kv head][dim][cell%32]; callers
    // get the reference's [cell][kv head][dim]
    const size_t per = static_cast<size_t>(c_.NHeadKV) * c_.HeadDim;
    const std::vector<uint16_t> t = read_back<uint16_t>(dev_, static_cast<uint16_t *>(vc_[l]) + static_cast<size_t>(slot) * n_kv_ * per, n_kv_ * per);
    std::vector<uint16_t> out(static_cast<size_t>(cells) * per);
    for (int c = 0; c < cells; c++)
        for (size_t hd = 0; hd < per; hd++) out[static_cast<size_t>(c) * per + hd] = t[(static_cast<size_t>(c / 32) * per + hd) * 32 + c % 32];
    return out;
}

// --------------------------------------------------------------------------------- Head -------

HeadGPU::HeadGPU(Device &dev, const Model &m, int maxRows) : dev_(dev), m_(m), c_(m.config()), max_rows_(maxRows) {
    if (maxRows < 1) throw Error("llm: HeadGPU needs room for at least one row");
    in_ = static_cast<float *>(dev.alloc(static_cast<size_t>(maxRows) * c_.NEmbd * 4));
    logits_ = static_cast<float *>(dev.alloc(static_cast<size_t>(maxRows) * c_.VocabSize * 4));
}

void HeadGPU::Resize(int rows) {
    if (rows < 1 || rows > max_rows_) throw Error("llm: HeadGPU: " + std::to_string(rows) + " rows, staged for " + std::to_string(max_rows_));
    rows_ = rows;
}

void HeadGPU::Upload(const std::vector<float> &x, int rows) {
    Resize(rows);
    if (x.size() != static_cast<size_t>(rows) * c_.NEmbd) throw Error("llm: HeadGPU.Upload: wrong length");
    dev_.upload(in_, x.data(), x.size() * 4);
}

std::vector<shv_op> HeadGPU::Dispatches(const float *in, int rows, std::vector<std::string> *labels) const {
    return DispatchesTo(in, rows, static_cast<const float *>(m_.Tensor("output_norm.weight").ptr), logits_, c_.VocabSize, labels);
}

std::vector<shv_op> HeadGPU::DispatchesTo(const float *in, int rows, const float *gamma, float *logits, int cols,
                                          std::vector<std::string> *labels) const {
    if (rows < 1 || cols < 1 || cols > c_.VocabSize) throw Error("llm: HeadGPU: " + std::to_string(rows) + " rows over " + std::to_string(cols) + " columns");
    const TensorView &w = m_.Tensor("output.weight");
    if (w.kind == TensorView::RAW) {
        // a head kept in the checkpoint's own type: matvec over rows expanded as Tensor.DequantizeRow expands them
        shv_gemv_args g{};
        g.w = w.ptr;
        g.x = in;
        g.y = logits;
        g.n = cols;
        g.k = c_.NEmbd;
        g.type = static_cast<int32_t>(w.ggml);
        g.n_tok = rows;
        g.gamma = gamma;
        g.eps = c_.RMSEps;
        g.x_stride = c_.NEmbd;
        g.y_stride = c_.VocabSize;
        if (labels) labels->push_back("head");
        return {make_op(SHV_OP_GEMV, g)};
    }
    shv_gemv_q4k_args p{};
    p.w = m_.Tensor("output.weight").ptr;
    p.x = in;
    p.y = logits;
    p.gamma = gamma;
    p.n = cols;
    p.k = c_.NEmbd;
    p.n_tok = rows;
    p.prologue = SHV_PRO_RMSNORM;
    p.eps = c_.RMSEps;
    p.x_stride = c_.NEmbd;
    p.y_stride = c_.VocabSize;
    if (labels) labels->push_back("head");
    return {make_op(SHV_OP_GEMV_Q4K, p)};
}

void HeadGPU::Run() {
    if (rows_ < 1) throw Error("llm: HeadGPU.Run before Upload");
    dev_.run(Dispatches(in_, rows_, nullptr));
}

std::vector<float> HeadGPU::Logits() const { return read_back<float>(dev_, logits_, static_cast<size_t>(rows_) * c_.VocabSize); }

// -------------------------------------------------------------------------------- Graph -------

// LLM_NO_PRERECORD=1 replays nothing: every pass is dispatched op by op, as the reference's
// knob of the same name does (llm/graph.go:306).  Profilers that cannot follow a graph launch
// see every kernel this way.
static bool no_prerecord() {
    const char *e = std::getenv("LLM_NO_PRERECORD");
    return e && e[0] == '1';
}

static uint64_t submit_pass(Device &dev, Pass &p, int iters, const char *what) {
    uint64_t ns = 0;
    if (no_prerecord()) {
        check(shv_dispatch_multi(dev.ctx(), p.ops.data(), static_cast<int>(p.ops.size()), iters, &ns, nullptr), what);
    } else {
        if (!p.rec) check(shv_prerecord(dev.ctx(), p.ops.data(), static_cast<int>(p.ops.size()), &p.rec), what);
        check(shv_prerecorded_submit(dev.ctx(), p.rec, iters, &ns), what);
    }
    return ns;
}

static void drop_passes(Device &dev, std::map<std::vector<int>, Pass> &passes) {
    for (auto &kv : passes)
        if (kv.second.rec) shv_prerecorded_destroy(dev.ctx(), kv.second.rec);
    passes.clear();
}

Graph::Graph(Device &dev, const Model &m, const GraphOpts &opts) : dev_(dev), m_(m), c_(m.config()), o_(opts) {
    layers_ = opts.Layers > 0 ? opts.Layers : c_.NLayer;
    if (layers_ > c_.NLayer) throw Error("llm: NewGraph: " + std::to_string(layers_) + " layers of a " + std::to_string(c_.NLayer) + "-layer model");
    if (o_.MaxTokens < 1 || o_.MaxTokens > 4096) throw Error("llm: NewGraph: MaxTokens " + std::to_string(o_.MaxTokens) + "; a pass carries 1..4096 rows");
    if (o_.Slots < 1 || o_.Slots > 32) throw Error("llm: NewGraph: Slots " + std::to_string(o_.Slots) + "; 1..32");
    if (o_.NKV < 2) throw Error("llm: NewGraph: NKV " + std::to_string(o_.NKV));
    if (o_.Speculative && (o_.SpecRows < 2 || o_.SpecRows > 8)) throw Error("llm: NewGraph: SpecRows " + std::to_string(o_.SpecRows) + "; 2..8");
    if (o_.HeadRows < 0 || o_.HeadRows > 14) throw Error("llm: NewGraph: HeadRows " + std::to_string(o_.HeadRows) + "; the sampler covers 14 rows a pass");
    // the widest pass anything here may ask for
    rows_max_ = std::max(o_.MaxTokens, std::max(o_.HeadRows, o_.Speculative ? o_.SpecRows : 1));
    const int planes = o_.Speculative ? o_.SpecRows + 1 : 1;
    const int head_rows = std::min(14, o_.HeadRows > 0 ? std::max(o_.HeadRows, o_.Speculative ? o_.SpecRows : 1) : rows_max_);
    seq_.assign(o_.Slots, Seq());
    x_ = static_cast<float *>(dev.alloc(static_cast<size_t>(rows_max_) * c_.NEmbd * 4));
    ids_stride_ = static_cast<size_t>(o_.NKV) + 2;
    ids_ = static_cast<int32_t *>(dev.alloc_zero(ids_stride_ * o_.Slots * 4));
    const size_t S = o_.Slots, R = rows_max_;
    ctl_ = static_cast<int32_t *>(dev.alloc_zero((3 * S + 3 * R) * 4));
    pos_ = ctl_;
    plane_ = ctl_ + S;
    slot_ix_ = ctl_ + 2 * S;
    row_pos_ = ctl_ + 3 * S;
    row_slot_ = row_pos_ + R;
    row_ids_ = row_slot_ + R;
    std::vector<int32_t> ix(S);
    for (size_t i = 0; i < S; i++) ix[i] = static_cast<int32_t>(i);
    dev.upload(slot_ix_, ix.data(), S * 4);
    // the rows' arg-maxes land in host memory: read after the pass's wait, no download
    best_ = static_cast<int32_t *>(dev.host_alloc(64 * 4));
    // A long pass goes through every block whole: one projection over all its rows, one walk of
    // the recurrence, one launch of the attention.  LLM_PASS_GROUPS=1 keeps the older order
    // instead, groups of kBlockRows rows through the attention / DeltaNet blocks one after the
    // other (the experts whole either way), for comparison.
    const char *pg = std::getenv("LLM_PASS_GROUPS");
    block_rows_ = pg && pg[0] == '1' ? std::min(rows_max_, kBlockRows) : rows_max_;
    // where each group of such a pass stands: [slot][group] positions, written with the
    // sequences' own before a prompt goes through and moved on by the long passes themselves
    groups_ = (rows_max_ + block_rows_ - 1) / block_rows_;
    if (groups_ > 1) grp_pos_ = static_cast<int32_t *>(dev.alloc_zero(static_cast<size_t>(o_.Slots) * groups_ * 4));
    moe_ = new MoEGPU(dev, m, rows_max_);
    dn_ = new DeltaNetGPU(dev, m, block_rows_, o_.Slots, pos_, planes, plane_);
    attn_ = new AttnGPU(dev, m, block_rows_, o_.NKV, o_.Slots, pos_);
    if (o_.AttnSplits > 0) attn_->SetSplits(o_.AttnSplits);
    if (!o_.NoHead) head_ = new HeadGPU(dev, m, head_rows);
    // One-row passes take the router's logits from the launch of the mixer's output projection
    // (48 launches fewer a step at 48 layers): the tables are made here, once, from the weights
    // as they stand, as the reference makes its banks when it stages a graph (llm/graph.go:635);
    // LLM_ROUTER_FOLD=0 keeps the router's own launch.
    const char *rf = std::getenv("LLM_ROUTER_FOLD");
    if (!(rf && rf[0] == '0')) {
        x2_ = static_cast<float *>(dev.alloc(static_cast<size_t>(MoEGPU::kFoldRows) * c_.NEmbd * 4));
        for (int l = 0; l < layers_; l++) moe_->Fold(l, m.Tensor(Model::Blk(l, c_.IsAttn(l) ? "attn_output" : "ssm_out")));
    }
    // the decode step of slot 0 is recorded up front, as NewGraph does (llm/graph.go:609)
    pass(0, 1, head_ ? kSample : kPrefill, false);
}

Graph::~Graph() {
    drop_passes(dev_, passes_);
    delete moe_;
    delete dn_;
    delete attn_;
    delete head_;
}

// The loop body of llm/graph.go:2330-2466 for a model without hyper-connection streams: the
// residual stream stays in one buffer, every block reads it through its RMSNorm prologue and
// adds its output back in place.  What follows the layers depends on the kind of pass:
//   kPrefill  nothing; the position moves on by the pass's rows
//   kSample   the head on the last row; its arg-max becomes the next token and the position moves
//   kRows     the head and arg-max on every row (ExtendRows); the position moves
//   kBatch    one row per sequence, positions and slots from the row tables (DecodeRows)
Pass &Graph::pass(int slot, int rows, Kind kind, bool spec) {
    const std::vector<int> key{slot, rows, static_cast<int>(kind), spec ? 1 : 0};
    auto it = passes_.find(key);
    if (it != passes_.end()) return it->second;
    if (rows < 1 || rows > rows_max_) throw Error("llm: a pass of " + std::to_string(rows) + " rows, the arenas hold " + std::to_string(rows_max_) + " — GraphOpts.MaxTokens");
    if ((kind == kRows || kind == kBatch) && (!head_ || rows > head_->MaxRows()))
        throw Error("llm: " + std::to_string(rows) + " rows, the head arena holds " + std::to_string(head_ ? head_->MaxRows() : 0) + " — GraphOpts.HeadRows");
    Pass p;
    PassRows r;
    r.spec = spec;
    shv_embed_args e{};
    e.table = m_.Tensor("token_embd.weight").ptr;
    e.type = static_cast<int32_t>(m_.Tensor("token_embd.weight").ggml);
    e.x = x_;
    e.n_tok = rows;
    e.n_embd = c_.NEmbd;
    e.vocab = c_.VocabSize;
    e.x_stride = c_.NEmbd;
    if (kind == kBatch) {
        r.pos = row_pos_;
        r.slot = row_slot_;
        r.n_seq = rows;
        r.seq_len = 1;
        e.ids = row_ids_;
    } else {
        r.pos = pos_ + slot;
        r.slot = slot_ix_ + slot;
        r.host_slot = slot;
        r.n_seq = 1;
        r.seq_len = rows;
        e.ids = ids_ + slot * ids_stride_;
        e.pos = pos_ + slot;
    }
    p.ops.push_back(make_op(SHV_OP_EMBED, e));
    p.labels.push_back("embed");
    if (rows > kBlockRows && (kind == kBatch || spec)) throw Error("llm: a pass of " + std::to_string(rows) + " rows is a plain prompt pass; batched and rewindable passes carry up to " + std::to_string(kBlockRows));
    for (int l = 0; l < layers_; l++) {
        // (rows of one sequence or one row each of several: LLM_BATCH_FOLD=0 keeps the router's launches in batched passes)
        static const bool batch_fold = [] { const char *e = std::getenv("LLM_BATCH_FOLD"); return !(e && e[0] == '0'); }();
        if (x2_ && moe_->Folded(l) && (rows == 1 || ((kind != kBatch || batch_fold) && rows <= MoEGPU::kFoldRows && moe_->FusedRouter(rows)))) {
            // the mixer writes the row beside the stream (its output projection reads the whole
            // residual row for the router's products while it writes), the MoE block brings it back
            PassRows rf = r;
            moe_->FoldInto(l, rf);
            auto sub = c_.IsAttn(l) ? attn_->Dispatches(l, x_, x2_, rf, &p.labels) : dn_->Dispatches(l, x_, x2_, rf, &p.labels);
            p.ops.insert(p.ops.end(), sub.begin(), sub.end());
            auto ffn = moe_->DispatchesFolded(l, x2_, x_, rows, &p.labels);
            p.ops.insert(p.ops.end(), ffn.begin(), ffn.end());
            continue;
        }
        if (rows <= block_rows_) {
            auto sub = c_.IsAttn(l) ? attn_->Dispatches(l, x_, x_, r, &p.labels) : dn_->Dispatches(l, x_, x_, r, &p.labels);
            p.ops.insert(p.ops.end(), sub.begin(), sub.end());
        } else {
            // every group reads its own position word, so it finds its cells, ring rows and
            // rotary angles where a pass of its own would
            for (int r0 = 0, j = 0; r0 < rows; r0 += block_rows_, j++) {
                PassRows g = r;
                g.pos = grp_pos_ + static_cast<size_t>(slot) * groups_ + j;
                g.seq_len = std::min(block_rows_, rows - r0);
                float *xg = x_ + static_cast<size_t>(r0) * c_.NEmbd;
                auto sub = c_.IsAttn(l) ? attn_->Dispatches(l, xg, xg, g, &p.labels) : dn_->Dispatches(l, xg, xg, g, &p.labels);
                p.ops.insert(p.ops.end(), sub.begin(), sub.end());
            }
        }
        auto ffn = moe_->Dispatches(l, x_, x_, rows, &p.labels);
        p.ops.insert(p.ops.end(), ffn.begin(), ffn.end());
    }
    shv_argmax_args am{};
    if (head_) {
        am.logits = head_->LogitsPort();
        am.best = best_;
        am.n = c_.VocabSize;
        am.logits_stride = c_.VocabSize;
    }
    shv_advance_args adv{pos_ + (slot < 0 ? 0 : slot), 1, rows};
    if (rows > block_rows_) {
        shv_advance_args ga{grp_pos_ + static_cast<size_t>(slot) * groups_, groups_, rows};
        p.ops.push_back(make_op(SHV_OP_ADVANCE, ga));
        p.labels.push_back("advance");
    }
    switch (kind) {
        case kPrefill:
            p.ops.push_back(make_op(SHV_OP_ADVANCE, adv));
            p.labels.push_back("advance");
            break;
        case kSample: {
            if (!head_) throw Error("llm: this graph was staged without a head");
            auto h = head_->Dispatches(x_ + static_cast<size_t>(rows - 1) * c_.NEmbd, 1, &p.labels);
            am.ids = ids_ + slot * ids_stride_;
            am.pos = pos_ + slot;
            am.n_rows = 1;
            am.advance = rows;
            // The vocabulary projection names the next token itself: its last block to finish does
            // what the arg-max launch would (LLM_HEAD_ARGMAX=0 keeps that launch).
            const char *ha = std::getenv("LLM_HEAD_ARGMAX");
            if (!(ha && ha[0] == '0') && h.size() == 1 && h[0].kind == SHV_OP_GEMV_Q4K) {
                shv_gemv_q4k_args g{};
                std::memcpy(&g, h[0].args, sizeof g);
                g.amax_best = am.best;
                g.amax_ids = am.ids;
                g.amax_pos = am.pos;
                g.amax_advance = am.advance;
                p.ops.push_back(make_op(SHV_OP_GEMV_Q4K, g));
                break;
            }
            p.ops.insert(p.ops.end(), h.begin(), h.end());
            p.ops.push_back(make_op(SHV_OP_ARGMAX, am));
            p.labels.push_back("argmax");
            break;
        }
        case kRows:
        case kBatch: {
            auto h = head_->Dispatches(x_, rows, &p.labels);
            p.ops.insert(p.ops.end(), h.begin(), h.end());
            am.n_rows = rows;
            p.ops.push_back(make_op(SHV_OP_ARGMAX, am));
            p.labels.push_back("argmax");
            if (kind == kRows) {
                p.ops.push_back(make_op(SHV_OP_ADVANCE, adv));
                p.labels.push_back("advance");
            }
            break;
        }
    }
    return passes_[key] = std::move(p);
}

uint64_t Graph::submit(Pass &p, int iters, const char *what) {
    const uint64_t ns = submit_pass(dev_, p, iters, what);
    Stats.GPUNanos += ns;
    Stats.Dispatches = static_cast<int>(p.ops.size());
    return ns;
}

int Graph::Dispatches() { return static_cast<int>(pass(slot_, 1, head_ ? kSample : kPrefill, false).ops.size()); }

// The host is the authority on where each sequence stands between calls; the recorded passes
// move the device copy themselves while they replay.
void Graph::put_pos() {
    std::vector<int32_t> v(2 * o_.Slots);
    for (int s = 0; s < o_.Slots; s++) {
        v[s] = seq_[s].past;
        v[o_.Slots + s] = seq_[s].plane;
    }
    dev_.upload(ctl_, v.data(), v.size() * 4);
    if (groups_ > 1) {
        std::vector<int32_t> g(static_cast<size_t>(o_.Slots) * groups_);
        for (int s = 0; s < o_.Slots; s++)
            for (int j = 0; j < groups_; j++) g[static_cast<size_t>(s) * groups_ + j] = seq_[s].past + j * block_rows_;
        dev_.upload(grp_pos_, g.data(), g.size() * 4);
    }
}

void Graph::Reset() {
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    dn_->ResetSlot(slot_);
    seq_[slot_] = Seq();
    put_pos();
}

void Graph::UseSlot(int s) {
    if (s < 0 || s >= o_.Slots) throw Error("llm: sequence slot " + std::to_string(s) + " of " + std::to_string(o_.Slots));
    if (spec_armed_ && s != slot_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    slot_ = s;
}

void Graph::check_ids(const std::vector<int32_t> &ids) const {
    for (int32_t id : ids)
        if (id < 0 || id >= c_.VocabSize) throw Error("llm: token " + std::to_string(id) + " is outside the vocabulary");
}

void Graph::Forward(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden) {
    Reset();
    Extend(ids, logits, hidden);
}

// The rows go through in chunks of MaxTokens; every chunk but the last is headless, the last one
// samples.  res_all, when given, receives every row's residual.
void Graph::extend(const std::vector<int32_t> &ids, float *res_all) {
    const int n = static_cast<int>(ids.size());
    Seq &q = seq_[slot_];
    if (n < 1) throw Error("llm: Graph.Extend: no tokens");
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past + n + 1 > o_.NKV) throw Error("llm: Graph.Extend: " + std::to_string(q.past + n) + " tokens do not fit " + std::to_string(o_.NKV) + " cells");
    check_ids(ids);
    dev_.upload(ids_ + slot_ * ids_stride_ + q.past, ids.data(), static_cast<size_t>(n) * 4);
    put_pos();
    const int M = o_.MaxTokens;
    const int last = n % M == 0 ? M : n % M;
    const int full = (n - last) / M;
    const size_t row_bytes = static_cast<size_t>(c_.NEmbd) * 4;
    if (full > 0) {
        Pass &p = pass(slot_, M, kPrefill, false);
        if (res_all) {
            for (int i = 0; i < full; i++) {
                submit(p, 1, "prefill");
                check(shv_copy(dev_.ctx(), res_all + static_cast<size_t>(i) * M * c_.NEmbd, x_, M * row_bytes), "keep residual");
            }
        } else {
            submit(p, full, "prefill");
        }
    }
    submit(pass(slot_, last, head_ ? kSample : kPrefill, false), 1, "last rows");
    if (res_all) check(shv_copy(dev_.ctx(), res_all + static_cast<size_t>(full) * M * c_.NEmbd, x_, last * row_bytes), "keep residual");
    Stats.Runs++;
    q.past += n;
    last_rows_ = last;
}

int Graph::StepRows() const { return head_ ? std::min(head_->MaxRows(), o_.Slots) : 0; }

void Graph::Extend(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden) {
    if (logits && !head_) throw Error("llm: Graph.Extend: the graph was staged without a head");
    extend(ids, nullptr);
    if (logits) {
        logits->resize(c_.VocabSize);
        dev_.download(logits->data(), head_->LogitsPort(), static_cast<size_t>(c_.VocabSize) * 4);
    }
    if (hidden) {
        hidden->resize(c_.NEmbd);
        dev_.download(hidden->data(), x_ + static_cast<size_t>(last_rows_ - 1) * c_.NEmbd, static_cast<size_t>(c_.NEmbd) * 4);
    }
}

const float *Graph::ForwardResidual(const std::vector<int32_t> &ids, std::vector<float> *logits) {
    if (logits && !head_) throw Error("llm: Graph.ForwardResidual: the graph was staged without a head");
    Reset();
    if (ids.size() > res_all_rows_) {
        // grown, never shrunk: the device's allocations live as long as the device
        res_all_rows_ = std::max<size_t>(ids.size(), 256);
        res_all_ = static_cast<float *>(dev_.alloc(res_all_rows_ * c_.NEmbd * 4));
    }
    extend(ids, res_all_);
    if (logits) {
        logits->resize(c_.VocabSize);
        dev_.download(logits->data(), head_->LogitsPort(), static_cast<size_t>(c_.VocabSize) * 4);
    }
    return res_all_;
}

const float *Graph::ExtendResidual(const std::vector<int32_t> &ids, std::vector<float> *logits) {
    if (logits && !head_) throw Error("llm: Graph.ExtendResidual: the graph was staged without a head");
    if (ids.size() > res_all_rows_) {
        res_all_rows_ = std::max<size_t>(ids.size(), 256);
        res_all_ = static_cast<float *>(dev_.alloc(res_all_rows_ * c_.NEmbd * 4));
    }
    extend(ids, res_all_);
    if (logits) {
        logits->resize(c_.VocabSize);
        dev_.download(logits->data(), head_->LogitsPort(), static_cast<size_t>(c_.VocabSize) * 4);
    }
    return res_all_;
}

void Graph::ExtendRows(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *res) {
    if (!head_) throw Error("llm: this graph was staged without a head");
    const int n = static_cast<int>(ids.size());
    Seq &q = seq_[slot_];
    if (n <= 0 || n > head_->MaxRows()) throw Error("llm: " + std::to_string(n) + " rows, the head arena holds " + std::to_string(head_->MaxRows()) + " — GraphOpts.HeadRows");
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past + n + 1 > o_.NKV) throw Error("llm: Graph.ExtendRows: " + std::to_string(q.past + n) + " tokens do not fit " + std::to_string(o_.NKV) + " cells");
    check_ids(ids);
    Pass &p = pass(slot_, n, kRows, spec_);
    dev_.upload(ids_ + slot_ * ids_stride_ + q.past, ids.data(), static_cast<size_t>(n) * 4);
    put_pos();
    submit(p, 1, "rows");
    Stats.Runs++;
    if (spec_) {
        spec_armed_ = true;
        spec_past_ = q.past;
        spec_rows_ = n;
    }
    q.past += n;
    last_rows_ = n;
    if (logits) {
        logits->resize(static_cast<size_t>(n) * c_.VocabSize);
        dev_.download(logits->data(), head_->LogitsPort(), logits->size() * 4);
    }
    if (res) {
        res->resize(static_cast<size_t>(n) * c_.NEmbd);
        dev_.download(res->data(), x_, res->size() * 4);
    }
}

void Graph::StageIds(int at, const std::vector<int32_t> &ids) {
    if (at < 0 || at + static_cast<int>(ids.size()) > o_.NKV) throw Error("llm: Graph.StageIds: positions " + std::to_string(at) + ".. do not fit " + std::to_string(o_.NKV) + " cells");
    check_ids(ids);
    dev_.upload(ids_ + slot_ * ids_stride_ + at, ids.data(), ids.size() * 4);
}

void Graph::ExtendRowsStaged(int n) {
    if (!head_) throw Error("llm: this graph was staged without a head");
    Seq &q = seq_[slot_];
    if (n <= 0 || n > head_->MaxRows()) throw Error("llm: " + std::to_string(n) + " rows, the head arena holds " + std::to_string(head_->MaxRows()) + " — GraphOpts.HeadRows");
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past + n + 1 > o_.NKV) throw Error("llm: Graph.ExtendRows: " + std::to_string(q.past + n) + " tokens do not fit " + std::to_string(o_.NKV) + " cells");
    Pass &p = pass(slot_, n, kRows, spec_);
    put_pos();
    submit(p, 1, "rows");
    Stats.Runs++;
    if (spec_) {
        spec_armed_ = true;
        spec_past_ = q.past;
        spec_rows_ = n;
    }
    q.past += n;
    last_rows_ = n;
}

void Graph::DecodeRows(const std::vector<int> &slots, const std::vector<int32_t> &ids, std::vector<float> *logits) {
    const int n = static_cast<int>(slots.size());
    if (n == 0 || n != static_cast<int>(ids.size())) throw Error("llm: " + std::to_string(n) + " slots and " + std::to_string(ids.size()) + " tokens");
    if (!head_) throw Error("llm: this graph was staged without a head");
    if (n > head_->MaxRows()) throw Error("llm: " + std::to_string(n) + " rows, the head arena holds " + std::to_string(head_->MaxRows()) + " — GraphOpts.HeadRows");
    if (spec_) throw Error("llm: a speculating graph cannot batch sequences");
    check_ids(ids);
    // checkBatch (llm/batch.go:45-63): a slot out of range or named twice, a position past the cache
    std::vector<int32_t> rows(3 * static_cast<size_t>(rows_max_), 0);
    std::vector<bool> seen(o_.Slots, false);
    for (int r = 0; r < n; r++) {
        const int s = slots[r];
        if (s < 0 || s >= o_.Slots) throw Error("llm: batch row on slot " + std::to_string(s) + " of " + std::to_string(o_.Slots));
        if (seen[s]) throw Error("llm: slot " + std::to_string(s) + " twice in one batch");
        seen[s] = true;
        if (seq_[s].past + 2 > o_.NKV) throw Error("llm: a token at position " + std::to_string(seq_[s].past) + " of a " + std::to_string(o_.NKV) + "-cell context");
        rows[r] = seq_[s].past;
        rows[rows_max_ + r] = s;
        rows[2 * rows_max_ + r] = ids[r];
    }
    Pass &p = pass(-1, n, kBatch, false);
    put_pos();
    dev_.upload(row_pos_, rows.data(), rows.size() * 4);
    for (int r = 0; r < n; r++) dev_.upload(ids_ + slots[r] * ids_stride_ + seq_[slots[r]].past, &ids[r], 4);
    submit(p, 1, "batched rows");
    Stats.Runs++;
    for (int r = 0; r < n; r++) seq_[slots[r]].past++;
    put_pos();
    last_rows_ = n;
    if (logits) {
        logits->resize(static_cast<size_t>(n) * c_.VocabSize);
        dev_.download(logits->data(), head_->LogitsPort(), logits->size() * 4);
    }
}

std::vector<int32_t> Graph::Argmaxes() const {
    dev_.sync();  // every pass is waited for when it is submitted; this costs nothing then
    return std::vector<int32_t>(best_, best_ + (last_rows_ > 0 ? last_rows_ : 1));
}

std::vector<int32_t> Graph::Generate(int n, uint64_t *gpu_nanos) {
    Seq &q = seq_[slot_];
    if (!head_) throw Error("llm: Graph.Generate: the graph was staged without a head");
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past < 1) throw Error("llm: Graph.Generate before a prompt");
    if (n < 1 || q.past + n + 1 > o_.NKV) throw Error("llm: Graph.Generate: " + std::to_string(n) + " more tokens do not fit the cache");
    // the last Extend already sampled the token at position past: it sits in ids[past], and
    // every replay consumes ids[pos] and appends ids[pos+1]
    uint64_t ns = 0;
    if (n > 1) {
        put_pos();
        ns = submit(pass(slot_, 1, kSample, false), n - 1, "generate");
    }
    if (gpu_nanos) *gpu_nanos = ns;
    std::vector<int32_t> out(n);
    dev_.download(out.data(), ids_ + slot_ * ids_stride_ + q.past, static_cast<size_t>(n) * 4);
    q.past += n - 1;
    last_rows_ = 1;
    return out;
}

std::vector<int32_t> Graph::Ids() const { return read_back<int32_t>(dev_, ids_ + slot_ * ids_stride_, seq_[slot_].past); }

// ---- rewindable passes (llm/graph.go:1122-1267) ----
// The DeltaNet state is the only thing a pass changes that a shorter sequence would still see:
// a cache cell or a projection-ring row past the end of the sequence is never read.  A rewindable
// pass therefore leaves the committed state plane alone and stores the state after each of its
// rows in the planes that follow it, and ending the pass is moving two integers.

void Graph::Speculate(bool on) {
    if (on == spec_) return;
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (on && dn_->Planes() < 2)
        throw Error("llm: this block was staged with one state slot; a rewindable pass needs two (GraphOpts.Speculative)");
    spec_ = on;
}

void Graph::SpeculateFirst(bool on) {
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    spec_first_ = on;
}

void Graph::Keep(int k) {
    if (!spec_armed_) throw Error("llm: nothing to keep; no speculative pass has run");
    if (!spec_first_) throw Error("llm: this pass did not store its prefixes apart (SpeculateFirst)");
    if (k < 1 || k > spec_rows_) throw Error("llm: keeping " + std::to_string(k) + " rows of a " + std::to_string(spec_rows_) + "-row pass");
    if (k == spec_rows_) return Commit();
    Seq &q = seq_[slot_];
    q.plane = (q.plane + k) % dn_->Planes();
    q.past = spec_past_ + k;
    put_pos();
    spec_armed_ = false;
}

void Graph::Commit() {
    if (!spec_armed_) throw Error("llm: nothing to commit; no speculative pass has run");
    Seq &q = seq_[slot_];
    q.plane = (q.plane + spec_rows_) % dn_->Planes();
    put_pos();
    spec_armed_ = false;
}

void Graph::Rewind() {
    if (!spec_armed_) throw Error("llm: nothing to rewind; no speculative pass has run");
    if (spec_first_) throw Error("llm: a keep-first pass is ended by KeepFirst or Commit");
    seq_[slot_].past = spec_past_;
    put_pos();
    spec_armed_ = false;
}

// One real decode step (the sequence advances by one token, as after Generate(1)), dispatched op
// by op so that every op has its own GPU time.
static std::vector<Stage> fold_stages(const Pass &p, const std::vector<uint64_t> &per, uint64_t total, std::map<std::string, uint64_t> *kinds_out) {
    std::map<std::string, uint64_t> kinds;
    std::vector<std::string> order;
    for (size_t i = 0; i < per.size(); i++) {
        if (!kinds.count(p.labels[i])) order.push_back(p.labels[i]);
        kinds[p.labels[i]] += per[i];
    }
    std::vector<Stage> out;
    for (const auto &k : order) out.push_back({k, kinds[k]});
    out.push_back({"total", total});
    if (kinds_out) *kinds_out = kinds;
    return out;
}

std::vector<Stage> Graph::ProfileStep() {
    Seq &q = seq_[slot_];
    if (!head_) throw Error("llm: Graph.ProfileStep: the graph was staged without a head");
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past < 1 || q.past + 2 > o_.NKV) throw Error("llm: Graph.ProfileStep: needs a prompt and a free cell");
    Pass &p = pass(slot_, 1, kSample, false);
    put_pos();
    std::vector<uint64_t> per(p.ops.size());
    uint64_t total = 0;
    check(shv_dispatch_multi(dev_.ctx(), p.ops.data(), static_cast<int>(p.ops.size()), 1, &total, per.data()), "profile step");
    q.past += 1;
    return fold_stages(p, per, total, &Stats.Kinds);
}

// A `rows`-row verification pass timed op by op and then discarded: the sequence is where it was.
std::vector<Stage> Graph::ProfileRows(int rows) {
    Seq &q = seq_[slot_];
    if (!head_) throw Error("llm: Graph.ProfileRows: the graph was staged without a head");
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (dn_->Planes() <= rows) throw Error("llm: Graph.ProfileRows: a discarded pass of " + std::to_string(rows) + " rows needs GraphOpts.Speculative with SpecRows >= " + std::to_string(rows));
    if (q.past < 1 || q.past + rows + 1 > o_.NKV) throw Error("llm: Graph.ProfileRows: needs a prompt and free cells");
    Pass &p = pass(slot_, rows, kRows, true);
    // the rows re-run the sequence's own next token `rows` times over: values do not matter here
    std::vector<int32_t> next(1);
    dev_.download(next.data(), ids_ + slot_ * ids_stride_ + q.past, 4);
    std::vector<int32_t> ids(rows, next[0]);
    put_pos();
    dev_.upload(ids_ + slot_ * ids_stride_ + q.past, ids.data(), ids.size() * 4);
    std::vector<uint64_t> per(p.ops.size());
    uint64_t total = 0;
    check(shv_dispatch_multi(dev_.ctx(), p.ops.data(), static_cast<int>(p.ops.size()), 1, &total, per.data()), "profile rows");
    put_pos();  // discarded: the position goes back, the committed plane never moved
    return fold_stages(p, per, total, nullptr);
}

void Graph::Checkpoint(struct Checkpoint &c) {
    const Seq &q = seq_[slot_];
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past == 0) throw Error("llm: nothing to checkpoint at position 0");
    c.past = q.past;
    c.ids.resize(q.past);
    dev_.download(c.ids.data(), ids_ + slot_ * ids_stride_, static_cast<size_t>(q.past) * 4);
    c.dn.resize(dn_->CarriedLen());
    dn_->SaveCarried(c.dn.data(), slot_, q.plane, q.past);
}

void Graph::Restore(const struct Checkpoint &c) {
    Seq &q = seq_[slot_];
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    bool same = c.past > 0 && c.past <= q.past && static_cast<int>(c.ids.size()) == c.past && c.dn.size() == dn_->CarriedLen();
    if (same) {
        std::vector<int32_t> have(c.past);
        dev_.download(have.data(), ids_ + slot_ * ids_stride_, static_cast<size_t>(c.past) * 4);
        same = have == c.ids;
    }
    if (!same) throw Error("llm: this slot no longer holds the checkpoint's tokens");
    dn_->RestoreCarried(c.dn.data(), slot_, q.plane, c.past);
    q.past = c.past;
    put_pos();
}

// One headless prompt chunk timed op by op; unlike ProfileRows it is a real Extend: the sequence
// advances by the chunk.
std::vector<Stage> Graph::ProfileChunk(const std::vector<int32_t> &ids) {
    const int n = static_cast<int>(ids.size());
    Seq &q = seq_[slot_];
    if (n < 1 || n > o_.MaxTokens) throw Error("llm: Graph.ProfileChunk: " + std::to_string(n) + " rows; 1.." + std::to_string(o_.MaxTokens));
    if (spec_armed_) throw Error("llm: a speculative pass is in flight; commit or rewind it first");
    if (q.past + n + 1 > o_.NKV) throw Error("llm: Graph.ProfileChunk: " + std::to_string(q.past + n) + " tokens do not fit " + std::to_string(o_.NKV) + " cells");
    check_ids(ids);
    dev_.upload(ids_ + slot_ * ids_stride_ + q.past, ids.data(), static_cast<size_t>(n) * 4);
    put_pos();
    Pass &p = pass(slot_, n, kPrefill, false);
    std::vector<uint64_t> per(p.ops.size());
    uint64_t total = 0;
    check(shv_dispatch_multi(dev_.ctx(), p.ops.data(), static_cast<int>(p.ops.size()), 1, &total, per.data()), "profile chunk");
    q.past += n;
    return fold_stages(p, per, total, nullptr);
}

// ------------------------------------------------------------------------------ MTPHead -------

MTPHead::MTPHead(Device &dev, const Model &m, HeadGPU &head, int maxTok, int nKV, int slots)
    : dev_(dev), m_(m), c_(m.config()), head_(head), max_tok_(maxTok), n_kv_(nKV), layer_(m.config().NLayer) {
    if (c_.NextN != 1) throw Error("llm: the model carries no draft block (nextn_predict_layers is " + std::to_string(c_.NextN) + ")");
    if (maxTok < 1 || maxTok > 64) throw Error("llm: MTPHead: " + std::to_string(maxTok) + " rows a call; 1..64");
    if (slots < 1) throw Error("llm: MTPHead: no slots");
    pasts_.assign(slots, 0);
    const size_t T = maxTok, E = c_.NEmbd;
    x_ = static_cast<float *>(dev.alloc(T * E * 4));
    h_ = static_cast<float *>(dev.alloc(T * E * 4));
    e_ = static_cast<float *>(dev.alloc(T * E * 4));
    logits_ = static_cast<float *>(dev.alloc(static_cast<size_t>(c_.VocabSize) * 4));
    const size_t S = slots;
    ctl_ = static_cast<int32_t *>(dev.alloc_zero((2 * S + T + 16) * 4));
    pos_ = ctl_;
    slot_ix_ = ctl_ + S;
    ids_ = ctl_ + 2 * S;
    best_ = static_cast<int32_t *>(dev.host_alloc(16 * 4));  // the draft's arg-max, read by the host after the pass's wait
    std::vector<int32_t> ix(S);
    for (size_t i = 0; i < S; i++) ix[i] = static_cast<int32_t>(i);
    dev.upload(slot_ix_, ix.data(), S * 4);
    attn_ = new AttnGPU(dev, m, maxTok, nKV, slots, pos_, layer_);
    moe_ = new MoEGPU(dev, m, maxTok);
}

MTPHead::~MTPHead() {
    drop_passes(dev_, passes_);
    delete attn_;
    delete moe_;
}

void MTPHead::Rewind(int n) {
    if (n < 0 || n > pasts_[slot_]) throw Error("llm: rewind to " + std::to_string(n) + " of " + std::to_string(pasts_[slot_]));
    pasts_[slot_] = n;
}

void MTPHead::UseSlot(int s) {
    if (s < 0 || s >= static_cast<int>(pasts_.size())) throw Error("llm: draft cache slot " + std::to_string(s) + " of " + std::to_string(pasts_.size()));
    slot_ = s;
}

void MTPHead::SetVocab(int k) {
    if (k < 0 || k > c_.VocabSize) throw Error("llm: a draft vocabulary of " + std::to_string(k) + " of " + std::to_string(c_.VocabSize));
    if (k != vocab_) drop_passes(dev_, passes_);
    vocab_ = k;
}

Pass &MTPHead::draft_pass(int n, bool head, int k, int32_t *ring) {
    // ring: the tokens come from the trunk's id ring at this head's position word, and the arg-max goes back there
    const std::vector<int> key{slot_, n, head ? 1 : 0, ring ? 1 + k : 0};
    auto it = passes_.find(key);
    if (it != passes_.end() && it->second.ring != ring) {
        if (it->second.rec) shv_prerecorded_destroy(dev_.ctx(), it->second.rec);
        passes_.erase(it);
        it = passes_.end();
    }
    if (it == passes_.end()) {
        Pass p;
        p.ring = ring;
        const int E = c_.NEmbd;
        shv_embed_args e{};
        e.table = m_.Tensor("token_embd.weight").ptr;
        e.type = static_cast<int32_t>(m_.Tensor("token_embd.weight").ggml);
        e.ids = ring ? ring : ids_;
        e.pos = ring ? pos_ + slot_ : nullptr;
        e.x = e_;
        e.n_tok = n;
        e.n_embd = E;
        e.vocab = c_.VocabSize;
        e.x_stride = E;
        p.ops.push_back(make_op(SHV_OP_EMBED, e));
        p.labels.push_back("embed");
        shv_gemv_q4k_args g{};
        g.w = m_.Tensor(Model::Blk(layer_, "nextn.eh_proj")).ptr;
        g.x = e_;
        g.z = h_;
        g.y = x_;
        g.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(layer_, "nextn.ehnorm_fused")).ptr);
        g.n = E;
        g.k = 2 * E;
        g.n_tok = n;
        g.prologue = SHV_PRO_RMSNORM_PAIR;
        g.eps = c_.RMSEps;
        g.x_stride = g.z_stride = g.y_stride = E;
        p.ops.push_back(make_op(SHV_OP_GEMV_Q4K, g));
        p.labels.push_back("mtp.eh_proj");
        PassRows r;
        r.pos = pos_ + slot_;
        r.slot = slot_ix_ + slot_;
        r.host_slot = slot_;
        r.seq_len = n;
        auto a = attn_->Dispatches(layer_, x_, x_, r, &p.labels);
        p.ops.insert(p.ops.end(), a.begin(), a.end());
        auto f = moe_->Dispatches(layer_, x_, x_, n, &p.labels);
        p.ops.insert(p.ops.end(), f.begin(), f.end());
        if (head) {
            const int cols = vocab_ > 0 ? vocab_ : c_.VocabSize;
            auto h = head_.DispatchesTo(x_ + static_cast<size_t>(n - 1) * E, 1,
                                        static_cast<const float *>(m_.Tensor(Model::Blk(layer_, "nextn.shared_head_norm")).ptr), logits_, cols, &p.labels);
            p.ops.insert(p.ops.end(), h.begin(), h.end());
            shv_argmax_args am{};
            am.logits = logits_;
            am.best = best_ + (ring ? k : 0);
            if (ring) {
                am.ids = ring;
                am.pos = pos_ + slot_;
                am.advance = n;
            }
            am.n_rows = 1;
            am.n = cols;
            am.logits_stride = c_.VocabSize;
            p.ops.push_back(make_op(SHV_OP_ARGMAX, am));
            p.labels.push_back("argmax");
        }
        it = passes_.emplace(key, std::move(p)).first;
    }
    return it->second;
}

void MTPHead::RowsChained(const float *hs, int n, int pos, int k, int32_t *ring) {
    if (!hs || !ring || n < 1 || n > max_tok_) throw Error("llm: MTPHead.RowsChained: " + std::to_string(n) + " rows, staged for " + std::to_string(max_tok_));
    if (k < 0 || k >= 16) throw Error("llm: MTPHead.RowsChained: draft " + std::to_string(k));
    const int at = pos >= 0 ? pos : pasts_[slot_];  // the device's position word follows the calls as pasts_ does
    if (at > pasts_[slot_]) throw Error("llm: MTPHead.Rows: position " + std::to_string(at) + " leaves a gap after the draft cache's " + std::to_string(pasts_[slot_]) + " cells");
    if (at + n + 1 > n_kv_) throw Error("llm: MTPHead.Rows: " + std::to_string(at + n) + " cells do not fit " + std::to_string(n_kv_));
    Pass &pass = draft_pass(n, true, k, ring);
    check(shv_copy(dev_.ctx(), h_, hs, static_cast<size_t>(n) * c_.NEmbd * 4), "draft input");
    if (pos >= 0) {
        const int32_t p32 = pos;
        dev_.upload(pos_ + slot_, &p32, 4);
    }
    if (!pass.rec) check(shv_prerecord(dev_.ctx(), pass.ops.data(), static_cast<int>(pass.ops.size()), &pass.rec), "draft");
    check(shv_prerecorded_launch(dev_.ctx(), pass.rec), "draft");
    Steps++;
    pasts_[slot_] = at + n;
}

int32_t MTPHead::Rows(const float *hs, const std::vector<int32_t> &ids, int pos, bool head) {
    const int n = static_cast<int>(ids.size());
    if (!hs || n < 1 || n > max_tok_) throw Error("llm: MTPHead.Rows: " + std::to_string(n) + " rows, staged for " + std::to_string(max_tok_));
    if (pos < 0 || pos > pasts_[slot_]) throw Error("llm: MTPHead.Rows: position " + std::to_string(pos) + " leaves a gap after the draft cache's " + std::to_string(pasts_[slot_]) + " cells");
    if (pos + n + 1 > n_kv_) throw Error("llm: MTPHead.Rows: " + std::to_string(pos + n) + " cells do not fit " + std::to_string(n_kv_));
    for (int32_t id : ids)
        if (id < 0 || id >= c_.VocabSize) throw Error("llm: token " + std::to_string(id) + " is outside the vocabulary");
    Pass &pass = draft_pass(n, head, 0, nullptr);
    // the block's input h may be this block's own output rows: it is copied aside first
    check(shv_copy(dev_.ctx(), h_, hs, static_cast<size_t>(n) * c_.NEmbd * 4), "draft input");
    dev_.upload(ids_, ids.data(), static_cast<size_t>(n) * 4);
    const int32_t p32 = pos;
    dev_.upload(pos_ + slot_, &p32, 4);
    GPUNanos += submit_pass(dev_, pass, 1, "draft");
    Steps++;
    pasts_[slot_] = pos + n;
    if (!head) return -1;
    return best_[0];  // submit_pass has waited for the pass
}

void MTPHead::RowsHost(const std::vector<float> &hs, const std::vector<int32_t> &ids, int pos, bool head, std::vector<float> *logits,
                       std::vector<float> *res) {
    const size_t n = ids.size(), E = c_.NEmbd;
    if (n < 1 || n > static_cast<size_t>(max_tok_) || hs.size() != n * E) throw Error("llm: the hidden state is " + std::to_string(hs.size()) + " values, want " + std::to_string(n * E));
    // staged through the embedding arena, which the pass overwrites only after h has been copied aside
    dev_.upload(e_, hs.data(), hs.size() * 4);
    Rows(e_, ids, pos, head);
    if (logits && head) {
        logits->resize(vocab_ > 0 ? vocab_ : c_.VocabSize);
        dev_.download(logits->data(), logits_, logits->size() * 4);
    }
    if (res) {
        res->resize(n * E);
        dev_.download(res->data(), x_, res->size() * 4);
    }
}

void MTPHead::LastLogits(std::vector<float> *out) {
    out->resize(vocab_ > 0 ? vocab_ : c_.VocabSize);
    dev_.download(out->data(), logits_, out->size() * 4);
}

// --------------------------------------------------------------------------- Speculator -------

Speculator::Speculator(Graph &g, MTPHead &d, int depth, int slot) : Depth(depth), g_(g), d_(d), slot_(slot) {
    if (depth < 1 || depth + 1 > g.MaxRows()) throw Error("llm: a draft depth of " + std::to_string(depth) + " needs passes of " + std::to_string(depth + 1) + " rows — GraphOpts.SpecRows");
    if (d.MaxRows() < depth + 1) throw Error("llm: the draft head is staged for " + std::to_string(d.MaxRows()) + " rows; a round owes up to " + std::to_string(depth + 1));
    if (slot >= g.Slots() || slot >= d.Slots())
        throw Error("llm: speculator slot " + std::to_string(slot) + "; the trunk holds " + std::to_string(g.Slots()) + " and the draft " + std::to_string(d.Slots()));
    // the owed rows (fewer than one draft call's worth: Owe settles at that) and the seed after them
    cap_rows_ = std::max(depth + 1, d.MaxRows()) + 2;
    if (const char *e = std::getenv("LLM_SPEC_CHAIN")) chained_ = e[0] != '0';
    h_ = static_cast<float *>(g.Dev().alloc(static_cast<size_t>(cap_rows_) * g.GetModel().config().NEmbd * 4));
    if (slot < 0) {
        g.Speculate(true);
        g.SpeculateFirst(true);
    }
}

void Speculator::use_slot() {
    if (slot_ >= 0) d_.UseSlot(slot_);
}

void Speculator::Prime(const std::vector<int32_t> &ids, int at, const float *res) {
    const int n = static_cast<int>(ids.size());
    const size_t E = g_.GetModel().config().NEmbd;
    if (n < 1 || !res) throw Error("llm: Speculator.Prime: no rows");
    use_slot();
    if (at == 0) owe_x_.clear();  // the slot's sequence starts over, and what its draft owed went with it
    if (at > 0 && !seeded_) throw Error("llm: priming from position " + std::to_string(at) + " without the residual before it");
    if (!owe_x_.empty()) throw Error("llm: priming the draft while it owes " + std::to_string(owe_x_.size()) + " rows; settle first");
    if (at > 0 && at != d_.Past()) throw Error("llm: priming the draft at " + std::to_string(at) + "; its cache holds " + std::to_string(d_.Past()));
    if (at == 0) {
        d_.Reset();
        g_.Dev().zero(h_, E * 4);
    }
    d_.Rows(h_, {ids[0]}, at, false);
    const int M = d_.MaxRows();
    for (int a = 1; a < n; a += M) {
        const int k = std::min(M, n - a);
        d_.Rows(res + static_cast<size_t>(a - 1) * E, std::vector<int32_t>(ids.begin() + a, ids.begin() + a + k), at + a, false);
    }
    check(shv_copy(g_.Dev().ctx(), h_, res + static_cast<size_t>(n - 1) * E, E * 4), "seed");
    seeded_ = true;
    pend_ = -1;
}

void Speculator::Owe(int32_t x, const float *h) {
    if (!seeded_) throw Error("llm: Speculator.Owe without the residual before the row");
    const size_t E = g_.GetModel().config().NEmbd;
    // the seed becomes the residual before x's position, h the new seed
    owe_x_.push_back(x);
    check(shv_copy(g_.Dev().ctx(), h_ + owe_x_.size() * E, h, E * 4), "owed row");
    // a round's first draft call carries the owed rows and the pending token: a long run of
    // plain steps is written as it fills a call (llm/spec.go:366-371)
    if (static_cast<int>(owe_x_.size()) >= d_.MaxRows()) settle_owed();
}

void Speculator::settle_owed() {
    const int n = static_cast<int>(owe_x_.size());
    if (n == 0) return;
    const size_t E = g_.GetModel().config().NEmbd;
    use_slot();
    const int at = past() - n, M = d_.MaxRows();
    for (int p0 = 0; p0 < n; p0 += M) {
        const int k = std::min(M, n - p0);
        d_.Rows(h_ + static_cast<size_t>(p0) * E, std::vector<int32_t>(owe_x_.begin() + p0, owe_x_.begin() + p0 + k), at + p0, false);
    }
    check(shv_copy(g_.Dev().ctx(), h_, h_ + static_cast<size_t>(n) * E, E * 4), "seed");
    owe_x_.clear();
}

void Speculator::Settle() {
    pend_ = -1;
    use_slot();
    settle_owed();
    // a deeper draft wrote cells past the trunk: they are masked once the position says so
    if (d_.Past() > past()) d_.Rewind(past());
}

std::vector<float> Speculator::Residual() const {
    const size_t E = g_.GetModel().config().NEmbd;
    std::vector<float> h(E);
    g_.Dev().download(h.data(), h_ + owe_x_.size() * E, E * 4);
    return h;
}

void Speculator::Rewind(int past, const std::vector<float> &h) {
    const size_t E = g_.GetModel().config().NEmbd;
    if (h.size() != E) throw Error("llm: rewinding the draft without the residual before " + std::to_string(past));
    use_slot();
    d_.Rewind(past);
    g_.Dev().upload(h_, h.data(), E * 4);
    seeded_ = true;
    pend_ = -1;
    owe_x_.clear();
}

std::vector<int32_t> Speculator::RoundFrom(int32_t first, const std::vector<int32_t> &forced, int limit) {
    if (!seeded_) throw Error("llm: a round without the trunk's residual");
    use_slot();
    if (static_cast<int>(owe_x_.size()) + 1 > d_.MaxRows()) settle_owed();
    pend_ = first;
    return Round(forced, limit);
}

int32_t Speculator::Start(const std::vector<int32_t> &prompt) {
    const int T = static_cast<int>(prompt.size());
    if (T < 1) throw Error("llm: Speculator.Start: no prompt");
    const size_t E = g_.GetModel().config().NEmbd;
    g_.Speculate(false);  // the prompt is committed as it runs
    std::vector<float> logits;  // the prompt's last row, when a sampler will want it
    const float *res = g_.ForwardResidual(prompt, sampler_ ? &logits : nullptr);
    // Prime (llm/spec.go:286-326): the draft's cell at position p is written from the trunk's
    // residual at p-1 and the token at p; cell 0 has nothing behind it and takes a zero residual.
    d_.Reset();
    g_.Dev().zero(h_, E * 4);
    d_.Rows(h_, {prompt[0]}, 0, false);
    const int M = d_.MaxRows();
    for (int a = 1; a < T; a += M) {
        const int n = std::min(M, T - a);
        d_.Rows(res + static_cast<size_t>(a - 1) * E, std::vector<int32_t>(prompt.begin() + a, prompt.begin() + a + n), a, false);
    }
    // the trunk's residual after the last prompt row seeds the first round
    check(shv_copy(g_.Dev().ctx(), h_, res + static_cast<size_t>(T - 1) * E, E * 4), "seed");
    owe_x_.clear();
    seeded_ = true;
    if (sampler_) {
        // the prompt enters the penalties' window, then its last row is sampled on the host
        sampler_->Accept(prompt.data(), T);
        pend_ = sampler_->Sample(logits.data(), static_cast<int>(logits.size()));
        sampler_->Accept(&pend_, 1);
    } else {
        // the token the prompt's last row sampled sits one past the sequence's end
        pend_ = g_.Generate(1, nullptr)[0];
    }
    g_.Speculate(true);
    g_.SpeculateFirst(true);
    Stats = SpecStats();
    Stats.Tokens = 1;
    return pend_;
}

void Speculator::UseSampler(Sampler *s, int64_t draft_seed) {
    if (!s || s->Greedy()) {
        sampler_ = nullptr;
        draft_sampler_.reset();
        return;
    }
    sampler_ = s;
    draft_sampler_ = s->DraftSampler(draft_seed);
}

void Speculator::SetSampler(Sampler *s, bool exact, int64_t draft_seed) {
    if (!s || s->Greedy()) {
        sampler_ = nullptr, exact_ = false;
        draft_sampler_.reset();
        return;
    }
    // a request keeps its draft sampler from round to round
    if (!exact && (s != sampler_ || exact_ || !draft_sampler_)) draft_sampler_ = s->DraftSampler(draft_seed);
    if (exact) draft_sampler_.reset();
    sampler_ = s, exact_ = exact;
}

// A round under a sampler (llm/spec.go:703-857 with llm/sample.go:183-250).  The passes are the
// greedy round's; what differs is who names the tokens: each draft is a draw from the draft
// sampler's distribution over the draft head's logits, each verified row goes through Verify.
std::vector<int32_t> Speculator::sampled_round(const std::vector<int32_t> &forced, int limit) {
    const size_t E = g_.GetModel().config().NEmbd;
    const int V = g_.GetModel().config().VocabSize;
    const int at = g_.Past();
    const int owed = static_cast<int>(owe_x_.size());
    const uint64_t d0 = d_.GPUNanos;
    std::vector<int32_t> rows{pend_};
    std::vector<int32_t> xs(owe_x_);
    xs.push_back(pend_);
    std::vector<Dist> q(Depth);
    std::vector<bool> drawn(Depth, false);
    std::vector<float> ql;
    int32_t dtok = d_.Rows(h_, xs, at - owed, true);
    for (int k = 0; k < Depth; k++) {
        if (k > 0) {
            std::vector<int32_t> one{rows[k]};
            dtok = d_.Rows(d_.ResPort() + (k == 1 ? static_cast<size_t>(owed) * E : 0), one, at + k, true);
        }
        if (k < static_cast<int>(forced.size())) {
            rows.push_back(forced[k]);  // not a draw from q: verified as a plain sample
        } else if (exact_) {
            rows.push_back(dtok);       // the draft head's arg-max: likewise
        } else {
            d_.LastLogits(&ql);
            rows.push_back(draft_sampler_->Propose(ql.data(), static_cast<int>(ql.size()), &q[k]));
            drawn[k] = true;
        }
    }
    Stats.DraftNanos += d_.GPUNanos - d0;

    const uint64_t v0 = g_.Stats.GPUNanos;
    std::vector<float> logits;
    g_.ExtendRows(rows, &logits, nullptr);
    Stats.VerifyNanos += g_.Stats.GPUNanos - v0;
    const int n = static_cast<int>(rows.size());
    Stats.Passes[std::min(n, 4)]++;
    Stats.Rounds++;
    if (n > 1) Stats.Drafted++;

    std::vector<int32_t> out;
    for (int i = 0; i < n; i++) {
        if (limit > 0 && static_cast<int>(out.size()) >= limit) break;
        float *row = logits.data() + static_cast<size_t>(i) * V;
        int32_t tok;
        if (i + 1 < n) tok = sampler_->Verify(row, V, rows[i + 1], drawn[i] ? &q[i] : nullptr);
        else tok = sampler_->Sample(row, V);
        sampler_->Accept(&tok, 1);
        out.push_back(tok);
        if (i + 1 == n) break;
        Stats.DraftedAt[std::min(i, 3)]++;
        if (rows[i + 1] != tok) break;
        Stats.AcceptedAt[std::min(i, 3)]++;
    }
    const int keep = static_cast<int>(out.size());
    if (keep > 1) Stats.Accepted++;
    g_.Keep(keep);
    check(shv_copy(g_.Dev().ctx(), h_, g_.ResPort(), static_cast<size_t>(keep) * E * 4), "seed");
    owe_x_.assign(rows.begin() + 1, rows.begin() + keep);
    d_.Rewind(std::min(d_.Past(), at + 1));
    pend_ = out[keep - 1];
    Stats.Tokens += keep;
    return out;
}

std::vector<int32_t> Speculator::Round(const std::vector<int32_t> &forced, int limit) {
    if (pend_ < 0) throw Error("llm: Speculator.Round before Start");
    use_slot();
    if (sampler_) return sampled_round(forced, limit);
    if (chained_ && !no_prerecord()) return chained_round(forced, limit);
    const size_t E = g_.GetModel().config().NEmbd;
    const int at = g_.Past();
    const int owed = static_cast<int>(owe_x_.size());
    // 1. the drafts: the owed rows and the first draft in one call, then each further draft from
    //    the draft's own residual
    const uint64_t d0 = d_.GPUNanos;
    std::vector<int32_t> rows{pend_};
    std::vector<int32_t> xs(owe_x_);
    xs.push_back(pend_);
    int32_t dtok = d_.Rows(h_, xs, at - owed, true);
    for (int k = 0; k < Depth; k++) {
        if (k > 0) {
            std::vector<int32_t> one{rows[k]};
            // the last row of the previous call is the residual this one chains on
            dtok = d_.Rows(d_.ResPort() + (k == 1 ? static_cast<size_t>(owed) * E : 0), one, at + k, true);
        }
        rows.push_back(k < static_cast<int>(forced.size()) ? forced[k] : dtok);
    }
    Stats.DraftNanos += d_.GPUNanos - d0;

    // 2. the verification pass
    const uint64_t v0 = g_.Stats.GPUNanos;
    g_.ExtendRows(rows, nullptr, nullptr);
    Stats.VerifyNanos += g_.Stats.GPUNanos - v0;
    return finish_round(rows, g_.Argmaxes(), at, limit);
}

// 3. row i's arg-max is the trunk's token at at+i+1; the pass is the sequence up to the first
//    draft it disagrees with
std::vector<int32_t> Speculator::finish_round(const std::vector<int32_t> &rows, const std::vector<int32_t> &best, int at, int limit) {
    const size_t E = g_.GetModel().config().NEmbd;
    const int n = static_cast<int>(rows.size());
    Stats.Passes[std::min(n, 4)]++;
    Stats.Rounds++;
    if (n > 1) Stats.Drafted++;
    std::vector<int32_t> out;
    for (int i = 0; i < n; i++) {
        if (limit > 0 && static_cast<int>(out.size()) >= limit) break;
        out.push_back(best[i]);
        if (i + 1 == n) break;
        Stats.DraftedAt[std::min(i, 3)]++;
        if (rows[i + 1] != best[i]) break;
        Stats.AcceptedAt[std::min(i, 3)]++;
    }
    const int keep = static_cast<int>(out.size());
    if (keep > 1) Stats.Accepted++;
    g_.Keep(keep);
    // the rows the draft's cache has not seen from the trunk's side (CatchUp, llm/spec.go:838-843),
    // then the residual the next draft is seeded from
    check(shv_copy(g_.Dev().ctx(), h_, g_.ResPort(), static_cast<size_t>(keep) * E * 4), "seed");
    owe_x_.assign(rows.begin() + 1, rows.begin() + keep);
    d_.Rewind(std::min(d_.Past(), at + 1));
    pend_ = out[keep - 1];
    Stats.Tokens += keep;
    return out;
}

// The greedy round without a wait between its passes.  Nothing the host decides depends on a draft before the
// verification pass has run: the draft head reads its tokens from the trunk's id ring, names the next one there
// itself and moves its own position word, the verification pass reads the same ring, and the host learns drafts and
// arg-maxes together after the one wait (what each call's wait cost: 25 us of launch and wake-up, three a round).
std::vector<int32_t> Speculator::chained_round(const std::vector<int32_t> &forced, int limit) {
    const size_t E = g_.GetModel().config().NEmbd;
    const int at = g_.Past();
    const int owed = static_cast<int>(owe_x_.size());
    int32_t *ring = g_.IdsPort();
    std::vector<int32_t> xs(owe_x_);
    xs.push_back(pend_);
    g_.StageIds(at - owed, xs);
    check(shv_stamp(g_.Dev().ctx(), 0), "stamp");
    for (int k = 0; k < Depth; k++) {
        if (k == 0) d_.RowsChained(h_, owed + 1, at - owed, 0, ring);
        else d_.RowsChained(d_.ResPort() + (k == 1 ? static_cast<size_t>(owed) * E : 0), 1, -1, k, ring);
        // a forced draft replaces the head's own in the ring before anything reads it
        if (k < static_cast<int>(forced.size())) g_.StageIds(at + k + 1, {forced[k]});
    }
    check(shv_stamp(g_.Dev().ctx(), 1), "stamp");
    const uint64_t v0 = g_.Stats.GPUNanos;
    g_.ExtendRowsStaged(Depth + 1);
    Stats.VerifyNanos += g_.Stats.GPUNanos - v0;
    uint64_t dns = 0;
    check(shv_stamp_elapsed(g_.Dev().ctx(), 0, 1, &dns), "stamp");
    Stats.DraftNanos += dns;
    d_.GPUNanos += dns;
    std::vector<int32_t> rows{pend_};
    for (int k = 0; k < Depth; k++) rows.push_back(k < static_cast<int>(forced.size()) ? forced[k] : d_.DraftAt(k));
    return finish_round(rows, g_.Argmaxes(), at, limit);
}

}  // namespace llm
