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
    shv_destroy(ctx_);
}

void *Device::alloc(size_t bytes) {
    void *p = nullptr;
    check(shv_alloc(ctx_, bytes < 256 ? 256 : bytes, &p), "alloc");
    owned_.push_back(p);
    allocated_ += bytes;
    return p;
}

void *Device::alloc_zero(size_t bytes) {
    void *p = alloc(bytes);
    zero(p, bytes < 256 ? 256 : bytes);
    return p;
}

void Device::upload(void *dst, const void *src, size_t bytes) { check(shv_upload(ctx_, dst, src, bytes), "upload"); }
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
    for (int l = 0; l < c.NLayer; l++) {
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

// ---------------------------------------------------------------------------------- MoE -------

MoEGPU::MoEGPU(Device &dev, const Model &m, int maxTokens) : dev_(dev), m_(m), c_(m.config()), max_tok_(maxTokens) {
    if (maxTokens < 1) throw Error("llm: MoEGPU needs room for at least one token");
    if (c_.NExpertUsed > c_.NExpert) throw Error("llm: MoEGPU: more experts used than there are");
    const size_t T = maxTokens;
    in_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    out_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    xn_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    logits_ = static_cast<float *>(dev.alloc(T * (c_.NExpert + 1) * 4));
    topk_ = static_cast<int32_t *>(dev.alloc(T * c_.NExpertUsed * 4));
    weights_ = static_cast<float *>(dev.alloc(T * (c_.NExpertUsed + 1) * 4));
    act_ = static_cast<float *>(dev.alloc(T * (c_.NExpertUsed + 1) * c_.FFNExpert * 4));
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
    shv_moe_up_args u{};
    u.xn = xn_;
    u.topk = topk_;
    u.gate_exps = m_.Tensor(Model::Blk(l, "ffn_gate_exps")).ptr;
    u.up_exps = m_.Tensor(Model::Blk(l, "ffn_up_exps")).ptr;
    u.gate_sh = m_.Tensor(Model::Blk(l, "ffn_gate_shexp")).ptr;
    u.up_sh = m_.Tensor(Model::Blk(l, "ffn_up_shexp")).ptr;
    u.act = act_;
    u.n_tok = nTok;
    u.n_embd = c_.NEmbd;
    u.n_used = c_.NExpertUsed;
    u.ffn = c_.FFNExpert;
    shv_moe_down_args d{};
    d.act = act_;
    d.topk = topk_;
    d.weights = weights_;
    d.down_exps = m_.Tensor(Model::Blk(l, "ffn_down_exps")).ptr;
    d.down_sh = m_.Tensor(Model::Blk(l, "ffn_down_shexp")).ptr;
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

DeltaNetGPU::DeltaNetGPU(Device &dev, const Model &m, int maxTokens, int slots, int32_t *pos)
    : dev_(dev), m_(m), c_(m.config()), max_tok_(maxTokens), slots_(slots), pos_(pos) {
    // refusals at construction, never at run (llm/gpu_deltanet.go:423-447)
    if (c_.SSMHeadDim != 128) throw Error("llm: DeltaNetGPU: head dimension " + std::to_string(c_.SSMHeadDim) + ", the step kernel is built for 128");
    if (c_.SSMConv != 4) throw Error("llm: DeltaNetGPU: conv kernel " + std::to_string(c_.SSMConv) + ", built for 4");
    if (maxTokens < 1 || maxTokens + c_.SSMConv - 1 > kRing) throw Error("llm: DeltaNetGPU: a pass of " + std::to_string(maxTokens) + " rows does not fit the projection ring");
    if (slots < 1) throw Error("llm: DeltaNetGPU: no slots");
    const size_t T = maxTokens;
    in_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    out_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    attn_ = static_cast<float *>(dev.alloc(T * c_.VWidth() * 4));
    ring_.assign(c_.NLayer, nullptr);
    state_.assign(c_.NLayer, nullptr);
    const size_t ring_bytes = static_cast<size_t>(slots) * kRing * c_.DNFusedRows() * 4;
    const size_t st_bytes = static_cast<size_t>(slots) * c_.SSMHeadV * c_.SSMHeadDim * c_.SSMHeadDim * 4;
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
    dev_.zero(ring_[l], static_cast<size_t>(slots_) * kRing * c_.DNFusedRows() * 4);
    dev_.zero(state_[l], static_cast<size_t>(slots_) * c_.SSMHeadV * c_.SSMHeadDim * c_.SSMHeadDim * 4);
}

void DeltaNetGPU::ResetAll() {
    for (int l = 0; l < c_.NLayer; l++)
        if (state_[l]) Reset(l);
}

std::vector<shv_op> DeltaNetGPU::Dispatches(int l, const float *in, float *out, int nTok, std::vector<std::string> *labels) const {
    if (!state_[l]) throw Error("llm: DeltaNetGPU: layer " + std::to_string(l) + " is not a DeltaNet layer");
    const int width = c_.DNFusedRows();
    shv_gemv_q4k_args p{};
    p.w = m_.Tensor(Model::Blk(l, "ssm_in_fused")).ptr;
    p.x = in;
    p.y = ring_[l];
    p.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "attn_norm")).ptr);
    p.pos = pos_;
    p.n = width;
    p.k = c_.NEmbd;
    p.n_tok = nTok;
    p.prologue = SHV_PRO_RMSNORM;
    p.eps = c_.RMSEps;
    p.x_stride = c_.NEmbd;
    p.y_stride = width;
    p.seq_len = nTok;
    p.ring_slots = kRing;
    p.ring_stride = width;
    shv_dn_step_args s{};
    s.ring = ring_[l];
    s.conv1d = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_conv1d")).ptr);
    s.a = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_a")).ptr);
    s.dt_bias = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_dt")).ptr);
    s.state = state_[l];
    s.out = attn_;
    s.pos = pos_;
    s.n_seq = 1;
    s.seq_len = nTok;
    s.n_head_k = c_.SSMHeadK;
    s.n_head_v = c_.SSMHeadV;
    s.head_dim = c_.SSMHeadDim;
    s.conv = c_.SSMConv;
    s.ring_slots = kRing;
    s.ring_stride = width;
    s.eps = c_.RMSEps;
    shv_gemv_q4k_args o{};
    o.w = m_.Tensor(Model::Blk(l, "ssm_out")).ptr;
    o.x = attn_;
    o.y = out;
    o.residual = in;
    o.gamma = static_cast<const float *>(m_.Tensor(Model::Blk(l, "ssm_norm")).ptr);
    o.z = ring_[l] + c_.ConvWidth();  // the z columns of a projection row
    o.pos = pos_;
    o.n = c_.NEmbd;
    o.k = c_.VWidth();
    o.n_tok = nTok;
    o.prologue = SHV_PRO_GATED_NORM;
    o.head_dim = c_.SSMHeadDim;
    o.eps = c_.RMSEps;
    o.x_stride = c_.VWidth();
    o.y_stride = c_.NEmbd;
    o.seq_len = nTok;
    o.ring_slots = kRing;
    o.ring_stride = width;
    o.z_ring = 1;
    if (labels) labels->insert(labels->end(), {"dn.qkv", "dn.step", "dn.out"});
    return {make_op(SHV_OP_GEMV_Q4K, p), make_op(SHV_OP_DN_STEP, s), make_op(SHV_OP_GEMV_Q4K, o)};
}

void DeltaNetGPU::Run(int layer) {
    if (n_tok_ < 1) throw Error("llm: DeltaNetGPU.Run before Upload");
    dev_.run(Dispatches(layer, in_, out_, n_tok_, nullptr));
}

std::vector<float> DeltaNetGPU::State(int l, int slot) const {
    if (!state_[l] || slot < 0 || slot >= slots_) throw Error("llm: DeltaNetGPU.State: no such layer or slot");
    const size_t n = static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim;
    return read_back<float>(dev_, state_[l] + slot * n, n);
}

void DeltaNetGPU::SetState(int l, const std::vector<float> &s, int slot) {
    const size_t n = static_cast<size_t>(c_.SSMHeadV) * c_.SSMHeadDim * c_.SSMHeadDim;
    if (!state_[l] || slot < 0 || slot >= slots_ || s.size() != n) throw Error("llm: DeltaNetGPU.SetState: no such layer or slot, or wrong length");
    dev_.upload(state_[l] + slot * n, s.data(), n * 4);
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

AttnGPU::AttnGPU(Device &dev, const Model &m, int maxTokens, int nKV, int slots, int32_t *pos)
    : dev_(dev), m_(m), c_(m.config()), max_tok_(maxTokens), n_kv_(nKV), slots_(slots), pos_(pos) {
    if (c_.HeadDim != 256) throw Error("llm: AttnGPU: head dimension " + std::to_string(c_.HeadDim) + ", the decode kernel is built for 256");
    if (c_.NHead != 8 * c_.NHeadKV) throw Error("llm: AttnGPU: the decode kernel is built for 8 query heads per KV head");
    if (maxTokens < 1 || nKV < maxTokens || slots < 1) throw Error("llm: AttnGPU: bad token, cell or slot count");
    SetSplits(0);
    const size_t T = maxTokens;
    in_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    out_ = static_cast<float *>(dev.alloc(T * c_.NEmbd * 4));
    qkv_ = static_cast<float *>(dev.alloc(T * c_.AttnFusedRows() * 4));
    ctx_ = static_cast<float *>(dev.alloc(T * c_.NHead * c_.HeadDim * 4));
    partial_ = static_cast<float *>(dev.alloc(static_cast<size_t>(c_.NHeadKV) * kMaxSplits * 8 * (c_.HeadDim + 2) * 4));
    const std::vector<float> rt = rope_table(nKV, c_.RopeDims, c_.RopeBase);
    rope_ = static_cast<float *>(dev.alloc(rt.size() * 4));
    dev.upload(rope_, rt.data(), rt.size() * 4);
    kc_.assign(c_.NLayer, nullptr);
    vc_.assign(c_.NLayer, nullptr);
    const size_t cb = static_cast<size_t>(slots) * nKV * c_.NHeadKV * c_.HeadDim * 2;
    for (int l = 0; l < c_.NLayer; l++) {
        if (!c_.IsAttn(l)) continue;
        kc_[l] = dev.alloc(cb);
        vc_[l] = dev.alloc(cb);
        cache_bytes_ += 2 * cb;
    }
}

void AttnGPU::SetSplits(int n) {
    // slices for the cache's capacity: about 128 cells each up to 256 slices (the kernel engages
    // only as many as the sequence's current length fills)
    if (n <= 0) n = std::min(256, std::max(8, (n_kv_ + 127) / 128));
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
    if (!kc_[l]) throw Error("llm: AttnGPU: layer " + std::to_string(l) + " is not an attention layer");
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
    a.kcache = kc_[l];
    a.vcache = vc_[l];
    a.partial = partial_;
    a.out = ctx_;
    a.pos = pos_;
    a.n_seq = 1;
    a.seq_len = nTok;
    a.n_head = c_.NHead;
    a.n_head_kv = c_.NHeadKV;
    a.head_dim = c_.HeadDim;
    a.rope_dims = c_.RopeDims;
    a.max_cells = n_kv_;
    a.qkv_stride = width;
    a.n_splits = splits_;
    a.eps = c_.RMSEps;
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
    if (!kc_[l] || cells > n_kv_ || slot >= slots_) throw Error("llm: AttnGPU.K: no such layer, cell or slot");
    const size_t per = static_cast<size_t>(c_.NHeadKV) * c_.HeadDim;
    return read_back<uint16_t>(dev_, static_cast<uint16_t *>(kc_[l]) + slot * n_kv_ * per, cells * per);
}

std::vector<uint16_t> AttnGPU::V(int l, int cells, int slot) const {
    if (!vc_[l] || cells > n_kv_ || slot >= slots_) throw Error("llm: AttnGPU.V: no such layer, cell or slot");
    const size_t per = static_cast<size_t>(c_.NHeadKV) * c_.HeadDim;
    return read_back<uint16_t>(dev_, static_cast<uint16_t *>(vc_[l]) + slot * n_kv_ * per, cells * per);
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
    shv_gemv_q4k_args p{};
    p.w = m_.Tensor("output.weight").ptr;
    p.x = in;
    p.y = logits_;
    p.gamma = static_cast<const float *>(m_.Tensor("output_norm.weight").ptr);
    p.n = c_.VocabSize;
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

static void submit(Device &dev, shv_prerecorded *rec, const std::vector<shv_op> &ops, int iters, uint64_t *ns, const char *what) {
    if (no_prerecord())
        check(shv_dispatch_multi(dev.ctx(), ops.data(), static_cast<int>(ops.size()), iters, ns, nullptr), what);
    else
        check(shv_prerecorded_submit(dev.ctx(), rec, iters, ns), what);
}

Graph::Graph(Device &dev, const Model &m, const GraphOpts &opts) : dev_(dev), m_(m), c_(m.config()), o_(opts) {
    layers_ = opts.Layers > 0 ? opts.Layers : c_.NLayer;
    if (layers_ > c_.NLayer) throw Error("llm: NewGraph: " + std::to_string(layers_) + " layers of a " + std::to_string(c_.NLayer) + "-layer model");
    if (o_.MaxTokens != 1) throw Error("llm: NewGraph: this build records one-row passes only (MaxTokens 1)");
    if (o_.Slots != 1) throw Error("llm: NewGraph: this build stages one sequence (Slots 1)");
    if (o_.NKV < 2) throw Error("llm: NewGraph: NKV " + std::to_string(o_.NKV));
    x_ = static_cast<float *>(dev.alloc(static_cast<size_t>(o_.MaxTokens) * c_.NEmbd * 4));
    ids_ = static_cast<int32_t *>(dev.alloc_zero((static_cast<size_t>(o_.NKV) + 2) * 4));
    pos_ = static_cast<int32_t *>(dev.alloc_zero(static_cast<size_t>(o_.Slots) * 4));
    best_ = static_cast<int32_t *>(dev.alloc_zero(64));
    moe_ = new MoEGPU(dev, m, o_.MaxTokens);
    dn_ = new DeltaNetGPU(dev, m, o_.MaxTokens, o_.Slots, pos_);
    attn_ = new AttnGPU(dev, m, o_.MaxTokens, o_.NKV, o_.Slots, pos_);
    if (o_.AttnSplits > 0) attn_->SetSplits(o_.AttnSplits);
    if (!o_.NoHead) head_ = new HeadGPU(dev, m, 1);
    record();
}

Graph::~Graph() {
    if (step_) shv_prerecorded_destroy(dev_.ctx(), step_);
    if (prefill_) shv_prerecorded_destroy(dev_.ctx(), prefill_);
    delete moe_;
    delete dn_;
    delete attn_;
    delete head_;
}

// The loop body of llm/graph.go:2330-2466 for a model without hyper-connection streams: the
// residual stream stays in one buffer, every block reads it through its RMSNorm prologue and
// adds its output back in place.
void Graph::record() {
    std::vector<shv_op> ops;
    std::vector<std::string> labels;
    shv_embed_args e{};
    e.table = m_.Tensor("token_embd.weight").ptr;
    e.ids = ids_;
    e.pos = pos_;
    e.x = x_;
    e.n_tok = 1;
    e.n_embd = c_.NEmbd;
    e.vocab = c_.VocabSize;
    e.x_stride = c_.NEmbd;
    ops.push_back(make_op(SHV_OP_EMBED, e));
    labels.push_back("embed");
    for (int l = 0; l < layers_; l++) {
        auto sub = c_.IsAttn(l) ? attn_->Dispatches(l, x_, x_, 1, &labels) : dn_->Dispatches(l, x_, x_, 1, &labels);
        ops.insert(ops.end(), sub.begin(), sub.end());
        auto ffn = moe_->Dispatches(l, x_, x_, 1, &labels);
        ops.insert(ops.end(), ffn.begin(), ffn.end());
    }
    prefill_ops_ = ops;
    shv_advance_args adv{pos_, 1, 1};
    prefill_ops_.push_back(make_op(SHV_OP_ADVANCE, adv));
    check(shv_prerecord(dev_.ctx(), prefill_ops_.data(), static_cast<int>(prefill_ops_.size()), &prefill_), "record prefill step");
    if (head_) {
        auto h = head_->Dispatches(x_, 1, &labels);
        ops.insert(ops.end(), h.begin(), h.end());
        shv_argmax_args am{};
        am.logits = head_->LogitsPort();
        am.best = best_;
        am.ids = ids_;
        am.pos = pos_;
        am.n_rows = 1;
        am.n = c_.VocabSize;
        am.logits_stride = c_.VocabSize;
        ops.push_back(make_op(SHV_OP_ARGMAX, am));
        labels.push_back("argmax");
        step_ops_ = ops;
        step_labels_ = labels;
        check(shv_prerecord(dev_.ctx(), step_ops_.data(), static_cast<int>(step_ops_.size()), &step_), "record decode step");
    }
}

void Graph::Reset() {
    dn_->ResetAll();
    const int32_t zero = 0;
    dev_.upload(pos_, &zero, 4);
    past_ = 0;
}

void Graph::Forward(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden) {
    Reset();
    Extend(ids, logits, hidden);
}

void Graph::Extend(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden) {
    const int n = static_cast<int>(ids.size());
    if (n < 1) throw Error("llm: Graph.Extend: no tokens");
    if (past_ + n + 1 > o_.NKV) throw Error("llm: Graph.Extend: " + std::to_string(past_ + n) + " tokens do not fit " + std::to_string(o_.NKV) + " cells");
    for (int32_t id : ids)
        if (id < 0 || id >= c_.VocabSize) throw Error("llm: Graph.Extend: token " + std::to_string(id) + " is outside the vocabulary");
    dev_.upload(ids_ + past_, ids.data(), static_cast<size_t>(n) * 4);
    const int32_t p = past_;
    dev_.upload(pos_, &p, 4);
    // every row but the last goes through the headless step; the last one samples
    uint64_t ns = 0;
    if (n > 1) submit(dev_, prefill_, prefill_ops_, n - 1, &ns, "prefill");
    Stats.GPUNanos += ns;
    if (head_) {
        submit(dev_, step_, step_ops_, 1, &ns, "decode step");
        Stats.Dispatches = static_cast<int>(step_ops_.size());
    } else {
        submit(dev_, prefill_, prefill_ops_, 1, &ns, "last row");
        Stats.Dispatches = static_cast<int>(prefill_ops_.size());
    }
    Stats.GPUNanos += ns;
    Stats.Runs++;
    past_ += n;
    if (logits) {
        if (!head_) throw Error("llm: Graph.Extend: the graph was staged without a head");
        logits->resize(c_.VocabSize);
        dev_.download(logits->data(), head_->LogitsPort(), static_cast<size_t>(c_.VocabSize) * 4);
    }
    if (hidden) {
        hidden->resize(c_.NEmbd);
        dev_.download(hidden->data(), x_, static_cast<size_t>(c_.NEmbd) * 4);
    }
}

std::vector<int32_t> Graph::Generate(int n, uint64_t *gpu_nanos) {
    if (!head_) throw Error("llm: Graph.Generate: the graph was staged without a head");
    if (past_ < 1) throw Error("llm: Graph.Generate before a prompt");
    if (n < 1 || past_ + n + 1 > o_.NKV) throw Error("llm: Graph.Generate: " + std::to_string(n) + " more tokens do not fit the cache");
    // the last Extend already sampled the token at position past_: it sits in ids[past_], and
    // every replay consumes ids[pos] and appends ids[pos+1]
    uint64_t ns = 0;
    if (n > 1) submit(dev_, step_, step_ops_, n - 1, &ns, "generate");
    if (gpu_nanos) *gpu_nanos = ns;
    std::vector<int32_t> out(n);
    dev_.download(out.data(), ids_ + past_, static_cast<size_t>(n) * 4);
    past_ += n - 1;
    Stats.GPUNanos += ns;
    return out;
}

std::vector<int32_t> Graph::Ids() const { return read_back<int32_t>(dev_, ids_, past_); }

// One real decode step (the sequence advances by one token, as after Generate(1)), dispatched op
// by op so that every op has its own GPU time.
std::vector<Stage> Graph::ProfileStep() {
    if (!head_) throw Error("llm: Graph.ProfileStep: the graph was staged without a head");
    if (past_ < 1 || past_ + 2 > o_.NKV) throw Error("llm: Graph.ProfileStep: needs a prompt and a free cell");
    std::vector<uint64_t> per(step_ops_.size());
    uint64_t total = 0;
    check(shv_dispatch_multi(dev_.ctx(), step_ops_.data(), static_cast<int>(step_ops_.size()), 1, &total, per.data()), "profile step");
    past_ += 1;
    std::map<std::string, uint64_t> kinds;
    std::vector<std::string> order;
    for (size_t i = 0; i < per.size(); i++) {
        if (!kinds.count(step_labels_[i])) order.push_back(step_labels_[i]);
        kinds[step_labels_[i]] += per[i];
    }
    Stats.Kinds = kinds;
    std::vector<Stage> out;
    for (const auto &k : order) out.push_back({k, kinds[k]});
    out.push_back({"total", total});
    return out;
}

}  // namespace llm
