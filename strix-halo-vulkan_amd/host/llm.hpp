// Host side of the token loop: the reference's Go op surface (llm/gpu_moe.go, gpu_deltanet.go,
// gpu_attn.go, gpu_head.go, graph.go) restated in C++ above the C ABI of include/shv_hip.h.
//
// The reference's host code is Go calling its device shim through cgo; no Go toolchain exists in
// the build image, so this layer stands where that Go code would and calls exactly the entry
// points a cgo binding would call.  Names, argument meaning and error behaviour follow the Go
// types: constructors refuse impossible shapes, Upload/Run/read-backs per block, Forward/Extend/
// Reset per graph.  Errors are C++ exceptions of type llm::Error carrying the reference's
// "llm: ..." message style.
#pragma once

#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "shv_hip.h"

namespace llm {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// vk.Device (vk/engine.go:266-311): owns the context; every block borrows it.
class Device {
public:
    explicit Device(int index = 0);
    ~Device();
    Device(const Device &) = delete;
    Device &operator=(const Device &) = delete;
    shv_ctx *ctx() const { return ctx_; }
    void *alloc(size_t bytes);  // tracked; released with the device
    void *alloc_zero(size_t bytes);
    void upload(void *dst, const void *src, size_t bytes);
    void download(void *dst, const void *src, size_t bytes);
    void zero(void *dst, size_t bytes);
    void sync();
    void run(const std::vector<shv_op> &ops);  // dispatch and block
    size_t allocated() const { return allocated_; }

private:
    shv_ctx *ctx_ = nullptr;
    std::vector<void *> owned_;
    size_t allocated_ = 0;
};

void check(int rc, const char *what);

template <typename T>
shv_op make_op(uint32_t kind, const T &args) {
    static_assert(sizeof(T) <= sizeof(shv_op::args), "argument block exceeds the op record");
    shv_op op{};
    op.kind = kind;
    __builtin_memcpy(op.args, &args, sizeof(T));
    return op;
}

// llm.Config (llm/model.go:14-29) plus the DeltaNet and attention shapes the reference reads
// from the checkpoint's metadata (llm/deltanet.go:75-95, llm/attn.go:45-68).
struct Config {
    int NLayer = 48;
    int NEmbd = 2048;
    int NHead = 16;
    int NHeadKV = 2;
    int HeadDim = 256;
    int RopeDims = 64;
    float RopeBase = 1e7f;
    int NExpert = 512;
    int NExpertUsed = 10;
    int FFNExpert = 512;
    int VocabSize = 151936;
    float RMSEps = 1e-6f;
    int SSMHeadDim = 128;  // ssm.state_size
    int SSMHeadK = 16;     // ssm.group_count
    int SSMHeadV = 32;     // ssm.time_step_rank
    int SSMConv = 4;       // ssm.conv_kernel
    int AttnEvery = 4;     // every 4th layer is full attention, the rest gated DeltaNet

    bool IsAttn(int layer) const { return (layer + 1) % AttnEvery == 0; }
    int QKWidth() const { return SSMHeadK * SSMHeadDim; }
    int VWidth() const { return SSMHeadV * SSMHeadDim; }
    int ConvWidth() const { return 2 * QKWidth() + VWidth(); }
    int DNFusedRows() const { return ConvWidth() + VWidth() + 2 * SSMHeadV; }  // qkv | z | alpha | beta
    int AttnFusedRows() const { return NHead * 2 * HeadDim + 2 * NHeadKV * HeadDim; }  // q|gate, k, v
};

// One tensor of the model in device memory.
struct TensorView {
    void *ptr = nullptr;
    uint64_t bytes = 0;
    enum Kind { F32, F16, Q4K } kind = F32;
    int64_t rows = 0, cols = 0;  // Q4K / F16 / F32 matrices: rows x cols; vectors: rows = 1
    float init_mean = 0.f, init_std = 0.02f;
};

// llm.Model (llm/model.go:52-131) for a model that lives in HBM: every tensor by its GGUF name.
class Model {
public:
    Model(Device &dev, const Config &cfg);
    const Config &config() const { return cfg_; }
    const TensorView &Tensor(const std::string &name) const;
    bool Has(const std::string &name) const { return tensors_.count(name) != 0; }
    const std::map<std::string, TensorView> &Tensors() const { return tensors_; }
    // Random-init weights of this architecture, drawn and quantised on the device: Q4_K tensors
    // ~N(0, 0.02) through the reference's quantiser, norm gammas ~ 1 + N(0, 0.1).
    void InitSynthetic(uint64_t seed);
    uint64_t WeightBytes() const;
    static std::string Blk(int layer, const char *name);

private:
    void add(const std::string &name, TensorView::Kind kind, int64_t rows, int64_t cols, float mean, float std);
    void alias(const std::string &name, const std::string &of, int64_t row0, int64_t rows);
    Device &dev_;
    Config cfg_;
    std::map<std::string, TensorView> tensors_;
};

// llm.Stage (llm/gpu.go:1578-1581)
struct Stage {
    std::string Kind;
    uint64_t GPUNanos = 0;
};

// ---- blocks ------------------------------------------------------------------------------------
// Each block mirrors its Go namesake: it owns its activation buffers, takes [nTok][NEmbd] float32
// through Upload, runs one layer with Run, and hands tensors back in the CPU reference's layouts.
// Dispatches() is what a graph records; `in` and `out` are residual-stream rows (out = in + block).

// llm.MoEGPU (llm/gpu_moe.go:708-774, NewMoEGPU :868)
class MoEGPU {
public:
    MoEGPU(Device &dev, const Model &m, int maxTokens);
    void Upload(const std::vector<float> &x, int nTok);  // x is the block input BEFORE its RMSNorm
    void Resize(int nTok);
    void Run(int layer);
    std::vector<Stage> Profile(int layer, int iters);
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, int nTok, std::vector<std::string> *labels) const;
    std::vector<float> Logits() const;    // [T][NExpert+1]
    std::vector<int32_t> TopK() const;    // [T][used]
    std::vector<float> Weights() const;   // [T][used+1]
    std::vector<float> Swiglu() const;    // [T][used+1][ffn]
    std::vector<float> Out() const;       // [T][NEmbd]
    float *InPort() const { return in_; }
    float *OutPort() const { return out_; }
    uint64_t ActivationBytes() const { return act_bytes_; }

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    int max_tok_, n_tok_ = 0;
    float *in_, *out_, *xn_, *logits_, *weights_, *act_;
    int32_t *topk_;
    uint64_t act_bytes_ = 0;
};

// llm.DeltaNetGPU (llm/gpu_deltanet.go:207-322, NewDeltaNetGPUBank :421)
class DeltaNetGPU {
public:
    static constexpr int kRing = 8;  // projection rows kept per slot: up to 5 rows a pass + 3 of history
    DeltaNetGPU(Device &dev, const Model &m, int maxTokens, int slots, int32_t *pos);
    void Upload(const std::vector<float> &x, int nTok);
    void Resize(int nTok);
    void Run(int layer);
    void Reset(int layer);
    void ResetAll();
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, int nTok, std::vector<std::string> *labels) const;
    std::vector<float> State(int layer, int slot = 0) const;  // S, [hv][d][d]
    void SetState(int layer, const std::vector<float> &s, int slot = 0);
    std::vector<float> Result() const;  // [T][hv*d] attention output before the gated norm
    std::vector<float> Out() const;     // [T][NEmbd]
    float *InPort() const { return in_; }
    float *OutPort() const { return out_; }
    uint64_t StateBytes() const { return state_bytes_; }

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    int max_tok_, slots_, n_tok_ = 0;
    int32_t *pos_;
    float *in_, *out_, *attn_;
    std::vector<float *> ring_, state_;  // per layer (nullptr on attention layers)
    uint64_t state_bytes_ = 0;
};

// llm.AttnGPU (llm/gpu_attn.go:403-539, NewAttnGPUBank :779)
class AttnGPU {
public:
    AttnGPU(Device &dev, const Model &m, int maxTokens, int nKV, int slots, int32_t *pos);
    void Upload(const std::vector<float> &x, int nTok);
    void Resize(int nTok);
    void Run(int layer);
    static constexpr int kMaxSplits = 512;  // what the decode kernel's merge has room for
    void SetSplits(int n);
    int Splits() const { return splits_; }
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, int nTok, std::vector<std::string> *labels) const;
    std::vector<float> Context() const;  // [T][NHead*HeadDim] before the gate
    std::vector<float> Out() const;
    std::vector<uint16_t> K(int layer, int cells, int slot = 0) const;  // fp16 bits, [cells][nkv][d]
    std::vector<uint16_t> V(int layer, int cells, int slot = 0) const;
    float *InPort() const { return in_; }
    float *OutPort() const { return out_; }
    uint64_t CacheBytes() const { return cache_bytes_; }

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    int max_tok_, n_kv_, slots_, splits_, n_tok_ = 0;
    int32_t *pos_;
    float *in_, *out_, *qkv_, *ctx_, *partial_, *rope_;
    std::vector<void *> kc_, vc_;
    uint64_t cache_bytes_ = 0;
};

// llm.HeadGPU (llm/gpu_head.go:54-100, NewHeadGPUBank :114)
class HeadGPU {
public:
    HeadGPU(Device &dev, const Model &m, int maxRows);
    void Upload(const std::vector<float> &x, int rows);
    void Resize(int rows);
    void Run();
    std::vector<shv_op> Dispatches(const float *in, int rows, std::vector<std::string> *labels) const;
    std::vector<float> Logits() const;  // [rows][vocab]
    int Vocab() const { return c_.VocabSize; }
    int MaxRows() const { return max_rows_; }
    float *LogitsPort() const { return logits_; }
    float *InPort() const { return in_; }

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    int max_rows_, rows_ = 0;
    float *in_, *logits_;
};

// llm.GraphOpts (llm/graph.go:58-126), the fields that apply here.
struct GraphOpts {
    int MaxTokens = 1;  // rows a pass may carry
    int NKV = 4096;     // attention cache cells per slot
    int Layers = 0;     // 0: all of the model's layers
    bool NoHead = false;
    int Slots = 1;
    int AttnSplits = 0;  // 0: chosen from NKV
};

// llm.GraphStats (llm/graph.go:536-566)
struct GraphStats {
    uint64_t GPUNanos = 0;
    int Dispatches = 0;
    int Runs = 0;
    std::map<std::string, uint64_t> Kinds;  // GPU time by dispatch label
};

// llm.Graph (llm/graph.go:184-289, NewGraph :609): the whole model as one recorded op sequence.
class Graph {
public:
    Graph(Device &dev, const Model &m, const GraphOpts &opts);
    ~Graph();
    // Forward resets the sequence and extends it (llm/graph.go:1695).
    void Forward(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden);
    // Extend appends ids to the sequence and returns the LAST row's logits (llm/graph.go:1709).
    void Extend(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden);
    // Greedy continuation (cmd/llm/generate.go:121-165): n replays of the recorded decode step with
    // the arg-max feeding the next step on the device; returns the n tokens and GPU time.
    std::vector<int32_t> Generate(int n, uint64_t *gpu_nanos);
    void Reset();
    int Past() const { return past_; }
    std::vector<int32_t> Ids() const;
    // One decode step dispatched op by op with a GPU time per op, folded by label
    // (DispatchMultiMarked + recorder.submit, vk/engine.go:913, llm/record.go:217-232).
    std::vector<Stage> ProfileStep();
    GraphStats Stats;
    void ResetStats() { Stats = GraphStats(); }
    int Dispatches() const { return static_cast<int>(step_ops_.size()); }
    MoEGPU &MoE() { return *moe_; }
    DeltaNetGPU &DeltaNet() { return *dn_; }
    AttnGPU &Attn() { return *attn_; }
    HeadGPU &Head() { return *head_; }

private:
    void record();
    Device &dev_;
    const Model &m_;
    Config c_;
    GraphOpts o_;
    int layers_, past_ = 0;
    float *x_ = nullptr;     // residual stream, [MaxTokens][NEmbd]
    int32_t *ids_ = nullptr; // the sequence's tokens by position
    int32_t *pos_ = nullptr; // [Slots] position of each slot's next row
    int32_t *best_ = nullptr;
    MoEGPU *moe_ = nullptr;
    DeltaNetGPU *dn_ = nullptr;
    AttnGPU *attn_ = nullptr;
    HeadGPU *head_ = nullptr;
    std::vector<shv_op> step_ops_, prefill_ops_;  // one token with the head + arg-max / without
    std::vector<std::string> step_labels_;
    shv_prerecorded *step_ = nullptr, *prefill_ = nullptr;
};

}  // namespace llm
