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
#include <functional>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "gguf.hpp"
#include "sample.hpp"
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
    void release(void *p, size_t bytes);  // an alloc() handed back early; bytes as asked for
    void *host_alloc(size_t bytes);       // pinned host memory the device can write; zeroed, released with the device
    void upload(void *dst, const void *src, size_t bytes);
    void download(void *dst, const void *src, size_t bytes);
    void zero(void *dst, size_t bytes);
    void sync();
    void run(const std::vector<shv_op> &ops);  // dispatch and block
    size_t allocated() const { return allocated_; }

private:
    shv_ctx *ctx_ = nullptr;
    std::vector<void *> owned_, host_owned_;
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
    int NextN = 0;         // nextn_predict_layers: 1 adds the draft head as block NLayer (llm/mtp.go:137)
    // The block-sparse indexer beside the trunk's full-attention layers (AttnConfig.IdxHeads /
    // IdxDim / TopK / Ratio, llm/attn.go:56-68; llm/model.go:385-405).  IdxRatio 0: dense layers.
    int IdxHeads = 0, IdxDim = 0, IdxTopK = 0, IdxRatio = 0;
    bool QSA(int layer) const { return IdxRatio > 0 && layer < NLayer && IsAttn(layer); }
    int IdxRows() const { return IdxHeads * IdxDim + IdxDim; }  // the queries' rows, then the key's

    // The draft block is a full-attention layer (llm/mtp.go:17-21).
    bool IsAttn(int layer) const { return layer >= NLayer || (layer + 1) % AttnEvery == 0; }
    int Blocks() const { return NLayer + NextN; }
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
    enum Kind { F32, F16, Q4K, RAW } kind = F32;  // RAW: rows in the ggml type `ggml`, as the checkpoint holds them
    uint32_t ggml = 0;           // the ggml type of the bytes at ptr
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

    // llm.Open's readConfig (llm/model.go:66-99): the model's shape from the checkpoint's own
    // metadata, keys under its general.architecture; the vocabulary is token_embd's row count.
    static Config ConfigFromGGUF(const gguf::Set &s);
    // Every tensor of this model from a mapped checkpoint into its device buffer, straight from
    // the mapping.  A fused projection is filled from its constituents (attn_q / attn_k / attn_v,
    // attn_qkv / attn_gate / ssm_alpha / ssm_beta, nextn.enorm / hnorm) when the file carries
    // those, as llama.cpp's converter writes them.  A tensor in the type the kernels stream
    // (Q4_K matrices, F32 vectors) is copied byte for byte.  An F32 tensor of the model in any
    // other type the dequantiser knows is expanded on the device.  The embedding table stays in
    // the checkpoint's own type (rows are expanded as they are gathered, llm/model.go:125-131).
    // A matrix the kernels stream as Q4_K that the checkpoint holds in another type is expanded
    // and fitted again by the round-to-nearest quantiser on the device — the reference's
    // transcode (llm/moebank.go:288-400, rtn arm), a loss on top of a loss — when `transcode`
    // allows it; Transcoded() names those tensors.  Throws, naming the tensor, on a missing
    // tensor, a shape that disagrees with the metadata, or a type that cannot be staged.
    // Expert banks (ffn_{gate,up,down}_{exps,shexp}) are the exception: the reference stages them in
    // the checkpoint's own type (llm/gpu_moe.go:673-688) and so does this — a bank in any type the
    // device expands stays as it is and the expert kernels read it through that type's arm —
    // unless `moe_plan` (the grammar of LLM_MOE_BANK, llm/moebank.go:55-63: family=q4_k,... with
    // a family naming a ceiling) narrows that family, which refits the banks wider than Q4_K.
    struct LoadOpts {
        bool transcode = true;
        std::string moe_plan;
        bool head_native = true;  // output.weight stays in the checkpoint's own type (LLM_HEAD_TYPE=q4_k refits it like the rest)
    };
    void LoadGGUF(const gguf::Set &s, const LoadOpts &o);
    void LoadGGUF(const gguf::Set &s, bool transcode = true) {
        LoadOpts o;
        o.transcode = transcode;
        LoadGGUF(s, o);
    }
    const std::vector<std::string> &Transcoded() const { return transcoded_; }
    // This model as one version-3 file the above reads back bit for bit: metadata keys as
    // ConfigFromGGUF reads them, constituents in place of fused tensors, expert banks 3-D.
    void SaveGGUF(const std::string &path, const std::string &arch = "qwen3next") const;

private:
    void add(const std::string &name, TensorView::Kind kind, int64_t rows, int64_t cols, float mean, float std);
    void alias(const std::string &name, const std::string &of, int64_t row0, int64_t rows);
    const std::string *base_of(const TensorView &alias) const;
    Device &dev_;
    Config cfg_;
    std::map<std::string, TensorView> tensors_;
    std::vector<std::string> transcoded_;
};

// llm.Stage (llm/gpu.go:1578-1581)
struct Stage {
    std::string Kind;
    uint64_t GPUNanos = 0;
};

// How the rows of a pass map to sequences (llm/batch.go:33-72): n_seq sequences of seq_len
// consecutive rows each; sequence s starts at position pos[s] on slot slot[s].  An ordinary pass
// is one sequence of nTok rows; a batched decode pass is nTok sequences of one row.  Both arrays
// live on the device, so a recorded pass follows the sequence without being re-recorded.
struct PassRows {
    const int32_t *pos = nullptr;
    const int32_t *slot = nullptr;  // nullptr: sequence s is slot s
    int host_slot = -1;             // a pass of one sequence whose slot the host knows when it records the pass: the
                                    // blocks then offset their per-slot memory themselves and the kernels are spared
                                    // a dependent load of the slot word
    int n_seq = 1, seq_len = 1;
    bool spec = false;              // DeltaNet: a rewindable pass (state goes to the other planes)
    // A pass of one to four rows of a sequence whose mixer's output projection also forms the logits of the layer's router
    // (MoEGPU::Fold): the table's rows, how many, and where the products go.  out must then be
    // another buffer than in.
    const float *fold = nullptr;
    int fold_rows = 0, fold_stride = 0;
    float *fold_out = nullptr;
    int rows() const { return n_seq * seq_len; }
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
    // The router's rows of `layer` carried through the output projection `w_out` (Q4_K [NEmbd][k])
    // that feeds the block: made once, when a graph is staged.  False (and nothing made) where the
    // shapes or types are not the ones the fused launch is built for.
    bool Fold(int layer, const TensorView &w_out);
    bool Folded(int layer) const { return layer >= 0 && layer < static_cast<int>(fold_.size()) && fold_[layer] != nullptr; }
    // What the mixer's output projection needs to form the logits (fields of PassRows)
    void FoldInto(int layer, PassRows &r) const;
    // The block on a one-row pass whose logits came with the output projection: gate/up (which
    // normalises the row itself) and down.  `in` is the row before its RMSNorm.
    std::vector<shv_op> DispatchesFolded(int layer, const float *in, float *out, int nTok, std::vector<std::string> *labels) const;
    static constexpr int kFoldRows = 4;  // rows of one sequence the fused launches take
    std::vector<float> Logits() const;    // [T][NExpert+1]
    std::vector<int32_t> TopK() const;    // [T][used]
    std::vector<float> Weights() const;   // [T][used+1]
    std::vector<float> Swiglu() const;    // [T][used+1][ffn]; of a pass short enough not to be grouped by expert (a grouped pass leaves operands there, not floats)
    std::vector<float> Out() const;       // [T][NEmbd]
    float *InPort() const { return in_; }
    float *OutPort() const { return out_; }
    uint64_t ActivationBytes() const { return act_bytes_; }
    // Where the top-k selection runs (MoEGPU.SetRouter, llm/gpu_moe.go:307): fused, in the prologue
    // of the gate/up kernel from the router's logits, or as a dispatch of its own after the router.
    // Fused on passes of one to four rows unless asked otherwise (mode 2): one launch fewer on the
    // step's critical path, the selection repeated by every workgroup with all four of its waves
    // (482 to 509 tok/s; a 2-row pass 2.32 to 2.28 ms, a 3-row pass 2.81 to 2.75); with the router's
    // rows on the mixer's output projection (Fold) two launches fewer, which pays at four rows too
    // (four sequences a pass 3.14 to 2.90 ms); beyond, where there is no such table, slower than a
    // dispatch of its own (eight rows 4.80 to 5.04 ms).
    void SetRouter(bool fused) { route_mode_ = fused ? 1 : 0; }
    bool FusedRouter(int rows = 1) const { return route_mode_ == 1 || (route_mode_ == 2 && rows <= kFoldRows); }

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    int max_tok_, n_tok_ = 0;
    float *in_, *out_, *xn_, *logits_, *weights_, *act_, *pairs_ = nullptr;
    int32_t *topk_, *group_ = nullptr;
    uint64_t act_bytes_ = 0;
    int route_mode_ = 2;  // 0 own dispatch, 1 fused, 2 fused for passes of up to four rows
    std::vector<float *> fold_;  // per layer [NExpert+1][k + NEmbd], or nullptr
    int fold_k_ = 0;
};

// llm.DeltaNetGPU (llm/gpu_deltanet.go:207-322, NewDeltaNetGPUBank :421)
class DeltaNetGPU {
public:
    static constexpr int kRing = 8;  // least projection rows kept per slot: up to 5 rows a pass + 3 of history
    // A pass of more rows than this (one sequence's prompt chunk) keeps its projection rows in one
    // ring sized for the whole pass and shared by all layers and slots; the conv's three rows of
    // history come from the slot's own ring before the step, and the pass's last three go back after.
    static constexpr int kSmallPass = 64;
    // planes > 1 stages the state copies a rewindable pass needs (WithDNSpecSlots,
    // llm/gpu_deltanet.go:380); plane is the device array naming each slot's committed copy.
    DeltaNetGPU(Device &dev, const Model &m, int maxTokens, int slots, int32_t *pos, int planes = 1, int32_t *plane = nullptr);
    void Upload(const std::vector<float> &x, int nTok);
    void Resize(int nTok);
    void Run(int layer);
    void Reset(int layer);
    void ResetAll();
    void ResetSlot(int slot);
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, int nTok, std::vector<std::string> *labels) const;
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, const PassRows &rows, std::vector<std::string> *labels) const;
    std::vector<float> State(int layer, int slot = 0, int plane = 0) const;  // S, [hv][d][d]
    void SetState(int layer, const std::vector<float> &s, int slot = 0, int plane = 0);
    int Planes() const { return planes_; }
    int RingSlots() const { return ring_slots_; }
    // What a sequence carries from one token to the next (DeltaNetGPU.CarriedLen / SaveCarried /
    // RestoreCarried, llm/gpu_deltanet.go): per DeltaNet layer the committed state plane and the
    // three projection rows before position `past` that the causal conv will still read.
    size_t CarriedLen() const;
    void SaveCarried(float *dst, int slot, int plane, int past) const;
    void RestoreCarried(const float *src, int slot, int plane, int past);
    std::vector<float> Result() const;  // [T][hv*d] attention output before the gated norm
    std::vector<float> Out() const;     // [T][NEmbd]
    float *InPort() const { return in_; }
    float *OutPort() const { return out_; }
    uint64_t StateBytes() const { return state_bytes_; }

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    int max_tok_, slots_, planes_, ring_slots_, n_tok_ = 0;
    int32_t *pos_, *plane_;
    float *in_, *out_, *attn_;
    float *row_ = nullptr;               // the projection row of a one-row pass, also kept outside the ring (the out projection's gate)
    float *big_ring_ = nullptr;          // the long pass's ring, [big_slots_][DNFusedRows]
    int big_slots_ = 0;
    float *work_ = nullptr;              // what the chunked step prepares of a pass's rows (q^, k^, v, log g, beta)
    int64_t work_floats_ = 0;
    std::vector<float *> ring_, state_;  // per layer (nullptr on attention layers)
    uint64_t state_bytes_ = 0;
};

// llm.AttnGPU (llm/gpu_attn.go:403-539, NewAttnGPUBank :779)
class AttnGPU {
public:
    // only_layer >= 0 stages that one block alone (the draft head's, llm/mtp.go:176-275)
    AttnGPU(Device &dev, const Model &m, int maxTokens, int nKV, int slots, int32_t *pos, int only_layer = -1);
    void Upload(const std::vector<float> &x, int nTok);
    void Resize(int nTok);
    void Run(int layer);
    static constexpr int kMaxSplits = 512;  // what the decode kernel's merge has room for
    size_t partial_records_ = 0;            // slice records (two rows of 8 heads each) the scratch holds
    void SetSplits(int n);
    int Splits() const { return splits_; }
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, int nTok, std::vector<std::string> *labels) const;
    std::vector<shv_op> Dispatches(int layer, const float *in, float *out, const PassRows &rows, std::vector<std::string> *labels) const;
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
    // the indexer of layers that have one: raw keys [slots][cells][IdxDim] binary16 and the pooled
    // blocks' keys [slots][cells/ratio + 1][IdxDim] per layer; projection rows, scores and the
    // selection's bit mask of one pass, shared by the layers
    std::vector<uint16_t *> idxc_;
    std::vector<float *> pooled_;
    float *qsa_work_ = nullptr, *qsa_score_ = nullptr;
    uint32_t *qsa_mask_ = nullptr;
    int mask_stride_ = 0;
};

// llm.HeadGPU (llm/gpu_head.go:54-100, NewHeadGPUBank :114)
class HeadGPU {
public:
    HeadGPU(Device &dev, const Model &m, int maxRows);
    void Upload(const std::vector<float> &x, int rows);
    void Resize(int rows);
    void Run();
    std::vector<shv_op> Dispatches(const float *in, int rows, std::vector<std::string> *labels) const;
    // the same projection through another norm and into another arena, over the first `cols`
    // vocabulary entries (RunCols, llm/gpu_head.go:499): what the draft head borrows
    std::vector<shv_op> DispatchesTo(const float *in, int rows, const float *gamma, float *logits, int cols,
                                     std::vector<std::string> *labels) const;
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
// Rows an attention or DeltaNet block takes in one go; a pass of more rows walks them in groups.
constexpr int kBlockRows = 64;

struct GraphOpts {
    int MaxTokens = 1;  // rows a pass may carry, up to 4096 (a longer prompt goes through in chunks of this)
    int NKV = 4096;     // attention cache cells per slot
    int Layers = 0;     // 0: all of the model's layers
    bool NoHead = false;
    int Slots = 1;            // sequences held side by side (UseSlot, DecodeRows)
    int AttnSplits = 0;       // 0: chosen from NKV
    int HeadRows = 0;         // rows ExtendRows / DecodeRows may carry; 0: MaxTokens
    bool Speculative = false; // stage the DeltaNet state planes rewindable passes need
    int SpecRows = 2;         // rows of a verification pass: draft depth + 1
};

// llm.GraphStats (llm/graph.go:536-566)
struct GraphStats {
    uint64_t GPUNanos = 0;
    int Dispatches = 0;
    int Runs = 0;
    std::map<std::string, uint64_t> Kinds;  // GPU time by dispatch label
};

// A recorded op sequence and its replayable form.
struct Pass {
    std::vector<shv_op> ops;
    std::vector<std::string> labels;
    shv_prerecorded *rec = nullptr;
    int32_t *ring = nullptr;  // a draft pass that reads its tokens from the trunk's id ring: which ring
};

// llm.Checkpoint (llm/graph.go:902-1003): a sequence's position, tokens and DeltaNet carry, in host
// memory; the KV cells need no copy, the ones past the checkpoint are simply written again.
struct Checkpoint {
    int past = 0;
    std::vector<int32_t> ids;
    std::vector<float> dn;
};

// llm.Graph (llm/graph.go:184-289, NewGraph :609): the whole model as recorded op sequences, one
// per (slot, row count, kind of pass), recorded the first time each is needed.
class Graph {
public:
    Graph(Device &dev, const Model &m, const GraphOpts &opts);
    ~Graph();
    // Forward resets the sequence and extends it (llm/graph.go:1695).
    void Forward(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden);
    // Extend appends ids to the sequence and returns the LAST row's logits (llm/graph.go:1709).
    void Extend(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *hidden);
    // ForwardResidual is Forward that also keeps the residual of EVERY prompt row on the device,
    // [T][NEmbd], which is what primes the draft head (llm/graph.go:1441-1450).
    const float *ForwardResidual(const std::vector<int32_t> &ids, std::vector<float> *logits);
    // ExtendResidual is the same for a sequence that goes on: ids appended, every row's residual kept
    // (llm/graph.go ExtendResidual, as backend/llm_sched.go:672 calls it for a chunk that primes a draft).
    const float *ExtendResidual(const std::vector<int32_t> &ids, std::vector<float> *logits);
    // ExtendRows appends ids and computes every row's logits: the verification pass
    // (llm/graph.go:1383-1429).  logits [n][vocab] and res [n][NEmbd] (the residual before the
    // final norm) are copied out when asked for; Argmaxes() and ResPort() serve a caller that
    // needs only the greedy tokens and leaves the residual on the device.
    void ExtendRows(const std::vector<int32_t> &ids, std::vector<float> *logits, std::vector<float> *res);
    // DecodeRows advances n sequences by one token each in one pass (llm/graph.go:1527-1666).
    void DecodeRows(const std::vector<int> &slots, const std::vector<int32_t> &ids, std::vector<float> *logits);
    // The same pass over ids that are on the device already: StageIds puts tokens at positions at.. of the live
    // slot's id ring without waiting for the device, IdsPort() is that ring for an op that names a token itself
    // (a draft head's arg-max), ExtendRowsStaged runs the n rows at positions past.. that the ring then holds.
    void StageIds(int at, const std::vector<int32_t> &ids);
    int32_t *IdsPort() const { return ids_ + slot_ * ids_stride_; }
    void ExtendRowsStaged(int n);
    std::vector<int32_t> Argmaxes() const;     // the greedy token of each row of the last ExtendRows / DecodeRows
    const float *ResPort() const { return x_; }  // residual rows of the last pass, on the device
    // Greedy continuation (cmd/llm/generate.go:121-165): n replays of the recorded decode step with
    // the arg-max feeding the next step on the device; returns the n tokens and GPU time.
    std::vector<int32_t> Generate(int n, uint64_t *gpu_nanos);
    void Reset();  // the live slot's sequence
    void UseSlot(int s);
    int Slots() const { return o_.Slots; }
    int Slot() const { return slot_; }
    int Past() const { return seq_[slot_].past; }
    int PastOf(int s) const { return seq_.at(s).past; }
    bool InFlight() const { return spec_armed_; }  // a rewindable pass has run and is neither kept nor committed
    int Plane() const { return seq_[slot_].plane; }  // the live slot's committed DeltaNet state plane
    int NKV() const { return o_.NKV; }
    int MaxRows() const { return rows_max_; }
    int StepRows() const;  // rows one DecodeRows pass may carry: 0 without a head
    std::vector<int32_t> Ids() const;
    // Rewindable passes (llm/graph.go:1122-1267).  While Speculate is on, ExtendRows leaves the
    // committed DeltaNet state alone and stores the state after each of its rows apart; exactly
    // one such pass may be in flight, ended by Commit (all rows), Keep(k) (the first k; needs
    // SpeculateFirst) or Rewind (none; refused under SpeculateFirst, as in the reference).
    void Speculate(bool on);
    bool Speculating() const { return spec_; }
    void SpeculateFirst(bool on);
    void Keep(int k);
    void KeepFirst() { Keep(1); }
    void Commit();
    void Rewind();
    // Checkpoint saves the live slot's sequence into `into` (llm/graph.go:1004-1031); Restore takes
    // the slot back to it and refuses unless the slot's sequence still starts with the
    // checkpoint's tokens (:1037-1062).  Neither may run while a rewindable pass is in flight.
    void Checkpoint(struct Checkpoint &into);
    void Restore(const struct Checkpoint &c);
    // One decode step dispatched op by op with a GPU time per op, folded by label
    // (DispatchMultiMarked + recorder.submit, vk/engine.go:913, llm/record.go:217-232).
    std::vector<Stage> ProfileStep();
    // GPU time of one `rows`-row verification pass relative to nothing: nanoseconds per op label.
    std::vector<Stage> ProfileRows(int rows);
    std::vector<Stage> ProfileChunk(const std::vector<int32_t> &ids);
    GraphStats Stats;
    void ResetStats() { Stats = GraphStats(); }
    int Dispatches();
    MoEGPU &MoE() { return *moe_; }
    DeltaNetGPU &DeltaNet() { return *dn_; }
    AttnGPU &Attn() { return *attn_; }
    HeadGPU &Head() { return *head_; }
    Device &Dev() { return dev_; }
    const Model &GetModel() const { return m_; }

private:
    enum Kind { kPrefill = 0, kSample = 1, kRows = 2, kBatch = 3 };
    struct Seq {
        int past = 0;
        int plane = 0;
    };
    Pass &pass(int slot, int rows, Kind kind, bool spec);
    uint64_t submit(Pass &p, int iters, const char *what);
    void put_pos();
    void check_ids(const std::vector<int32_t> &ids) const;
    void extend(const std::vector<int32_t> &ids, float *res_all);
    Device &dev_;
    const Model &m_;
    Config c_;
    GraphOpts o_;
    int layers_, rows_max_, block_rows_ = 1, groups_ = 1, slot_ = 0;
    int32_t *grp_pos_ = nullptr;
    std::vector<Seq> seq_;
    bool spec_ = false, spec_first_ = false, spec_armed_ = false;
    int spec_past_ = 0, spec_rows_ = 0;
    int last_rows_ = 0;
    float *x_ = nullptr;       // residual stream, [rows_max][NEmbd]
    float *x2_ = nullptr;      // a one-row pass's row between a layer's mixer and its MoE block (router fold)
    float *res_all_ = nullptr; // ForwardResidual's rows
    size_t res_all_rows_ = 0;
    int32_t *ids_ = nullptr;   // [Slots][NKV+2] the sequences' tokens by position
    int32_t *ctl_ = nullptr;   // pos[Slots] | plane[Slots] | slot index[Slots] | row pos[rows] | row slot[rows] | row ids[rows]
    int32_t *pos_ = nullptr, *plane_ = nullptr, *slot_ix_ = nullptr, *row_pos_ = nullptr, *row_slot_ = nullptr, *row_ids_ = nullptr;
    int32_t *best_ = nullptr;
    size_t ids_stride_ = 0;
    MoEGPU *moe_ = nullptr;
    DeltaNetGPU *dn_ = nullptr;
    AttnGPU *attn_ = nullptr;
    HeadGPU *head_ = nullptr;
    std::map<std::vector<int>, Pass> passes_;
};

// llm.MTPHead (llm/mtp.go:84-134, NewMTPHeadSlots :151): the draft block staged beside the trunk.
// For a model without hyper-connection streams the wiring is qwen3next's (llm/mtp.go:31-33):
//     x   = eh_proj . concat(RMSNorm(embd(token), enorm), RMSNorm(h, hnorm))
//     x  += Attn(RMSNorm(x, attn_norm));  x += MoE(RMSNorm(x, ffn_norm))
//     logits = lm_head . RMSNorm(x, shared_head_norm)           (the trunk's lm_head, borrowed)
// h is the trunk's residual after the previous token, or this block's own x when drafts chain.
// Its only carried state is a one-layer KV cache per slot, which Rewind moves for free.
class MTPHead {
public:
    MTPHead(Device &dev, const Model &m, HeadGPU &head, int maxTok, int nKV, int slots);
    ~MTPHead();
    // n rows at positions pos..pos+n-1: hs is [n][NEmbd] ON THE DEVICE (the trunk's ResPort() or
    // ResPort() of this head), ids the token at each position.  With head, the last row's logits
    // are computed and its greedy token returned (-1 otherwise).  (MTPHead.Rows, llm/mtp.go:542)
    int32_t Rows(const float *hs, const std::vector<int32_t> &ids, int pos, bool head);
    // the reference's host-side signature: hs from host memory, logits and residual copied back
    void RowsHost(const std::vector<float> &hs, const std::vector<int32_t> &ids, int pos, bool head,
                  std::vector<float> *logits, std::vector<float> *res);
    // Rows for a caller that does not wait (a greedy round): the n tokens are read from `ring` (the trunk's id ring
    // of the sequence) at positions pos..pos+n-1, the head's arg-max is stored as the token at pos+n there, kept
    // for DraftAt(k) and moves this head's position word on, so that the call for draft k+1 (n = 1, pos < 0: the
    // position the device holds) needs nothing from the host.  Returns without waiting for the device.
    void RowsChained(const float *hs, int n, int pos, int k, int32_t *ring);
    int32_t DraftAt(int k) const { return best_[k]; }  // valid once the stream has been waited for
    const float *ResPort() const { return x_; }  // [n][NEmbd] of the last call
    void LastLogits(std::vector<float> *out);     // the last head call's logits, over the drafted prefix of the vocabulary
    int Past() const { return pasts_[slot_]; }
    void Rewind(int n);
    void Reset() { pasts_[slot_] = 0; }
    int Slots() const { return static_cast<int>(pasts_.size()); }
    void UseSlot(int s);
    int MaxRows() const { return max_tok_; }
    void SetVocab(int k);  // draft over a prefix of the vocabulary (llm/mtp.go:675); 0: all of it
    int Steps = 0;
    uint64_t GPUNanos = 0;

private:
    Device &dev_;
    const Model &m_;
    Config c_;
    HeadGPU &head_;
    int max_tok_, n_kv_, layer_, slot_ = 0, vocab_ = 0;
    std::vector<int> pasts_;
    AttnGPU *attn_ = nullptr;
    MoEGPU *moe_ = nullptr;
    float *x_, *h_, *e_, *logits_;
    int32_t *ctl_, *pos_, *slot_ix_, *ids_, *best_;
    std::map<std::vector<int>, Pass> passes_;
    Pass &draft_pass(int n, bool head, int k, int32_t *ring);
};

// llm.SpecStats (llm/spec.go:67-112), the counters that exist without a sampler.
struct SpecStats {
    int Rounds = 0, Drafted = 0, Accepted = 0, Tokens = 0;
    int Passes[5] = {0, 0, 0, 0, 0};
    int DraftedAt[4] = {0, 0, 0, 0}, AcceptedAt[4] = {0, 0, 0, 0};
    uint64_t DraftNanos = 0, VerifyNanos = 0;
};

// llm.Speculator (llm/spec.go:221-857): the draft head proposes Depth tokens, one verification
// pass of Depth+1 rows checks them, the longest agreeing prefix is kept.  Greedy by default: every
// token it emits is the trunk's own arg-max over the trunk's own sequence.  With a sampler
// (UseSampler) the draft draws its proposals from its own sampler's distribution q and the trunk
// keeps each with probability min(1, p/q), else redraws from max(0, p - q) (Sampler::Verify), so
// the tokens are distributed as the trunk's sampler's whatever the draft proposes; the rows'
// logits then come to the host, where the reference keeps its sampler too.
class Speculator {
public:
    // slot >= 0: the speculator of one sequence slot of a served graph (NewSlotSpeculator,
    // llm/spec.go:258): it drafts in that slot of the draft's cache and leaves Graph.Speculate to
    // its caller, who also runs plain and batched passes on the same graph.
    Speculator(Graph &g, MTPHead &d, int depth, int slot = -1);
    // Prefill the prompt through the trunk and the draft (Start + Prime, llm/spec.go:300-420);
    // returns the first generated token.
    int32_t Start(const std::vector<int32_t> &prompt);
    // One round (llm/spec.go:703-857): the tokens it emitted, 1..Depth+1 of them.  `forced`, when
    // not empty, replaces the draft head's proposals (the draft still runs): the reference's
    // `propose` hook, which tests use to drive every acceptance length.
    // limit > 0: the round keeps at most that many tokens (a request's remaining budget).
    std::vector<int32_t> Round(const std::vector<int32_t> &forced = {}, int limit = 0);
    // s == nullptr or a greedy sampler: back to arg-max.  The sampler is borrowed; the draft's is made
    // from it (Sampler::DraftSampler) with its own seed.  Takes effect at the next Start.
    void UseSampler(Sampler *s, int64_t draft_seed);
    // The sampler of the rounds from here on, for a caller that serves several requests (nullptr or a
    // greedy one: arg-max).  exact: the drafts are the draft head's arg-max and every verified row
    // is ONE plain draw of s, kept while it equals the draft after it, so a seeded request consumes
    // its random stream exactly as a loop of plain steps does (backend/llm_spec_test.go:24-31);
    // otherwise the drafts are drawn and verified by speculative sampling, as UseSampler arranges.
    void SetSampler(Sampler *s, bool exact, int64_t draft_seed);
    void Stop() { g_.Speculate(false); }
    // ---- the served loop's pieces (llm/spec.go:285-456) ----
    // Prime writes the draft's cells at positions at .. at+n-1 from a chunk the trunk has just run:
    // res is ExtendResidual's, row r the trunk's residual at at+r, on the device.  Position `at`
    // is seeded from the residual this speculator holds, or zeros at position 0.
    void Prime(const std::vector<int32_t> &ids, int at, const float *res);
    // Owe records a plain decode step the trunk ran on this slot, token x and the trunk's residual
    // at that row (on the device): the draft catches up at the next round or at Settle.
    void Owe(int32_t x, const float *h);
    // Settle writes the draft's cells for the rows it owes; nothing is pending after it.
    void Settle();
    // The trunk's residual one row before its position, which a checkpoint keeps beside the
    // trunk's state so that Rewind can resume from it.
    std::vector<float> Residual() const;
    void Rewind(int past, const std::vector<float> &h);
    // One round from `first`, the token named last and not yet run (Round, llm/spec.go:349).
    std::vector<int32_t> RoundFrom(int32_t first, const std::vector<int32_t> &forced = {}, int limit = 0);
    bool Seeded() const { return seeded_; }
    int Owed() const { return static_cast<int>(owe_x_.size()); }
    SpecStats Stats;
    int Depth;

private:
    Graph &g_;
    MTPHead &d_;
    int32_t pend_ = -1;
    int slot_ = -1, cap_rows_ = 0;
    bool seeded_ = false;
    float *h_ = nullptr;  // [cap_rows_][NEmbd]: the owed rows' residuals, then the trunk's last one
    std::vector<int32_t> owe_x_;
    void use_slot();
    int past() const { return slot_ >= 0 ? g_.PastOf(slot_) : g_.Past(); }
    void settle_owed();
    Sampler *sampler_ = nullptr;
    bool exact_ = false;
    std::unique_ptr<Sampler> draft_sampler_;
    std::vector<int32_t> sampled_round(const std::vector<int32_t> &forced, int limit);
    // the greedy round handed to the device in one go: drafts and verification back to back, one wait
    bool chained_ = true;  // LLM_SPEC_CHAIN=0: every draft call and the verification pass waited for in turn
    std::vector<int32_t> chained_round(const std::vector<int32_t> &forced, int limit);
    std::vector<int32_t> finish_round(const std::vector<int32_t> &rows, const std::vector<int32_t> &best, int at, int limit);
};

}  // namespace llm
