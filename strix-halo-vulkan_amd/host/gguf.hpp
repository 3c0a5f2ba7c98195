// gguf.hpp — GGUF checkpoints mapped read-only, the host side of weight staging: the reference's
// package gguf (gguf/gguf.go) restated in C++.  A file is a magic, a version, two counts, a table
// of typed key/value pairs, a table of tensor descriptors, padding to general.alignment and one
// data section every descriptor's offset is relative to.  Weights are never copied on the host: a
// Tensor's Data points into the mapping and goes from there straight into a device buffer.
//
// Shapes are in ggml order: Dims[0] is the fastest-varying axis, the row length of a 2-D weight.
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace gguf {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

constexpr uint64_t kDefaultAlignment = 32;  // gguf/gguf.go:48
constexpr const char *kKeyAlignment = "general.alignment";
constexpr const char *kKeyArchitecture = "general.architecture";
constexpr const char *kKeySplitNo = "split.no";
constexpr const char *kKeySplitCount = "split.count";
constexpr const char *kKeySplitTensors = "split.tensors.count";

// ggml tensor types by their file-format numbers (gguf/gguf.go:55-88).
enum Type : uint32_t {
    F32 = 0, F16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9, Q2_K = 10, Q3_K = 11,
    Q4_K = 12, Q5_K = 13, Q6_K = 14, Q8_K = 15, IQ2_XXS = 16, IQ2_XS = 17, IQ3_XXS = 18, IQ1_S = 19,
    IQ4_NL = 20, IQ3_S = 21, IQ2_S = 22, IQ4_XS = 23, I8 = 24, I16 = 25, I32 = 26, I64 = 27, F64 = 28,
    IQ1_M = 29, BF16 = 30, TQ1_0 = 34, TQ2_0 = 35, MXFP4 = 39,
};

// Block geometry of a type (gguf/gguf.go:95-134): elements a block holds, bytes it takes.
struct TypeInfo {
    const char *name;
    int elems;
    int nbytes;
};
const TypeInfo *Info(uint32_t type);        // nullptr for a type the table does not know
std::string TypeName(uint32_t type);        // "?<n>" for an unknown one (gguf/gguf.go:138-144)
inline bool Known(uint32_t type) { return Info(type) != nullptr; }
inline bool Quantised(uint32_t type) { const TypeInfo *i = Info(type); return i && i->elems > 1; }
int64_t SizeOf(uint32_t type, int64_t n);   // bytes of n elements; throws on an unknown type or a partial block

// One entry of the tensor table (gguf/gguf.go:175-246).  Data aliases the mapped shard.
struct Tensor {
    std::string Name;
    uint32_t Type = 0;
    std::vector<int64_t> Dims;
    const uint8_t *Data = nullptr;
    uint64_t Bytes = 0;
    int Shard = 0;

    int64_t Elems() const;
    int64_t Rows() const;      // the product of every axis but the first
    int64_t RowBytes() const;  // 0 when Dims[0] is not whole blocks
    const uint8_t *Row(int64_t i) const { return Data + i * RowBytes(); }
    // The pages of this tensor will be read at random: one page a fault instead of a readahead window.
    void AdviseRandom() const;
};

// A metadata value, widened as the reference widens it (gguf/gguf.go:528-651): every integer
// width to uint64 / int64, both float widths to double; arrays keep one widened element type.
struct Value {
    enum Kind { None = 0, Uint, Int, Float, Bool, Str, Uints, Ints, Floats, Bools, Strs } kind = None;
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    bool b = false;
    std::string s;
    std::vector<uint64_t> us;
    std::vector<int64_t> is;
    std::vector<double> fs;
    std::vector<uint8_t> bs;
    std::vector<std::string> ss;
    uint64_t Len() const;
};

// The typed getters both File and Set answer (gguf/gguf.go:653-726).
class KV {
public:
    virtual ~KV() = default;
    virtual const Value *Find(const std::string &key) const = 0;
    bool Uint(const std::string &key, uint64_t *out) const;   // any integer width; a negative one is no answer
    bool Int(const std::string &key, int64_t *out) const;
    bool Float(const std::string &key, double *out) const;    // integers widen
    bool Str(const std::string &key, std::string *out) const;
    bool Bool(const std::string &key, bool *out) const;
    const std::vector<std::string> *Strings(const std::string &key) const;
    const std::vector<uint64_t> *Uints(const std::string &key) const;
    const std::vector<int64_t> *Ints(const std::string &key) const;
    const std::vector<double> *Floats(const std::string &key) const;
};

// One mapped file: a whole checkpoint or one shard of a split one (gguf/gguf.go:248-428).
class File : public KV {
public:
    static std::unique_ptr<File> Open(const std::string &path);
    ~File() override;
    File(const File &) = delete;
    File &operator=(const File &) = delete;

    std::string Path;
    uint32_t Version = 0;
    uint64_t Alignment = kDefaultAlignment;
    int64_t DataStart = 0;  // file offset of the data section
    std::vector<Tensor> Tensors;

    const std::vector<std::string> &Keys() const { return order_; }
    const Value *Find(const std::string &key) const override;
    const Tensor &Get(const std::string &name) const;
    bool Has(const std::string &name) const { return by_name_.count(name) != 0; }

private:
    File() = default;
    void parse();
    std::map<std::string, Value> kv_;
    std::vector<std::string> order_;
    std::map<std::string, size_t> by_name_;
    const uint8_t *map_ = nullptr;
    size_t size_ = 0;
};

// A checkpoint that may be split over several shards, llama.cpp's convention
// `<base>-00001-of-00004.gguf` (gguf/gguf.go:726-930): opened from any one shard or from a
// directory holding exactly one checkpoint; shard 1 carries the metadata.
class Set : public KV {
public:
    static std::unique_ptr<Set> Open(const std::string &path);
    std::vector<std::unique_ptr<File>> Files;
    std::vector<const Tensor *> Tensors;

    const File &KVFile() const { return *Files.at(0); }
    const Value *Find(const std::string &key) const override { return KVFile().Find(key); }
    const std::vector<std::string> &Keys() const { return KVFile().Keys(); }
    const Tensor &Get(const std::string &name) const;
    bool Has(const std::string &name) const { return by_name_.count(name) != 0; }
    int Len() const { return static_cast<int>(Tensors.size()); }
    int64_t Params() const;
    int64_t Bytes() const;
    std::string Arch() const;

private:
    void checkSplit() const;
    std::map<std::string, const Tensor *> by_name_;
};

// Writes a version-3 file: metadata in the order given, every tensor at the next multiple of the
// alignment.  A tensor's bytes come from a callback at write time, one tensor in memory at a time.
class Writer {
public:
    explicit Writer(uint64_t alignment = kDefaultAlignment);
    void PutU32(const std::string &key, uint32_t v);
    void PutI32(const std::string &key, int32_t v);
    void PutU64(const std::string &key, uint64_t v);
    void PutF32(const std::string &key, float v);
    void PutBool(const std::string &key, bool v);
    void PutStr(const std::string &key, const std::string &v);
    void PutStrs(const std::string &key, const std::vector<std::string> &v);
    void PutI32s(const std::string &key, const std::vector<int32_t> &v);
    void AddTensor(const std::string &name, uint32_t type, const std::vector<int64_t> &dims, std::function<void(uint8_t *dst, uint64_t bytes)> fill);
    void Write(const std::string &path) const;

private:
    struct Entry {
        std::string name;
        uint32_t type;
        std::vector<int64_t> dims;
        uint64_t bytes, offset;
        std::function<void(uint8_t *, uint64_t)> fill;
    };
    void key(const std::string &k, uint32_t vt);
    uint64_t align_;
    uint64_t n_kv_ = 0, data_ = 0;
    std::vector<uint8_t> kv_;
    std::vector<Entry> tensors_;
};

}  // namespace gguf
