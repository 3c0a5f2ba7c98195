// GGUF reader and writer: see gguf.hpp.
#include "gguf.hpp"

#include <dirent.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>

namespace gguf {

namespace {

struct TypeRow {
    uint32_t type;
    TypeInfo info;
};
// ggml-common.h's block geometry (gguf/gguf.go:101-134)
const TypeRow kTypes[] = {
    {F32, {"F32", 1, 4}},          {F16, {"F16", 1, 2}},          {BF16, {"BF16", 1, 2}},        {F64, {"F64", 1, 8}},
    {I8, {"I8", 1, 1}},            {I16, {"I16", 1, 2}},          {I32, {"I32", 1, 4}},          {I64, {"I64", 1, 8}},
    {Q4_0, {"Q4_0", 32, 18}},      {Q4_1, {"Q4_1", 32, 20}},      {Q5_0, {"Q5_0", 32, 22}},      {Q5_1, {"Q5_1", 32, 24}},
    {Q8_0, {"Q8_0", 32, 34}},      {Q8_1, {"Q8_1", 32, 36}},      {IQ4_NL, {"IQ4_NL", 32, 18}},  {MXFP4, {"MXFP4", 32, 17}},
    {Q2_K, {"Q2_K", 256, 84}},     {Q3_K, {"Q3_K", 256, 110}},    {Q4_K, {"Q4_K", 256, 144}},    {Q5_K, {"Q5_K", 256, 176}},
    {Q6_K, {"Q6_K", 256, 210}},    {Q8_K, {"Q8_K", 256, 292}},    {IQ4_XS, {"IQ4_XS", 256, 136}}, {IQ3_S, {"IQ3_S", 256, 110}},
    {IQ3_XXS, {"IQ3_XXS", 256, 98}}, {IQ2_XXS, {"IQ2_XXS", 256, 66}}, {IQ2_XS, {"IQ2_XS", 256, 74}}, {IQ2_S, {"IQ2_S", 256, 82}},
    {IQ1_S, {"IQ1_S", 256, 50}},   {IQ1_M, {"IQ1_M", 256, 56}},   {TQ1_0, {"TQ1_0", 256, 54}},   {TQ2_0, {"TQ2_0", 256, 66}},
};

std::string fmt(const char *f, ...) __attribute__((format(printf, 1, 2)));
std::string fmt(const char *f, ...) {
    char buf[768];
    va_list ap;
    va_start(ap, f);
    std::vsnprintf(buf, sizeof(buf), f, ap);
    va_end(ap);
    return buf;
}

// metadata value tags (gguf/gguf.go:502-518)
enum ValueType : uint32_t { vtU8, vtI8, vtU16, vtI16, vtU32, vtI32, vtF32, vtBool, vtStr, vtArray, vtU64, vtI64, vtF64 };

// walks the little-endian header with every read bounds-checked (gguf/gguf.go:431-500)
struct Reader {
    const uint8_t *b;
    size_t n, o = 0;

    void need(size_t k) const {
        if (k > n - o) throw Error(fmt("truncated at offset %zu, wanted %zu more bytes of %zu", o, k, n));
    }
    template <typename T>
    T le() {
        need(sizeof(T));
        T v;
        std::memcpy(&v, b + o, sizeof(T));  // the hosts this runs on are little-endian
        o += sizeof(T);
        return v;
    }
    std::string str() {
        const uint64_t len = le<uint64_t>();
        if (len > n) throw Error(fmt("string length %llu exceeds the file", static_cast<unsigned long long>(len)));
        need(len);
        std::string s(reinterpret_cast<const char *>(b + o), len);
        o += len;
        return s;
    }
    // one scalar, widened into v; returns the widened kind
    Value::Kind scalar(uint32_t t, Value &v) {
        switch (t) {
            case vtU8: v.u = le<uint8_t>(); return Value::Uint;
            case vtI8: v.i = le<int8_t>(); return Value::Int;
            case vtU16: v.u = le<uint16_t>(); return Value::Uint;
            case vtI16: v.i = le<int16_t>(); return Value::Int;
            case vtU32: v.u = le<uint32_t>(); return Value::Uint;
            case vtI32: v.i = le<int32_t>(); return Value::Int;
            case vtF32: v.f = le<float>(); return Value::Float;
            case vtBool: v.b = le<uint8_t>() != 0; return Value::Bool;
            case vtStr: v.s = str(); return Value::Str;
            case vtU64: v.u = le<uint64_t>(); return Value::Uint;
            case vtI64: v.i = le<int64_t>(); return Value::Int;
            case vtF64: v.f = le<double>(); return Value::Float;
        }
        throw Error(fmt("unknown value type %u", t));
    }
    Value value(uint32_t t) {
        Value v;
        if (t != vtArray) {
            v.kind = scalar(t, v);
            return v;
        }
        const uint32_t et = le<uint32_t>();
        const uint64_t cnt = le<uint64_t>();
        if (et == vtArray) throw Error("nested arrays are not in the GGUF grammar");
        if (et > vtF64) throw Error(fmt("unknown array element type %u", et));
        // every element takes at least its fixed size of the bytes that are left, so a count the
        // file cannot hold is refused before anything is reserved for it
        static const uint8_t kSize[] = {1, 1, 2, 2, 4, 4, 4, 1, 8, 0, 8, 8, 8};
        if (cnt > (n - o) / kSize[et]) throw Error(fmt("array of %llu elements exceeds the file", static_cast<unsigned long long>(cnt)));
        Value e;
        switch (et) {
            case vtStr: v.kind = Value::Strs; v.ss.reserve(cnt); break;
            case vtBool: v.kind = Value::Bools; v.bs.reserve(cnt); break;
            case vtF32: case vtF64: v.kind = Value::Floats; v.fs.reserve(cnt); break;
            case vtI8: case vtI16: case vtI32: case vtI64: v.kind = Value::Ints; v.is.reserve(cnt); break;
            default: v.kind = Value::Uints; v.us.reserve(cnt); break;
        }
        for (uint64_t i = 0; i < cnt; i++) {
            scalar(et, e);
            switch (v.kind) {
                case Value::Strs: v.ss.push_back(std::move(e.s)); break;
                case Value::Bools: v.bs.push_back(e.b); break;
                case Value::Floats: v.fs.push_back(e.f); break;
                case Value::Ints: v.is.push_back(e.i); break;
                default: v.us.push_back(e.u); break;
            }
        }
        return v;
    }
};

bool exists(const std::string &p) {
    struct stat st;
    return ::stat(p.c_str(), &st) == 0;
}

std::string dir_of(const std::string &p) {
    const size_t s = p.find_last_of('/');
    return s == std::string::npos ? "." : s == 0 ? "/" : p.substr(0, s);
}
std::string base_of(const std::string &p) {
    const size_t s = p.find_last_of('/');
    return s == std::string::npos ? p : p.substr(s + 1);
}

// `<base>-NNNNN-of-MMMMM.gguf` (gguf/gguf.go:740): the shard suffix llama-gguf-split writes
bool split_name(const std::string &file, std::string *stem, std::string *no, std::string *count) {
    const size_t tail = 1 + 5 + 4 + 5 + 5;  // "-NNNNN" "-of-" "MMMMM" ".gguf"
    if (file.size() < tail) return false;
    const size_t at = file.size() - tail;
    const std::string t = file.substr(at);
    if (t[0] != '-' || t.compare(6, 4, "-of-") != 0 || t.compare(15, 5, ".gguf") != 0) return false;
    for (int i = 0; i < 5; i++)
        if (!isdigit(static_cast<unsigned char>(t[1 + i])) || !isdigit(static_cast<unsigned char>(t[10 + i]))) return false;
    *stem = file.substr(0, at);
    *no = t.substr(1, 5);
    *count = t.substr(10, 5);
    return true;
}

// the one checkpoint in a directory: a single .gguf or the first shard of one split set (gguf/gguf.go:822-843)
std::string sole_checkpoint(const std::string &dir) {
    DIR *d = ::opendir(dir.c_str());
    if (!d) throw Error("gguf: " + dir + ": " + std::strerror(errno));
    std::vector<std::string> candidates;
    while (const dirent *e = ::readdir(d)) {
        const std::string f = e->d_name;
        if (f.size() < 5 || f.compare(f.size() - 5, 5, ".gguf") != 0) continue;
        std::string stem, no, count;
        if (!split_name(f, &stem, &no, &count) || no == "00001") candidates.push_back(dir + "/" + f);
    }
    ::closedir(d);
    std::sort(candidates.begin(), candidates.end());
    if (candidates.empty()) throw Error("gguf: no .gguf checkpoint under " + dir);
    if (candidates.size() > 1) throw Error(fmt("gguf: %s holds %zu checkpoints, name one", dir.c_str(), candidates.size()));
    return candidates[0];
}

// one shard's path expanded into every shard of its set (gguf/gguf.go:845-863)
std::vector<std::string> shard_paths(const std::string &path) {
    std::string stem, no, count;
    if (!split_name(base_of(path), &stem, &no, &count)) return {path};
    const int n = std::atoi(count.c_str());
    if (n < 1) throw Error("gguf: " + path + ": unreadable shard count " + count);
    std::vector<std::string> out;
    for (int i = 0; i < n; i++) {
        out.push_back(fmt("%s/%s-%05d-of-%05d.gguf", dir_of(path).c_str(), stem.c_str(), i + 1, n));
        if (!exists(out.back())) throw Error(fmt("gguf: %s: shard %d of %d is missing", path.c_str(), i + 1, n));
    }
    return out;
}

}  // namespace

const TypeInfo *Info(uint32_t type) {
    for (const TypeRow &r : kTypes)
        if (r.type == type) return &r.info;
    return nullptr;
}

std::string TypeName(uint32_t type) {
    const TypeInfo *i = Info(type);
    return i ? i->name : "?" + std::to_string(type);
}

int64_t SizeOf(uint32_t type, int64_t n) {
    const TypeInfo *i = Info(type);
    if (!i) throw Error(fmt("gguf: unknown ggml type %u", type));
    if (n < 0 || n % i->elems != 0) throw Error(fmt("gguf: %lld elements is not a whole number of %s blocks of %d", static_cast<long long>(n), i->name, i->elems));
    return n / i->elems * i->nbytes;
}

int64_t Tensor::Elems() const {
    int64_t n = 1;
    for (int64_t d : Dims) n *= d;
    return n;
}
int64_t Tensor::Rows() const {
    int64_t n = 1;
    for (size_t i = 1; i < Dims.size(); i++) n *= Dims[i];
    return n;
}
int64_t Tensor::RowBytes() const {
    const TypeInfo *i = Info(Type);
    if (!i || Dims.empty() || Dims[0] % i->elems != 0) return 0;
    return Dims[0] / i->elems * i->nbytes;
}
void Tensor::AdviseRandom() const {
    if (!Bytes) return;
    const uintptr_t page = static_cast<uintptr_t>(::sysconf(_SC_PAGESIZE));
    const uintptr_t base = reinterpret_cast<uintptr_t>(Data);
    // whole pages only: the partial ones at either end belong to a neighbouring tensor (gguf/gguf.go:196-208)
    const uintptr_t lo = (base + page - 1) & ~(page - 1), hi = (base + Bytes) & ~(page - 1);
    if (hi <= lo) return;
    if (::madvise(reinterpret_cast<void *>(lo), hi - lo, MADV_RANDOM) != 0) throw Error(std::string("gguf: madvise: ") + std::strerror(errno));
}

uint64_t Value::Len() const {
    switch (kind) {
        case Uints: return us.size();
        case Ints: return is.size();
        case Floats: return fs.size();
        case Bools: return bs.size();
        case Strs: return ss.size();
        default: return 0;
    }
}

bool KV::Uint(const std::string &key, uint64_t *out) const {
    const Value *v = Find(key);
    if (v && v->kind == Value::Uint) return *out = v->u, true;
    if (v && v->kind == Value::Int && v->i >= 0) return *out = static_cast<uint64_t>(v->i), true;
    return false;
}
bool KV::Int(const std::string &key, int64_t *out) const {
    const Value *v = Find(key);
    if (v && v->kind == Value::Int) return *out = v->i, true;
    if (v && v->kind == Value::Uint) return *out = static_cast<int64_t>(v->u), true;
    return false;
}
bool KV::Float(const std::string &key, double *out) const {
    const Value *v = Find(key);
    if (v && v->kind == Value::Float) return *out = v->f, true;
    if (v && v->kind == Value::Uint) return *out = static_cast<double>(v->u), true;
    if (v && v->kind == Value::Int) return *out = static_cast<double>(v->i), true;
    return false;
}
bool KV::Str(const std::string &key, std::string *out) const {
    const Value *v = Find(key);
    if (v && v->kind == Value::Str) return *out = v->s, true;
    return false;
}
bool KV::Bool(const std::string &key, bool *out) const {
    const Value *v = Find(key);
    if (v && v->kind == Value::Bool) return *out = v->b, true;
    return false;
}
const std::vector<std::string> *KV::Strings(const std::string &key) const {
    const Value *v = Find(key);
    return v && v->kind == Value::Strs ? &v->ss : nullptr;
}
const std::vector<uint64_t> *KV::Uints(const std::string &key) const {
    const Value *v = Find(key);
    return v && v->kind == Value::Uints ? &v->us : nullptr;
}
const std::vector<int64_t> *KV::Ints(const std::string &key) const {
    const Value *v = Find(key);
    return v && v->kind == Value::Ints ? &v->is : nullptr;
}
const std::vector<double> *KV::Floats(const std::string &key) const {
    const Value *v = Find(key);
    return v && v->kind == Value::Floats ? &v->fs : nullptr;
}

// ---------------------------------------------------------------------------------- File -------

std::unique_ptr<File> File::Open(const std::string &path) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) throw Error("gguf: " + path + ": " + std::strerror(errno));
    struct stat st;
    if (::fstat(fd, &st) != 0) {
        ::close(fd);
        throw Error("gguf: " + path + ": " + std::strerror(errno));
    }
    if (st.st_size < 24) {
        ::close(fd);
        throw Error("gguf: " + path + " is too short to hold a header");
    }
    // the whole file, header included, so a tensor's Data is the mapping plus its absolute offset
    void *m = ::mmap(nullptr, static_cast<size_t>(st.st_size), PROT_READ, MAP_SHARED, fd, 0);
    ::close(fd);
    if (m == MAP_FAILED) throw Error("gguf: " + path + ": mmap: " + std::strerror(errno));
    std::unique_ptr<File> f(new File());
    f->Path = path;
    f->map_ = static_cast<const uint8_t *>(m);
    f->size_ = static_cast<size_t>(st.st_size);
    try {
        f->parse();
    } catch (const Error &e) {
        throw Error("gguf: " + path + ": " + e.what());
    }
    return f;
}

File::~File() {
    if (map_) ::munmap(const_cast<uint8_t *>(map_), size_);
}

void File::parse() {
    Reader r{map_, size_};
    if (std::memcmp(map_, "GGUF", 4) != 0) throw Error("not a GGUF file (bad magic)");
    r.o = 4;
    Version = r.le<uint32_t>();
    if (Version < 2 || Version > 3) throw Error(fmt("unsupported GGUF version %u", Version));
    const uint64_t n_tensor = r.le<uint64_t>(), n_kv = r.le<uint64_t>();
    for (uint64_t i = 0; i < n_kv; i++) {
        std::string k;
        try {
            k = r.str();
        } catch (const Error &e) {
            throw Error(fmt("metadata key %llu: %s", static_cast<unsigned long long>(i), e.what()));
        }
        try {
            const uint32_t vt = r.le<uint32_t>();
            Value v = r.value(vt);
            if (!kv_.count(k)) order_.push_back(k);
            kv_[k] = std::move(v);
        } catch (const Error &e) {
            throw Error("metadata \"" + k + "\": " + e.what());
        }
    }
    uint64_t a;
    if (Uint(kKeyAlignment, &a)) {
        if (a == 0 || (a & (a - 1)) != 0) throw Error(fmt("general.alignment %llu is not a power of two", static_cast<unsigned long long>(a)));
        Alignment = a;
    }
    // the table is read before the data section's start is known: the table is what ends the header
    struct Desc {
        std::string name;
        uint32_t type;
        std::vector<int64_t> dims;
        uint64_t offset;
    };
    if (n_tensor > size_) throw Error(fmt("%llu tensors exceed the file", static_cast<unsigned long long>(n_tensor)));
    std::vector<Desc> descs;
    descs.reserve(n_tensor);
    for (uint64_t i = 0; i < n_tensor; i++) {
        Desc d;
        try {
            d.name = r.str();
        } catch (const Error &e) {
            throw Error(fmt("tensor %llu: %s", static_cast<unsigned long long>(i), e.what()));
        }
        try {
            const uint32_t nd = r.le<uint32_t>();
            if (nd == 0 || nd > 4) throw Error(fmt("has %u dimensions, ggml allows 1-4", nd));
            for (uint32_t j = 0; j < nd; j++) d.dims.push_back(static_cast<int64_t>(r.le<uint64_t>()));
            d.type = r.le<uint32_t>();
            d.offset = r.le<uint64_t>();
        } catch (const Error &e) {
            throw Error("tensor \"" + d.name + "\": " + e.what());
        }
        descs.push_back(std::move(d));
    }
    DataStart = static_cast<int64_t>((r.o + Alignment - 1) & ~(Alignment - 1));
    Tensors.reserve(descs.size());
    for (Desc &d : descs) {
        Tensor t;
        t.Name = d.name;
        t.Type = d.type;
        t.Dims = d.dims;
        // a product that cannot be a size within this file is refused before it can wrap
        int64_t n = 1;
        for (int64_t x : d.dims) {
            if (x < 0 || (x != 0 && n > (int64_t{1} << 56) / x)) throw Error("tensor \"" + d.name + "\": its dimensions overflow");
            n *= x;
        }
        int64_t nbytes;
        try {
            nbytes = SizeOf(d.type, n);
        } catch (const Error &e) {
            throw Error("tensor \"" + d.name + "\": " + e.what());
        }
        const uint64_t lo = static_cast<uint64_t>(DataStart) + d.offset, hi = lo + static_cast<uint64_t>(nbytes);
        if (lo < static_cast<uint64_t>(DataStart) || hi < lo || hi > size_)
            throw Error(fmt("tensor \"%s\" spans [%llu,%llu), past the end of a %zu byte file", d.name.c_str(),
                            static_cast<unsigned long long>(lo), static_cast<unsigned long long>(hi), size_));
        t.Data = map_ + lo;
        t.Bytes = static_cast<uint64_t>(nbytes);
        if (by_name_.count(d.name)) throw Error("tensor \"" + d.name + "\" appears twice");
        by_name_[d.name] = Tensors.size();
        Tensors.push_back(std::move(t));
    }
}

const Value *File::Find(const std::string &key) const {
    auto it = kv_.find(key);
    return it == kv_.end() ? nullptr : &it->second;
}

const Tensor &File::Get(const std::string &name) const {
    auto it = by_name_.find(name);
    if (it == by_name_.end()) throw Error("gguf: " + Path + ": no tensor named \"" + name + "\"");
    return Tensors[it->second];
}

// ----------------------------------------------------------------------------------- Set -------

std::unique_ptr<Set> Set::Open(const std::string &path_in) {
    std::string path = path_in;
    struct stat st;
    if (::stat(path.c_str(), &st) != 0) throw Error("gguf: " + path + ": " + std::strerror(errno));
    if (S_ISDIR(st.st_mode)) path = sole_checkpoint(path);
    std::unique_ptr<Set> s(new Set());
    int shard = 0;
    for (const std::string &p : shard_paths(path)) {
        s->Files.push_back(File::Open(p));
        for (Tensor &t : s->Files.back()->Tensors) {
            if (s->by_name_.count(t.Name)) throw Error("gguf: tensor \"" + t.Name + "\" appears in more than one shard of " + path);
            t.Shard = shard;
            s->by_name_[t.Name] = &t;
            s->Tensors.push_back(&t);
        }
        shard++;
    }
    s->checkSplit();
    return s;
}

// The shards form one complete checkpoint (gguf/gguf.go:795-819): consecutive split.no, an agreed
// split.count and the promised tensor total.  A download that stopped after three of four shards
// still opens shard by shard; only these keys notice.
void Set::checkSplit() const {
    uint64_t v;
    if (Files.size() == 1) {
        if (Files[0]->Uint(kKeySplitCount, &v) && v > 1)
            throw Error(fmt("gguf: %s is shard 1 of %llu but no siblings were found", Files[0]->Path.c_str(), static_cast<unsigned long long>(v)));
        return;
    }
    for (size_t i = 0; i < Files.size(); i++) {
        const File &f = *Files[i];
        if (!f.Uint(kKeySplitNo, &v)) throw Error("gguf: " + f.Path + " has no split.no");
        if (v != i) throw Error(fmt("gguf: %s is split.no=%llu, expected %zu", f.Path.c_str(), static_cast<unsigned long long>(v), i));
        if (f.Uint(kKeySplitCount, &v) && v != Files.size())
            throw Error(fmt("gguf: %s says split.count=%llu but %zu shards were opened", f.Path.c_str(), static_cast<unsigned long long>(v), Files.size()));
    }
    if (Files[0]->Uint(kKeySplitTensors, &v) && v != Tensors.size())
        throw Error(fmt("gguf: %s says split.tensors.count=%llu but %zu tensors were read", Files[0]->Path.c_str(), static_cast<unsigned long long>(v), Tensors.size()));
}

const Tensor &Set::Get(const std::string &name) const {
    auto it = by_name_.find(name);
    if (it == by_name_.end()) throw Error("gguf: no tensor named \"" + name + "\"");
    return *it->second;
}
int64_t Set::Params() const {
    int64_t n = 0;
    for (const Tensor *t : Tensors) n += t->Elems();
    return n;
}
int64_t Set::Bytes() const {
    int64_t n = 0;
    for (const Tensor *t : Tensors) n += static_cast<int64_t>(t->Bytes);
    return n;
}
std::string Set::Arch() const {
    std::string a;
    Str(kKeyArchitecture, &a);
    return a;
}

// -------------------------------------------------------------------------------- Writer -------

namespace {
template <typename T>
void put(std::vector<uint8_t> &b, T v) {
    const uint8_t *p = reinterpret_cast<const uint8_t *>(&v);
    b.insert(b.end(), p, p + sizeof(T));
}
void put_str(std::vector<uint8_t> &b, const std::string &s) {
    put<uint64_t>(b, s.size());
    b.insert(b.end(), s.begin(), s.end());
}
}  // namespace

Writer::Writer(uint64_t alignment) : align_(alignment) {
    if (alignment == 0 || (alignment & (alignment - 1)) != 0) throw Error("gguf: the alignment must be a power of two");
    if (alignment != kDefaultAlignment) PutU32(kKeyAlignment, static_cast<uint32_t>(alignment));
}
void Writer::key(const std::string &k, uint32_t vt) {
    put_str(kv_, k);
    put<uint32_t>(kv_, vt);
    n_kv_++;
}
void Writer::PutU32(const std::string &k, uint32_t v) { key(k, vtU32); put(kv_, v); }
void Writer::PutI32(const std::string &k, int32_t v) { key(k, vtI32); put(kv_, v); }
void Writer::PutU64(const std::string &k, uint64_t v) { key(k, vtU64); put(kv_, v); }
void Writer::PutF32(const std::string &k, float v) { key(k, vtF32); put(kv_, v); }
void Writer::PutBool(const std::string &k, bool v) { key(k, vtBool); put<uint8_t>(kv_, v ? 1 : 0); }
void Writer::PutStr(const std::string &k, const std::string &v) { key(k, vtStr); put_str(kv_, v); }
void Writer::PutStrs(const std::string &k, const std::vector<std::string> &v) {
    key(k, vtArray);
    put<uint32_t>(kv_, vtStr);
    put<uint64_t>(kv_, v.size());
    for (const std::string &s : v) put_str(kv_, s);
}
void Writer::PutI32s(const std::string &k, const std::vector<int32_t> &v) {
    key(k, vtArray);
    put<uint32_t>(kv_, vtI32);
    put<uint64_t>(kv_, v.size());
    for (int32_t x : v) put(kv_, x);
}

void Writer::AddTensor(const std::string &name, uint32_t type, const std::vector<int64_t> &dims, std::function<void(uint8_t *, uint64_t)> fill) {
    if (dims.empty() || dims.size() > 4) throw Error("gguf: tensor \"" + name + "\": ggml allows 1-4 dimensions");
    int64_t n = 1;
    for (int64_t d : dims) n *= d;
    Entry e{name, type, dims, static_cast<uint64_t>(SizeOf(type, n)), 0, std::move(fill)};
    data_ = (data_ + align_ - 1) & ~(align_ - 1);
    e.offset = data_;
    data_ += e.bytes;
    tensors_.push_back(std::move(e));
}

void Writer::Write(const std::string &path) const {
    std::vector<uint8_t> head;
    head.insert(head.end(), {'G', 'G', 'U', 'F'});
    put<uint32_t>(head, 3);
    put<uint64_t>(head, tensors_.size());
    put<uint64_t>(head, n_kv_);
    head.insert(head.end(), kv_.begin(), kv_.end());
    for (const Entry &e : tensors_) {
        put_str(head, e.name);
        put<uint32_t>(head, static_cast<uint32_t>(e.dims.size()));
        for (int64_t d : e.dims) put<uint64_t>(head, static_cast<uint64_t>(d));
        put<uint32_t>(head, e.type);
        put<uint64_t>(head, e.offset);
    }
    head.resize((head.size() + align_ - 1) & ~(align_ - 1), 0);
    FILE *f = std::fopen(path.c_str(), "wb");
    if (!f) throw Error("gguf: " + path + ": " + std::strerror(errno));
    bool ok = std::fwrite(head.data(), 1, head.size(), f) == head.size();
    uint64_t at = 0;
    std::vector<uint8_t> buf;
    for (const Entry &e : tensors_) {
        if (!ok) break;
        buf.assign(e.offset - at, 0);  // padding up to this tensor's offset
        ok = std::fwrite(buf.data(), 1, buf.size(), f) == buf.size();
        buf.assign(e.bytes, 0);
        try {
            if (e.fill) e.fill(buf.data(), e.bytes);
        } catch (...) {
            std::fclose(f);
            throw;
        }
        ok = ok && std::fwrite(buf.data(), 1, buf.size(), f) == buf.size();
        at = e.offset + e.bytes;
    }
    ok = (std::fclose(f) == 0) && ok;
    if (!ok) throw Error("gguf: " + path + ": short write");
}

}  // namespace gguf
