#include "text.hpp"

#include <algorithm>
#include <cstdio>
#include <cstring>

#include "gguf.hpp"

namespace llm {
namespace text {

namespace {

#include "unicode_tables.inc"

constexpr uint32_t kRuneError = 0xFFFD;

template <size_t N>
bool in_ranges(const uint32_t (&t)[N][2], uint32_t c) {
    size_t lo = 0, hi = N;
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (c < t[mid][0]) hi = mid;
        else if (c > t[mid][1]) lo = mid + 1;
        else return true;
    }
    return false;
}
bool is_letter(uint32_t c) { return in_ranges(kUnicodeLetter, c); }
bool is_mark(uint32_t c) { return in_ranges(kUnicodeMark, c); }
bool is_number(uint32_t c) { return in_ranges(kUnicodeNumber, c); }
bool is_space(uint32_t c) { return in_ranges(kUnicodeSpace, c); }

// One code point from s at i, as Go's range over a string reads it: a byte that starts no valid sequence is
// U+FFFD and one byte long.
uint32_t next_rune(const std::string &s, size_t i, size_t *len) {
    const auto b = [&](size_t k) { return static_cast<uint8_t>(s[k]); };
    const uint8_t c = b(i);
    *len = 1;
    if (c < 0x80) return c;
    const size_t left = s.size() - i;
    const auto cont = [&](size_t k) { return (b(k) & 0xC0) == 0x80; };
    if (c >= 0xC2 && c <= 0xDF && left >= 2 && cont(i + 1)) {
        *len = 2;
        return ((c & 0x1Fu) << 6) | (b(i + 1) & 0x3Fu);
    }
    if (c >= 0xE0 && c <= 0xEF && left >= 3 && cont(i + 1) && cont(i + 2)) {
        const uint32_t r = ((c & 0x0Fu) << 12) | ((b(i + 1) & 0x3Fu) << 6) | (b(i + 2) & 0x3Fu);
        if (r >= 0x800 && !(r >= 0xD800 && r <= 0xDFFF)) {
            *len = 3;
            return r;
        }
    }
    if (c >= 0xF0 && c <= 0xF4 && left >= 4 && cont(i + 1) && cont(i + 2) && cont(i + 3)) {
        const uint32_t r = ((c & 0x07u) << 18) | ((b(i + 1) & 0x3Fu) << 12) | ((b(i + 2) & 0x3Fu) << 6) | (b(i + 3) & 0x3Fu);
        if (r >= 0x10000 && r <= 0x10FFFF) {
            *len = 4;
            return r;
        }
    }
    return kRuneError;
}

void put_rune(std::string &out, uint32_t r) {
    if (r > 0x10FFFF || (r >= 0xD800 && r <= 0xDFFF)) r = kRuneError;
    if (r < 0x80) out += static_cast<char>(r);
    else if (r < 0x800) {
        out += static_cast<char>(0xC0 | (r >> 6));
        out += static_cast<char>(0x80 | (r & 0x3F));
    } else if (r < 0x10000) {
        out += static_cast<char>(0xE0 | (r >> 12));
        out += static_cast<char>(0x80 | ((r >> 6) & 0x3F));
        out += static_cast<char>(0x80 | (r & 0x3F));
    } else {
        out += static_cast<char>(0xF0 | (r >> 18));
        out += static_cast<char>(0x80 | ((r >> 12) & 0x3F));
        out += static_cast<char>(0x80 | ((r >> 6) & 0x3F));
        out += static_cast<char>(0x80 | (r & 0x3F));
    }
}

std::vector<uint32_t> runes_of(const std::string &s) {
    std::vector<uint32_t> r;
    r.reserve(s.size());
    for (size_t i = 0; i < s.size();) {
        size_t n;
        r.push_back(next_rune(s, i, &n));
        i += n;
    }
    return r;
}

// strings.TrimSpace: Unicode white space off both ends
std::string trim_space(const std::string &s) {
    size_t first = std::string::npos, last_end = 0;  // the span from the first to the last code point that is no space
    for (size_t i = 0; i < s.size();) {
        size_t n;
        const uint32_t r = next_rune(s, i, &n);
        if (!is_space(r)) {
            if (first == std::string::npos) first = i;
            last_end = i + n;
        }
        i += n;
    }
    return first == std::string::npos ? std::string() : s.substr(first, last_end - first);
}
bool ascii_blank(char c) { return c == ' ' || c == '\t' || c == '\r' || c == '\n'; }
std::string trim_left_blank(const std::string &s) {
    size_t a = 0;
    while (a < s.size() && ascii_blank(s[a])) a++;
    return s.substr(a);
}
std::string trim_right_blank(const std::string &s) {
    size_t b = s.size();
    while (b > 0 && ascii_blank(s[b - 1])) b--;
    return s.substr(0, b);
}
bool has_prefix(const std::string &s, const std::string &p) { return s.size() >= p.size() && s.compare(0, p.size(), p) == 0; }
bool has_suffix(const std::string &s, const std::string &p) { return s.size() >= p.size() && s.compare(s.size() - p.size(), p.size(), p) == 0; }

// ------------------------------------------------------------------------------------ JSON ----
struct Parser {
    const std::string &s;
    size_t i = 0;
    explicit Parser(const std::string &src) : s(src) {}
    [[noreturn]] void fail(const std::string &what) const { throw Error("llm: invalid JSON at byte " + std::to_string(i) + ": " + what); }
    void ws() {
        while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r')) i++;
    }
    static int hex(char c) { return c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : -1; }
    bool u4(size_t at, uint32_t *v) const {
        if (at + 4 > s.size()) return false;
        uint32_t r = 0;
        for (int k = 0; k < 4; k++) {
            const int h = hex(s[at + k]);
            if (h < 0) return false;
            r = r * 16 + static_cast<uint32_t>(h);
        }
        *v = r;
        return true;
    }
    std::string string() {
        if (i >= s.size() || s[i] != '"') fail("a string was expected");
        i++;
        std::string out;
        for (;;) {
            if (i >= s.size()) fail("unterminated string");
            const uint8_t c = static_cast<uint8_t>(s[i]);
            if (c == '"') {
                i++;
                return out;
            }
            if (c < 0x20) fail("control character in a string");
            if (c == '\\') {
                if (i + 1 >= s.size()) fail("unterminated escape");
                const char e = s[i + 1];
                i += 2;
                switch (e) {
                    case '"': out += '"'; break;
                    case '\\': out += '\\'; break;
                    case '/': out += '/'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'n': out += '\n'; break;
                    case 'r': out += '\r'; break;
                    case 't': out += '\t'; break;
                    case 'u': {
                        uint32_t r;
                        if (!u4(i, &r)) fail("bad \\u escape");
                        i += 4;
                        if (r >= 0xD800 && r <= 0xDBFF) {  // a high surrogate: with the low one behind it, one code point
                            uint32_t lo;
                            if (i + 6 <= s.size() && s[i] == '\\' && s[i + 1] == 'u' && u4(i + 2, &lo) && lo >= 0xDC00 && lo <= 0xDFFF) {
                                i += 6;
                                r = 0x10000 + ((r - 0xD800) << 10) + (lo - 0xDC00);
                            } else r = kRuneError;
                        } else if (r >= 0xDC00 && r <= 0xDFFF) r = kRuneError;
                        put_rune(out, r);
                        break;
                    }
                    default: fail("unknown escape");
                }
                continue;
            }
            size_t n;
            const uint32_t r = next_rune(s, i, &n);
            if (r == kRuneError && n == 1) put_rune(out, kRuneError);  // a byte that is no UTF-8: the replacement character
            else out.append(s, i, n);
            i += n;
        }
    }
    std::string number() {
        const size_t a = i;
        if (i < s.size() && s[i] == '-') i++;
        if (i >= s.size()) fail("a number was expected");
        if (s[i] == '0') i++;
        else if (s[i] >= '1' && s[i] <= '9') {
            while (i < s.size() && s[i] >= '0' && s[i] <= '9') i++;
        } else fail("a number was expected");
        if (i < s.size() && s[i] == '.') {
            i++;
            if (i >= s.size() || s[i] < '0' || s[i] > '9') fail("digits after the point");
            while (i < s.size() && s[i] >= '0' && s[i] <= '9') i++;
        }
        if (i < s.size() && (s[i] == 'e' || s[i] == 'E')) {
            i++;
            if (i < s.size() && (s[i] == '+' || s[i] == '-')) i++;
            if (i >= s.size() || s[i] < '0' || s[i] > '9') fail("digits in the exponent");
            while (i < s.size() && s[i] >= '0' && s[i] <= '9') i++;
        }
        return s.substr(a, i - a);
    }
    JValue value(int depth) {
        if (depth > 512) fail("nested too deep");
        ws();
        if (i >= s.size()) fail("a value was expected");
        JValue v;
        const size_t a = i;
        const char c = s[i];
        if (c == '{') {
            v.kind = JValue::Object;
            i++;
            ws();
            if (i < s.size() && s[i] == '}') i++;
            else
                for (;;) {
                    ws();
                    std::string key = string();
                    ws();
                    if (i >= s.size() || s[i] != ':') fail("':' was expected");
                    i++;
                    v.members.emplace_back(std::move(key), value(depth + 1));
                    ws();
                    if (i < s.size() && s[i] == ',') {
                        i++;
                        continue;
                    }
                    if (i < s.size() && s[i] == '}') {
                        i++;
                        break;
                    }
                    fail("',' or '}' was expected");
                }
        } else if (c == '[') {
            v.kind = JValue::Array;
            i++;
            ws();
            if (i < s.size() && s[i] == ']') i++;
            else
                for (;;) {
                    v.items.push_back(value(depth + 1));
                    ws();
                    if (i < s.size() && s[i] == ',') {
                        i++;
                        continue;
                    }
                    if (i < s.size() && s[i] == ']') {
                        i++;
                        break;
                    }
                    fail("',' or ']' was expected");
                }
        } else if (c == '"') {
            v.kind = JValue::String;
            v.str = string();
        } else if (c == '-' || (c >= '0' && c <= '9')) {
            v.kind = JValue::Number;
            v.str = number();
        } else if (s.compare(i, 4, "true") == 0) {
            v.kind = JValue::Bool, v.b = true, i += 4;
        } else if (s.compare(i, 5, "false") == 0) {
            v.kind = JValue::Bool, v.b = false, i += 5;
        } else if (s.compare(i, 4, "null") == 0) {
            v.kind = JValue::Null, i += 4;
        } else fail("a value was expected");
        v.raw = s.substr(a, i - a);
        return v;
    }
};

void py_string(std::string &b, const std::string &s) {
    b += '"';
    for (size_t i = 0; i < s.size();) {
        size_t n;
        const uint32_t r = next_rune(s, i, &n);
        i += n;
        switch (r) {
            case '"': b += "\\\""; break;
            case '\\': b += "\\\\"; break;
            case '\b': b += "\\b"; break;
            case '\f': b += "\\f"; break;
            case '\n': b += "\\n"; break;
            case '\r': b += "\\r"; break;
            case '\t': b += "\\t"; break;
            default:
                if (r < 0x20) {
                    char buf[8];
                    std::snprintf(buf, sizeof buf, "\\u%04x", r);
                    b += buf;
                } else put_rune(b, r);
        }
    }
    b += '"';
}

void py_value(std::string &b, const JValue &v) {
    switch (v.kind) {
        case JValue::Object:
            b += '{';
            for (size_t i = 0; i < v.members.size(); i++) {
                if (i) b += ", ";
                py_string(b, v.members[i].first);
                b += ": ";
                py_value(b, v.members[i].second);
            }
            b += '}';
            break;
        case JValue::Array:
            b += '[';
            for (size_t i = 0; i < v.items.size(); i++) {
                if (i) b += ", ";
                py_value(b, v.items[i]);
            }
            b += ']';
            break;
        case JValue::String: py_string(b, v.str); break;
        case JValue::Number: b += v.str; break;
        case JValue::Bool: b += v.b ? "true" : "false"; break;
        case JValue::Null: b += "null"; break;
    }
}

}  // namespace

const JValue *JValue::Get(const std::string &key) const {
    for (const auto &m : members)
        if (m.first == key) return &m.second;
    return nullptr;
}

JValue ParseJSON(const std::string &s) {
    Parser p(s);
    JValue v = p.value(0);
    p.ws();
    if (p.i != s.size()) throw Error("llm: trailing content after a JSON value");
    return v;
}

bool ValidJSON(const std::string &s) {
    try {
        ParseJSON(s);
        return true;
    } catch (const Error &) {
        return false;
    }
}

std::string PyJSON(const std::string &raw) {
    std::string b;
    py_value(b, ParseJSON(raw));
    return b;
}

std::string GoJSONString(const std::string &s) {
    static const char *hexd = "0123456789abcdef";
    std::string b = "\"";
    for (size_t i = 0; i < s.size();) {
        const uint8_t c = static_cast<uint8_t>(s[i]);
        if (c < 0x80) {
            i++;
            switch (c) {
                case '\\': b += "\\\\"; break;
                case '"': b += "\\\""; break;
                case '\b': b += "\\b"; break;
                case '\f': b += "\\f"; break;
                case '\n': b += "\\n"; break;
                case '\r': b += "\\r"; break;
                case '\t': b += "\\t"; break;
                default:
                    if (c < 0x20 || c == '<' || c == '>' || c == '&') {
                        b += "\\u00";
                        b += hexd[c >> 4];
                        b += hexd[c & 15];
                    } else b += static_cast<char>(c);
            }
            continue;
        }
        size_t n;
        const uint32_t r = next_rune(s, i, &n);
        if (r == kRuneError && n == 1) b += "\\ufffd";
        else if (r == 0x2028) b += "\\u2028";
        else if (r == 0x2029) b += "\\u2029";
        else b.append(s, i, n);
        i += n;
    }
    b += '"';
    return b;
}

// ------------------------------------------------------------------------- pre-tokenizer ----
namespace {

using Runes = std::vector<uint32_t>;

size_t space_run(const Runes &r, size_t i) {
    while (i < r.size() && is_space(r[i])) i++;
    return i;
}

// 1: (?i:'s|'t|'re|'ve|'m|'ll|'d)
size_t match_contraction(const Runes &r, size_t i, bool) {
    if (r[i] != '\'') return 0;
    static const char *const suffixes[] = {"s", "t", "re", "ve", "m", "ll", "d"};
    for (const char *c : suffixes) {
        const size_t n = std::strlen(c);
        if (r.size() - i - 1 < n) continue;
        bool ok = true;
        for (size_t j = 0; j < n && ok; j++) {
            uint32_t ch = r[i + 1 + j];
            if (ch >= 'A' && ch <= 'Z') ch += 32;  // the only upper-case letters whose lower case is one of these
            ok = ch == static_cast<uint8_t>(c[j]);
        }
        if (ok) return 1 + n;
    }
    return 0;
}
// 2: [^\r\n\p{L}\p{N}]?\p{L}+ (qwen35: [\p{L}\p{M}]+)
size_t match_word(const Runes &r, size_t i, bool marks) {
    const uint32_t c = r[i];
    const size_t lead = (c != '\r' && c != '\n' && !is_letter(c) && !is_number(c)) ? 1 : 0;
    for (int attempt = 0; attempt < 2; attempt++) {
        const size_t skip = attempt == 0 ? lead : 0;
        size_t j = i + skip;
        while (j < r.size() && (is_letter(r[j]) || (marks && is_mark(r[j])))) j++;
        if (j > i + skip) return j - i;
        if (skip == 0) break;
    }
    return 0;
}
// 3: \p{N}
size_t match_number(const Runes &r, size_t i, bool) { return is_number(r[i]) ? 1 : 0; }
// 4:  ?[^\s\p{L}\p{N}]+[\r\n]* (qwen35: \p{M} out of the class too)
size_t match_symbols(const Runes &r, size_t i, bool marks) {
    const size_t space = r[i] == ' ' ? 1 : 0;
    for (int attempt = 0; attempt < 2; attempt++) {
        const size_t skip = attempt == 0 ? space : 0;
        size_t j = i + skip;
        while (j < r.size() && !is_space(r[j]) && !is_letter(r[j]) && !is_number(r[j]) && !(marks && is_mark(r[j]))) j++;
        if (j > i + skip) {
            while (j < r.size() && (r[j] == '\r' || r[j] == '\n')) j++;
            return j - i;
        }
        if (skip == 0) break;
    }
    return 0;
}
// 5: \s*[\r\n]+
size_t match_newlines(const Runes &r, size_t i, bool) {
    if (!is_space(r[i])) return 0;
    const size_t end = space_run(r, i);
    for (size_t j = end; j-- > i;)
        if (r[j] == '\r' || r[j] == '\n') return j + 1 - i;
    return 0;
}
// 6: \s+(?!\S)
size_t match_trailing_space(const Runes &r, size_t i, bool) {
    if (!is_space(r[i])) return 0;
    const size_t end = space_run(r, i);
    if (end == r.size()) return end - i;
    if (end - i >= 2) return end - i - 1;
    return 0;
}
// 7: \s+
size_t match_space(const Runes &r, size_t i, bool) { return is_space(r[i]) ? space_run(r, i) - i : 0; }

}  // namespace

std::vector<std::string> Split(const std::string &text, bool marks) {
    // the alternatives in the order the regex writes them: a backtracking engine takes the first that matches
    static size_t (*const alternatives[])(const Runes &, size_t, bool) = {match_contraction, match_word, match_number, match_symbols,
                                                                         match_newlines, match_trailing_space, match_space};
    const Runes r = runes_of(text);
    std::vector<std::string> out;
    for (size_t i = 0; i < r.size();) {
        size_t n = 0;
        for (auto alt : alternatives)
            if ((n = alt(r, i, marks)) > 0) break;
        if (n == 0) n = 1;
        std::string piece;
        for (size_t k = i; k < i + n; k++) put_rune(piece, r[k]);
        out.push_back(std::move(piece));
        i += n;
    }
    return out;
}

// ------------------------------------------------------------------------------ tokenizer ----
Tokenizer Tokenizer::FromVocab(const Vocab &v) {
    if (v.Tokens.empty()) throw Error("tokenizer: the vocabulary is empty");
    if (!v.Types.empty() && v.Types.size() != v.Tokens.size())
        throw Error("tokenizer: " + std::to_string(v.Types.size()) + " token types for " + std::to_string(v.Tokens.size()) + " tokens");
    Tokenizer t;
    if (v.Pre == "qwen2" || v.Pre.empty()) t.marks_ = false;
    else if (v.Pre == "qwen35") t.marks_ = true;
    else throw Error("tokenizer: pre-tokenizer \"" + v.Pre + "\" is not implemented (qwen2, qwen35)");
    t.tokens_ = v.Tokens;
    t.vocab_.reserve(v.Tokens.size());
    for (size_t id = 0; id < v.Tokens.size(); id++) t.vocab_.emplace(v.Tokens[id], static_cast<int32_t>(id));  // the first id of a duplicate wins
    t.ranks_.reserve(v.Merges.size());
    for (size_t i = 0; i < v.Merges.size(); i++) {
        const std::string &m = v.Merges[i];
        const size_t sp = m.find(' ');
        if (sp == std::string::npos || sp == 0 || sp == m.size() - 1 || m.find(' ', sp + 1) != std::string::npos)
            throw Error("tokenizer: merge " + std::to_string(i) + " is \"" + m + "\", want two space-separated halves");
        std::string key = m.substr(0, sp);
        key += '\0';
        key += m.substr(sp + 1);
        t.ranks_[key] = static_cast<int>(i);  // a repeated pair keeps its last index, as the map assignment does
    }
    std::set<std::string> special(v.Specials.begin(), v.Specials.end());
    for (size_t id = 0; id < v.Tokens.size(); id++) {
        if (!v.Types.empty() && (v.Types[id] == TokenControl || v.Types[id] == TokenUserDefined)) special.insert(v.Tokens[id]);
        if (special.count(v.Tokens[id])) t.special_id_[v.Tokens[id]] = static_cast<int32_t>(id);  // the last id of a duplicated special
    }
    for (const auto &kv : t.special_id_) t.specials_.push_back(kv.first);
    std::sort(t.specials_.begin(), t.specials_.end(), [](const std::string &a, const std::string &b) {
        if (a.size() != b.size()) return a.size() > b.size();
        return a < b;
    });
    // GPT-2's bytes_to_unicode: the printable bytes map to themselves, the other 68 to U+0100 upward
    uint32_t next = 256;
    for (int b = 0; b < 256; b++) {
        const bool printable = (b >= '!' && b <= '~') || (b >= 0xA1 && b <= 0xAC) || (b >= 0xAE && b <= 0xFF);
        t.byte_to_rune_[b] = printable ? static_cast<uint32_t>(b) : next++;
        t.rune_to_byte_[t.byte_to_rune_[b]] = static_cast<uint8_t>(b);
    }
    return t;
}

Tokenizer Tokenizer::FromGGUF(const gguf::KV &kv) {
    const auto *tokens = kv.Strings("tokenizer.ggml.tokens");
    if (!tokens) throw Error("llm: the checkpoint has no tokenizer.ggml.tokens");
    const auto *merges = kv.Strings("tokenizer.ggml.merges");
    if (!merges) throw Error("llm: the checkpoint has no tokenizer.ggml.merges");
    Vocab v;
    v.Tokens = *tokens;
    v.Merges = *merges;
    kv.Str("tokenizer.ggml.pre", &v.Pre);
    if (const auto *raw = kv.Ints("tokenizer.ggml.token_type")) {
        v.Types.assign(raw->begin(), raw->end());
    } else if (const auto *rawu = kv.Uints("tokenizer.ggml.token_type")) {
        v.Types.assign(rawu->begin(), rawu->end());
    }
    return FromVocab(v);
}

bool Tokenizer::ID(const std::string &token, int32_t *id) const {
    auto s = special_id_.find(token);
    if (s != special_id_.end()) {
        *id = s->second;
        return true;
    }
    auto v = vocab_.find(token);
    if (v == vocab_.end()) return false;
    *id = v->second;
    return true;
}

std::vector<int32_t> Tokenizer::Encode(const std::string &text) const {
    std::vector<int32_t> ids;
    size_t from = 0;
    while (from < text.size()) {
        // the earliest added token in what is left, the longest of those that start there
        size_t best = std::string::npos;
        const std::string *tok = nullptr;
        for (const std::string &s : specials_) {
            const size_t at = text.find(s, from);
            if (at == std::string::npos || (best != std::string::npos && at >= best)) continue;
            best = at, tok = &s;
        }
        if (!tok) {
            const auto more = encodeOrdinary(text.substr(from));
            ids.insert(ids.end(), more.begin(), more.end());
            return ids;
        }
        if (best > from) {
            const auto more = encodeOrdinary(text.substr(from, best - from));
            ids.insert(ids.end(), more.begin(), more.end());
        }
        ids.push_back(special_id_.at(*tok));
        from = best + tok->size();
    }
    return ids;
}

std::vector<int32_t> Tokenizer::encodeOrdinary(const std::string &text) const {
    std::vector<int32_t> ids;
    for (const std::string &piece : Split(text, marks_)) {
        std::string mapped;
        for (unsigned char c : piece) put_rune(mapped, byte_to_rune_[c]);
        for (const std::string &tok : bpe(mapped)) {
            auto it = vocab_.find(tok);
            if (it == vocab_.end()) throw Error("tokenizer: \"" + tok + "\" is not in the vocabulary");
            ids.push_back(it->second);
        }
    }
    return ids;
}

// Each round finds the lowest-rank adjacent pair anywhere in the word and merges every non-overlapping
// occurrence of it (zimage/tokenizer/tokenizer.go:369-401).
std::vector<std::string> Tokenizer::bpe(const std::string &word) const {
    std::vector<std::string> syms;
    for (size_t i = 0; i < word.size();) {
        size_t n;
        next_rune(word, i, &n);
        syms.push_back(word.substr(i, n));
        i += n;
    }
    std::string key;
    while (syms.size() > 1) {
        int best_rank = -1;
        size_t best_at = std::string::npos;
        for (size_t i = 0; i + 1 < syms.size(); i++) {
            key.assign(syms[i]);
            key += '\0';
            key += syms[i + 1];
            auto it = ranks_.find(key);
            if (it == ranks_.end() || (best_at != std::string::npos && it->second >= best_rank)) continue;
            best_rank = it->second, best_at = i;
        }
        if (best_at == std::string::npos) break;
        const std::string a = syms[best_at], b = syms[best_at + 1];
        std::vector<std::string> out;
        out.reserve(syms.size());
        for (size_t i = 0; i < syms.size();) {
            if (i + 1 < syms.size() && syms[i] == a && syms[i + 1] == b) {
                out.push_back(a + b);
                i += 2;
            } else out.push_back(syms[i++]);
        }
        syms.swap(out);
    }
    return syms;
}

std::string Tokenizer::Decode(const std::vector<int32_t> &ids) const {
    std::string out;
    for (int32_t id : ids) {
        if (id < 0 || static_cast<size_t>(id) >= tokens_.size() || tokens_[id].empty())
            throw Error("tokenizer: id " + std::to_string(id) + " is not in the vocabulary");
        const std::string &tok = tokens_[id];
        if (special_id_.count(tok)) {
            out += tok;
            continue;
        }
        for (size_t i = 0; i < tok.size();) {
            size_t n;
            const uint32_t r = next_rune(tok, i, &n);
            i += n;
            auto b = rune_to_byte_.find(r);
            if (b == rune_to_byte_.end()) throw Error("tokenizer: token \"" + tok + "\" holds a character that is not byte-level");
            out += static_cast<char>(b->second);
        }
    }
    return out;
}

std::set<int32_t> EndOfGeneration(const gguf::KV &kv, const Tokenizer &tok) {
    std::set<int32_t> eog;
    uint64_t v;
    for (const char *k : {"tokenizer.ggml.eos_token_id", "tokenizer.ggml.eot_token_id", "tokenizer.ggml.eom_token_id"})
        if (kv.Uint(k, &v)) eog.insert(static_cast<int32_t>(v));
    for (const char *name : {"<|endoftext|>", "<|im_end|>", "<|eot_id|>", "<|end|>"}) {
        int32_t id;
        if (tok.ID(name, &id)) eog.insert(id);
    }
    return eog;
}

// -------------------------------------------------------------------------- chat template ----
const char *const ImageMarkup = "<|vision_start|><|image_pad|><|vision_end|>";

namespace {

// The reasoning instructions, the tool block's preamble and its rules: the template's own text, which the
// model was trained against (llm/chat.go:150-179).
const char *const kXhighInstructions =
    "Reasoning effort is set to xhigh. Please think carefully through the task, "
    "validate key assumptions, consider plausible alternatives, and prioritize correctness, "
    "consistency, and clarity in the final answer.";
const char *const kLowInstructions =
    "Reasoning effort is set to low. Keep your thinking brief and focused, "
    "moving directly to the conclusion without unnecessary elaboration.";
const char *const kToolsPreamble = "# Tools\n\nYou have access to the following functions:\n\n<tools>";
const char *const kToolsRules =
    "\n\nIf you choose to call a function ONLY reply in the following format with NO suffix:\n\n"
    "<tool_call>\n<function=example_function_name>\n<parameter=example_parameter_1>\nvalue_1\n</parameter>\n"
    "<parameter=example_parameter_2>\nThis is the value for the second parameter\nthat can span\n"
    "multiple lines\n</parameter>\n</function>\n</tool_call>\n\n<IMPORTANT>\nReminder:\n"
    "- Function calls MUST follow the specified format: an inner <function=...></function> block "
    "must be nested within <tool_call></tool_call> XML tags\n"
    "- Required parameters MUST be specified\n"
    "- You may provide optional reasoning for your function call in natural language BEFORE the "
    "function call, but NOT after\n"
    "- If there is no function call available, answer the question like normal with your current "
    "knowledge and do not tell the user about function calls\n</IMPORTANT>";
const std::string kThinkClose = "</think>", kCallOpen = "<tool_call>", kCallClose = "</tool_call>";

// The template's render_content(message.content, do_vision_count, is_system_content), untrimmed.
std::string content_of(const ChatMessage &m, bool counting, int *seen, bool add_id, bool system) {
    if (!m.HasParts) return m.Content;
    std::string b;
    for (const ChatPart &p : m.Parts) {
        if (!p.Image) {
            b += p.Text;
            continue;
        }
        if (system) throw Error("llm: a system message cannot contain images");
        if (counting) ++*seen;
        if (add_id) b += "Picture " + std::to_string(*seen) + ": ";
        b += ImageMarkup;
    }
    return b;
}

std::string reasoning_instructions(const ChatOpts &opt) {
    if (opt.NoThinking) return "";
    std::string effort = opt.Effort.empty() ? "xhigh" : opt.Effort;
    if (effort == "high") effort = "xhigh";
    if (effort == "xhigh") return kXhighInstructions;
    if (effort == "low") return kLowInstructions;
    if (effort == "medium") return "";
    throw Error("llm: unexpected reasoning effort \"" + effort + "\"; supported are xhigh (default), medium and low");
}

// The last user turn that is a question rather than a tool result (llm/chat.go:354-370).
int last_query_index(const std::vector<ChatMessage> &msgs, bool add_id) {
    for (int i = static_cast<int>(msgs.size()) - 1; i >= 0; i--) {
        if (msgs[i].Role != "user") continue;
        int seen = 0;
        const std::string c = trim_space(content_of(msgs[i], false, &seen, add_id, false));
        if (has_prefix(c, "<tool_response>") && has_suffix(c, "</tool_response>")) continue;
        return i;
    }
    return static_cast<int>(msgs.size()) - 1;
}

// A JSON string unquoted, anything else as Python writes JSON.
std::string render_arg(const std::string &v) {
    if (v.empty()) return "";
    if (v[0] == '"') {
        const JValue j = ParseJSON(v);
        return j.str;
    }
    return PyJSON(v);
}

}  // namespace

std::string RenderChat(const std::vector<ChatMessage> &msgs, const ChatOpts &opt) {
    if (msgs.empty()) throw Error("llm: no messages provided");
    // the leading run of system and developer turns is merged into one
    size_t num_sys = 0;
    std::string system;
    for (size_t i = 0; i < msgs.size(); i++) {
        const ChatMessage &m = msgs[i];
        if (num_sys != i || (m.Role != "system" && m.Role != "developer")) break;
        int seen = 0;
        const std::string c = trim_space(content_of(m, false, &seen, opt.AddVisionID, true));
        if (!c.empty()) {
            if (!system.empty()) system += '\n';
            system += c;
        }
        num_sys++;
    }
    const std::string instructions = reasoning_instructions(opt);

    std::string b;
    if (!opt.Tools.empty()) {
        b += "<|im_start|>system\n";
        if (!instructions.empty()) b += instructions + "\n\n";
        b += kToolsPreamble;
        for (size_t i = 0; i < opt.Tools.size(); i++) {
            try {
                b += "\n" + PyJSON(opt.Tools[i]);
            } catch (const Error &e) {
                throw Error("llm: tool " + std::to_string(i) + ": " + e.what());
            }
        }
        b += "\n</tools>";
        b += kToolsRules;
        if (!system.empty()) b += "\n\n" + system;
        b += "<|im_end|>\n";
    } else if (!system.empty()) {
        b += "<|im_start|>system\n";
        if (!instructions.empty()) b += instructions + "\n\n";
        b += system + "<|im_end|>\n";
    } else if (!instructions.empty()) {
        b += "<|im_start|>system\n" + instructions + "<|im_end|>\n";
    }

    const int last_query = last_query_index(msgs, opt.AddVisionID);
    int images = 0;
    for (size_t i = 0; i < msgs.size(); i++) {
        if (i < num_sys) continue;
        const ChatMessage &m = msgs[i];
        const std::string content = trim_space(content_of(m, true, &images, opt.AddVisionID, false));
        if (m.Role == "system" || m.Role == "developer") {
            throw Error("llm: a system message must be at the beginning of the conversation");
        } else if (m.Role == "user") {
            b += "<|im_start|>user\n" + content + "<|im_end|>\n";
        } else if (m.Role == "assistant") {
            if (!opt.DropThinking || static_cast<int>(i) > last_query)
                b += "<|im_start|>assistant\n<think>\n" + trim_space(m.Reasoning) + "\n</think>\n\n" + content;
            else b += "<|im_start|>assistant\n" + content;
            for (size_t j = 0; j < m.ToolCalls.size(); j++) {
                const ChatToolCall &call = m.ToolCalls[j];
                if (call.Name.empty()) throw Error("llm: tool call " + std::to_string(j) + " is missing a function name");
                if (j > 0) b += "\n<tool_call>\n<function=" + call.Name + ">\n";
                else if (!content.empty()) b += "\n\n<tool_call>\n<function=" + call.Name + ">\n";
                else b += "<tool_call>\n<function=" + call.Name + ">\n";
                for (const ChatArg &a : call.Args) {
                    std::string v;
                    try {
                        v = render_arg(a.Value);
                    } catch (const Error &e) {
                        throw Error("llm: tool call \"" + call.Name + "\", argument \"" + a.Name + "\": " + e.what());
                    }
                    b += "<parameter=" + a.Name + ">\n" + v + "\n</parameter>\n";
                }
                b += "</function>\n</tool_call>";
            }
            b += "<|im_end|>\n";
        } else if (m.Role == "tool") {
            // a run of tool results is one user turn: opened at the first of them, closed at the last
            if (i > 0 && msgs[i - 1].Role != "tool") b += "<|im_start|>user";
            b += "\n<tool_response>\n" + content + "\n</tool_response>";
            if (i == msgs.size() - 1 || msgs[i + 1].Role != "tool") b += "<|im_end|>\n";
        } else {
            throw Error("llm: unexpected message role \"" + m.Role + "\"");
        }
    }
    if (!opt.NoGenerationPrompt) {
        b += "<|im_start|>assistant\n";
        b += opt.NoThinking ? "<think>\n\n</think>\n\n" : "<think>\n";
    }
    return b;
}

std::vector<ChatArg> ParseToolArguments(const std::string &in) {
    const std::string s = trim_space(in);
    std::vector<ChatArg> out;
    if (s.empty()) return out;
    Parser p(s);
    p.ws();
    if (p.i >= s.size() || s[p.i] != '{') {
        // the reference reads one token first: what is no JSON at all fails there, a value of another kind here
        Parser q(s);
        q.value(0);
        throw Error("llm: tool arguments are not a JSON object");
    }
    // the object alone: the reference's decoder stops at the closing brace and never looks past it
    const JValue v = p.value(0);
    for (const auto &m : v.members) out.push_back({m.first, m.second.raw});
    return out;
}

// --------------------------------------------------------------------- reading a completion ----
namespace {

// How many bytes at the end of s could still be the beginning of marker.
size_t partial_suffix(const std::string &s, const std::string &marker) {
    size_t n = marker.size() - 1;
    if (n > s.size()) n = s.size();
    for (; n > 0; n--)
        if (s.compare(s.size() - n, n, marker, 0, n) == 0) return n;
    return 0;
}
size_t trailing_space(const std::string &s) { return s.size() - trim_right_blank(s).size(); }

// A JSON Schema `type`: a string, or a list of them, which counts as a string only if every arm is one (or null).
std::string schema_type(const JValue *t) {
    if (!t) return "";
    if (t->kind == JValue::String) return t->str;
    if (t->kind != JValue::Array || t->items.empty()) return "";
    for (const JValue &a : t->items) {
        if (a.kind != JValue::String) return "";
        if (a.str != "string" && a.str != "null") return "";
    }
    return "string";
}

std::map<std::string, std::map<std::string, std::string>> tool_params(const std::vector<std::string> &tools) {
    std::map<std::string, std::map<std::string, std::string>> out;
    for (const std::string &raw : tools) {
        JValue t;
        try {
            t = ParseJSON(raw);
        } catch (const Error &) {
            continue;
        }
        if (t.kind != JValue::Object) continue;
        // OpenAI's {"type":"function","function":{...}} or the bare function object
        const JValue *fn = t.Get("function");
        const JValue *src = (fn && fn->kind == JValue::Object) ? fn : &t;
        const JValue *name = src->Get("name");
        if (!name || name->kind != JValue::String || name->str.empty()) continue;
        std::map<std::string, std::string> types;
        const JValue *params = src->Get("parameters");
        const JValue *props = params && params->kind == JValue::Object ? params->Get("properties") : nullptr;
        if (props && props->kind == JValue::Object)
            for (const auto &m : props->members) types[m.first] = m.second.kind == JValue::Object ? schema_type(m.second.Get("type")) : "";
        out[name->str] = types;
    }
    return out;
}

// One rendered parameter back to JSON: a string parameter is the text as it stands, anything else is taken as
// JSON where it is JSON (llm/chatdecode.go:361-375).
std::string arg_json(const std::string &value, const std::string &typ) {
    if (typ != "string") {
        const std::string trimmed = trim_space(value);
        if (!trimmed.empty() && ValidJSON(trimmed)) return trimmed;
    }
    return GoJSONString(value);
}

bool parse_one_call(const std::string &body, const std::map<std::string, std::map<std::string, std::string>> &params, ChatCall *out) {
    const std::string fopen = "<function=";
    const size_t open = body.find(fopen);
    if (open == std::string::npos) return false;
    std::string rest = body.substr(open + fopen.size());
    size_t gt = rest.find('>');
    if (gt == std::string::npos) return false;
    const std::string name = trim_space(rest.substr(0, gt));
    if (name.empty()) return false;
    rest = rest.substr(gt + 1);
    const size_t fclose = rest.find("</function>");
    if (fclose != std::string::npos) rest = rest.substr(0, fclose);
    static const std::map<std::string, std::string> none;
    auto pt = params.find(name);
    const auto &types = pt == params.end() ? none : pt->second;
    std::string args = "{";
    int n = 0;
    const std::string popen = "<parameter=", pclose = "</parameter>";
    for (;;) {
        const size_t p = rest.find(popen);
        if (p == std::string::npos) break;
        rest = rest.substr(p + popen.size());
        gt = rest.find('>');
        if (gt == std::string::npos) break;
        const std::string key = trim_space(rest.substr(0, gt));
        rest = rest.substr(gt + 1);
        const size_t shut = rest.find(pclose);
        if (shut == std::string::npos) break;
        // the template writes a line break after the opening tag and before the closing one: the format's, not the value's
        std::string value = rest.substr(0, shut);
        if (has_prefix(value, "\n")) value = value.substr(1);
        if (has_suffix(value, "\n")) value = value.substr(0, value.size() - 1);
        rest = rest.substr(shut + pclose.size());
        if (n++ > 0) args += ',';
        args += GoJSONString(key);
        args += ':';
        auto ty = types.find(key);
        args += arg_json(value, ty == types.end() ? "" : ty->second);
    }
    args += '}';
    out->Name = name;
    out->Arguments = args;
    return true;
}

std::vector<ChatCall> parse_tool_calls(std::string s, const std::map<std::string, std::map<std::string, std::string>> &params) {
    std::vector<ChatCall> out;
    for (;;) {
        const size_t i = s.find(kCallOpen);
        if (i == std::string::npos) return out;
        s = s.substr(i + kCallOpen.size());
        const size_t end = s.find(kCallClose);
        if (end == std::string::npos) return out;  // a call cut off by the token limit is dropped, not half reported
        const std::string body = s.substr(0, end);
        s = s.substr(end + kCallClose.size());
        ChatCall call;
        if (parse_one_call(body, params, &call)) out.push_back(call);
    }
}

}  // namespace

ChatDecoder::ChatDecoder(const std::vector<std::string> &tools, bool thinking) : params_(tool_params(tools)), state_(thinking ? Think : Content) {}

void ChatDecoder::StopAt(const std::vector<std::string> &seqs) {
    stop_.clear();
    for (const std::string &s : seqs)
        if (!s.empty()) stop_.push_back(s);
}

std::string ChatDecoder::answer(const std::string &s) {
    if (!lead_) return s;
    const std::string t = trim_left_blank(s);
    if (!t.empty()) {
        lead_ = false;
        return t;
    }
    return "";
}

void ChatDecoder::Write(const std::string &s, std::string *reasoning, std::string *content) {
    reasoning->clear();
    content->clear();
    pend_ += s;
    for (;;) {
        switch (state_) {
            case Think: {
                const size_t i = pend_.find(kThinkClose);
                if (i != std::string::npos) {
                    *reasoning += pend_.substr(0, i);
                    pend_ = pend_.substr(i + kThinkClose.size());
                    state_ = Content;
                    continue;
                }
                const size_t held = partial_suffix(pend_, kThinkClose);
                *reasoning += pend_.substr(0, pend_.size() - held);
                pend_ = pend_.substr(pend_.size() - held);
                return;
            }
            case Content: {
                // the blank line the template puts between </think> and the answer goes before anything is matched
                if (lead_) {
                    const std::string trimmed = trim_left_blank(pend_);
                    if (trimmed.empty()) {
                        pend_.clear();
                        return;
                    }
                    pend_ = trimmed;
                }
                // whichever marker comes first ends the answer
                size_t at = pend_.find(kCallOpen);
                std::string stop;
                for (const std::string &seq : stop_) {
                    const size_t i = pend_.find(seq);
                    if (i != std::string::npos && (at == std::string::npos || i < at)) at = i, stop = seq;
                }
                if (at != std::string::npos && !stop.empty()) {
                    *content += answer(pend_.substr(0, at));
                    pend_.clear();
                    stopped_ = stop;
                    state_ = StoppedState;
                    return;
                }
                if (at != std::string::npos) {
                    *content += answer(trim_right_blank(pend_.substr(0, at)));
                    call_ += pend_.substr(at);
                    pend_.clear();
                    state_ = Call;
                    return;
                }
                size_t held = std::max(partial_suffix(pend_, kCallOpen), trailing_space(pend_));
                for (const std::string &seq : stop_) held = std::max(held, partial_suffix(pend_, seq));
                *content += answer(pend_.substr(0, pend_.size() - held));
                pend_ = pend_.substr(pend_.size() - held);
                return;
            }
            case StoppedState:
                pend_.clear();
                return;
            case Call:
                call_ += pend_;
                pend_.clear();
                return;
        }
    }
}

void ChatDecoder::Close(std::string *reasoning, std::string *content, std::vector<ChatCall> *calls) {
    reasoning->clear();
    content->clear();
    calls->clear();
    if (state_ == Think) *reasoning = pend_;
    else if (state_ == Content) *content = answer(pend_);
    pend_.clear();
    if (!call_.empty()) *calls = parse_tool_calls(call_, params_);
}

// ------------------------------------------------------------------------------- streaming ----
namespace {

// utf8.FullRune: whether p begins with a whole encoding; one that is invalid counts as whole (it reads as one
// replacement character and a width of one).
bool full_rune(const std::string &p, size_t at) {
    const size_t n = p.size() - at;
    if (n == 0) return false;
    const uint8_t c = static_cast<uint8_t>(p[at]);
    size_t need = 1;
    uint8_t lo = 0x80, hi = 0xBF;
    if (c >= 0xC2 && c <= 0xDF) need = 2;
    else if (c >= 0xE0 && c <= 0xEF) {
        need = 3;
        if (c == 0xE0) lo = 0xA0;
        if (c == 0xED) hi = 0x9F;
    } else if (c >= 0xF0 && c <= 0xF4) {
        need = 4;
        if (c == 0xF0) lo = 0x90;
        if (c == 0xF4) hi = 0x8F;
    }
    if (n >= need) return true;
    if (n > 1) {
        const uint8_t b1 = static_cast<uint8_t>(p[at + 1]);
        if (b1 < lo || b1 > hi) return true;
    }
    if (n > 2) {
        const uint8_t b2 = static_cast<uint8_t>(p[at + 2]);
        if (b2 < 0x80 || b2 > 0xBF) return true;
    }
    return false;
}

}  // namespace

std::string Utf8Stream::Write(const std::string &piece) {
    tail_ += piece;
    size_t cut = tail_.size();
    // a character is at most four bytes, so only the last one can be partial: find where it starts
    for (size_t i = 1; i <= 4 && i <= tail_.size(); i++) {
        const size_t start = tail_.size() - i;
        if ((static_cast<uint8_t>(tail_[start]) & 0xC0) == 0x80) continue;
        if (!full_rune(tail_, start)) cut = start;
        break;
    }
    std::string out = tail_.substr(0, cut);
    tail_.erase(0, cut);
    return out;
}

ChatStream::Finish ChatStream::Push(int32_t id, std::string *reasoning, std::string *content) {
    reasoning->clear();
    content->clear();
    if (finish_ != Running) return finish_;
    if (eog_.count(id)) return finish_ = EndOfText;
    const std::string whole = text_.Write(tok_->Piece(id));
    if (!whole.empty()) dec_.Write(whole, reasoning, content);
    if (!dec_.Stopped().empty()) finish_ = StopSequence;
    return finish_;
}

}  // namespace text
}  // namespace llm
