// The text on either side of the token loop: the checkpoint's byte-level BPE tokenizer and its stop set
// (llm/tokenizer.go, zimage/tokenizer/{tokenizer,split,vocab}.go), the chat template as the reference
// transcribed it (llm/chat.go, llm/pyjson.go) and the reader that splits a streamed completion into
// reasoning, answer and tool calls (llm/chatdecode.go).  Host code, as in the reference: nothing here touches
// the GPU.
#pragma once

#include <cstdint>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace gguf {
class KV;
}

namespace llm {
namespace text {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// ---- JSON as the template needs it: member order and number literals kept as they arrived ----
struct JValue {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    bool b = false;
    std::string str;  // String: the decoded text; Number: the literal as written
    std::vector<JValue> items;
    std::vector<std::pair<std::string, JValue>> members;
    std::string raw;  // the value's own bytes in the input (encoding/json's RawMessage)
    const JValue *Get(const std::string &key) const;  // first member of that name, or nullptr
};
JValue ParseJSON(const std::string &s);   // one value, nothing but white space after it; throws Error
bool ValidJSON(const std::string &s);     // json.Valid
std::string PyJSON(const std::string &raw);       // Python's json.dumps(x, ensure_ascii=False) of the value (llm/pyjson.go:31-43)
std::string GoJSONString(const std::string &s);   // encoding/json's Marshal of a string (HTML-safe escapes and all)

// ---- tokenizer (zimage/tokenizer) ----
enum TokenType { TokenUndefined = 0, TokenNormal = 1, TokenUnknown = 2, TokenControl = 3, TokenUserDefined = 4, TokenUnused = 5, TokenByte = 6 };

struct Vocab {
    std::vector<std::string> Tokens;    // by id, over the byte-level alphabet
    std::vector<std::string> Merges;    // "left right", lowest index merges first
    std::vector<int32_t> Types;         // one TokenType an id, or empty
    std::vector<std::string> Specials;  // tokens to match whole besides those Types marks
    std::string Pre;                    // tokenizer.ggml.pre: "qwen2", "" or "qwen35"
};

// The pre-tokenizer's pieces (zimage/tokenizer/split.go:35-54); marks: the qwen35 classes.
std::vector<std::string> Split(const std::string &text, bool marks);

class Tokenizer {
  public:
    static Tokenizer FromVocab(const Vocab &v);                 // zimage/tokenizer/vocab.go:62-136
    static Tokenizer FromGGUF(const gguf::KV &kv);              // LoadTokenizer, llm/tokenizer.go:22-40
    int Size() const { return static_cast<int>(tokens_.size()); }
    bool ID(const std::string &token, int32_t *id) const;
    std::vector<int32_t> Encode(const std::string &text) const;  // added tokens written out in the text are one id each
    std::string Decode(const std::vector<int32_t> &ids) const;
    std::string Piece(int32_t id) const { return Decode({id}); }  // one token's bytes (may end inside a UTF-8 sequence)
    bool Marks() const { return marks_; }

  private:
    std::vector<int32_t> encodeOrdinary(const std::string &text) const;
    std::vector<std::string> bpe(const std::string &word) const;
    std::unordered_map<std::string, int32_t> vocab_;
    std::vector<std::string> tokens_;
    std::unordered_map<std::string, int> ranks_;  // "a\0b" -> priority
    std::vector<std::string> specials_;           // longest first, then by name
    std::unordered_map<std::string, int32_t> special_id_;
    uint32_t byte_to_rune_[256];
    std::unordered_map<uint32_t, uint8_t> rune_to_byte_;
    bool marks_ = false;
};

// The tokens that end a generation (llm/tokenizer.go:52-68): the metadata's eos / eot / eom ids and, by name,
// <|endoftext|>, <|im_end|>, <|eot_id|>, <|end|> wherever the vocabulary has them.
std::set<int32_t> EndOfGeneration(const gguf::KV &kv, const Tokenizer &tok);

// ---- chat template (llm/chat.go) ----
struct ChatPart {
    std::string Text;
    bool Image = false;
};
struct ChatArg {
    std::string Name;
    std::string Value;  // the JSON that arrived
};
struct ChatToolCall {
    std::string Name;
    std::vector<ChatArg> Args;
};
struct ChatMessage {
    std::string Role, Content;
    std::vector<ChatPart> Parts;
    bool HasParts = false;  // Parts, not Content, is the turn (Go: Parts != nil)
    std::string Reasoning;
    std::vector<ChatToolCall> ToolCalls;
};
struct ChatOpts {
    std::vector<std::string> Tools;  // each entry of the request's tools array, as JSON
    std::string Effort;
    bool NoThinking = false, DropThinking = false, NoGenerationPrompt = false, AddVisionID = false;
};
extern const char *const ImageMarkup;
std::string RenderChat(const std::vector<ChatMessage> &msgs, const ChatOpts &opt);  // throws Error where the template raises
std::vector<ChatArg> ParseToolArguments(const std::string &s);                      // llm/chat.go:399-434

// ---- reading a completion back (llm/chatdecode.go) ----
struct ChatCall {
    std::string Name, Arguments;
};
class ChatDecoder {
  public:
    ChatDecoder(const std::vector<std::string> &tools, bool thinking);
    void StopAt(const std::vector<std::string> &seqs);
    const std::string &Stopped() const { return stopped_; }
    void Write(const std::string &s, std::string *reasoning, std::string *content);
    void Close(std::string *reasoning, std::string *content, std::vector<ChatCall> *calls);

  private:
    std::string answer(const std::string &s);
    enum State { Think, Content, Call, StoppedState };
    std::map<std::string, std::map<std::string, std::string>> params_;
    State state_;
    std::string pend_, call_;
    bool lead_ = true;
    std::vector<std::string> stop_;
    std::string stopped_;
};

// The tokens are bytes: a character's bytes come in several tokens routinely.  Write returns the part of the stream
// that is whole characters by now and keeps at most three bytes back (utf8Stream, backend/llm.go:1003-1032).
class Utf8Stream {
  public:
    std::string Write(const std::string &piece);

  private:
    std::string tail_;
};

// The text side of the emit loop (backend/llm.go:561-590): a sampled id becomes its bytes, whole characters go to the
// completion reader, and what that releases is this token's delta.
class ChatStream {
  public:
    enum Finish { Running = 0, EndOfText = 1, StopSequence = 2 };
    ChatStream(const Tokenizer *tok, std::set<int32_t> eog, const std::vector<std::string> &tools, bool thinking)
        : tok_(tok), eog_(std::move(eog)), dec_(tools, thinking) {}
    void StopAt(const std::vector<std::string> &seqs) { dec_.StopAt(seqs); }
    // An end-of-generation id or a stop sequence finishes the stream; ids pushed after that change nothing.
    Finish Push(int32_t id, std::string *reasoning, std::string *content);
    const std::string &Stopped() const { return dec_.Stopped(); }
    void Close(std::string *reasoning, std::string *content, std::vector<ChatCall> *calls) { dec_.Close(reasoning, content, calls); }

  private:
    const Tokenizer *tok_;
    std::set<int32_t> eog_;
    ChatDecoder dec_;
    Utf8Stream text_;
    Finish finish_ = Running;
};

}  // namespace text
}  // namespace llm
