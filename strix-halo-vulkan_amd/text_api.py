"""ctypes binding of the text layer in host/text.hpp (the shvtext_* entry points of host/shv_llm.h): the
checkpoint's byte-level BPE tokenizer and stop set (llm/tokenizer.go, zimage/tokenizer), the chat template and
Python-style JSON (llm/chat.go, llm/pyjson.go) and the streamed-completion reader (llm/chatdecode.go).  Nothing
here touches a device."""
import ctypes as C
import json

from . import llm_api

_bound = False


def _lib():
    global _bound
    L = llm_api.load()
    if _bound:
        return L
    vp, cp, u64, i32 = C.c_void_p, C.c_char_p, C.c_uint64, C.c_int32
    P = C.POINTER
    L.shvtext_free.argtypes = [vp]
    L.shvtext_free.restype = None
    L.shvtext_tokenizer_from_vocab.argtypes = [P(cp), P(u64), C.c_int, P(cp), P(u64), C.c_int, P(i32), P(cp), C.c_int, cp, P(vp)]
    L.shvtext_tokenizer_from_gguf.argtypes = [vp, P(vp), P(i32), C.c_int, P(C.c_int)]
    L.shvtext_tokenizer_free.argtypes = [vp]
    L.shvtext_tokenizer_free.restype = None
    L.shvtext_tokenizer_size.argtypes = [vp]
    L.shvtext_tokenizer_id.argtypes = [vp, cp, P(i32)]
    L.shvtext_encode.argtypes = [vp, cp, u64, P(P(i32)), P(C.c_int)]
    L.shvtext_decode.argtypes = [vp, P(i32), C.c_int, P(vp), P(u64)]
    L.shvtext_split.argtypes = [cp, u64, C.c_int, P(vp), P(u64), P(P(i32)), P(C.c_int)]
    L.shvtext_pyjson.argtypes = [cp, P(vp)]
    L.shvtext_parse_tool_arguments.argtypes = [cp, P(vp)]
    L.shvtext_render_chat.argtypes = [cp, P(vp)]
    L.shvtext_decoder_new.argtypes = [cp, C.c_int, P(vp)]
    L.shvtext_decoder_free.argtypes = [vp]
    L.shvtext_decoder_free.restype = None
    L.shvtext_decoder_stop_at.argtypes = [vp, P(cp), P(u64), C.c_int]
    L.shvtext_decoder_stopped.argtypes = [vp, P(u64)]
    L.shvtext_decoder_stopped.restype = vp
    L.shvtext_decoder_write.argtypes = [vp, cp, u64, P(vp), P(u64), P(vp), P(u64)]
    L.shvtext_decoder_close.argtypes = [vp, P(vp), P(u64), P(vp), P(u64), P(vp)]
    L.shvtext_stream_new.argtypes = [vp, P(i32), C.c_int, cp, C.c_int, P(vp)]
    L.shvtext_stream_free.argtypes = [vp]
    L.shvtext_stream_free.restype = None
    L.shvtext_stream_stop_at.argtypes = [vp, P(cp), P(u64), C.c_int]
    L.shvtext_stream_push.argtypes = [vp, i32, P(vp), P(u64), P(vp), P(u64), P(C.c_int)]
    L.shvtext_stream_stopped.argtypes = [vp, P(u64)]
    L.shvtext_stream_stopped.restype = vp
    L.shvtext_stream_close.argtypes = [vp, P(vp), P(u64), P(vp), P(u64), P(vp)]
    _bound = True
    return L


def _take(L, p, n=None):
    """The bytes of a string the library handed out, which is then freed."""
    if not p.value:
        return b""
    b = C.string_at(p.value, n.value) if n is not None else C.string_at(p.value)
    L.shvtext_free(p)
    return b


def _bytes(s):
    return s if isinstance(s, (bytes, bytearray)) else s.encode("utf-8", "surrogatepass")


def _strings(items):
    raw = [_bytes(s) for s in items]
    arr = (C.c_char_p * max(1, len(raw)))(*raw)
    lens = (C.c_uint64 * max(1, len(raw)))(*[len(r) for r in raw])
    return arr, lens, len(raw)


class Tokenizer:
    """tokenizer.Tokenizer: Encode / Decode / ID / Size."""

    def __init__(self, handle, eog=None):
        self.L, self.h, self.eog = _lib(), handle, eog

    @classmethod
    def from_vocab(cls, tokens, merges, types=None, specials=(), pre=""):
        L = _lib()
        ta, tl, nt = _strings(tokens)
        ma, ml, nm = _strings(merges)
        sa, _, ns = _strings(specials)
        ty = (C.c_int32 * nt)(*types) if types is not None else None
        h = C.c_void_p()
        llm_api._check(L.shvtext_tokenizer_from_vocab(ta, tl, nt, ma, ml, nm, ty, sa, ns, _bytes(pre), C.byref(h)))
        return cls(h)

    @classmethod
    def from_gguf(cls, gguf_file):
        """LoadTokenizer and EndOfGeneration over an open gguf_api.GGUF."""
        L = _lib()
        h, n = C.c_void_p(), C.c_int()
        ids = (C.c_int32 * 16)()
        llm_api._check(L.shvtext_tokenizer_from_gguf(gguf_file.h, C.byref(h), ids, 16, C.byref(n)))
        return cls(h, set(ids[:min(n.value, 16)]))

    def close(self):
        if self.h:
            self.L.shvtext_tokenizer_free(self.h)
            self.h = None

    def size(self):
        return self.L.shvtext_tokenizer_size(self.h)

    def id(self, token):
        v = C.c_int32()
        return v.value if self.L.shvtext_tokenizer_id(self.h, _bytes(token), C.byref(v)) else None

    def encode(self, text):
        b = _bytes(text)
        p, n = C.POINTER(C.c_int32)(), C.c_int()
        llm_api._check(self.L.shvtext_encode(self.h, b, len(b), C.byref(p), C.byref(n)))
        ids = [p[i] for i in range(n.value)]
        self.L.shvtext_free(C.cast(p, C.c_void_p))
        return ids

    def decode_bytes(self, ids):
        arr = (C.c_int32 * max(1, len(ids)))(*ids)
        p, n = C.c_void_p(), C.c_uint64()
        llm_api._check(self.L.shvtext_decode(self.h, arr, len(ids), C.byref(p), C.byref(n)))
        return _take(self.L, p, n)

    def decode(self, ids):
        return self.decode_bytes(ids).decode("utf-8", "replace")


def split(text, marks=False):
    """The pre-tokenizer's pieces, as bytes."""
    L = _lib()
    b = _bytes(text)
    out, n_out, lens, n = C.c_void_p(), C.c_uint64(), C.POINTER(C.c_int32)(), C.c_int()
    llm_api._check(L.shvtext_split(b, len(b), 1 if marks else 0, C.byref(out), C.byref(n_out), C.byref(lens), C.byref(n)))
    sizes = [lens[i] for i in range(n.value)]
    L.shvtext_free(C.cast(lens, C.c_void_p))
    allb = _take(L, out, n_out)
    pieces, at = [], 0
    for s in sizes:
        pieces.append(allb[at:at + s])
        at += s
    return pieces


def pyjson(raw):
    L = _lib()
    p = C.c_void_p()
    llm_api._check(L.shvtext_pyjson(_bytes(raw), C.byref(p)))
    return _take(L, p).decode("utf-8")


def parse_tool_arguments(s):
    """[(name, value JSON as it arrived)] in the object's order."""
    L = _lib()
    p = C.c_void_p()
    llm_api._check(L.shvtext_parse_tool_arguments(_bytes(s), C.byref(p)))
    raw = _take(L, p).decode("utf-8")
    # the values are embedded as they arrived: cut them out of the array by a decoder that reports positions
    dec, out, i = json.JSONDecoder(), [], 1
    while raw[i] != "]":
        if raw[i] == ",":
            i += 1
        assert raw.startswith('{"name":', i)
        name, j = dec.raw_decode(raw, i + len('{"name":'))
        assert raw.startswith(',"value":', j)
        _, k = dec.raw_decode(raw, j + len(',"value":'))
        out.append((name, raw[j + len(',"value":'):k]))
        i = k + 1
    return out


def render_chat(messages, tools=None, **opts):
    """RenderChat.  messages: dicts with role, content | parts, reasoning, tool_calls [{name, args: [{name, value}]}];
    opts: effort, no_thinking, drop_thinking, no_generation_prompt, add_vision_id."""
    L = _lib()
    req = {"messages": messages, "tools": tools or [], "opts": opts}
    p = C.c_void_p()
    llm_api._check(L.shvtext_render_chat(json.dumps(req, ensure_ascii=False).encode("utf-8"), C.byref(p)))
    return _take(L, p).decode("utf-8")


class ChatDecoder:
    """llm.ChatDecoder: write pieces, get (reasoning, content) back; close for the held-back tail and the calls."""

    def __init__(self, tools=None, thinking=False):
        self.L = _lib()
        self.h = C.c_void_p()
        tj = json.dumps(tools, ensure_ascii=False).encode("utf-8") if tools else None
        llm_api._check(self.L.shvtext_decoder_new(tj, 1 if thinking else 0, C.byref(self.h)))

    def __del__(self):
        if getattr(self, "h", None):
            self.L.shvtext_decoder_free(self.h)
            self.h = None

    def stop_at(self, seqs):
        arr, lens, n = _strings(seqs)
        llm_api._check(self.L.shvtext_decoder_stop_at(self.h, arr, lens, n))

    def stopped(self):
        n = C.c_uint64()
        p = self.L.shvtext_decoder_stopped(self.h, C.byref(n))
        return C.string_at(p, n.value).decode("utf-8")

    def write(self, piece):
        b = _bytes(piece)
        r, rn, c, cn = C.c_void_p(), C.c_uint64(), C.c_void_p(), C.c_uint64()
        llm_api._check(self.L.shvtext_decoder_write(self.h, b, len(b), C.byref(r), C.byref(rn), C.byref(c), C.byref(cn)))
        return _take(self.L, r, rn).decode("utf-8", "replace"), _take(self.L, c, cn).decode("utf-8", "replace")

    def close(self):
        r, rn, c, cn, j = C.c_void_p(), C.c_uint64(), C.c_void_p(), C.c_uint64(), C.c_void_p()
        llm_api._check(self.L.shvtext_decoder_close(self.h, C.byref(r), C.byref(rn), C.byref(c), C.byref(cn), C.byref(j)))
        calls = [(d["name"], d["arguments"]) for d in json.loads(_take(self.L, j).decode("utf-8"))]
        return _take(self.L, r, rn).decode("utf-8", "replace"), _take(self.L, c, cn).decode("utf-8", "replace"), calls


class ChatStream:
    """The emit loop's text side: push sampled ids, get (reasoning delta, content delta, finish) back; finish is 0 while
    running, 1 at an end-of-generation id, 2 at a stop sequence."""

    def __init__(self, tokenizer, eog=None, tools=None, thinking=False):
        self.L, self.tok = _lib(), tokenizer
        eog = sorted(tokenizer.eog or []) if eog is None else sorted(eog)
        arr = (C.c_int32 * max(1, len(eog)))(*eog)
        tj = json.dumps(tools, ensure_ascii=False).encode("utf-8") if tools else None
        self.h = C.c_void_p()
        llm_api._check(self.L.shvtext_stream_new(tokenizer.h, arr, len(eog), tj, 1 if thinking else 0, C.byref(self.h)))

    def __del__(self):
        if getattr(self, "h", None):
            self.L.shvtext_stream_free(self.h)
            self.h = None

    def stop_at(self, seqs):
        arr, lens, n = _strings(seqs)
        llm_api._check(self.L.shvtext_stream_stop_at(self.h, arr, lens, n))

    def push(self, token_id):
        r, rn, c, cn, fin = C.c_void_p(), C.c_uint64(), C.c_void_p(), C.c_uint64(), C.c_int()
        llm_api._check(self.L.shvtext_stream_push(self.h, int(token_id), C.byref(r), C.byref(rn), C.byref(c), C.byref(cn), C.byref(fin)))
        # a model may write bytes that are no character at all; those reach the caller as they would reach a JSON encoder
        return _take(self.L, r, rn).decode("utf-8", "replace"), _take(self.L, c, cn).decode("utf-8", "replace"), fin.value

    def stopped(self):
        n = C.c_uint64()
        p = self.L.shvtext_stream_stopped(self.h, C.byref(n))
        return C.string_at(p, n.value).decode("utf-8")

    def close(self):
        r, rn, c, cn, j = C.c_void_p(), C.c_uint64(), C.c_void_p(), C.c_uint64(), C.c_void_p()
        llm_api._check(self.L.shvtext_stream_close(self.h, C.byref(r), C.byref(rn), C.byref(c), C.byref(cn), C.byref(j)))
        calls = [(d["name"], d["arguments"]) for d in json.loads(_take(self.L, j).decode("utf-8"))]
        return _take(self.L, r, rn).decode("utf-8", "replace"), _take(self.L, c, cn).decode("utf-8", "replace"), calls
