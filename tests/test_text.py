"""The text layer (host/text.hpp behind the shvtext_* C entry points): tokenizer, stop set, chat template,
Python-style JSON, the streamed-completion reader.  CPU only.

What pins what.  The reference's own tokenizer and chat-template tests read dumps that are not in its tree
(reference/out/tokenizer/cases.json, reference/out/chat/cases.json are made from checkpoints), so:
  * the pre-tokenizer is held to the regexes it hand-rolls (zimage/tokenizer/tokenizer.go:222-225), run by the `regex`
    module, which has the lookahead Go's engine lacks;
  * Encode is held to the Hugging Face `tokenizers` library on a byte-level BPE trained here, with the same Split
    regex in front: an independent implementation of the same published algorithm;
  * pyJSON, ParseToolArguments and the completion reader are held to the literal cases of llm/chat_test.go and
    llm/chatdecode_test.go, which need no dump;
  * RenderChat's refusals are the reference's (llm/chat_test.go:137-160); its renderings have no golden text to be held
    to here (the template lives in the checkpoint's metadata): PARITY UNPINNED for those, which are checked for the
    structure llm/chat.go states and against Python's json.dumps for the tool block."""
import json
import random

import pytest

import gguf_file as GF
import shv

T = shv.pkg.text_api
G = shv.pkg.gguf_api

QWEN2 = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"
QWEN35 = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?[\p{L}\p{M}]+|\p{N}| ?[^\s\p{L}\p{M}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"

CORPUS = [
    "Hello, world!", "a cat", " leading space", "trailing space ", "two  spaces", "tabs\tand\nnewlines\r\n\r\nmixed  \n  x",
    "I'm sure they're here; we've said it's John's, he'll say he'd. DON'T SHOUT, I'LL", "'quoted' 'tis 'sblood",
    "2024-01-15 12:30 3.14159 ١٢٣ ４５ ⅷ ²", "naïve café résumé Ünïcödé", "é ä́ combining", "日本語のテキスト 中文 한국어",
    "emoji 😀👍🏽 family 👨‍👩‍👧", "math ∑∫√ ≤≥ →← {}[]() <>", "#include <stdio.h>\nint main() { return 0; }\n",
    "snake_case camelCase kebab-case", "   ", "\n", "", "x", " ", "a b c　d", "line1\n\n\nline2\n   \n", "end\n",
    "!!!???...", "$100 50% #tag @user", "Привет мир", "مرحبا بالعالم", "שלום עולם", "ไทย ภาษา", "ελληνικά",
    "<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n", "text<|endoftext|>more<|im_end|>", "<|im_start|><|im_start|>",
    "half <|im_sta and rt|>", "tab\t\t\tx", "a\r\nb\rc", "'S 'T 'RE 'Ve 'lL", "don't'll've", "١'s", "_'s_", " sep ",
]


def _random_texts(n, seed):
    rng = random.Random(seed)
    pool = list("abcdefXYZ 0123456789\t\n\r'.,!?-_()<>|") + ["é", "ß", "Ж", "中", "日", "́", "̈", "٣", "²", " ", " ", "😀",
                                                                "'s", "'re", " ", "  ", "\n\n", "<|im_end|>", "'", "''"]
    return ["".join(rng.choice(pool) for _ in range(rng.randint(1, 40))) for _ in range(n)]


def _random_code_points(n, seed):
    """Strings over the whole code space, every general category drawn equally often (a third ASCII): what decides
    a piece is the class of each character, and the classes' tables are ranges over all planes."""
    import unicodedata
    rng = random.Random(seed)
    cats = {}
    for cp in range(0x110000):
        if not 0xD800 <= cp <= 0xDFFF:
            cats.setdefault(unicodedata.category(chr(cp)), []).append(cp)
    names = sorted(cats)

    def one():
        if rng.random() < 0.35:
            return rng.choice("abcXYZ 019\t\n\r'.,-sStTrReEvVmMlLdD")
        return chr(rng.choice(cats[rng.choice(names)]))
    return ["".join(one() for _ in range(rng.randint(1, 24))) for _ in range(n)]


@pytest.mark.parametrize("marks,pattern", [(False, QWEN2), (True, QWEN35)], ids=["qwen2", "qwen35"])
def test_the_pre_tokenizer_is_the_regex_it_hand_rolls(marks, pattern):
    regex = pytest.importorskip("regex")
    rx = regex.compile(pattern)
    for text in CORPUS + _random_texts(600, 5 + marks) + _random_code_points(3000, 11 + marks):
        want = [m.group(0).encode("utf-8") for m in rx.finditer(text)]
        got = T.split(text, marks)
        assert got == want, (text, got, want)
        assert b"".join(got) == text.encode("utf-8")   # the pieces tile the input


def test_a_mark_joins_the_letters_before_it_only_under_qwen35():
    """zimage/tokenizer/split.go:30-31: "e" + U+0301 is one piece under qwen35 and two under qwen2."""
    assert T.split("é", True) == ["é".encode()]
    assert T.split("é", False) == [b"e", "́".encode()]


def test_bytes_that_are_no_utf8_become_the_replacement_character():
    """Go's []rune(text) reads a byte that starts no sequence as U+FFFD, and string() writes that back."""
    assert b"".join(T.split(b"ab\xff\xfecd", False)) == "ab��cd".encode()
    assert b"".join(T.split(b"\xe4\xb8", False)) == "��".encode()          # a sequence cut short
    assert b"".join(T.split(b"\xed\xa0\x80", False)) == "���".encode()  # a surrogate half is no code point


@pytest.fixture(scope="module")
def trained():
    """A byte-level BPE trained by the `tokenizers` library with qwen2's Split in front, and the same vocabulary and
    merge table handed to FromVocab as a GGUF would state them."""
    tk = pytest.importorskip("tokenizers")
    from tokenizers import Regex, Tokenizer, decoders, models, pre_tokenizers, trainers
    specials = ["<|endoftext|>", "<|im_start|>", "<|im_end|>", "<|im_start|>x"]   # one a prefix of another
    hf = Tokenizer(models.BPE())
    hf.pre_tokenizer = pre_tokenizers.Sequence([pre_tokenizers.Split(Regex(QWEN2), behavior="isolated"),
                                                pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    hf.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=900, initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), special_tokens=specials,
                                  show_progress=False)
    training = [t for t in CORPUS if "<|" not in t] * 3 + _random_texts(300, 99) + [
        "the quick brown fox jumps over the lazy dog " * 4, "she sells sea shells by the sea shore " * 4,
        "to be or not to be that is the question " * 4, "1234567890 " * 5, "    indented code\n        more indented\n" * 3]
    hf.train_from_iterator([t for t in training if "<|" not in t], trainer)
    model = json.loads(hf.to_str())["model"]
    vocab = hf.get_vocab(with_added_tokens=True)
    tokens = [None] * len(vocab)
    for tok, i in vocab.items():
        tokens[i] = tok
    merges = [m if isinstance(m, str) else " ".join(m) for m in model["merges"]]
    types = [3 if t in specials else 1 for t in tokens]
    mine = T.Tokenizer.from_vocab(tokens, merges, types, pre="qwen2")
    yield hf, mine, tokens, merges, types, specials
    mine.close()


def test_encode_is_what_the_tokenizers_library_encodes(trained):
    hf, mine, tokens, merges, _, _ = trained
    assert len(merges) > 300 and mine.size() == len(tokens)
    longer = 0
    for text in CORPUS + _random_texts(500, 7):
        want = hf.encode(text, add_special_tokens=False).ids
        got = mine.encode(text)
        assert got == want, (text, got, want)
        longer += len(got) < len(text.encode())
        assert mine.decode_bytes(got) == text.encode("utf-8")   # the byte-level alphabet makes the round trip exact
    assert longer > 100   # merges happened: the comparison is not one of single bytes


def test_added_tokens_in_the_text_are_one_id_each_and_the_longest_wins(trained):
    _, mine, tokens, _, _, _ = trained
    start, end, startx = mine.id("<|im_start|>"), mine.id("<|im_end|>"), mine.id("<|im_start|>x")
    assert None not in (start, end, startx)
    ids = mine.encode("<|im_start|>user\na cat<|im_end|>\n")
    assert ids[0] == start and ids.count(end) == 1
    assert mine.encode("<|im_start|>x")[0] == startx          # not <|im_start|> followed by "x"
    assert mine.encode("<|im_start|>y")[0] == start
    assert mine.decode(ids) == "<|im_start|>user\na cat<|im_end|>\n"
    assert mine.id("no such token") is None


def test_breaking_the_tokenizer_is_noticed(trained):
    """The reference's negative control (zimage/tokenizer/tokenizer_test.go:203-245): each break is a plausible mistake,
    and the corpus has to catch it."""
    hf, _, tokens, merges, types, _ = trained
    texts = [t for t in CORPUS if t]
    want = [hf.encode(t, add_special_tokens=False).ids for t in texts]
    breaks = {"no merges": (tokens, [], types, "qwen2"), "merge order reversed": (tokens, merges[::-1], types, "qwen2"),
              "special tokens ignored": (tokens, merges, None, "qwen2")}
    for name, (tk, mg, ty, pre) in breaks.items():
        broken = T.Tokenizer.from_vocab(tk, mg, ty, pre=pre)
        caught = 0
        for t, w in zip(texts, want):
            try:
                caught += broken.encode(t) != w
            except shv.pkg.ShvError:
                caught += 1
        broken.close()
        assert caught > 0, name


def test_from_vocab_refuses_what_the_reference_refuses():
    """zimage/tokenizer/vocab.go:62-104."""
    E = shv.pkg.ShvError
    with pytest.raises(E, match="vocabulary is empty"):
        T.Tokenizer.from_vocab([], [])
    with pytest.raises(E, match='pre-tokenizer "llama3" is not implemented'):
        T.Tokenizer.from_vocab(["a"], [], pre="llama3")
    for bad in ("ab", " ab", "ab ", "a b c"):
        with pytest.raises(E, match="want two space-separated halves"):
            T.Tokenizer.from_vocab(["a", "b"], [bad])
    t = T.Tokenizer.from_vocab(["a", "b", "a"], ["a b"])      # the first id of a duplicate wins
    assert t.id("a") == 0
    with pytest.raises(E, match="is not in the vocabulary"):
        t.encode("ab")                                         # the merge makes "ab", which has no id
    with pytest.raises(E, match="id 7 is not in the vocabulary"):
        t.decode([7])
    t.close()


def test_tokenizer_and_stop_set_out_of_a_checkpoints_metadata(trained, tmp_path):
    """LoadTokenizer and EndOfGeneration (llm/tokenizer.go:22-68): the stop set is the metadata's eos / eot / eom ids AND
    the tokens llama.cpp flags by name wherever the vocabulary has them."""
    hf, _, tokens, merges, types, _ = trained
    w = GF.Writer()
    w.put("general.architecture", GF.STR, "qwen3next")
    w.put_array("tokenizer.ggml.tokens", GF.STR, tokens)
    w.put_array("tokenizer.ggml.merges", GF.STR, merges)
    w.put_array("tokenizer.ggml.token_type", GF.I32, types)
    w.put("tokenizer.ggml.pre", GF.STR, "qwen2")
    w.put("tokenizer.ggml.eos_token_id", GF.U32, 5)
    w.put("tokenizer.ggml.eot_token_id", GF.U32, 6)
    path = tmp_path / "tok.gguf"
    w.write(path)
    f = G.GGUF(path, single=True)
    tok = T.Tokenizer.from_gguf(f)
    assert tok.eog == {5, 6, tok.id("<|endoftext|>"), tok.id("<|im_end|>")}
    text = "the quick brown fox<|im_end|>"
    assert tok.encode(text) == hf.encode(text, add_special_tokens=False).ids
    tok.close()
    f.close()
    # a checkpoint without a merge table is refused
    w2 = GF.Writer()
    w2.put_array("tokenizer.ggml.tokens", GF.STR, tokens)
    w2.write(tmp_path / "nomerges.gguf")
    f2 = G.GGUF(tmp_path / "nomerges.gguf", single=True)
    with pytest.raises(shv.pkg.ShvError, match="no tokenizer.ggml.merges"):
        T.Tokenizer.from_gguf(f2)
    f2.close()


# ---- Python's json.dumps, the template's tojson (llm/pyjson.go; cases of llm/chat_test.go:196-210) ----
PYJSON_CASES = [
    ('{"a":1,"b":[1,2],"c":{"d":true}}', '{"a": 1, "b": [1, 2], "c": {"d": true}}'),
    ('{"a":"<b> & </b>"}', '{"a": "<b> & </b>"}'),
    ('{"a":"café °C"}', '{"a": "café °C"}'),
    ('{"a":"tab\\there\\nand"}', '{"a": "tab\\there\\nand"}'),
    ('{"a":1.50,"b":1e3,"c":null}', '{"a": 1.50, "b": 1e3, "c": null}'),
    ('[]', '[]'),
    ('{}', '{}'),
]


def test_pyjson_literal_cases_of_the_reference():
    for raw, want in PYJSON_CASES:
        assert T.pyjson(raw) == want


def test_pyjson_is_pythons_own_dumps():
    """Held to the function it restates: json.dumps(x, ensure_ascii=False) over values whose number literals Python
    writes back as they came."""
    values = [{"type": "function", "function": {"name": "get_weather", "description": "Get the weather in a city, in °C",
                                                 "parameters": {"type": "object", "properties": {"city": {"type": "string", "description": "e.g. Wimbledon"},
                                                                                                 "days": {"type": "integer"}, "units": {"type": ["string", "null"]}},
                                                                "required": ["city"]}}},
              {"q": 'Search the web for "documents" & things', "ctl": "\u0001\u001f\b\f", "sep": "  ", "emoji": "😀", "nest": [[], {}, [None, True, False, -3, 7]]},
              "plain", 12, None, [1, [2, [3, [4]]]], {"z": 1, "a": 2, "m": 3}]
    for v in values:
        for compact in (json.dumps(v), json.dumps(v, ensure_ascii=False, separators=(",", ":")), json.dumps(v, indent=2)):
            assert T.pyjson(compact) == json.dumps(v, ensure_ascii=False)
    for bad in ('{"a":1} x', '{"a":}', '[1,]', '{"a" 1}', '"unterminated', '{"a":tru}', '01', '"\\x"', ''):
        with pytest.raises(shv.pkg.ShvError):
            T.pyjson(bad)


def test_tool_arguments_keep_the_objects_order():
    """llm/chat_test.go:166-191."""
    args = T.parse_tool_arguments('{"z": 1, "a": "two", "m": {"k": [1,2]}}')
    assert [n for n, _ in args] == ["z", "a", "m"]
    assert args[2][1] == '{"k": [1,2]}'
    with pytest.raises(shv.pkg.ShvError, match="not a JSON object"):
        T.parse_tool_arguments("[1,2]")
    assert T.parse_tool_arguments("  ") == []


# ---- the chat template (llm/chat.go) ----
XHIGH = ("Reasoning effort is set to xhigh. Please think carefully through the task, validate key assumptions, consider plausible "
         "alternatives, and prioritize correctness, consistency, and clarity in the final answer.")


def test_render_chat_refuses_what_the_template_refuses():
    """llm/chat_test.go:137-160: the template's own raise_exception calls."""
    E = shv.pkg.ShvError
    cases = {
        "no messages": ([], {}),
        "system in the middle": ([{"role": "user", "content": "hi"}, {"role": "system", "content": "be terse"}], {}),
        "unknown role": ([{"role": "narrator", "content": "hi"}], {}),
        "unknown effort": ([{"role": "user", "content": "hi"}], {"effort": "ultra"}),
        "an image in a system message": ([{"role": "system", "parts": [{"text": "see "}, {"image": True}]}, {"role": "user", "content": "hi"}], {}),
        "nameless tool call": ([{"role": "user", "content": "hi"}, {"role": "assistant", "tool_calls": [{}]}], {}),
    }
    for name, (msgs, opts) in cases.items():
        with pytest.raises(E):
            T.render_chat(msgs, **opts)
            pytest.fail(name)


def test_render_chat_structure():
    """PARITY UNPINNED (no rendering of the checkpoint's template to hold these to): the structure llm/chat.go:195-322
    states, case by case."""
    user = [{"role": "user", "content": "  hi  "}]
    gen = "<|im_start|>assistant\n<think>\n"
    # default effort is xhigh, "high" is its alias, medium has no instructions and then no system turn at all
    assert T.render_chat(user) == "<|im_start|>system\n" + XHIGH + "<|im_end|>\n<|im_start|>user\nhi<|im_end|>\n" + gen
    assert T.render_chat(user, effort="high") == T.render_chat(user)
    assert T.render_chat(user, effort="medium") == "<|im_start|>user\nhi<|im_end|>\n" + gen
    assert T.render_chat(user, effort="low").startswith("<|im_start|>system\nReasoning effort is set to low. ")
    # no thinking: no instructions, and the block is closed before the model can open it
    assert T.render_chat(user, no_thinking=True) == "<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n"
    assert T.render_chat(user, effort="medium", no_generation_prompt=True) == "<|im_start|>user\nhi<|im_end|>\n"
    # the leading run of system and developer turns is merged, trimmed, joined by one line break, after the instructions
    msgs = [{"role": "system", "content": " be terse \n"}, {"role": "developer", "content": "and kind"}, {"role": "system", "content": "   "}] + user
    assert T.render_chat(msgs).startswith("<|im_start|>system\n" + XHIGH + "\n\nbe terse\nand kind<|im_end|>\n<|im_start|>user\n")
    assert T.render_chat(msgs, effort="medium").startswith("<|im_start|>system\nbe terse\nand kind<|im_end|>\n")
    # an assistant turn keeps its reasoning; with drop_thinking only after the last real question
    hist = [{"role": "user", "content": "q1"}, {"role": "assistant", "content": "a1", "reasoning": " r1 "},
            {"role": "user", "content": "q2"}, {"role": "assistant", "content": "a2", "reasoning": "r2"}]
    kept = T.render_chat(hist, effort="medium", no_generation_prompt=True)
    assert kept == ("<|im_start|>user\nq1<|im_end|>\n<|im_start|>assistant\n<think>\nr1\n</think>\n\na1<|im_end|>\n"
                    "<|im_start|>user\nq2<|im_end|>\n<|im_start|>assistant\n<think>\nr2\n</think>\n\na2<|im_end|>\n")
    dropped = T.render_chat(hist, effort="medium", no_generation_prompt=True, drop_thinking=True)
    assert dropped == ("<|im_start|>user\nq1<|im_end|>\n<|im_start|>assistant\na1<|im_end|>\n"
                       "<|im_start|>user\nq2<|im_end|>\n<|im_start|>assistant\n<think>\nr2\n</think>\n\na2<|im_end|>\n")
    # images: one pad in place, numbered across the conversation when asked
    pics = [{"role": "user", "parts": [{"text": "look "}, {"image": True}, {"text": " and "}, {"image": True}]},
            {"role": "user", "parts": [{"image": True}]}]
    markup = "<|vision_start|><|image_pad|><|vision_end|>"
    assert T.render_chat(pics, effort="medium", no_generation_prompt=True) == (
        "<|im_start|>user\nlook " + markup + " and " + markup + "<|im_end|>\n<|im_start|>user\n" + markup + "<|im_end|>\n")
    assert T.render_chat(pics, effort="medium", no_generation_prompt=True, add_vision_id=True) == (
        "<|im_start|>user\nlook Picture 1: " + markup + " and Picture 2: " + markup + "<|im_end|>\n<|im_start|>user\nPicture 3: " + markup + "<|im_end|>\n")


def test_render_chat_tool_block_calls_and_results():
    """PARITY UNPINNED as above.  The tool block carries each tool as Python writes JSON; a call's string argument is
    written raw and anything else as JSON; a run of tool results is one user turn."""
    tool = {"type": "function", "function": {"name": "get_weather", "description": "in °C <now>", "parameters": {
        "type": "object", "properties": {"city": {"type": "string"}, "days": {"type": "integer"}}}}}
    msgs = [{"role": "system", "content": "be terse"}, {"role": "user", "content": "weather?"},
            {"role": "assistant", "content": "I will look.", "reasoning": "need a tool", "tool_calls": [
                {"name": "get_weather", "args": [{"name": "city", "value": "Wimbledon\nLondon"}, {"name": "days", "value": 2},
                                                 {"name": "where", "value": {"lat": 51.4, "ok": True}}]},
                {"name": "get_weather", "args": []}]},
            {"role": "tool", "content": "rain"}, {"role": "tool", "content": "sun "}, {"role": "user", "content": "thanks"}]
    out = T.render_chat(msgs, tools=[tool], effort="low")
    head, rest = out.split("<|im_end|>\n", 1)
    assert head.startswith("<|im_start|>system\nReasoning effort is set to low. ")
    assert "\n\n# Tools\n\nYou have access to the following functions:\n\n<tools>\n" + json.dumps(tool, ensure_ascii=False) + "\n</tools>\n\nIf you choose" in head
    assert head.endswith("</IMPORTANT>\n\nbe terse")
    assert rest == (
        "<|im_start|>user\nweather?<|im_end|>\n"
        "<|im_start|>assistant\n<think>\nneed a tool\n</think>\n\nI will look.\n\n"
        "<tool_call>\n<function=get_weather>\n<parameter=city>\nWimbledon\nLondon\n</parameter>\n<parameter=days>\n2\n</parameter>\n"
        "<parameter=where>\n{\"lat\": 51.4, \"ok\": true}\n</parameter>\n</function>\n</tool_call>"
        "\n<tool_call>\n<function=get_weather>\n</function>\n</tool_call><|im_end|>\n"
        "<|im_start|>user\n<tool_response>\nrain\n</tool_response>\n<tool_response>\nsun\n</tool_response><|im_end|>\n"
        "<|im_start|>user\nthanks<|im_end|>\n<|im_start|>assistant\n<think>\n")
    # a call with no prose before it opens without the blank line
    bare = T.render_chat([{"role": "user", "content": "q"}, {"role": "assistant", "tool_calls": [{"name": "f", "args": []}]}],
                         effort="medium", no_generation_prompt=True)
    assert bare.endswith("<|im_start|>assistant\n<think>\n\n</think>\n\n<tool_call>\n<function=f>\n</function>\n</tool_call><|im_end|>\n")
    # drop_thinking: a user turn that is only a tool response is not the last question
    conv = [{"role": "user", "content": "q"}, {"role": "assistant", "content": "a", "reasoning": "r"},
            {"role": "user", "content": "<tool_response>\nx\n</tool_response>"}, {"role": "assistant", "content": "b", "reasoning": "s"}]
    out = T.render_chat(conv, effort="medium", no_generation_prompt=True, drop_thinking=True)
    assert out.count("<think>") == 2    # both assistant turns come after the last real question


# ---- reading a completion back (llm/chatdecode.go; the cases of llm/chatdecode_test.go) ----
def feed(d, pieces):
    r, c = "", ""
    for p in pieces:
        rr, cc = d.write(p)
        r, c = r + rr, c + cc
    rr, cc, calls = d.close()
    return r + rr, c + cc, calls


THINK_CASES = [
    ("whole", True, ["Two and two.</think>\n\nIt is 4."], "Two and two.", "It is 4."),
    ("marker split across tokens", True, ["Two and", " two.<", "/th", "ink>", "\n\n", "It is ", "4."], "Two and two.", "It is 4."),
    ("no close", True, ["Still thinking"], "Still thinking", ""),
    ("not thinking", False, ["It is 4."], "", "It is 4."),
    ("empty reasoning", True, ["</think>\n\nIt is 4."], "", "It is 4."),
    ("a less-than that is not a marker", True, ["if a <", "b then", "</think>", "\n\n", "1 <", " 2"], "if a <b then", "1 < 2"),
    ("trailing whitespace is the answer's", True, ["x</think>\n\nline\n\n"], "x", "line\n\n"),
]


@pytest.mark.parametrize("name,thinking,pieces,want_r,want_c", THINK_CASES, ids=[c[0] for c in THINK_CASES])
def test_decoder_splits_thinking(name, thinking, pieces, want_r, want_c):
    r, c, calls = feed(T.ChatDecoder(None, thinking), pieces)
    assert (r, c, calls) == (want_r, want_c, [])


def test_decoder_holds_back_a_partial_marker():
    d = T.ChatDecoder(None, False)
    assert d.write("done. <tool_c")[1] == "done. "
    assert d.write("all>\n<function=f>\n</function>\n</tool_call>")[1] == ""
    _, content, calls = d.close()
    assert content == "" and [n for n, _ in calls] == ["f"]


WEATHER = {"type": "function", "function": {"name": "get_weather", "parameters": {"type": "object", "properties": {
    "city": {"type": "string"}, "days": {"type": "integer"}, "exact": {"type": "boolean"}, "where": {"type": "object"},
    "note": {"type": ["string", "null"]}}}}}


def test_decoder_tool_calls_are_typed_by_the_schema():
    gen = ("I will look it up.\n\n<tool_call>\n<function=get_weather>\n<parameter=city>\nWimbledon\n</parameter>\n"
           "<parameter=days>\n2\n</parameter>\n<parameter=exact>\ntrue\n</parameter>\n"
           "<parameter=where>\n{\"lat\": 51.4, \"lon\": -0.2}\n</parameter>\n<parameter=note>\n123\n</parameter>\n</function>\n</tool_call>")
    _, content, calls = feed(T.ChatDecoder([WEATHER], False), [gen])
    assert content == "I will look it up."
    assert calls == [("get_weather", '{"city":"Wimbledon","days":2,"exact":true,"where":{"lat": 51.4, "lon": -0.2},"note":"123"}')]
    json.loads(calls[0][1])
    # the same generation a byte at a time: the calls are the same; the blank line in front of the call, which a whole
    # piece trims, is forwarded when "<" arrives on its own (the held-back tail is then the partial marker alone, as in
    # the reference's own "done. <tool_c" case, which emits "done. " with its space)
    r, c, calls2 = feed(T.ChatDecoder([WEATHER], False), list(gen))
    assert (r, c, calls2) == ("", content + "\n\n", calls)


def test_decoder_two_calls_and_a_multi_line_argument():
    tools = [{"name": "search", "parameters": {"properties": {"query": {"type": "string"}}}}]
    gen = ("<tool_call>\n<function=search>\n<parameter=query>\nline one\nline two\n</parameter>\n</function>\n</tool_call>\n"
           "<tool_call>\n<function=search>\n<parameter=query>\nagain\n</parameter>\n</function>\n</tool_call>")
    _, _, calls = feed(T.ChatDecoder(tools, False), [gen])
    assert calls == [("search", '{"query":"line one\\nline two"}'), ("search", '{"query":"again"}')]


def test_decoder_drops_a_truncated_call_and_types_an_unknown_tools_arguments_by_their_looks():
    _, content, calls = feed(T.ChatDecoder(None, False), ["<tool_call>\n<function=search>\n<parameter=query>\nline on"])
    assert (content, calls) == ("", [])
    gen = "<tool_call>\n<function=mystery>\n<parameter=a>\n7\n</parameter>\n<parameter=b>\nseven\n</parameter>\n</function>\n</tool_call>"
    _, _, calls = feed(T.ChatDecoder(None, False), [gen])
    assert calls == [("mystery", '{"a":7,"b":"seven"}')]
    # a string value goes out as encoding/json writes strings: <, > and & escaped, the line separators too
    gen = "<tool_call>\n<function=mystery>\n<parameter=h>\n<b> &  \n</parameter>\n</function>\n</tool_call>"
    _, _, calls = feed(T.ChatDecoder(None, False), [gen])
    assert calls == [("mystery", '{"h":"\\u003cb\\u003e \\u0026 \\u2028"}')]
    assert json.loads(calls[0][1]) == {"h": "<b> &  "}


STOP_CASES = [
    ("whole", ["END"], ["the answer ENDand more"], "the answer ", "END"),
    ("split across tokens", ["END"], ["the ans", "wer E", "N", "D more"], "the answer ", "END"),
    ("a blank line", ["\n\n"], ["one line\n", "\nthe rest"], "one line", "\n\n"),
    ("never matched", ["END"], ["the answer"], "the answer", ""),
    ("the earliest of several", ["ZZZ", "END"], ["the answer END then ZZZ"], "the answer ", "END"),
    ("a partial match is still the answer", ["END"], ["the answer EN"], "the answer EN", ""),
]


@pytest.mark.parametrize("name,stop,pieces,want,want_at", STOP_CASES, ids=[c[0] for c in STOP_CASES])
def test_decoder_stop_sequences(name, stop, pieces, want, want_at):
    d = T.ChatDecoder(None, False)
    d.stop_at(stop + [""])    # empty strings are ignored
    _, content, calls = feed(d, pieces)
    assert (content, d.stopped(), calls) == (want, want_at, [])


def test_decoder_does_not_watch_stop_sequences_in_the_reasoning():
    d = T.ChatDecoder(None, True)
    d.stop_at(["\n\n"])
    r, c, _ = feed(d, ["first thought\n\nsecond thought</think>\n\nThe answer\n\nmore"])
    assert (r, c, d.stopped()) == ("first thought\n\nsecond thought", "The answer", "\n\n")


# ---- the emit loop's text side (backend/llm.go:561-590, utf8Stream :1003-1032) ----
def test_stream_keeps_a_characters_bytes_together_and_stops_at_the_stop_set(trained):
    _, mine, _, _, _, _ = trained
    end = mine.id("<|im_end|>")
    text = "thinking 🍵</think>\n\nThe answer is 茶 🍵, naïve.\n"
    ids = mine.encode(text)
    pieces = [mine.decode_bytes([i]) for i in ids]
    assert sum(1 for p in pieces if p.decode("utf-8", "replace").count("\ufffd")) >= 6   # the tea cup and the ideograph came apart into bytes
    st = T.ChatStream(mine, eog={end}, thinking=True)
    r, c = "", ""
    for i in ids + [end, ids[0]]:                   # an id after the end changes nothing
        rr, cc, fin = st.push(i)
        for delta in (rr, cc):
            delta.encode("utf-8")                   # every delta is whole characters
            assert "�" not in delta
        r, c = r + rr, c + cc
    rr, cc, calls = st.close()
    assert fin == 1 and (r + rr, c + cc, calls) == ("thinking 🍵", "The answer is 茶 🍵, naïve.\n", [])


def test_stream_stop_sequence_and_tool_call(trained):
    _, mine, _, _, _, _ = trained
    st = T.ChatStream(mine, eog=set(), thinking=False)
    st.stop_at(["STOP"])
    out, fin = "", 0
    for i in mine.encode("one two STOP three"):
        _, cc, fin = st.push(i)
        out += cc
        if fin:
            break
    assert (out, fin, st.stopped()) == ("one two ", 2, "STOP")
    tools = [{"name": "search", "parameters": {"properties": {"query": {"type": "string"}, "n": {"type": "integer"}}}}]
    st = T.ChatStream(mine, eog=set(), tools=tools, thinking=False)
    gen = "Let me look.\n\n<tool_call>\n<function=search>\n<parameter=query>\n茶 tea\n</parameter>\n<parameter=n>\n3\n</parameter>\n</function>\n</tool_call>"
    out = ""
    for i in mine.encode(gen):
        _, cc, fin = st.push(i)
        out += cc
    _, cc, calls = st.close()
    assert (out + cc).rstrip() == "Let me look." and fin == 0
    assert calls == [("search", '{"query":"茶 tea","n":3}')]
