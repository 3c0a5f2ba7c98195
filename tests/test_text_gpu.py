"""A chat request through the token loop: template, tokenizer, prefill, greedy decode on the GPU, and the sampled ids
back through the streamed-completion reader (the path of backend/llm.go:397-620 with the HTTP layer left out).  The
model is a reduced random-init one whose vocabulary is a byte-level BPE trained here, so the text it writes is noise:
what is held is that the loop's text side loses nothing and invents nothing."""
import json

import numpy as np
import pytest

import shv

pytestmark = pytest.mark.gpu
LA = shv.pkg.llm_api
T = shv.pkg.text_api

QWEN2 = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"


def _tokenizer():
    pytest.importorskip("tokenizers")
    from tokenizers import Regex, Tokenizer, models, pre_tokenizers, trainers
    specials = ["<|endoftext|>", "<|im_start|>", "<|im_end|>"]
    hf = Tokenizer(models.BPE())
    hf.pre_tokenizer = pre_tokenizers.Sequence([pre_tokenizers.Split(Regex(QWEN2), behavior="isolated"),
                                                pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    trainer = trainers.BpeTrainer(vocab_size=700, initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), special_tokens=specials, show_progress=False)
    hf.train_from_iterator(["the quick brown fox jumps over the lazy dog " * 4, "system user assistant think tool call function " * 4,
                            "Reasoning effort is set to xhigh. Please think carefully through the task. " * 3], trainer)
    vocab = hf.get_vocab(with_added_tokens=True)
    tokens = [None] * len(vocab)
    for t, i in vocab.items():
        tokens[i] = t
    merges = [m if isinstance(m, str) else " ".join(m) for m in json.loads(hf.to_str())["model"]["merges"]]
    return T.Tokenizer.from_vocab(tokens, merges, [3 if t in specials else 1 for t in tokens], pre="qwen2"), len(tokens)


def test_chat_request_through_the_token_loop():
    tok, n_vocab = _tokenizer()
    cfg = LA.Config(n_layer=4, n_expert=16, n_expert_used=4, vocab=n_vocab, nkv=512)
    m = LA.LLM(cfg)
    try:
        m.init_synthetic(77)
        m.stage()
        prompt = T.render_chat([{"role": "system", "content": "be terse"}, {"role": "user", "content": "the quick brown fox?"}])
        ids = tok.encode(prompt)
        assert tok.decode(ids) == prompt and ids[0] == tok.id("<|im_start|>")
        m.reset()
        m.extend(np.array(ids, np.int32))
        out, _ = m.generate(48)
        out = [int(t) for t in out]
        eog = {tok.id("<|endoftext|>"), tok.id("<|im_end|>")}
        st = T.ChatStream(tok, eog=eog, thinking=True)
        r, c, fin, used = "", "", 0, 0
        for t in out:
            if t >= n_vocab:        # the model's table is padded past the vocabulary: such an id has no text, as in the reference
                with pytest.raises(shv.pkg.ShvError, match="not in the vocabulary"):
                    st.push(t)
                break
            rr, cc, fin = st.push(t)
            r, c, used = r + rr, c + cc, used + 1
            if fin:
                break
        rr, cc, calls = st.close()
        r, c = r + rr, c + cc
        # the same ids decoded in one piece and read in one piece: the streamed reading lost and invented nothing
        upto = used - 1 if fin == 1 else used
        whole = tok.decode_bytes(out[:upto]).decode("utf-8", "replace")
        d = T.ChatDecoder(None, True)
        wr, wc = d.write(whole)
        cr, cc2, wcalls = d.close()
        keep = lambda s: s.replace("�", "")    # a generation cut inside a character: the streamed reader holds the partial bytes back
        assert keep(r) == keep(wr + cr) and keep(c) == keep(wc + cc2) and calls == wcalls
        assert used > 0
        print("chat loop: %d prompt ids, %d generated, %d read, finish %d, %d chars of reasoning, %d of answer" % (len(ids), len(out), used, fin, len(r), len(c)))
    finally:
        m.close()
        tok.close()
