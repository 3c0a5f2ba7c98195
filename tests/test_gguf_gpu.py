"""Checkpoints through the GGUF container onto the device: a model written out and read back
(llm.Open, llm/model.go:52-99) is the same bytes in HBM and decodes the same tokens; constituents
fill fused projections; float tensors in other types are expanded by the device dequantiser; a
split checkpoint loads like a whole one; a tensor of any accepted type goes from the mapping
through the any-type GEMV."""
import numpy as np
import pytest

import gguf_file as GF
import oracle_lib as O
import shv
from test_dequant_gpu import random_tensor

pytestmark = pytest.mark.gpu
LA = shv.pkg.llm_api
G = shv.pkg.gguf_api
ShvError = shv.api.ShvError


def small_cfg(**kw):
    d = dict(n_layer=4, n_expert=16, n_expert_used=4, vocab=4096, nkv=128)
    d.update(kw)
    return LA.Config(**d)


@pytest.fixture(scope="module")
def saved(tmp_path_factory):
    cfg = small_cfg(nextn=1)
    m = LA.LLM(cfg)
    m.init_synthetic(77)
    m.stage()
    path = tmp_path_factory.mktemp("gguf") / "model.gguf"
    m.save_gguf(path)
    yield m, cfg, str(path)
    m.close()


def _greedy(m, prompt, n):
    m.reset()
    lg, _ = m.extend(prompt)
    ids, _ = m.generate(n)
    return lg, ids


def _rewrite(parsed, path, tensors=None, drop=(), extra_kv=()):
    """The parsed file written again by the tests' own writer, with some tensors replaced or left out."""
    w = GF.Writer()
    for k, v in list(parsed["kv"].items()) + list(extra_kv):
        w.put(k, GF.STR if isinstance(v, str) else GF.F32 if isinstance(v, float) else GF.U32, v)
    for name, (typ, dims, data) in parsed["tensors"].items():
        if name in drop:
            continue
        if tensors and name in tensors:
            typ, dims, data = tensors[name]
        w.tensor(name, typ, dims, data)
    return w.write(path)


def test_saved_file_is_a_plain_gguf_of_constituents(saved):
    m, cfg, path = saved
    p = GF.parse(path)
    assert p["version"] == 3 and p["kv"]["general.architecture"] == "qwen3next"
    kv = p["kv"]
    assert kv["qwen3next.block_count"] == 5 and kv["qwen3next.nextn_predict_layers"] == 1
    assert kv["qwen3next.embedding_length"] == cfg.n_embd and kv["qwen3next.expert_count"] == 16
    assert kv["qwen3next.ssm.state_size"] == cfg.ssm_head_dim and kv["qwen3next.full_attention_interval"] == 4
    names = set(p["tensors"])
    assert not [n for n in names if "fused" in n]
    for n in ("blk.3.attn_q.weight", "blk.3.attn_k.weight", "blk.3.attn_v.weight", "blk.0.attn_qkv.weight",
              "blk.0.attn_gate.weight", "blk.0.ssm_alpha.weight", "blk.0.ssm_beta.weight", "blk.4.nextn.enorm.weight",
              "blk.4.nextn.hnorm.weight", "token_embd.weight", "output.weight"):
        assert n in names, n
    typ, dims, data = p["tensors"]["blk.1.ffn_down_exps.weight"]
    assert typ == 12 and dims == [cfg.ffn_expert, cfg.n_embd, cfg.n_expert]
    assert p["tensors"]["output_norm.weight"][1] == [cfg.n_embd]
    assert p["tensors"]["token_embd.weight"][:2] == (1, [cfg.n_embd, cfg.vocab])
    for n, (typ, dims, data) in p["tensors"].items():
        assert np.array_equal(np.frombuffer(data, np.uint8), m.download(n).view(np.uint8)), n


def test_checkpoint_reads_back_bit_for_bit_and_decodes_the_same_tokens(saved):
    m, cfg, path = saved
    r = LA.LLM(small_cfg(n_layer=1, n_expert=2, vocab=7), gguf=path)   # the shape comes from the file
    try:
        for f, _ in LA.Config._fields_:
            if f not in ("layers", "no_head", "attn_splits", "max_tokens", "slots", "head_rows", "speculative", "spec_rows"):
                assert getattr(r.cfg, f) == getattr(cfg, f), f
        a, b = m.tensors(), r.tensors()
        assert [t[0] for t in a] == [t[0] for t in b]
        for t in a:
            assert np.array_equal(m.download(t[0]).view(np.uint8), r.download(t[0]).view(np.uint8)), t[0]
        r.stage()
        prompt = np.random.default_rng(3).integers(0, cfg.vocab, size=9).astype(np.int32)
        lg0, ids0 = _greedy(m, prompt, 16)
        lg1, ids1 = _greedy(r, prompt, 16)
        assert np.array_equal(lg0.view(np.uint32), lg1.view(np.uint32))
        assert np.array_equal(ids0, ids1)
    finally:
        r.close()


def test_split_checkpoint_loads_like_a_whole_one(saved, tmp_path):
    m, cfg, path = saved
    p = GF.parse(path)
    names = list(p["tensors"])
    cut = [names[:len(names) // 3], names[len(names) // 3:2 * len(names) // 3], names[2 * len(names) // 3:]]
    for i, part in enumerate(cut):
        extra = [("split.no", i), ("split.count", 3), ("split.tensors.count", len(names))]
        q = dict(p, kv=p["kv"] if i == 0 else {})
        _rewrite(q, tmp_path / ("m-%05d-of-00003.gguf" % (i + 1)), drop=set(names) - set(part), extra_kv=extra)
    r = LA.LLM(small_cfg(), gguf=tmp_path / "m-00002-of-00003.gguf")
    try:
        for t in m.tensors():
            assert np.array_equal(m.download(t[0]).view(np.uint8), r.download(t[0]).view(np.uint8)), t[0]
    finally:
        r.close()


def test_float_tensors_of_other_types_are_expanded_on_the_device(saved, tmp_path):
    m, cfg, path = saved
    p = GF.parse(path)
    swap = {}

    def as_type(name, typ):
        _, dims, data = p["tensors"][name]
        v = np.frombuffer(data, np.float32)
        if typ == 1:
            raw = v.astype(np.float16).view(np.uint8)
        elif typ == 30:
            raw = (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
        else:       # Q8_0 blocks of 32: d = max|x| / 127
            blk = v.reshape(-1, 32)
            d = (np.abs(blk).max(axis=1) / 127).astype(np.float16)
            q = np.round(blk / np.maximum(d.astype(np.float32), 1e-30)[:, None]).clip(-127, 127).astype(np.int8)
            raw = np.concatenate([d.view(np.uint8).reshape(-1, 2), q.view(np.uint8)], axis=1).reshape(-1)
        swap[name] = (typ, dims, raw.tobytes())

    as_type("output_norm.weight", 30)
    as_type("blk.0.attn_norm.weight", 1)
    as_type("blk.2.ffn_gate_inp.weight", 8)
    as_type("blk.1.ssm_conv1d.weight", 1)
    r = LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "mixed.gguf", tensors=swap))
    try:
        for name, (typ, dims, raw) in swap.items():
            want = O.dequant(typ, np.frombuffer(raw, np.uint8), int(np.prod(dims)))
            assert np.array_equal(r.download(name).view(np.uint32), want.view(np.uint32)), name
        assert np.array_equal(r.download("blk.1.attn_norm.weight"), m.download("blk.1.attn_norm.weight"))
    finally:
        r.close()


def test_load_refuses_what_it_cannot_stage(saved, tmp_path, monkeypatch):
    m, cfg, path = saved
    p = GF.parse(path)
    with pytest.raises(ShvError, match=r"rows of blk\.3\.attn_qkv_fused"):
        LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "nok.gguf", drop={"blk.3.attn_k.weight"}))
    with pytest.raises(ShvError, match=r"0 of 1 rows of output_norm"):
        LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "nonorm.gguf", drop={"output_norm.weight"}))
    _, dims, data = p["tensors"]["blk.0.ssm_out.weight"]
    n = int(np.prod(dims))
    q8 = (8, dims, bytes(n // 32 * 34))
    monkeypatch.setenv("LLM_TRANSCODE", "0")
    with pytest.raises(ShvError, match="Q8_0 in the checkpoint; the kernels stream it as Q4_K"):
        LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "q8.gguf", tensors={"blk.0.ssm_out.weight": q8}))
    monkeypatch.delenv("LLM_TRANSCODE")
    _, dims, data = p["tensors"]["blk.0.ffn_up_shexp.weight"]
    n = int(np.prod(dims))
    q2 = (10, dims, bytes(n // 256 * 84))
    with pytest.raises(ShvError, match="blk.0.ffn_up_shexp.weight"):
        LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "q2.gguf", tensors={"blk.0.ffn_up_shexp.weight": q2}))
    _, edims, _ = p["tensors"]["token_embd.weight"]
    with pytest.raises(ShvError, match="not a type the device expands"):
        LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "e2.gguf", tensors={"token_embd.weight": (10, edims, bytes(int(np.prod(edims)) // 256 * 84))}))
    short = (0, [cfg.n_embd // 2], bytes(cfg.n_embd * 2))
    with pytest.raises(ShvError, match="the metadata makes it"):
        LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "shape.gguf", tensors={"output_norm.weight": short}))
    q = dict(p, kv={k: v for k, v in p["kv"].items() if k != "qwen3next.ssm.state_size"})
    with pytest.raises(ShvError, match="states no qwen3next.ssm.state_size"):
        LA.LLM(small_cfg(), gguf=_rewrite(q, tmp_path / "nokey.gguf"))
    q = dict(p, kv={k: v for k, v in p["kv"].items() if k != "general.architecture"})
    with pytest.raises(ShvError, match="no general.architecture"):
        LA.LLM(small_cfg(), gguf=_rewrite(q, tmp_path / "noarch.gguf"))


BANK_WORDS = ("_exps.", "_shexp.")


@pytest.mark.parametrize("plan", ["", "down_exps=q4_k,gate_exps=q4_k,up_shexp=q4_k"])
def test_checkpoint_of_mixed_types_is_staged_and_decodes_as_the_cpu_does(saved, tmp_path, monkeypatch, plan):
    """What a converter's mixed recipe looks like: the embedding table in Q8_0, the head in Q6_K,
    expert banks in Q5_K / Q8_0 / IQ4_NL / Q5_1, one constituent of a fused projection in Q5_0, others
    in F16 and Q4_1.  The table stays in its own type (rows expanded by the gather,
    llm/model.go:125-131) and so do the expert banks (llm/gpu_moe.go:673-688), read through their
    types' arms; every other such matrix is expanded and fitted again as Q4_K, bit for bit what the
    CPU's dequantiser (gguf/dequant.go:52-98) followed by the CPU's quantiser
    (llm/quantk.go:115-179) gives.  Under a plan (LLM_MOE_BANK, llm/moebank.go:55-63) the families
    it names are refitted too, where they are wider than Q4_K.  Either way the model decodes what
    the CPU model decodes from the weights as staged."""
    m, cfg, path = saved
    p = GF.parse(path)
    recipe = {"token_embd.weight": "Q8_0", "output.weight": "Q6_K", "blk.0.ffn_down_exps.weight": "Q5_K",
              "blk.1.ffn_gate_exps.weight": "Q8_0", "blk.2.ffn_down_exps.weight": "IQ4_NL", "blk.1.ffn_up_shexp.weight": "Q5_1",
              "blk.3.attn_k.weight": "Q5_0", "blk.0.attn_gate.weight": "F16", "blk.2.ssm_out.weight": "Q4_1",
              "blk.4.nextn.eh_proj.weight": "BF16"}
    swap, f32 = {}, {}
    for i, (name, tname) in enumerate(recipe.items()):
        typ = O.GGML_TYPES[tname]
        _, dims, _ = p["tensors"][name]
        n = int(np.prod(dims))
        if tname in ("F16", "BF16"):
            v = (np.random.default_rng(50 + i).standard_normal(n) * 0.02).astype(np.float32)
            raw = v.astype(np.float16).view(np.uint8) if tname == "F16" else (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
        else:
            raw = random_tensor(tname, n, seed=60 + i, scale=2e-4)
        if name == "token_embd.weight":
            # scales of 2^-6: every expanded value is a binary16 too, so the CPU model's binary16 table holds the same rows
            blocks = raw.reshape(-1, 34)
            blocks[:, 0], blocks[:, 1] = 0x00, 0x24
        swap[name] = (typ, dims, raw.tobytes())
        f32[name] = O.dequant(typ, raw, n)
    if plan:
        monkeypatch.setenv("LLM_MOE_BANK", plan)
    # a family's ceiling leaves a bank no wider than Q4_K alone: IQ4_NL stays whatever the plan says
    refit_banks = {"blk.0.ffn_down_exps.weight", "blk.1.ffn_gate_exps.weight", "blk.1.ffn_up_shexp.weight"} if plan else set()
    native = ({n for n in recipe if any(w in n for w in BANK_WORDS)} - refit_banks) | {"output.weight"}   # the head keeps its type too
    r = LA.LLM(small_cfg(), gguf=_rewrite(p, tmp_path / "recipe.gguf", tensors=swap))
    try:
        assert sorted(r.transcoded()) == sorted(n for n in recipe if n != "token_embd.weight" and n not in native)
        assert r.tensor_type("token_embd.weight") == 8 and r.tensor_type("output.weight") == 14
        for name in recipe:
            if name == "token_embd.weight" or name in native:
                assert r.tensor_type(name) == swap[name][0], name
                assert np.array_equal(r.download(name), np.frombuffer(swap[name][2], np.uint8)), name
                continue
            k = swap[name][1][0]
            want = O.quantize_q4k(f32[name].reshape(-1, k))
            assert r.tensor_type(name) == 12
            assert np.array_equal(r.download(name).view(np.uint8), want.reshape(-1)), name
        assert np.array_equal(r.download("blk.3.attn_q.weight"), m.download("blk.3.attn_q.weight"))
        # saved again, the file names the types now in memory and holds the same bytes
        r.save_gguf(tmp_path / "again.gguf")
        again = GF.parse(tmp_path / "again.gguf")
        for name in native | {"token_embd.weight"}:
            assert again["tensors"][name][0] == swap[name][0] and again["tensors"][name][2] == swap[name][2], name
        # the token loop against the CPU loop over the weights as staged
        r.stage()
        tensors = {t[0]: r.download(t[0]) for t in r.tensors()}
        table = f32["token_embd.weight"].astype(np.float16)
        assert np.array_equal(table.astype(np.float32), f32["token_embd.weight"])
        tensors["token_embd.weight"] = table.view(np.uint16)
        # the CPU model walks its layers with any Q4_K head (its logits are not used): the head in the checkpoint's type
        # is matvec over the CPU's dequantised rows of it (llm/hc.go:255-264), applied to the CPU's own residual stream
        head = f32["output.weight"].reshape(cfg.vocab, cfg.n_embd)
        tensors["output.weight"] = O.quantize_q4k(head)
        om = O.OracleModel(cfg, tensors, max_cells=cfg.nkv, bank_types={n: swap[n][0] for n in native if n != "output.weight"})
        prompt = np.random.default_rng(5).integers(0, cfg.vocab, size=7).astype(np.int32)
        r.reset()
        lg_gpu, hd_gpu = r.extend(prompt, want_hidden=True)
        _, hd_cpu = om.extend(prompt)
        xn = O.rmsnorm(hd_cpu.reshape(1, -1), tensors["output_norm.weight"], cfg.rms_eps)[0]
        lg_cpu = (head.astype(np.float64) @ xn.astype(np.float64)).astype(np.float32)
        assert O.rel_l2(hd_gpu, hd_cpu) <= 1e-3 and O.rel_l2(lg_gpu, lg_cpu) <= 1e-3
        tok = int(O.lib().shv_ref_argmax(O.F(lg_cpu), cfg.vocab))
        ids, _ = r.generate(1)
        top2 = np.sort(lg_cpu)[-2:]
        assert ids[0] == tok or top2[1] - top2[0] < 1e-4
    finally:
        r.close()


def test_the_head_in_its_own_type_or_refitted(saved, tmp_path, monkeypatch):
    """A checkpoint's vocabulary projection in Q8_0 stays Q8_0 in HBM and the head's launch reads it through that type's
    arm, for one row and for the rows of a pass; LLM_HEAD_TYPE=q4_k refits it like any other dense matrix (and says so)."""
    m, cfg, path = saved
    p = GF.parse(path)
    _, dims, _ = p["tensors"]["output.weight"]
    raw = random_tensor("Q8_0", int(np.prod(dims)), seed=77, scale=2e-4)
    head = O.dequant(O.GGML_TYPES["Q8_0"], raw, int(np.prod(dims))).reshape(cfg.vocab, cfg.n_embd)
    out = _rewrite(p, tmp_path / "head.gguf", tensors={"output.weight": (O.GGML_TYPES["Q8_0"], dims, raw.tobytes())})
    r = LA.LLM(small_cfg(head_rows=5), gguf=out)
    try:
        assert r.tensor_type("output.weight") == 8 and "output.weight" not in r.transcoded()
        assert np.array_equal(r.download("output.weight"), raw)
        r.stage()
        gamma = r.download("output_norm.weight")
        rows = np.random.default_rng(9).integers(0, cfg.vocab, size=5).astype(np.int32)
        _, lg_rows, res = r.extend_rows(rows, want_logits=True, want_res=True)
        for t in range(5):
            xn = O.rmsnorm(res[t:t + 1], gamma, cfg.rms_eps)[0]
            assert O.rel_l2(lg_rows[t], head.astype(np.float64) @ xn.astype(np.float64)) <= 1e-4, t
        # the recorded one-row step: logits of its row, and the token it names is their first maximum
        lg, hd = r.extend(rows[:1], want_hidden=True)
        want = head.astype(np.float64) @ O.rmsnorm(hd.reshape(1, -1), gamma, cfg.rms_eps)[0].astype(np.float64)
        assert O.rel_l2(lg, want) <= 1e-4
        ids, _ = r.generate(1)
        top2 = np.sort(lg)[-2:]
        assert ids[0] == int(np.argmax(lg)) or top2[1] - top2[0] < 1e-5
    finally:
        r.close()
    monkeypatch.setenv("LLM_HEAD_TYPE", "q4_k")
    r = LA.LLM(small_cfg(), gguf=out)
    try:
        assert r.tensor_type("output.weight") == 12 and "output.weight" in r.transcoded()
        assert np.array_equal(r.download("output.weight").view(np.uint8), O.quantize_q4k(head).reshape(-1))
    finally:
        r.close()
    monkeypatch.setenv("LLM_HEAD_TYPE", "q6_k")
    with pytest.raises(ShvError, match="LLM_HEAD_TYPE"):
        LA.LLM(small_cfg(), gguf=out)


def test_a_bank_plan_is_held_to_the_grammar(saved, monkeypatch):
    m, cfg, path = saved
    for plan, msg in (("down_exps", "is not family=format"), ("ffn_down=q4_k", "names family"), ("down_exps=q5_1", "q4_k is the format")):
        monkeypatch.setenv("LLM_MOE_BANK", plan)
        with pytest.raises(ShvError, match=msg):
            LA.LLM(small_cfg(), gguf=path)
    monkeypatch.delenv("LLM_MOE_BANK")
    monkeypatch.setenv("LLM_MOE_BANK_QUANT", "imatrix")
    with pytest.raises(ShvError, match="no importance matrix"):
        LA.LLM(small_cfg(), gguf=path)


@pytest.mark.parametrize("name", ["Q8_0", "Q6_K", "Q5_K", "IQ4_NL", "BF16"])
def test_gemv_over_a_mapped_tensor(ctx, tmp_path, name):
    """A tensor's bytes straight from the mapping into HBM and through the any-type GEMV, against
    matvec over the CPU's dequantised rows (llm/hc.go:255-264)."""
    typ, n, k = O.GGML_TYPES[name], 96, 1024
    w = GF.Writer()
    w.tensor("pad", 0, [3], bytes(12))                   # pushes the next tensor off the file's natural alignment
    w.tensor("w", typ, [k, n], random_tensor(name, n * k, seed=typ + 9).tobytes())
    with G.GGUF(w.write(tmp_path / "w.gguf")) as f:
        t = f.get("w")
        assert t.type == typ and t.rows == n and t.dims[0] == k
        x = np.random.default_rng(1).standard_normal(k).astype(np.float32)
        y = ctx.alloc(n * 4)
        ctx.gemv(t.type, ctx.upload(np.array(t.data())), ctx.upload(x), y, n, k)
        want = O.dequant(typ, np.array(t.data()), n * k).reshape(n, k).astype(np.float64) @ x
        assert O.rel_l2(y.read(np.float32, n), want) <= 1e-5
