"""Token-loop glue ops: embedding gather, greedy arg-max (llm/sample.go:359-367), advance."""
import numpy as np
import pytest

import oracle_lib as O
import shv
from test_dequant_gpu import random_tensor

pytestmark = pytest.mark.gpu
A = shv.api


def _argmax(ctx, logits):
    logits = np.ascontiguousarray(logits, np.float32)
    rows, n = logits.shape
    best = ctx.alloc(rows * 4)
    ctx.enqueue(A.OP_ARGMAX, A.ArgmaxArgs(ctx.upload(logits).ptr, best.ptr, None, None, rows, n, n))
    return best.read(np.int32, rows)


def test_argmax_first_maximum_wins(ctx):
    rng = np.random.default_rng(1)
    L = O.lib()
    for n in (1, 7, 1000, 151936):
        x = rng.standard_normal((3, n)).astype(np.float32)
        want = [L.shv_ref_argmax(O.F(np.ascontiguousarray(r)), n) for r in x]
        assert list(_argmax(ctx, x)) == want == list(np.argmax(x, axis=1))
    # ties go to the lowest id (llm/sample_test.go:17), wherever the block boundaries fall
    x = np.zeros((1, 151936), np.float32)
    x[0, [5, 700, 1024, 151935]] = 3.0
    assert _argmax(ctx, x)[0] == 5
    x[0, 5] = 0.0
    assert _argmax(ctx, x)[0] == 700
    # NaN never wins; a row with nothing above -inf returns 0
    x = np.full((2, 4096), -np.inf, np.float32)
    x[0, 100] = np.nan
    x[0, 200] = -1e30
    assert list(_argmax(ctx, x)) == [200, 0]
    assert _argmax(ctx, np.full((1, 300), np.nan, np.float32))[0] == 0


def test_argmax_feeds_the_next_step(ctx):
    logits = np.zeros((1, 5000), np.float32)
    logits[0, 4321] = 1.0
    ids = ctx.upload(np.array([11, 22, 33, -1, -1], np.int32))
    pos = ctx.upload(np.array([2], np.int32))
    best = ctx.alloc(4)
    ctx.enqueue(A.OP_ARGMAX, A.ArgmaxArgs(ctx.upload(logits).ptr, best.ptr, ids.ptr, pos.ptr, 1, 5000, 5000))
    assert best.read(np.int32, 1)[0] == 4321
    assert list(ids.read(np.int32, 5)) == [11, 22, 33, 4321, -1]
    assert pos.read(np.int32, 1)[0] == 3
    ctx.enqueue(A.OP_ADVANCE, A.AdvanceArgs(pos.ptr, 1, 4))
    assert pos.read(np.int32, 1)[0] == 7


def test_embedding_gather(ctx):
    rng = np.random.default_rng(2)
    vocab, H = 1000, 2048
    table = rng.standard_normal((vocab, H)).astype(np.float16)
    ids = np.array([3, 999, 0, 17, 5000], np.int32)
    d_x = ctx.alloc(4 * H * 4)
    d_t, d_ids = ctx.upload(table), ctx.upload(ids)
    ctx.enqueue(A.OP_EMBED, A.EmbedArgs(d_t.ptr, d_ids.ptr, None, d_x.ptr, 4, H, vocab, H, 1))
    got = d_x.read(np.float32, 4 * H).reshape(4, H)
    assert np.array_equal(got, table[ids[:4]].astype(np.float32))
    # position-relative read, and an id outside the vocabulary is NaN rather than a wild read
    ctx.enqueue(A.OP_EMBED, A.EmbedArgs(d_t.ptr, d_ids.ptr, ctx.upload(np.array([3], np.int32)).ptr, d_x.ptr,
                                        2, H, vocab, H, 1))
    got = d_x.read(np.float32, 2 * H).reshape(2, H)
    assert np.array_equal(got[0], table[17].astype(np.float32)) and np.isnan(got[1]).all()


@pytest.mark.parametrize("name", ["F32", "BF16", "Q8_0", "Q4_1", "Q5_0", "Q5_1", "IQ4_NL", "Q4_K", "Q5_K", "Q6_K"])
def test_embedding_gather_from_a_table_of_any_type(ctx, name):
    """Rows of a table kept in the checkpoint's own type, against Tensor.DequantizeRow
    (llm/model.go:125-131): bit for bit, the row stride of the output honoured."""
    typ, vocab, H = O.GGML_TYPES[name], 300, 768
    raw = random_tensor(name, vocab * H, seed=typ + 40)
    want = O.dequant(typ, raw, vocab * H).reshape(vocab, H)
    ids = np.array([7, 299, 0, -1, 123, 300], np.int32)
    stride = H + 64
    d_x = ctx.upload(np.full(len(ids) * stride, 5.0, np.float32))
    ctx.enqueue(A.OP_EMBED, A.EmbedArgs(ctx.upload(raw).ptr, ctx.upload(ids).ptr, None, d_x.ptr, len(ids), H, vocab, stride, typ))
    got = d_x.read(np.float32, len(ids) * stride).reshape(len(ids), stride)
    assert np.all(got[:, H:] == 5.0)
    for t, i in enumerate(ids):
        if 0 <= i < vocab:
            assert np.array_equal(got[t, :H].view(np.uint32), want[i].view(np.uint32)), (t, i)
        else:
            assert np.isnan(got[t, :H]).all()
    with pytest.raises(A.ShvError, match="embed: a row of 100 elements"):
        ctx.enqueue(A.OP_EMBED, A.EmbedArgs(ctx.upload(raw).ptr, ctx.upload(ids).ptr, None, d_x.ptr, 1, 100, vocab, 100, 12))


def test_vocabulary_projection_names_the_next_token_itself(ctx):
    """shv_gemv_q4k with amax_best: the launch's last block does what shv_argmax does over the row
    the launch wrote — first maximum, ties to the lower id, NaN never wins, the next token stored
    and the position advanced — and the logits are the plain launch's bit for bit.  Twice in a
    row, so that the arrival counter is seen to re-arm."""
    rng = np.random.default_rng(12)
    n, k = 151936, 2048
    f = ctx.alloc(n * k * 4)
    ctx.enqueue(A.OP_FILL_NORMAL, A.FillNormalArgs(f.ptr, n * k, 99, 0.0, 0.02))
    w = ctx.alloc(n * (k // 256 * 144))
    ctx.enqueue(A.OP_QUANTIZE_Q4K, A.QuantizeQ4KArgs(f.ptr, w.ptr, n, k))
    ctx.sync()
    f.free()
    # rows 100 and 7000 become copies of row 140000: three equal logits, the lowest id must win if they are the maximum
    rb = k // 256 * 144
    wb = w.read(np.uint8, n * rb).reshape(n, rb)
    wb[100] = wb[140000]
    wb[7000] = wb[140000]
    w.write(wb)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    d_gamma = ctx.upload(gamma)
    y0, y1, best = ctx.alloc(n * 4), ctx.alloc(n * 4), ctx.alloc(4)
    ids, pos = ctx.upload(np.full(16, -1, np.int32)), ctx.upload(np.array([3], np.int32))
    row140k = O.dequant_q4k(wb[140000:140001], k)[0]
    for trial, x in enumerate((rng.standard_normal(k).astype(np.float32), (row140k / gamma * 50).astype(np.float32))):
        dx = ctx.upload(x)
        ctx.gemv_q4k(w, dx, y0, n, k, prologue=A.PRO_RMSNORM, gamma=d_gamma)
        g = A.gemv_args(w, dx, y1, n, k, 1, A.PRO_RMSNORM, d_gamma)
        g.amax_best, g.amax_ids, g.amax_pos, g.amax_advance = best.ptr, ids.ptr, pos.ptr, 1 + trial
        ctx.enqueue(A.OP_GEMV_Q4K, g)
        lg = y0.read(np.float32, n)
        assert np.array_equal(lg, y1.read(np.float32, n))
        want = int(np.argmax(lg))
        assert best.read(np.int32, 1)[0] == want
        if trial == 1:
            assert want == 100, "the row aligned with x should win, at its lowest copy"
    got_ids = list(ids.read(np.int32, 8))
    assert got_ids[:4] == [-1] * 4 and got_ids[4] >= 0 and got_ids[5] == -1 and got_ids[6] == 100 and got_ids[7] == -1
    assert pos.read(np.int32, 1)[0] == 6
    # NaN in, NaN out everywhere: nothing is `>` -inf and the reference returns 0
    x = np.full(k, np.nan, np.float32)
    g = A.gemv_args(w, ctx.upload(x), y1, n, k, 1, A.PRO_RMSNORM, d_gamma)
    g.amax_best = best.ptr
    ctx.enqueue(A.OP_GEMV_Q4K, g)
    assert best.read(np.int32, 1)[0] == 0
    with pytest.raises(A.ShvError, match="one plain row"):
        g.n_tok = 2
        ctx.enqueue(A.OP_GEMV_Q4K, g)


def test_small_uploads_that_do_not_wait_arrive_in_order(ctx):
    """shv_upload_async: a pass's control words go through pinned staging and the call returns at once.  What a
    later download or op of the context sees is what blocking uploads would have left: several hundred of them in a
    row (more than the staging ring holds, so it wraps and waits), overlapping destinations where the last write
    wins, a source buffer reused right after each call, and a transfer above the limit taking the blocking road."""
    rng = np.random.default_rng(3)
    buf = ctx.alloc(4096 * 4)
    want = np.zeros(4096, np.int32)
    buf.write(want)
    src = np.zeros(128, np.int32)
    for i in range(700):
        n = int(rng.integers(1, 129))
        at = int(rng.integers(0, 4096 - n))
        src[:n] = rng.integers(-2 ** 31, 2 ** 31 - 1, size=n)
        buf.write_async(src[:n], byte_offset=at * 4)
        want[at:at + n] = src[:n]
        src[:] = -1                                     # the call has copied what it needs
    assert np.array_equal(buf.read(np.int32, 4096), want)
    big = rng.integers(0, 100, size=1000).astype(np.int32)   # 4000 bytes: above the limit
    buf.write_async(big)
    want[:1000] = big
    assert np.array_equal(buf.read(np.int32, 4096), want)
    # an op enqueued right behind an upload sees it: the arg-max of the row just written
    row = np.zeros(100, np.float32)
    logits, best = ctx.alloc(400), ctx.alloc(16)
    for winner in (7, 93, 0, 41):
        row[:] = 0
        row[winner] = 1
        logits.write_async(row)
        ctx.enqueue(A.OP_ARGMAX, A.ArgmaxArgs(logits.ptr, best.ptr, None, None, 1, 100, 100))
        assert int(best.read(np.int32, 1)[0]) == winner


def test_stamps_time_work_that_was_launched_without_a_wait(ctx):
    """shv_stamp / shv_stamp_elapsed: the GPU time between two points of the stream, for passes handed over with
    shv_prerecorded_launch.  More work between the stamps takes longer; a stamp that was never made, a number out of
    range and stamps the stream has not reached yet are refused."""
    pos = ctx.alloc(16).zero()
    op = A.make_op(A.OP_ADVANCE, A.AdvanceArgs(pos.ptr, 1, 1))
    one, many = ctx.prerecord([op]), ctx.prerecord([op] * 200)
    with pytest.raises(A.ShvError):
        ctx.stamp(4)
    with pytest.raises(A.ShvError, match="never made"):
        ctx.stamp_elapsed(2, 3)
    ctx.stamp(0)
    one.launch()
    ctx.stamp(1)
    many.launch()
    ctx.stamp(2)
    ctx.sync()
    short, long_ = ctx.stamp_elapsed(0, 1), ctx.stamp_elapsed(1, 2)
    assert 0 < short < long_ and long_ > 100_000, (short, long_)      # 200 dependent launches: hundreds of microseconds
    assert int(pos.read(np.int32, 1)[0]) == 201
    one.destroy()
    many.destroy()
