//go:build shv_hip

// Package hip binds libshv_hip.so (include/shv_hip.h) for the reference's Go host code: it offers
// package llm what package vk offers it (vk/engine.go) for the token loop's ops.
//
// NOT COMPILED IN THIS REPOSITORY: the build image has no Go toolchain, so this file has been
// checked by eye against the header only.  It is the binding a maintainer of the reference adds
// beside vk/ (build tag shv_hip); llm/gpu_moe_hip.go next to it shows one block's op list built
// on it.  The C++ mirror in host/llm.cpp is the same code compiled and tested.
package hip

/*
#cgo CFLAGS:  -I${SRCDIR}/../../../include
#cgo LDFLAGS: -L${SRCDIR}/../.. -lshv_hip -Wl,-rpath,${SRCDIR}/../..
#include <stdlib.h>
#include <string.h>
#include "shv_hip.h"
*/
import "C"

import (
	"errors"
	"runtime"
	"time"
	"unsafe"
)

// Device is vk.Device's counterpart (vk/engine.go:266): one GPU, one in-order stream.
type Device struct{ ctx *C.shv_ctx }

func lastErr() error { return errors.New(C.GoString(C.shv_last_error())) }

// call runs f on a locked OS thread: shv_last_error is thread-local.
func call(f func() C.int) error {
	runtime.LockOSThread()
	defer runtime.UnlockOSThread()
	if f() != C.SHV_OK {
		return lastErr()
	}
	return nil
}

// Open is vk.NewInstance + vk.NewDevice (vk/engine.go:53,266).
func Open(index int) (*Device, error) {
	d := &Device{}
	if err := call(func() C.int { return C.shv_init(C.int(index), &d.ctx) }); err != nil {
		return nil, err
	}
	return d, nil
}

func (d *Device) Close()      { C.shv_destroy(d.ctx); d.ctx = nil }
func (d *Device) Sync() error { return call(func() C.int { return C.shv_sync(d.ctx) }) }

// Buffer is vk.Buffer's counterpart (vk/engine.go:319-634): a device address and a length.
type Buffer struct {
	dev  *Device
	ptr  unsafe.Pointer
	size uint64
}

// NewBuffer is vk.NewBuffer (vk/engine.go:457).
func (d *Device) NewBuffer(size uint64) (*Buffer, error) {
	b := &Buffer{dev: d, size: size}
	if err := call(func() C.int { return C.shv_alloc(d.ctx, C.size_t(size), &b.ptr) }); err != nil {
		return nil, err
	}
	return b, nil
}

// Slice is free: ops take addresses, not (buffer, offset, range) descriptors.
func (b *Buffer) Slice(off, n uint64) *Buffer { return &Buffer{b.dev, unsafe.Add(b.ptr, off), n} }
func (b *Buffer) Addr() unsafe.Pointer          { return b.ptr }
func (b *Buffer) Size() uint64                  { return b.size }
func (b *Buffer) Destroy()                      { C.shv_free(b.dev.ctx, b.ptr); b.ptr = nil }

// Write / Read are Buffer.Write* / Read* (vk/engine.go:477-626) for any element type.
func (b *Buffer) Write(src []byte) error {
	return call(func() C.int { return C.shv_upload(b.dev.ctx, b.ptr, unsafe.Pointer(&src[0]), C.size_t(len(src))) })
}

// WriteSoon is Write for a pass's control words and ids: up to 512 bytes are copied aside and handed to the
// stream, and the call does not wait for the device (the reference writes such words into host-visible memory).
func (b *Buffer) WriteSoon(src []byte) error {
	return call(func() C.int { return C.shv_upload_async(b.dev.ctx, b.ptr, unsafe.Pointer(&src[0]), C.size_t(len(src))) })
}
func (b *Buffer) Read(dst []byte) error {
	return call(func() C.int { return C.shv_download(b.dev.ctx, unsafe.Pointer(&dst[0]), b.ptr, C.size_t(len(dst))) })
}
func (b *Buffer) Zero() error {
	return call(func() C.int { return C.shv_zero(b.dev.ctx, b.ptr, C.size_t(b.size)) })
}

// Op is vk.MultiDispatch's counterpart (vk/engine.go:848-860): kind, flags and up to 248 bytes of
// arguments, passed to the kernel by value.  There are no pipelines or descriptor sets to make.
type Op C.shv_op

const Overlap = 1 // MultiDispatch.Overlap: accepted, ops still run in list order

func mk(kind C.uint32_t, args unsafe.Pointer, n C.size_t) Op {
	var op C.shv_op
	op.kind = kind
	C.memcpy(unsafe.Pointer(&op.args[0]), args, n)
	return Op(op)
}

func fp(b *Buffer) *C.float {
	if b == nil {
		return nil
	}
	return (*C.float)(b.ptr)
}
func ip(b *Buffer) *C.int32_t {
	if b == nil {
		return nil
	}
	return (*C.int32_t)(b.ptr)
}
func vp(b *Buffer) unsafe.Pointer {
	if b == nil {
		return nil
	}
	return b.ptr
}

// Prologues of the Q4_K projection (what the reference runs as llm_rmsnorm.comp, llm_dn_norm.comp
// and llm_attn_gate.comp before its GEMV).
const (
	ProNone       = C.SHV_PRO_NONE
	ProRMSNorm    = C.SHV_PRO_RMSNORM
	ProGatedNorm  = C.SHV_PRO_GATED_NORM
	ProMulSigmoid = C.SHV_PRO_MUL_SIGMOID
	ProRMSNormPair = C.SHV_PRO_RMSNORM_PAIR
)

// GemvOpts are the optional fields of shv_gemv_q4k_args.
type GemvOpts struct {
	Prologue            int
	Gamma, Z, Residual  *Buffer
	Pos, Slot           *Buffer // device int32: each sequence's position and slot
	Eps                 float32
	HeadDim             int
	XStride, YStride    int
	ZStride             int
	SeqLen              int
	RingSlots, RingStride int // y (or, with ZRing, z) is a ring of projection rows addressed by position
	ZRing               bool
	YFlat               *Buffer // one-row ring output: the row once more at a fixed address
	// The router's logits in the same launch (the mixer's output projection of a pass of one to
	// three rows): Fold is the layer's table made by RouterFold, FoldOut receives FoldRows products
	// a row, FoldStride floats apart; Residual must not be y.
	Fold, FoldOut        *Buffer
	FoldRows, FoldStride int
	// The greedy sampler in the same launch (a one-row vocabulary projection): what Argmax does
	// with best / ids / pos / advance.
	AmaxBest, AmaxIds, AmaxPos *Buffer
	AmaxAdvance                int
}

// GemvQ4K is llm_gemv_q4k.comp / llm_gemm_q4k.comp: y[t] = W pro(x[t]) (+ residual[t]) for rows
// t < rows; three rows and more run on the matrix cores by themselves.
func GemvQ4K(w, x, y *Buffer, n, k, rows int, o GemvOpts) Op {
	var a C.shv_gemv_q4k_args
	a.w, a.x, a.y = w.ptr, fp(x), fp(y)
	a.residual, a.gamma, a.z = fp(o.Residual), fp(o.Gamma), fp(o.Z)
	a.pos, a.slot = ip(o.Pos), ip(o.Slot)
	a.n, a.k, a.n_tok = C.int32_t(n), C.int32_t(k), C.int32_t(rows)
	a.prologue, a.head_dim, a.eps = C.int32_t(o.Prologue), C.int32_t(o.HeadDim), C.float(o.Eps)
	a.x_stride, a.y_stride, a.z_stride = C.int32_t(pick(o.XStride, k)), C.int32_t(pick(o.YStride, n)), C.int32_t(pick(o.ZStride, k))
	a.seq_len, a.ring_slots, a.ring_stride = C.int32_t(o.SeqLen), C.int32_t(o.RingSlots), C.int32_t(o.RingStride)
	if o.ZRing {
		a.z_ring = 1
	}
	a.y_flat = fp(o.YFlat)
	a.fold, a.fold_out = fp(o.Fold), fp(o.FoldOut)
	a.fold_rows, a.fold_stride = C.int32_t(o.FoldRows), C.int32_t(o.FoldStride)
	a.amax_best, a.amax_ids, a.amax_pos = ip(o.AmaxBest), ip(o.AmaxIds), ip(o.AmaxPos)
	a.amax_advance = C.int32_t(o.AmaxAdvance)
	return mk(C.SHV_OP_GEMV_Q4K, unsafe.Pointer(&a), C.sizeof_shv_gemv_q4k_args)
}

func pick(v, def int) int {
	if v != 0 {
		return v
	}
	return def
}

// MoERouter is llm_moe_router.comp + llm_moe_route.comp: xn = rmsnorm(h) * gamma, the logits of
// the n_expert experts and of the shared expert's gate, and (unless deferred to MoEUp) the top-k.
func MoERouter(h, gamma, router, sharedGate, xn, logits, topk, weights *Buffer, rows, nEmbd, nExpert, nUsed int, eps float32, deferRoute bool) Op {
	var a C.shv_moe_router_args
	a.h, a.gamma, a.router, a.shared_gate = fp(h), fp(gamma), fp(router), fp(sharedGate)
	a.xn, a.logits, a.topk, a.weights = fp(xn), fp(logits), ip(topk), fp(weights)
	a.n_tok, a.n_embd, a.n_expert, a.n_used = C.int32_t(rows), C.int32_t(nEmbd), C.int32_t(nExpert), C.int32_t(nUsed)
	a.eps, a.h_stride = C.float(eps), C.int32_t(nEmbd)
	if deferRoute {
		a.defer_route = 1
	}
	return mk(C.SHV_OP_MOE_ROUTER, unsafe.Pointer(&a), C.sizeof_shv_moe_router_args)
}

// RouterFold makes a layer's table [R diag(gamma) W | R diag(gamma)] (nExpert rows of k + nEmbd
// floats) from the float32 router, the post-attention norm's gamma and the Q4_K output projection
// W [nEmbd][k]; scratch holds nEmbd * k floats and may be freed afterwards.  Run once when the
// graph is staged, where the reference makes its dense banks (llm/bank_q4.go:172-266).
func RouterFold(router, gamma, wOut, out, scratch *Buffer, nExpert, nEmbd, k int) Op {
	var a C.shv_router_fold_args
	a.router, a.gamma, a.w_out = fp(router), fp(gamma), vp(wOut)
	a.out, a.scratch = fp(out), fp(scratch)
	a.n_expert, a.n_embd, a.k = C.int32_t(nExpert), C.int32_t(nEmbd), C.int32_t(k)
	return mk(C.SHV_OP_ROUTER_FOLD, unsafe.Pointer(&a), C.sizeof_shv_router_fold_args)
}

// MoENorm is what MoEUp needs when the router's logits came from the output projection (GemvOpts.Fold):
// xn is then the un-normalised residual row; the kernel normalises it, scales the logits by the same
// factor and forms the shared expert's gate.
type MoENorm struct {
	Gamma, SharedGate *Buffer
	Eps               float32
}

// WithNorm sets those fields on an op made by MoEUp.
func (o Op) WithNorm(n MoENorm) Op {
	a := (*C.shv_moe_up_args)(unsafe.Pointer(&o.args[0]))
	a.gamma, a.shared_gate, a.eps = fp(n.Gamma), fp(n.SharedGate), C.float(n.Eps)
	return o
}

// MoEBanks names the six expert banks and their ggml types (gguf.Tensor.Type).
type MoEBanks struct {
	GateExps, UpExps, DownExps, GateSh, UpSh, DownSh *Buffer
	Types                                            [6]int32
}

// MoEUp is llm_moe_gemv.comp MODE 0 + llm_moe_act.comp: act[t][s] = silu(Wg x) * (Wu x) for the
// token's experts and the shared one.  logits/weights non-nil: every block routes its token first.
// group non-nil (2*nExpert + 1 + rows*nUsed ints): a pass of 128 rows and more goes grouped by
// expert on the matrix cores.  packed: such a pass leaves act as the operands the grouped MoEDown
// reads instead of floats (MoEDown must follow at once, with groupReady and packed too).
func MoEUp(xn, topk *Buffer, b MoEBanks, act *Buffer, rows, nEmbd, nUsed, ffn, nExpert int, logits, weights, group *Buffer, packed bool) Op {
	var a C.shv_moe_up_args
	a.xn, a.topk = fp(xn), ip(topk)
	a.gate_exps, a.up_exps, a.gate_sh, a.up_sh = vp(b.GateExps), vp(b.UpExps), vp(b.GateSh), vp(b.UpSh)
	a.act = fp(act)
	a.n_tok, a.n_embd, a.n_used, a.ffn, a.n_expert = C.int32_t(rows), C.int32_t(nEmbd), C.int32_t(nUsed), C.int32_t(ffn), C.int32_t(nExpert)
	a.logits, a.weights, a.group = fp(logits), fp(weights), ip(group)
	a.gate_type, a.up_type, a.gate_sh_type, a.up_sh_type = C.int32_t(b.Types[0]), C.int32_t(b.Types[1]), C.int32_t(b.Types[3]), C.int32_t(b.Types[4])
	if packed {
		a.act_packed = 1
	}
	return mk(C.SHV_OP_MOE_UP, unsafe.Pointer(&a), C.sizeof_shv_moe_up_args)
}

// MoEDown is llm_moe_gemv.comp MODE 1 + llm_moe_combine.comp (+ the residual add).
func MoEDown(act, topk, weights *Buffer, b MoEBanks, residual, out *Buffer, rows, nEmbd, nUsed, ffn, nExpert int, group, pairs *Buffer, groupReady, packed bool) Op {
	var a C.shv_moe_down_args
	a.act, a.topk, a.weights = fp(act), ip(topk), fp(weights)
	a.down_exps, a.down_sh = vp(b.DownExps), vp(b.DownSh)
	a.residual, a.out = fp(residual), fp(out)
	a.n_tok, a.n_embd, a.n_used, a.ffn, a.n_expert = C.int32_t(rows), C.int32_t(nEmbd), C.int32_t(nUsed), C.int32_t(ffn), C.int32_t(nExpert)
	a.res_stride, a.out_stride = C.int32_t(nEmbd), C.int32_t(nEmbd)
	a.down_type, a.down_sh_type = C.int32_t(b.Types[2]), C.int32_t(b.Types[5])
	a.group, a.pairs = ip(group), fp(pairs)
	if groupReady {
		a.group_ready = 1
	}
	if packed {
		a.act_packed = 1
	}
	return mk(C.SHV_OP_MOE_DOWN, unsafe.Pointer(&a), C.sizeof_shv_moe_down_args)
}

// PassRows says which rows a pass carries (llm::PassRows in host/llm.hpp; the reference's rowSet,
// llm/graph.go:1383-1429): NSeq sequences of SeqLen consecutive rows, their positions and slots in
// device memory, and whether the pass is rewindable.
type PassRows struct {
	NSeq, SeqLen int
	Pos, Slot    *Buffer // device int32 per sequence; Slot nil: sequence s is slot s
	Spec         bool
}

// DNStepArgs are the fields of shv_dn_step_args a caller sets (llm_dn_conv.comp + llm_dn_scan.comp).
type DNStepArgs struct {
	Ring, Conv1D, A, DtBias, State, Out *Buffer
	Rows                                PassRows
	HeadK, HeadV, HeadDim, Conv         int
	RingSlots, RingStride               int
	Eps                                 float32
	Plane                               *Buffer // device int32 per slot: the committed state plane
	Planes                              int
	Work                                *Buffer // scratch of the chunked form; nil keeps every pass row by row
}

// DNStep is the gated delta rule over the ring rows of a pass.
func DNStep(d DNStepArgs) Op {
	var a C.shv_dn_step_args
	a.ring, a.conv1d, a.a, a.dt_bias = fp(d.Ring), fp(d.Conv1D), fp(d.A), fp(d.DtBias)
	a.state, a.out = fp(d.State), fp(d.Out)
	a.pos, a.slot = ip(d.Rows.Pos), ip(d.Rows.Slot)
	a.n_seq, a.seq_len = C.int32_t(d.Rows.NSeq), C.int32_t(d.Rows.SeqLen)
	a.n_head_k, a.n_head_v, a.head_dim, a.conv = C.int32_t(d.HeadK), C.int32_t(d.HeadV), C.int32_t(d.HeadDim), C.int32_t(d.Conv)
	a.ring_slots, a.ring_stride, a.eps = C.int32_t(d.RingSlots), C.int32_t(d.RingStride), C.float(d.Eps)
	a.plane, a.n_planes = ip(d.Plane), C.int32_t(d.Planes)
	if d.Rows.Spec {
		a.spec = 1
	}
	if d.Work != nil {
		a.work, a.work_floats = fp(d.Work), C.int64_t(d.Work.size/4)
	}
	return mk(C.SHV_OP_DN_STEP, unsafe.Pointer(&a), C.sizeof_shv_dn_step_args)
}

// AttnArgs are the fields of shv_attn_decode_args a caller sets (llm_attn_pack.comp,
// llm_attn_wmma.comp -DSPLITK, llm_attn_combine.comp in one op).
type AttnArgs struct {
	QKV, QNorm, KNorm, Rope      *Buffer
	KCache, VCache, Partial, Out *Buffer
	Rows                         PassRows
	NHead, NHeadKV, HeadDim      int
	RopeDims, MaxCells           int
	QKVStride, Splits            int
	Eps                          float32
	Mask                         *Buffer // the block-sparse indexer's selection (QSAIndex), or nil
	MaskStride                   int
}

// AttnDecode appends the rows' cells and attends over each sequence's cache.
func AttnDecode(d AttnArgs) Op {
	var a C.shv_attn_decode_args
	a.qkv, a.q_norm, a.k_norm, a.rope = fp(d.QKV), fp(d.QNorm), fp(d.KNorm), fp(d.Rope)
	a.kcache, a.vcache, a.partial, a.out = vp(d.KCache), vp(d.VCache), fp(d.Partial), fp(d.Out)
	a.pos, a.slot = ip(d.Rows.Pos), ip(d.Rows.Slot)
	a.n_seq, a.seq_len = C.int32_t(d.Rows.NSeq), C.int32_t(d.Rows.SeqLen)
	a.n_head, a.n_head_kv, a.head_dim = C.int32_t(d.NHead), C.int32_t(d.NHeadKV), C.int32_t(d.HeadDim)
	a.rope_dims, a.max_cells = C.int32_t(d.RopeDims), C.int32_t(d.MaxCells)
	a.qkv_stride, a.n_splits, a.eps = C.int32_t(d.QKVStride), C.int32_t(d.Splits), C.float(d.Eps)
	if d.Mask != nil {
		a.mask = (*C.uint32_t)(d.Mask.ptr)
		a.mask_stride = C.int32_t(d.MaskStride)
	}
	return mk(C.SHV_OP_ATTN_DECODE, unsafe.Pointer(&a), C.sizeof_shv_attn_decode_args)
}

// QSAArgs are the fields of shv_qsa_index_args (indexerAt / selected / topK, llm/attn.go:247-443).
type QSAArgs struct {
	X, Gamma, W, QNorm, KNorm, Rope *Buffer
	IdxCache, Pooled                *Buffer
	Rows                            PassRows
	Work, Score, Mask               *Buffer
	NEmbd, IdxHeads, IdxDim         int
	TopK, Ratio, RopeDims, MaxCells int
	MaskStride                      int
	Eps                             float32
}

// QSAIndex makes the per-row selection mask of an attention layer with a compression ratio.
func QSAIndex(d QSAArgs) Op {
	var a C.shv_qsa_index_args
	a.x, a.gamma, a.w, a.q_norm, a.k_norm, a.rope = fp(d.X), fp(d.Gamma), fp(d.W), fp(d.QNorm), fp(d.KNorm), fp(d.Rope)
	a.idxcache, a.pooled = vp(d.IdxCache), fp(d.Pooled)
	a.pos, a.slot = ip(d.Rows.Pos), ip(d.Rows.Slot)
	a.work, a.score, a.mask = fp(d.Work), fp(d.Score), (*C.uint32_t)(vp(d.Mask))
	a.n_seq, a.seq_len, a.n_embd = C.int32_t(d.Rows.NSeq), C.int32_t(d.Rows.SeqLen), C.int32_t(d.NEmbd)
	a.idx_heads, a.idx_dim, a.top_k, a.ratio = C.int32_t(d.IdxHeads), C.int32_t(d.IdxDim), C.int32_t(d.TopK), C.int32_t(d.Ratio)
	a.rope_dims, a.max_cells, a.mask_stride, a.eps = C.int32_t(d.RopeDims), C.int32_t(d.MaxCells), C.int32_t(d.MaskStride), C.float(d.Eps)
	return mk(C.SHV_OP_QSA_INDEX, unsafe.Pointer(&a), C.sizeof_shv_qsa_index_args)
}

// RingRows copies count rows of n floats between two rings of projection rows addressed by the sequence's
// position (a long pass's ring and the sequence's own small one).
func RingRows(src, dst, pos *Buffer, srcSlots, dstSlots, stride, n, first, count int) Op {
	var a C.shv_ring_rows_args
	a.src, a.dst, a.pos = fp(src), fp(dst), ip(pos)
	a.src_slots, a.dst_slots, a.stride, a.n = C.int32_t(srcSlots), C.int32_t(dstSlots), C.int32_t(stride), C.int32_t(n)
	a.first, a.count = C.int32_t(first), C.int32_t(count)
	return mk(C.SHV_OP_RING_ROWS, unsafe.Pointer(&a), C.sizeof_shv_ring_rows_args)
}

// Embed gathers rows of the embedding table (Model.Embedding + HCGPU.UploadInit): ids[pos[0]..] when pos is given.
func Embed(table, ids, pos, x *Buffer, rows, nEmbd, vocab, typ int) Op {
	var a C.shv_embed_args
	a.table, a.ids, a.pos, a.x = vp(table), ip(ids), ip(pos), fp(x)
	a.n_tok, a.n_embd, a.vocab, a.x_stride, a._type = C.int32_t(rows), C.int32_t(nEmbd), C.int32_t(vocab), C.int32_t(nEmbd), C.int32_t(typ)
	return mk(C.SHV_OP_EMBED, unsafe.Pointer(&a), C.sizeof_shv_embed_args)
}

// Argmax is Argmax (llm/sample.go:359-367) over rows of logits; with ids and pos, one row's result is stored
// as the sequence's next token and its position advanced.
func Argmax(logits, best, ids, pos *Buffer, rows, n, stride, advance int) Op {
	var a C.shv_argmax_args
	a.logits, a.best, a.ids, a.pos = fp(logits), ip(best), ip(ids), ip(pos)
	a.n_rows, a.n, a.logits_stride, a.advance = C.int32_t(rows), C.int32_t(n), C.int32_t(stride), C.int32_t(advance)
	return mk(C.SHV_OP_ARGMAX, unsafe.Pointer(&a), C.sizeof_shv_argmax_args)
}

// Raw wraps an argument block the caller filled itself (shv_dn_step_args, shv_attn_decode_args,
// shv_embed_args, shv_argmax_args, shv_advance_args, shv_ring_rows_args): llm/gpu_deltanet.go and
// llm/gpu_attn.go build theirs field by field exactly as the functions above do.
func Raw(kind uint32, args unsafe.Pointer, n uintptr) Op { return mk(C.uint32_t(kind), args, C.size_t(n)) }

// DispatchMultiMarked is vk.DispatchMultiMarked (vk/engine.go:913): run the ops once, return the
// GPU time of the whole and of each op.
func (d *Device) DispatchMultiMarked(ops []Op) (total time.Duration, perOp []time.Duration, err error) {
	ns := make([]C.uint64_t, len(ops))
	var tot C.uint64_t
	err = call(func() C.int {
		return C.shv_dispatch_multi(d.ctx, (*C.shv_op)(unsafe.Pointer(&ops[0])), C.int(len(ops)), 1, &tot, &ns[0])
	})
	if err != nil {
		return 0, nil, err
	}
	perOp = make([]time.Duration, len(ops))
	for i, v := range ns {
		perOp[i] = time.Duration(v)
	}
	return time.Duration(tot), perOp, nil
}

// DispatchMultiTimed is vk.DispatchMultiTimed (vk/engine.go:893).
func (d *Device) DispatchMultiTimed(ops []Op, iters int) (time.Duration, error) {
	var tot C.uint64_t
	err := call(func() C.int {
		return C.shv_dispatch_multi(d.ctx, (*C.shv_op)(unsafe.Pointer(&ops[0])), C.int(len(ops)), C.int(iters), &tot, nil)
	})
	return time.Duration(tot), err
}

// Prerecorded is vk.Prerecorded (vk/engine.go:997-1086): the op list recorded once (a HIP graph).
type Prerecorded struct {
	dev *Device
	p   *C.shv_prerecorded
}

func (d *Device) NewPrerecorded(ops []Op) (*Prerecorded, error) {
	r := &Prerecorded{dev: d}
	err := call(func() C.int {
		return C.shv_prerecord(d.ctx, (*C.shv_op)(unsafe.Pointer(&ops[0])), C.int(len(ops)), &r.p)
	})
	if err != nil {
		return nil, err
	}
	return r, nil
}

// Submit replays iters times, waits, and returns the GPU time.
func (p *Prerecorded) Submit(iters int) (time.Duration, error) {
	var ns C.uint64_t
	err := call(func() C.int { return C.shv_prerecorded_submit(p.dev.ctx, p.p, C.int(iters), &ns) })
	return time.Duration(ns), err
}

// Launch replays once without waiting: decode steps queue back to back, the token feeds back on the device.
func (p *Prerecorded) Launch() error {
	return call(func() C.int { return C.shv_prerecorded_launch(p.dev.ctx, p.p) })
}

// Stamp marks the point the stream has reached (i in 0..3); StampElapsed is the GPU time between two stamps once the
// stream has been waited for: the time of work handed over with Launch.
func (d *Device) Stamp(i int) error { return call(func() C.int { return C.shv_stamp(d.ctx, C.int(i)) }) }
func (d *Device) StampElapsed(from, to int) (time.Duration, error) {
	var ns C.uint64_t
	err := call(func() C.int { return C.shv_stamp_elapsed(d.ctx, C.int(from), C.int(to), &ns) })
	return time.Duration(ns), err
}
func (p *Prerecorded) Count() int { return int(C.shv_prerecorded_count(p.p)) }
func (p *Prerecorded) Destroy()   { C.shv_prerecorded_destroy(p.dev.ctx, p.p); p.p = nil }
