//go:build shv_hip

// The other three blocks' op lists and the pass that strings them together, over package hip: what
// DeltaNetGPU.graph (llm/gpu_deltanet.go:1268), AttnGPU.graph (llm/gpu_attn.go:2200), HeadGPU.graph
// (llm/gpu_head.go:433) and Graph.layers / extendPrerecorded (llm/graph.go:2330, :1791-1890) build as
// []vk.MultiDispatch.  As in gpu_moe_hip.go the structs, their staging and their public methods stay;
// the arenas become hip.Buffers and graph() returns []hip.Op.
//
// NOT COMPILED IN THIS REPOSITORY (no Go toolchain in the build image).  DeltaNetGPU::Dispatches,
// AttnGPU::Dispatches, HeadGPU::DispatchesTo and Graph::pass in host/llm.cpp are these functions in
// C++, compiled and tested against the oracle.
package llm

import (
	"fmt"

	"strix-halo-vulkan/hip"
)

// fold names a layer's router table and where the logits go, when the router's rows ride on the
// mixer's output projection (MoEGPU::FoldInto in host/llm.cpp); the zero value leaves them out.
type fold struct {
	table, out   *hip.Buffer
	rows, stride int
}

// deltanetHIP is what DeltaNetGPU holds when it is built over package hip.
type deltanetHIP struct {
	dev *hip.Device
	cfg Config
	// per layer: ssm_in_fused (q | k | v | z | alpha | beta rows of one Q4_K matrix), attn_norm, ssm_conv1d,
	// ssm_a, ssm_dt, ssm_norm, ssm_out, the projection ring [slots][ringSlots][width] and the state
	// [slots][planes][hv][d][d]
	inFused, attnNorm, conv1d, a, dt, norm, out []*hip.Buffer
	ring, state                                 []*hip.Buffer
	attn, row                                   *hip.Buffer // the rule's raw output; the one-row pass's projection row at a fixed address
	plane                                       *hip.Buffer // device int32 per slot: the committed plane (rewindable passes)
	bigRing, work                               *hip.Buffer // a long pass's ring and the chunked rule's scratch; nil without them
	ringSlots, bigSlots, planes                 int
}

const smallPass = 16 // rows up to which a pass writes the sequence's own ring (kSmallPass in host/llm.cpp)

// graph is DeltaNetGPU.graph for one layer and one pass: in-projection with the RMSNorm prologue into the
// ring, the gated delta rule, out-projection with the gated-norm prologue and the residual.
func (g *deltanetHIP) graph(layer int, in, out *hip.Buffer, r hip.PassRows, f fold) ([]hip.Op, []string, error) {
	if layer < 0 || layer >= len(g.inFused) || g.state[layer] == nil {
		return nil, nil, fmt.Errorf("llm: layer %d is not a DeltaNet layer", layer)
	}
	c := g.cfg
	rows := r.NSeq * r.SeqLen
	if r.Spec && r.SeqLen >= g.planes {
		return nil, nil, fmt.Errorf("llm: a rewindable pass of %d rows needs %d state planes, %d are staged", r.SeqLen, r.SeqLen+1, g.planes)
	}
	width := c.DNFusedRows()
	big := rows > smallPass
	if big && (r.NSeq != 1 || r.Spec || g.bigRing == nil) {
		return nil, nil, fmt.Errorf("llm: a pass of %d rows is one sequence's plain prompt chunk", rows)
	}
	ring, ringSlots := g.ring[layer], g.ringSlots
	if big {
		ring, ringSlots = g.bigRing, g.bigSlots
	}
	flat := rows == 1
	p := hip.GemvOpts{Prologue: hip.ProRMSNorm, Gamma: g.attnNorm[layer], Eps: c.RMSEps, Pos: r.Pos, Slot: r.Slot,
		XStride: c.NEmbd, YStride: width, SeqLen: r.SeqLen, RingSlots: ringSlots, RingStride: width}
	if flat {
		p.YFlat = g.row // the out projection then finds its gate without waiting for the position word
	}
	step := hip.DNStepArgs{Ring: ring, Conv1D: g.conv1d[layer], A: g.a[layer], DtBias: g.dt[layer], State: g.state[layer], Out: g.attn,
		Rows: r, HeadK: c.SSMHeadK, HeadV: c.SSMHeadV, HeadDim: c.SSMHeadDim, Conv: c.SSMConv, RingSlots: ringSlots, RingStride: width,
		Eps: c.RMSEps, Plane: g.plane, Planes: g.planes, Work: g.work}
	o := hip.GemvOpts{Prologue: hip.ProGatedNorm, Gamma: g.norm[layer], Residual: in, Eps: c.RMSEps, HeadDim: c.SSMHeadDim,
		XStride: c.VWidth(), YStride: c.NEmbd, Fold: f.table, FoldOut: f.out, FoldRows: f.rows, FoldStride: f.stride}
	if flat {
		o.Z, o.ZStride = g.row.Slice(uint64(c.ConvWidth())*4, uint64(c.VWidth())*4), width
	} else {
		o.Z = ring.Slice(uint64(c.ConvWidth())*4, ring.Size()-uint64(c.ConvWidth())*4)
		o.Pos, o.Slot, o.SeqLen, o.RingSlots, o.RingStride, o.ZRing = r.Pos, r.Slot, r.SeqLen, ringSlots, width, true
	}
	ops := []hip.Op{
		hip.GemvQ4K(g.inFused[layer], in, ring, width, c.NEmbd, rows, p),
		hip.DNStep(step),
		hip.GemvQ4K(g.out[layer], g.attn, out, c.NEmbd, c.VWidth(), rows, o),
	}
	kinds := []string{"dn.qkv", "dn.step", "dn.out"}
	if big {
		// the conv's history into the pass's ring, and the pass's last rows back into the sequence's own
		hist := c.SSMConv - 1
		ops = []hip.Op{hip.RingRows(g.ring[layer], g.bigRing, r.Pos, g.ringSlots, g.bigSlots, width, c.ConvWidth(), -hist, hist), ops[0], ops[1],
			hip.RingRows(g.bigRing, g.ring[layer], r.Pos, g.bigSlots, g.ringSlots, width, c.ConvWidth(), rows-hist, hist), ops[2]}
		kinds = []string{"dn.hist", "dn.qkv", "dn.step", "dn.hist", "dn.out"}
	}
	return ops, kinds, nil
}

// attnHIP is what AttnGPU holds when it is built over package hip.
type attnHIP struct {
	dev *hip.Device
	cfg Config
	// per layer: attn_qkv_fused (q|gate per head, then k, then v), attn_norm, attn_q_norm, attn_k_norm,
	// attn_output, the caches K [slot][cell][kv head][dim] and V in 32-cell tiles, both binary16
	qkvFused, attnNorm, qNorm, kNorm, out []*hip.Buffer
	kc, vc                                []*hip.Buffer
	// with a compression ratio: the indexer's fused q|k projection (float32), its norms, key cache and pooled blocks
	idxW, idxQNorm, idxKNorm, idxCache, pooled []*hip.Buffer
	qsaWork, qsaScore, qsaMask                 *hip.Buffer
	maskStride                                 int
	qkv, ctx, partial, rope                    *hip.Buffer
	nKV, splits                                int
}

// graph is AttnGPU.graph for one layer and one pass: fused projection with the RMSNorm prologue, (the
// indexer,) attention with head norms, rotation, cache write and split scores, out-projection with the
// sigmoid gate and the residual.
func (g *attnHIP) graph(layer int, in, out *hip.Buffer, r hip.PassRows, f fold) ([]hip.Op, []string, error) {
	if layer < 0 || layer >= len(g.kc) || g.kc[layer] == nil {
		return nil, nil, fmt.Errorf("llm: layer %d is not an attention layer staged here", layer)
	}
	c := g.cfg
	rows := r.NSeq * r.SeqLen
	width := c.AttnFusedRows()
	ops := []hip.Op{hip.GemvQ4K(g.qkvFused[layer], in, g.qkv, width, c.NEmbd, rows,
		hip.GemvOpts{Prologue: hip.ProRMSNorm, Gamma: g.attnNorm[layer], Eps: c.RMSEps, XStride: c.NEmbd, YStride: width})}
	kinds := []string{"attn.qkv"}
	a := hip.AttnArgs{QKV: g.qkv, QNorm: g.qNorm[layer], KNorm: g.kNorm[layer], Rope: g.rope, KCache: g.kc[layer], VCache: g.vc[layer],
		Partial: g.partial, Out: g.ctx, Rows: r, NHead: c.NHead, NHeadKV: c.NHeadKV, HeadDim: c.HeadDim, RopeDims: c.RopeDims,
		MaxCells: g.nKV, QKVStride: width, Splits: g.splits, Eps: c.RMSEps}
	if g.idxCache != nil && g.idxCache[layer] != nil {
		ops = append(ops, hip.QSAIndex(hip.QSAArgs{X: in, Gamma: g.attnNorm[layer], W: g.idxW[layer], QNorm: g.idxQNorm[layer],
			KNorm: g.idxKNorm[layer], Rope: g.rope, IdxCache: g.idxCache[layer], Pooled: g.pooled[layer], Rows: r, Work: g.qsaWork,
			Score: g.qsaScore, Mask: g.qsaMask, NEmbd: c.NEmbd, IdxHeads: c.IdxHeads, IdxDim: c.IdxDim, TopK: c.IdxTopK, Ratio: c.IdxRatio,
			RopeDims: c.RopeDims, MaxCells: g.nKV, MaskStride: g.maskStride, Eps: c.RMSEps}))
		kinds = append(kinds, "attn.index")
		a.Mask, a.MaskStride = g.qsaMask, g.maskStride
	}
	ops = append(ops, hip.AttnDecode(a), hip.GemvQ4K(g.out[layer], g.ctx, out, c.NEmbd, c.NHead*c.HeadDim, rows,
		hip.GemvOpts{Prologue: hip.ProMulSigmoid, Z: g.qkv, Residual: in, HeadDim: c.HeadDim, XStride: c.NHead * c.HeadDim,
			YStride: c.NEmbd, ZStride: width, Fold: f.table, FoldOut: f.out, FoldRows: f.rows, FoldStride: f.stride}))
	return ops, append(kinds, "attn.attn", "attn.out"), nil
}

// headHIP is what HeadGPU holds when it is built over package hip.
type headHIP struct {
	cfg                     Config
	outputNorm, output      *hip.Buffer // output_norm, the Q4_K vocabulary projection
	logits, best, ids, pos  *hip.Buffer
}

// graph is HeadGPU.graph: the vocabulary projection with the final norm as its prologue.  A decode step's
// one row also names the next token in the same launch (what Argmax and SetPast do on the host in the
// reference); other passes take the arg-max of their rows as an op of its own.
func (g *headHIP) graph(in *hip.Buffer, rows int, sample bool) ([]hip.Op, []string) {
	c := g.cfg
	o := hip.GemvOpts{Prologue: hip.ProRMSNorm, Gamma: g.outputNorm, Eps: c.RMSEps, XStride: c.NEmbd, YStride: c.VocabSize}
	if sample && rows == 1 {
		o.AmaxBest, o.AmaxIds, o.AmaxPos, o.AmaxAdvance = g.best, g.ids, g.pos, 1
		return []hip.Op{hip.GemvQ4K(g.output, in, g.logits, c.VocabSize, c.NEmbd, 1, o)}, []string{"head"}
	}
	ops := []hip.Op{hip.GemvQ4K(g.output, in, g.logits, c.VocabSize, c.NEmbd, rows, o)}
	if !sample {
		return ops, []string{"head"}
	}
	return append(ops, hip.Argmax(g.logits, g.best, nil, nil, rows, c.VocabSize, c.VocabSize, 0)), []string{"head", "argmax"}
}

// graphHIP is the part of Graph that records a pass: the blocks, the residual stream x (and the second
// row buffer x2 the folded router needs: its projection reads the whole residual row while it writes),
// the token ids and positions on the device.
type graphHIP struct {
	dev       *hip.Device
	cfg       Config
	dn        *deltanetHIP
	attn      *attnHIP
	moe       *moeHIP
	head      *headHIP
	embd      *hip.Buffer // token_embd in the checkpoint's own type
	embdType  int
	x, x2     *hip.Buffer
	ids, pos  *hip.Buffer
	foldTable []*hip.Buffer // per layer, made once by hip.RouterFold when the graph is staged; nil: the router keeps its launch
	logits    *hip.Buffer   // the MoE block's router logits, rows of n_expert + 1 floats
}

// layers is Graph.layers (llm/graph.go:2330) without hyper-connection streams: per layer the mixer on
// RMSNorm(x) and the MoE block on RMSNorm(x), each adding to x.  One to four rows (of one sequence or one each of several) with a
// folded router take the two-op MoE block; everything else the three-op one.
func (g *graphHIP) layers(r hip.PassRows) ([]hip.Op, []string, error) {
	c := g.cfg
	rows := r.NSeq * r.SeqLen
	ops := []hip.Op{hip.Embed(g.embd, g.ids, g.pos, g.x, rows, c.NEmbd, c.VocabSize, g.embdType)}
	kinds := []string{"embed"}
	for l := 0; l < c.NLayer; l++ {
		folded := g.foldTable != nil && g.foldTable[l] != nil && rows <= 4
		var f fold
		mixOut := g.x
		if folded {
			f = fold{table: g.foldTable[l], out: g.logits, rows: c.NExpert, stride: c.NExpert + 1}
			mixOut = g.x2
		}
		var sub []hip.Op
		var names []string
		var err error
		if c.IsAttn(l) {
			sub, names, err = g.attn.graph(l, g.x, mixOut, r, f)
		} else {
			sub, names, err = g.dn.graph(l, g.x, mixOut, r, f)
		}
		if err != nil {
			return nil, nil, err
		}
		ops, kinds = append(ops, sub...), append(kinds, names...)
		g.moe.rows = rows
		ffn, names, err := g.moe.graph(l, mixOut, g.x)
		if err != nil {
			return nil, nil, err
		}
		if folded {
			// the router's launch goes; gate/up takes the un-normalised row, normalises it, scales the logits
			// by the same factor and forms the shared expert's gate
			ffn = []hip.Op{ffn[1].WithNorm(hip.MoENorm{Gamma: g.moe.norm[l], SharedGate: g.moe.sharedGate[l], Eps: c.RMSEps}), ffn[2]}
			names = names[1:]
		}
		ops, kinds = append(ops, ffn...), append(kinds, names...)
	}
	return ops, kinds, nil
}

// record is Graph.record + extendPrerecorded (llm/graph.go:312, :1791-1890) for the decode step: one
// recorded sequence whose every replay consumes ids[pos] and stores ids[pos+1], so K tokens are K
// submissions with no host work in between.
func (g *graphHIP) record() (*hip.Prerecorded, error) {
	r := hip.PassRows{NSeq: 1, SeqLen: 1, Pos: g.pos}
	ops, _, err := g.layers(r)
	if err != nil {
		return nil, err
	}
	head, _ := g.head.graph(g.x, 1, true)
	return g.dev.NewPrerecorded(append(ops, head...))
}
