//go:build shv_hip

// The MoE block's op list over package hip: what MoEGPU.graph (llm/gpu_moe.go:1695) builds as
// []vk.MultiDispatch — router GEMM, route, grouped or per-token GEMV twice, activation, combine,
// residual add — is three ops here.  The struct, its staging (stage, alloc) and its public methods
// (Upload, Run, Profile, Dispatches, llm/gpu_moe.go:1896-1990) stay as they are; only the arenas
// become hip.Buffers and graph() returns []hip.Op.
//
// NOT COMPILED IN THIS REPOSITORY (no Go toolchain in the build image).  MoEGPU::Dispatches in
// host/llm.cpp is this function in C++, compiled and tested against the oracle.
package llm

import (
	"fmt"

	"strix-halo-vulkan/hip"
)

// moeHIP is what MoEGPU holds when it is built over package hip instead of package vk.
type moeHIP struct {
	dev *hip.Device
	cfg Config
	// per layer: post_attention_norm, ffn_gate_inp, ffn_gate_inp_shexp and the six banks, as the
	// bytes of the GGUF tensors (no repacking: bank_q4.go's fragment tiling is not used)
	norm, router, sharedGate []*hip.Buffer
	banks                    []hip.MoEBanks
	// arenas for up to maxRows rows
	xn, logits, topk, weights, act *hip.Buffer
	group, pairs                   *hip.Buffer // workspaces of the grouped path; nil keeps every pass per (token, slot)
	rows                           int
	routeInUp                      bool // passes of one to four rows make their selection inside MoEUp (LLM_MOE_ROUTE=rows)
}

// graph is MoEGPU.graph for one layer: in and out are the residual stream's rows (out may be in).
func (g *moeHIP) graph(layer int, in, out *hip.Buffer) ([]hip.Op, []string, error) {
	if layer < 0 || layer >= len(g.banks) {
		return nil, nil, fmt.Errorf("llm: layer %d of %d", layer, len(g.banks))
	}
	c := g.cfg
	// Types is (gate, up, down, shared gate, shared up, shared down): the gate/up launch goes its
	// Q4_K road only when all four of its banks are Q4_K, the down launch only when both of its are
	ty := g.banks[layer].Types
	q4k := ty[0] == ggmlQ4K && ty[1] == ggmlQ4K && ty[3] == ggmlQ4K && ty[4] == ggmlQ4K
	downQ4K := ty[2] == ggmlQ4K && ty[5] == ggmlQ4K
	// passes of one to four rows route in the expert kernel itself; banks of another type take the router's selection
	fused := g.routeInUp && g.rows <= 4 && q4k
	var lg, wt, grp *hip.Buffer
	if fused {
		lg, wt = g.logits, g.weights
	} else {
		grp = g.group
	}
	ready := !fused && q4k && g.group != nil
	packed := ready && downQ4K && g.pairs != nil // both projections Q4_K, one right after the other: act goes over as operands
	ops := []hip.Op{
		hip.MoERouter(in, g.norm[layer], g.router[layer], g.sharedGate[layer], g.xn, g.logits, g.topk, g.weights,
			g.rows, c.NEmbd, c.NExpert, c.NExpertUsed, c.RMSEps, fused),
		hip.MoEUp(g.xn, g.topk, g.banks[layer], g.act, g.rows, c.NEmbd, c.NExpertUsed, c.FFNExpert, c.NExpert, lg, wt, grp, packed),
		hip.MoEDown(g.act, g.topk, g.weights, g.banks[layer], in, out, g.rows, c.NEmbd, c.NExpertUsed, c.FFNExpert, c.NExpert,
			g.group, g.pairs, ready, packed),
	}
	return ops, []string{"moe.router", "moe.up", "moe.down"}, nil
}

// Run is MoEGPU.Run (llm/gpu_moe.go:1903): one submission for the block, or none when the graph
// is recording a whole pass and takes the ops into its own list.
func (g *moeHIP) Run(layer int, in, out *hip.Buffer) error {
	ops, kinds, err := g.graph(layer, in, out)
	if err != nil {
		return err
	}
	if _, err := g.dev.DispatchMultiTimed(ops, 1); err != nil {
		return fmt.Errorf("llm: moe, %d ops (%v): %w", len(ops), kinds, err)
	}
	return nil
}

// Profile is MoEGPU.Profile (llm/gpu_moe.go:1930): the GPU time of each op.
func (g *moeHIP) Profile(layer int, in, out *hip.Buffer) ([]Stage, error) {
	ops, kinds, err := g.graph(layer, in, out)
	if err != nil {
		return nil, err
	}
	_, per, err := g.dev.DispatchMultiMarked(ops)
	if err != nil {
		return nil, err
	}
	st := make([]Stage, len(ops))
	for i := range ops {
		st[i] = Stage{Kind: kinds[i], GPU: per[i]}
	}
	return st, nil
}

const ggmlQ4K = 12 // gguf.TypeQ4_K
