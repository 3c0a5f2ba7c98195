/*
 * shv_oracle.h — CPU restatement of strix-halo-vulkan's Go/CPU reference for the
 * language-model token loop.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test suite, the smoke
 * check and the benchmark's CPU-baseline leg may call it, and only as the checker
 * or the reported baseline; the HIP library never links or loads it.
 *
 * Every function follows one function of the reference (cited file:line, paths
 * relative to the reference tree).  Arithmetic is kept at the reference's widths:
 * float32 accumulators stay float32, sums the reference takes in float64 stay
 * float64, exp/sigmoid go through double and are rounded once.  Build with
 * -ffp-contract=off: the reference runs on amd64, where Go never fuses a
 * multiply-add.
 *
 * Pinning (what fixes each function besides having been read):
 *   f32_to_f16 / f16_to_f32 / f16_round   golden table f32_to_f16.txt (10 575 pairs) + all 65 536 halves
 *   scale_min_k4 / dequant_q4k            ggml to_float vectors (dequant_q4k_{in,ref}.bin), bit-exact
 *   quantize_q4k                          ggml quantize_chunk vectors (quant_q4k_{in,ref}.bin), bit-exact
 *   matvec / gemv_q4k                     float64 dot product, brute force
 *   softmax / route                       closed forms, constructed ties, numpy on tie-free input
 *   moe_block                             dense brute force over dequantised experts
 *   rmsnorm / head_norm / silu / sigmoid / softplus   float64 libm + the two softplus edge cases
 *   deltanet_layer / delta_rule           chunk-split bit-identity, closed form (g=0, beta=1,
 *                                         orthonormal k), independent float64 recurrence
 *   rope / attn_layer                     textbook NeoX rotation, independent float64 attention
 *   argmax                                numpy.argmax + constructed ties
 * The reference holds no golden vector for route, moe_block, deltanet_layer,
 * attn_layer, rope or argmax that can be used without its 111 GB checkpoint, so
 * for those the restatement is pinned by mathematics only: "parity unpinned"
 * against reference-held vectors.
 */
#ifndef SHV_ORACLE_H
#define SHV_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SHV_Q4K_BLOCK 256      /* weights in a super-block */
#define SHV_Q4K_BYTES 144      /* bytes in a super-block   */

/* ---- IEEE binary16, safetensors/safetensors.go:425-496, llm/hc.go:318-360 ---- */
uint16_t shv_ref_f32_to_f16(float f);
float    shv_ref_f16_to_f32(uint16_t h);
float    shv_ref_f16_round(float x);

/* ---- Q4_K, gguf/dequant.go:238-276 ---- */
void shv_ref_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m);
void shv_ref_dequant_q4k(const uint8_t *data, int64_t nblocks, float *dst);
/* ggml type numbers of the tensor types the loader accepts (gguf/gguf.go, gguf/dequant.go:103-110) */
enum {
    SHV_GGML_F32 = 0, SHV_GGML_F16 = 1, SHV_GGML_Q4_1 = 3, SHV_GGML_Q5_0 = 6, SHV_GGML_Q5_1 = 7, SHV_GGML_Q8_0 = 8,
    SHV_GGML_Q4_K = 12, SHV_GGML_Q5_K = 13, SHV_GGML_Q6_K = 14, SHV_GGML_IQ4_NL = 20, SHV_GGML_BF16 = 30
};
int64_t shv_ref_type_bytes(int type, int64_t n);
/* y = W x, rows of W in any accepted type (0 = Q4_K): DequantizeRow then llm/hc.go:255-264 */
int shv_ref_gemv_any(float *y, int type, const uint8_t *w, const float *x, int n, int k, int threads);
int shv_ref_dequant(int type, const uint8_t *data, int64_t n, float *dst);

/* ---- Q4_K quantiser (round-to-nearest arm), llm/quantk.go:115-179, llm/sim.go:982-1060,
 *      llm/quantk.go:211-226, llm/moebank.go:489-532 ---- */
float shv_ref_make_qkx_quants(const float *x, int n, int nmax, const float *w, uint8_t *lv,
                              uint8_t *laux, float rmin, float rdelta, int nstep, float *the_min);
void  shv_ref_quantize_q4k_row(const float *row, int64_t k, uint8_t *dst);
/* rows in parallel (OpenMP); each row is quantised exactly as above */
void  shv_ref_quantize_q4k(const float *w, int64_t rows, int64_t k, uint8_t *dst);

/* ---- dense helpers, llm/hc.go:176-190,255-268, llm/deltanet.go:450-455, llm/attn.go:510-522 ---- */
void  shv_ref_matvec(float *y, const float *w, const float *x, int n, int k);
/* y = W x for Q4_K rows: dequantise a row (gguf/dequant.go:119-124) then the sequential
 * float32 dot of matvec.  threads<=1 is the reference's single goroutine; larger values
 * split the ROWS into one contiguous chunk per thread (llm/hc.go:232-252), same values. */
void  shv_ref_gemv_q4k(float *y, const uint8_t *w, const float *x, int n, int k, int threads);
float shv_ref_sigmoid(float x);
float shv_ref_silu(float x);
float shv_ref_softplus(float x);
void  shv_ref_rmsnorm(float *dst, const float *src, const float *gamma, int n, float eps);
void  shv_ref_head_norm(float *x, const float *gamma, int dim, int n, float eps);
int32_t shv_ref_argmax(const float *logits, int64_t n);  /* llm/sample.go:359-367 */

/* ---- MoE block, llm/moe.go:215-461 ---- */
typedef struct {
    int n_embd, n_expert, n_used, ffn_expert, ffn_shared;
} shv_ref_moe_cfg;

typedef struct {
    const float   *router;       /* [n_expert][n_embd] f32 */
    const float   *shared_gate;  /* [n_embd] f32 */
    const uint8_t *gate_exps;    /* Q4_K rows: expert e row j = e*ffn_expert + j, n_embd long */
    const uint8_t *up_exps;      /* same */
    const uint8_t *down_exps;    /* Q4_K rows: e*n_embd + j, ffn_expert long */
    const uint8_t *gate_sh, *up_sh, *down_sh;  /* shared expert, same shapes for one expert */
    int types[6];                /* ggml type of gate_exps, up_exps, down_exps, gate_sh, up_sh, down_sh; 0 = Q4_K */
} shv_ref_moe_w;

void shv_ref_softmax(float *dst, const float *src, int n);
/* Route: logits/probs [T][n_expert], topk [T][n_used], weights_norm [T][n_used]. */
void shv_ref_moe_route(const shv_ref_moe_cfg *c, const shv_ref_moe_w *w, const float *x, int n_tok,
                       float *logits, float *probs, int32_t *topk, float *weights_norm);
/* Whole block over every token.  Optional traces may be NULL:
 * swiglu [T][n_used][ffn], moe_out [T][n_embd] (routed half only), sh_gate_sig [T]. */
void shv_ref_moe_block(const shv_ref_moe_cfg *c, const shv_ref_moe_w *w, const float *x, int n_tok,
                       float *out, float *logits, int32_t *topk, float *weights_norm,
                       float *swiglu, float *moe_out, float *sh_gate_sig, int threads);

/* ---- gated DeltaNet layer, llm/deltanet.go:212-455 ---- */
typedef struct {
    int n_embd, head_dim, n_head_k, n_head_v, conv;
    float eps;
    int qk_norm_max;  /* 0 = L2Rsqrt (the model), 1 = L2Max (ggml_l2_norm) */
} shv_ref_dn_cfg;

typedef struct {
    const uint8_t *qkv;    /* Q4_K [2*hk*d + hv*d][n_embd] */
    const uint8_t *z;      /* Q4_K [hv*d][n_embd] */
    const uint8_t *alpha;  /* Q4_K [hv][n_embd] */
    const uint8_t *beta;   /* Q4_K [hv][n_embd] */
    const uint8_t *out;    /* Q4_K [n_embd][hv*d] */
    const float *conv1d;   /* [conv_width][conv] */
    const float *a;        /* [hv]  (already -exp(A_log)) */
    const float *dt_bias;  /* [hv] */
    const float *norm;     /* [d] */
} shv_ref_dn_w;

/* state_conv [conv_width][conv-1] (column 0 oldest), state_s [hv][d][d] holding S[i][j] at
 * [j*d+i]; both advanced in place.  Optional traces (NULL to skip): qkv_mixed [T][cw],
 * qnorm/knorm [T][hk][d], gate/beta_sig [T][hv], attn_out [T][hv][d], final [T][hv*d].
 * head_map_divide=1 swaps the reference's h%hk map for h/(hv/hk): the negative control
 * of llm/deltanet_test.go:234-268. */
void shv_ref_deltanet_layer(const shv_ref_dn_cfg *c, const shv_ref_dn_w *w, const float *xn,
                            int n_tok, float *state_conv, float *state_s, float *result,
                            float *qkv_mixed, float *qnorm, float *knorm, float *gate,
                            float *beta_sig, float *attn_out, float *final_out,
                            int head_map_divide, int threads);
/* the recurrence alone on prepared q,k,v,gate,beta (llm/deltanet.go:365-403) */
void shv_ref_delta_rule(int d, int n_head_k, int n_head_v, int n_tok, const float *qnorm,
                        const float *knorm, const float *v, const float *gate,
                        const float *beta_sig, float *state_s, float *out, const int *k_of);

/* ---- gated full attention, dense path, llm/attn.go:135-219,444-586 ---- */
typedef struct {
    int n_embd, n_head, n_head_kv, head_dim, rope_dims;
    float rope_base;
    int sections[4];
    float eps;
    /* the block-sparse indexer beside the layer (llm/attn.go:56-68): ratio 0 is a dense layer */
    int idx_heads, idx_dim, top_k, ratio;
} shv_ref_attn_cfg;

typedef struct {
    const uint8_t *q;   /* Q4_K [n_head*2*d][n_embd]: per head d query rows then d gate rows */
    const uint8_t *k;   /* Q4_K [n_head_kv*d][n_embd] */
    const uint8_t *v;   /* Q4_K [n_head_kv*d][n_embd] */
    const uint8_t *o;   /* Q4_K [n_embd][n_head*d] */
    const float *q_norm, *k_norm;  /* [d] */
    /* the indexer's tensors (llm/attn.go:90-93), float32: never quantised in the reference either */
    const float *idx_q;            /* [idx_heads*idx_dim][n_embd] */
    const float *idx_k;            /* [idx_dim][n_embd] */
    const float *idx_q_norm, *idx_k_norm;  /* [idx_dim] */
} shv_ref_attn_w;

/* x is [n_tok][n_heads][head_dim], rotated in place at text positions pos[t]. */
void shv_ref_rope(const shv_ref_attn_cfg *c, float *x, const int32_t *pos, int n_heads,
                  int head_dim, int n_tok);
/* n_tok new rows at positions past..past+n_tok-1 over an fp16 cache that already holds
 * `past` cells.  kcache/vcache are [cells][n_head_kv][head_dim] binary16 bit patterns; the
 * new rows' K (after norm and rope) and V are rounded to halves and appended, then each row
 * attends causally to cells 0..its own.  With past=0 this is AttnLayerAt under exact
 * matvecs and the fp16-cache arm of llm/attn.go:176-184.  Optional traces: q_rot
 * [T][n_head][d], pregate [T][n_head*d]. */
void shv_ref_attn_layer(const shv_ref_attn_cfg *c, const shv_ref_attn_w *w, const float *xn,
                        int n_tok, int past, uint16_t *kcache, uint16_t *vcache, float *out,
                        float *q_rot, float *pregate, int threads);

/* ---- the block-sparse indexer, llm/attn.go:221-443 (indexerAt, selected) and :588-682 (topK,
 * topKThreshold, f2ui) ----
 * The radix select: the key of the n-th largest of x[0..len) under the order-preserving map f2ui,
 * by four 8-bit histogram passes (llm/attn.go:637-670). */
uint32_t shv_ref_f2ui(float v);
uint32_t shv_ref_topk_threshold(const float *x, int len, int n);
/* The selection itself (llm/attn.go:615-632): every index strictly above the threshold in
 * ascending order, then indices equal to it in ascending order until n are taken.  sel receives
 * min(n, len) indices; returns how many of them are strictly above. */
int shv_ref_topk(const float *x, int len, int n, int32_t *sel);
/* The layer with its indexer (cfg.ratio > 0), generalised like shv_ref_attn_layer to a cache that
 * already holds `past` cells: with past = 0 this is AttnLayerAt with Ratio > 0 under exact
 * matvecs, the fp16 KV cache and the fp16 indexer-key cache (llm/attn.go:273-285; the reference
 * couples those roundings and its int8 activations under one switch, which is split here as for
 * the dense layer; the scores are formed in float32, the Exact arm of :330-356).
 * idxcache is [n_kv][idx_dim] binary16: the raw indexer keys, appended like K and V.  n_kv is the
 * padded cell count the block structure, bias and top-k width are cut against (:124-133).
 * Row i (position p = past + i) sees the cells its selection names among 0..p.
 * Optional traces: topk [n_tok][width] ascending cell lists (width = min(top_k + ratio - 1, n_kv)),
 * above [n_tok], score [n_tok][ceil(n_kv/ratio)] the pre-bias block scores. */
void shv_ref_attn_layer_qsa(const shv_ref_attn_cfg *c, const shv_ref_attn_w *w, const float *xn,
                            int n_tok, int past, uint16_t *kcache, uint16_t *vcache, uint16_t *idxcache,
                            int n_kv, float *out, float *q_rot, float *pregate, int32_t *topk,
                            int32_t *above, float *score, int threads);

/* ---- the token loop over the synthetic Qwen3-Next-shape model ----
 * The reference's loop body is llm/graph.go:2330-2466 (per layer: mix -> DeltaNet or attention ->
 * combine -> mix -> MoE -> combine; then the head, :1762) and its driver cmd/llm/generate.go:121-165
 * (prefill, Argmax, extend).  BASELINE's model has no hyper-connection streams, so "mix" is a plain
 * RMSNorm (llm/hc.go:176-190 with hc=1) and "combine" a residual add:
 *     x = float32(embd[id])
 *     x += Block_l(RMSNorm(x, attn_norm_l))     Block = DeltaNet, or attention on every attn_every-th layer
 *     x += MoE_l(RMSNorm(x, ffn_norm_l))
 *     logits = lm_head * RMSNorm(x, out_norm)
 * The composition is this repository's reading of that shape: "parity unpinned" against any
 * reference-held vector, like the blocks it is made of. */
typedef struct {
    int n_layer, n_embd, vocab;
    int attn_every;      /* layer l is full attention when (l+1) % attn_every == 0 */
    float eps;
    int max_cells;       /* KV cache capacity per attention layer */
    shv_ref_moe_cfg moe;
    shv_ref_dn_cfg dn;
    shv_ref_attn_cfg attn;
} shv_ref_model_cfg;

typedef struct {
    const float *attn_norm;  /* [n_embd] */
    const float *ffn_norm;   /* [n_embd] */
    shv_ref_dn_w dn;         /* used on DeltaNet layers   */
    shv_ref_attn_w attn;     /* used on attention layers  */
    shv_ref_moe_w moe;
} shv_ref_layer_w;

typedef struct {
    const uint16_t *embd;    /* binary16 [vocab][n_embd] */
    const float *out_norm;   /* [n_embd] */
    const uint8_t *lm_head;  /* Q4_K [vocab][n_embd] */
    const shv_ref_layer_w *layers;
} shv_ref_model_w;

/* Per-layer state; entries of the other kind of layer are NULL. */
typedef struct {
    float **dn_conv;      /* [n_layer] -> [conv_width][conv-1] */
    float **dn_s;         /* [n_layer] -> [hv][d][d] */
    uint16_t **kcache;    /* [n_layer] -> [max_cells][n_head_kv][head_dim] */
    uint16_t **vcache;
    int past;             /* tokens already in the sequence */
    uint16_t **idxcache;  /* [n_layer] -> [max_cells][idx_dim], attention layers of a model with an indexer; else NULL */
} shv_ref_model_state;

/* Extend the sequence by n_tok tokens (Graph.Extend, llm/graph.go:1709-1777): logits [vocab] and
 * hidden [n_embd] (the residual stream before the final norm) of the LAST row; either may be NULL. */
void shv_ref_model_extend(const shv_ref_model_cfg *c, const shv_ref_model_w *w, shv_ref_model_state *st,
                          const int32_t *ids, int n_tok, float *logits, float *hidden, int threads);
/* The same pass with EVERY row's logits [n_tok][vocab] and residual [n_tok][n_embd] (Graph.ExtendRows,
 * llm/graph.go:1383-1429: the verification pass of the speculative loop); either may be NULL. */
void shv_ref_model_extend_rows(const shv_ref_model_cfg *c, const shv_ref_model_w *w, shv_ref_model_state *st,
                               const int32_t *ids, int n_tok, float *logits_rows, float *hidden_rows, int threads);

/* ---- the draft head (MTPHead.Rows, llm/mtp.go:31-53,542-673) for a model without hyper-connection
 * streams, which is qwen3next's wiring as llm/mtp.go:31-33 names it:
 *     x   = eh_proj . concat(RMSNorm(embd(id), enorm), RMSNorm(h, hnorm))
 *     x  += Attn(RMSNorm(x, attn_norm))        one full-attention block with a KV cache of its own
 *     x  += MoE(RMSNorm(x, ffn_norm))
 *     logits = lm_head . RMSNorm(x, shared_head_norm)      (the trunk's lm_head)
 * hs is [n_tok][n_embd], the residual behind each row; rows sit at positions pos..pos+n_tok-1 of the
 * draft's own cache.  res receives every row's x, logits the LAST row's.  "parity unpinned": the
 * reference's own wiring is for its four-stream model and has no numerical oracle either
 * (llm/mtp.go:23-29); this composition is pinned only through the blocks it is made of. */
typedef struct {
    const float *enorm, *hnorm;   /* [n_embd] */
    const uint8_t *eh_proj;       /* Q4_K [n_embd][2*n_embd] */
    const float *head_norm;       /* [n_embd] */
    shv_ref_layer_w layer;        /* attention weights, norms and MoE of the draft block */
} shv_ref_mtp_w;

void shv_ref_mtp_rows(const shv_ref_model_cfg *c, const shv_ref_model_w *w, const shv_ref_mtp_w *mw,
                      uint16_t *kcache, uint16_t *vcache, const float *hs, const int32_t *ids, int n_tok,
                      int pos, float *logits, float *res, int threads);

#ifdef __cplusplus
}
#endif
#endif
