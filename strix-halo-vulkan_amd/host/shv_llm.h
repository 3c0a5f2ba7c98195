/*
 * shv_llm.h — flat C entry points over the C++ host layer (llm.hpp), so that tests and the
 * benchmark can drive llm::Graph from ctypes.  This is the harness's door into the host layer,
 * not the drop-in boundary: the boundary is include/shv_hip.h, which this layer itself calls.
 * Every function returns 0 on success, -1 otherwise with shvllm_last_error() set.
 */
#ifndef SHV_LLM_H
#define SHV_LLM_H

#include <stdint.h>

#include "shv_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct shvllm shvllm;

typedef struct {
    int32_t n_layer, n_embd, n_head, n_head_kv, head_dim, rope_dims;
    float rope_base;
    int32_t n_expert, n_expert_used, ffn_expert, vocab;
    float rms_eps;
    int32_t ssm_head_dim, ssm_head_k, ssm_head_v, ssm_conv, attn_every;
    int32_t nkv, layers, no_head, attn_splits;   /* GraphOpts: cells, layer truncation, head, slices */
    int32_t max_tokens, slots, head_rows;        /* GraphOpts: rows a pass, sequences, rows with logits */
    int32_t speculative, spec_rows;              /* GraphOpts: rewindable passes and their width */
    int32_t nextn;                               /* 1: the model carries the draft block */
} shvllm_config;

const char *shvllm_last_error(void);
int shvllm_open(int device, const shvllm_config *cfg, shvllm **out);  /* device + model (unset weights) */
void shvllm_close(shvllm *h);
shv_ctx *shvllm_ctx(shvllm *h);
int shvllm_init_synthetic(shvllm *h, uint64_t seed);
int shvllm_tensor_count(shvllm *h);
int shvllm_tensor_at(shvllm *h, int i, const char **name, void **dptr, uint64_t *bytes, int32_t *kind,
                     int64_t *rows, int64_t *cols, int32_t *is_alias);
int shvllm_tensor(shvllm *h, const char *name, void **dptr, uint64_t *bytes);
uint64_t shvllm_weight_bytes(shvllm *h);
int shvllm_stage(shvllm *h);   /* NewGraph: allocate state, record the decode step */
int shvllm_reset(shvllm *h);
int shvllm_extend(shvllm *h, const int32_t *ids, int n, float *logits, float *hidden);
int shvllm_generate(shvllm *h, int n, int32_t *out_ids, uint64_t *gpu_nanos);
int shvllm_past(shvllm *h);
int shvllm_dispatches(shvllm *h);
/* one timed decode step: up to max entries of (label, nanoseconds); returns the count in *n */
int shvllm_profile_step(shvllm *h, char (*labels)[32], uint64_t *nanos, int max, int *n);
/* read-backs for parity checks */
int shvllm_dn_state(shvllm *h, int layer, float *dst);                   /* [hv][d][d] */
int shvllm_kv(shvllm *h, int layer, int cells, uint16_t *k, uint16_t *v); /* [cells][nkv][d] halves */
uint64_t shvllm_gpu_nanos(shvllm *h);

/* multi-row passes, sequence slots and rewindable passes (Graph.ExtendRows / DecodeRows / UseSlot /
 * Speculate / SpeculateFirst / Keep / Commit / Rewind).  Output pointers may be NULL. */
int shvllm_extend_rows(shvllm *h, const int32_t *ids, int n, float *logits, float *res, int32_t *best);
int shvllm_decode_rows(shvllm *h, const int32_t *slots, const int32_t *ids, int n, float *logits, int32_t *best);
int shvllm_use_slot(shvllm *h, int slot);
int shvllm_speculate(shvllm *h, int on);
int shvllm_speculate_first(shvllm *h, int on);
int shvllm_keep(shvllm *h, int k);
int shvllm_commit(shvllm *h);
/* Graph.Checkpoint / Restore (llm/graph.go:1004-1062): the live slot's position, tokens and
 * DeltaNet carry saved to host memory, and the slot taken back to them (refused unless its
 * sequence still starts with the checkpoint's tokens). */
typedef struct shvllm_checkpoint shvllm_checkpoint_t;
int shvllm_checkpoint(shvllm *h, shvllm_checkpoint_t **out);
int shvllm_restore(shvllm *h, const shvllm_checkpoint_t *c);
void shvllm_checkpoint_free(shvllm_checkpoint_t *c);
int shvllm_rewind(shvllm *h);
int shvllm_plane(shvllm *h);
int shvllm_ids(shvllm *h, int32_t *dst, int max, int *n);
int shvllm_dn_state_at(shvllm *h, int layer, int slot, int plane, float *dst);
int shvllm_kv_at(shvllm *h, int layer, int slot, int cells, uint16_t *k, uint16_t *v);
int shvllm_profile_rows(shvllm *h, int rows, char (*labels)[32], uint64_t *nanos, int max, int *n);
/* One headless prompt chunk of `rows` ids (at most max_tokens), timed op by op; the sequence advances. */
int shvllm_profile_chunk(shvllm *h, const int32_t *ids, int rows, char (*labels)[32], uint64_t *nanos, int max, int *n);

/* the draft head (MTPHead) and the greedy speculative loop (Speculator) over the staged graph */
int shvllm_mtp_stage(shvllm *h, int max_tok, int vocab_prefix);
int shvllm_mtp_rows(shvllm *h, const float *hs, const int32_t *ids, int n, int pos, int head, float *logits, float *res);
int shvllm_mtp_rewind(shvllm *h, int n);
int shvllm_mtp_past(shvllm *h);
int shvllm_spec_open(shvllm *h, int depth);
int shvllm_spec_start(shvllm *h, const int32_t *prompt, int n, int32_t *first);
/* one round; forced (n_forced of them, may be 0) replaces the draft head's proposals */
int shvllm_spec_round(shvllm *h, const int32_t *forced, int n_forced, int32_t *out, int max, int *n_out);
/* counts: rounds, drafted, accepted, tokens, passes[5], drafted_at[4], accepted_at[4] (17 values);
 * nanos: draft, verify */
int shvllm_spec_stats(shvllm *h, int32_t *counts, uint64_t *nanos);

#ifdef __cplusplus
}
#endif
#endif
