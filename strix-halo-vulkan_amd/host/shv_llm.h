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

#ifdef __cplusplus
}
#endif
#endif
