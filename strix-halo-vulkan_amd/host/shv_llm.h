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
    int32_t idx_heads, idx_dim, idx_top_k, idx_ratio;  /* the block-sparse indexer of the trunk's attention layers; ratio 0: none */
} shvllm_config;

const char *shvllm_last_error(void);
int shvllm_open(int device, const shvllm_config *cfg, shvllm **out);  /* device + model (unset weights) */
void shvllm_close(shvllm *h);
shv_ctx *shvllm_ctx(shvllm *h);
int shvllm_init_synthetic(shvllm *h, uint64_t seed);
/* llm.Open (llm/model.go:52-64): a checkpoint (a .gguf, any shard of a split one, or a directory
 * holding one) mapped, its shape read from its metadata and every tensor staged in device memory.
 * The model fields of *opts are ignored; its graph fields (nkv ... spec_rows) are kept. */
int shvllm_open_gguf(int device, const char *path, const shvllm_config *opts, shvllm **out);
int shvllm_get_config(shvllm *h, shvllm_config *out);
/* this model written as one GGUF file that shvllm_open_gguf reads back bit for bit */
int shvllm_save_gguf(shvllm *h, const char *path);
int shvllm_tensor_count(shvllm *h);
int shvllm_tensor_at(shvllm *h, int i, const char **name, void **dptr, uint64_t *bytes, int32_t *kind,
                     int64_t *rows, int64_t *cols, int32_t *is_alias);
int shvllm_tensor(shvllm *h, const char *name, void **dptr, uint64_t *bytes);
int shvllm_tensor_type(shvllm *h, const char *name, int32_t *ggml_type);  /* the ggml type of the bytes in device memory */
/* Matrices the checkpoint held in a type other than Q4_K, expanded and fitted again as Q4_K when the
 * model was opened (TranscodeMoE's round-to-nearest arm, llm/moebank.go:288-400): their count, and
 * their names, one a line, into buf when it is given.  LLM_TRANSCODE=0 makes the open refuse them. */
int shvllm_transcoded(shvllm *h, char *buf, size_t cap);
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
/* the sampler the loop's tokens are drawn with (Sampler + DraftSampler + Verify); temp <= 0: greedy again.
 * Call before shvllm_spec_start. */
int shvllm_spec_sampler(shvllm *h, float temp, int top_k, float top_p, float min_p, float repeat_penalty, float presence_penalty,
                        int64_t seed, int64_t draft_seed);
int shvllm_spec_start(shvllm *h, const int32_t *prompt, int n, int32_t *first);
/* one round; forced (n_forced of them, may be 0) replaces the draft head's proposals */
int shvllm_spec_round(shvllm *h, const int32_t *forced, int n_forced, int32_t *out, int max, int *n_out);
/* counts: rounds, drafted, accepted, tokens, passes[5], drafted_at[4], accepted_at[4] (17 values);
 * nanos: draft, verify */
int shvllm_spec_stats(shvllm *h, int32_t *counts, uint64_t *nanos);

/* ---- the scheduler (backend/llm_sched.go:201-898): several conversations interleaved on one graph.
 * A request acquires a slot, queues a prefill and then decode steps; the caller's one device thread
 * calls shvllm_sched_pump, which picks the next pass by the policy (interactive strictly before
 * background, then least device time, background prefill in preempt chunks, pending decode steps
 * of one class in one pass), runs it on the graph and books it.  With h NULL the object is the
 * policy alone over `slots` slots: shvllm_sched_next says what would run, shvllm_sched_finish books
 * a duration the caller supplies, and no device is touched.  Times are milliseconds on a clock of
 * the caller's choosing; pump uses the steady clock.  Not thread-safe: one caller at a time. ---- */
typedef struct shvllm_sched shvllm_sched;
typedef struct shvllm_sched_opts {
    int32_t batch, preempt_chunk, reserve, no_batch_decode;
    double coalesce_ms;
    int32_t spec_depth;  /* tokens a speculative round drafts (needs shvllm_mtp_stage and a graph staged for rewindable
                            passes of spec_depth + 1 rows); 0: decode by plain steps only */
} shvllm_sched_opts;
#define SHVLLM_SCHED_MAX_ROWS 64
typedef struct shvllm_sched_pass {
    int32_t kind;      /* 0 nothing, 1 one chunk of one unit, 2 a batched decode pass, 3 a speculative round of `unit` on `slot` */
    int32_t unit, slot, pos, n, fresh, restore, take, step; /* kind 1 */
    int32_t n_units;   /* kind 2 */
    int32_t units[SHVLLM_SCHED_MAX_ROWS], slots[SHVLLM_SCHED_MAX_ROWS];
    double wait_ms;    /* kind 0: > 0 while a batch waits for conversations still sampling */
    int32_t prime, tracked; /* kind 1 with spec_depth: the chunk primes the slot's draft; the draft was caught up when handed out */
} shvllm_sched_pass;
typedef struct shvllm_sched_job {
    int32_t cls, slot, reused, restored, stepping;
    double served_ms;
    uint64_t arrival;
} shvllm_sched_job;
int shvllm_sched_open(shvllm *h, int slots, const shvllm_sched_opts *opts, shvllm_sched **out);
void shvllm_sched_close(shvllm_sched *s);
/* cls 0 interactive, 1 background; mark: prompt position of the slot's checkpoint, 0 for none */
int shvllm_sched_acquire(shvllm_sched *s, int cls, const int32_t *prompt, int n, int mark, double now_ms, int *job);
int shvllm_sched_release(shvllm_sched *s, int job, double now_ms);
int shvllm_sched_job_info(shvllm_sched *s, int job, shvllm_sched_job *out);
int shvllm_sched_run(shvllm_sched *s, int job, const int32_t *ids, int n, int fresh, int *unit);
int shvllm_sched_step(shvllm_sched *s, int job, int32_t id, int *unit);
/* a decode step that may run as a speculative round (backend/llm_sched.go:455-464): the unit ends with the round's
 * tokens (shvllm_sched_unit_tokens; the last is pending like a sampled one) or, run as a plain step, with logits.
 * room: tokens the request may still take.  The round names its tokens by arg-max. */
int shvllm_sched_decode(shvllm_sched *s, int job, int32_t id, int room, int *unit);
/* the same with the request's sampler (borrowed until the unit is done), which names the round's tokens and takes
 * them into its window itself: exact != 0 for a seeded request (every verified row is one plain draw, so the random
 * stream is consumed as plain steps consume it), else the drafts are drawn with a sampler seeded by draft_seed and
 * verified by speculative sampling.  A unit that ran as a plain step returns logits as ever. */
struct shvsampler;
int shvllm_sched_decode_sampled(shvllm_sched *s, int job, int32_t id, int room, struct shvsampler *sampler, int exact, int64_t draft_seed, int *unit);
int shvllm_sched_withdraw(shvllm_sched *s, int unit);
int shvllm_sched_next(shvllm_sched *s, double now_ms, shvllm_sched_pass *out);
int shvllm_sched_finish(shvllm_sched *s, double took_ms, int ok, double now_ms);  /* books the pass shvllm_sched_next handed out last */
/* the same for a round (kind 3) the caller ran itself: the tokens it drew */
int shvllm_sched_finish_round(shvllm_sched *s, double took_ms, int ok, double now_ms, const int32_t *toks, int n);
int shvllm_sched_pump(shvllm_sched *s, shvllm_sched_pass *out);
/* state: 0 queued, 1 done, 2 failed; logits [vocab] when done and given; left: ids not yet run */
int shvllm_sched_unit(shvllm_sched *s, int unit, int *state, int *left, double *busy_ms, float *logits, int max);
int shvllm_sched_unit_tokens(shvllm_sched *s, int unit, int32_t *dst, int max, int *n);  /* a round's tokens; n 0 for a unit that ran as a step */
int shvllm_sched_forget(shvllm_sched *s, int unit);
/* counts: restores, batched passes, rows in them, passes, jobs waiting for a slot, units queued */
int shvllm_sched_counts(shvllm_sched *s, int32_t counts[6]);
int shvllm_sched_held(shvllm_sched *s, int slot, int32_t *dst, int max, int *n, int *ckpt_len);
/* counts: speculative rounds, tokens they drew; tracked: whether the slot's draft covers what the slot holds */
int shvllm_sched_round_counts(shvllm_sched *s, int32_t counts[2]);
int shvllm_sched_tracked(shvllm_sched *s, int slot, int *tracked);

/* ---- the host sampler (llm.Sampler, llm/sample.go): penalties -> top_k -> top_p -> min_p -> temp -> draw,
 * and speculative sampling's Verify.  No device involved; rows are host floats and come back unchanged. ---- */
typedef struct shvsampler shvsampler;
shvsampler *shvsampler_new(float temp, int top_k, float top_p, int64_t seed);   /* NewSampler */
void shvsampler_free(shvsampler *s);
void shvsampler_set(shvsampler *s, float min_p, float repeat_penalty, float presence_penalty);
int shvsampler_greedy(shvsampler *s);
void shvsampler_accept(shvsampler *s, const int32_t *ids, int n);
int32_t shvsampler_sample(shvsampler *s, float *logits, int n);
/* the distribution Sample draws from, most likely first; returns its length (ids/p take up to max) */
int shvsampler_dist(shvsampler *s, float *logits, int n, int32_t *ids, float *p, int max);
shvsampler *shvsampler_draft(shvsampler *s, int64_t seed);                       /* DraftSampler; NULL when greedy */
int32_t shvsampler_propose(shvsampler *s, float *logits, int n);                 /* keeps its distribution in s */
int shvsampler_last_dist(shvsampler *s, int32_t *ids, float *p, int max);
/* Verify against the distribution of proposer's last propose; proposer NULL (or greedy) is Sample */
int32_t shvsampler_verify(shvsampler *s, float *logits, int n, int32_t draft, shvsampler *proposer);
/* loops for the distribution tests: counts[id]++ per draw; speculate_many returns how often the draft was kept */
void shvsampler_sample_many(shvsampler *s, float *logits, int n, int draws, int32_t *counts);
int64_t shvsampler_speculate_many(shvsampler *s, shvsampler *ds, float *pl, float *ql, int n, int draws, int32_t *counts);
int32_t shvsampler_argmax(const float *logits, int n);
int shvsampler_top_n(const float *logits, int n, int k, int32_t *dst);
int shvsampler_top_k_of(const float *logits, int n, int k, int32_t *dst);

/* ---- the GGUF container by itself (package gguf, gguf/gguf.go): no device involved ---------- */
typedef struct shvgguf shvgguf;
int shvgguf_open(const char *path, shvgguf **out);   /* OpenSet: a file, any shard, or a directory */
int shvgguf_open_file(const char *path, shvgguf **out); /* Open: this one file, no sibling shards */
void shvgguf_close(shvgguf *g);
int shvgguf_files(shvgguf *g);
int shvgguf_file_info(shvgguf *g, int i, const char **path, uint32_t *version, uint64_t *alignment, int64_t *data_start);
int shvgguf_len(shvgguf *g);
int64_t shvgguf_params(shvgguf *g);
int64_t shvgguf_bytes(shvgguf *g);
const char *shvgguf_arch(shvgguf *g);
/* tensor i of the joined table; dims has room for 4 */
int shvgguf_tensor_at(shvgguf *g, int i, const char **name, uint32_t *type, int32_t *n_dims, int64_t *dims,
                      const void **data, uint64_t *bytes, int32_t *shard, int64_t *rows, int64_t *row_bytes);
int shvgguf_find(shvgguf *g, const char *name);      /* index, or -1 */
int shvgguf_advise_random(shvgguf *g, int i);
int shvgguf_key_count(shvgguf *g);
const char *shvgguf_key_at(shvgguf *g, int i);
/* metadata: 1 = found and of a kind the getter answers, 0 = not.  kind: 0 none, 1 uint, 2 int, 3 float,
 * 4 bool, 5 string, 6 uints, 7 ints, 8 floats, 9 bools, 10 strings (widths widen as File.Uint/Int/Float do) */
int shvgguf_kind(shvgguf *g, const char *key);
int shvgguf_uint(shvgguf *g, const char *key, uint64_t *out);
int shvgguf_int(shvgguf *g, const char *key, int64_t *out);
int shvgguf_float(shvgguf *g, const char *key, double *out);
int shvgguf_bool(shvgguf *g, const char *key, int32_t *out);
int shvgguf_str(shvgguf *g, const char *key, const char **out, uint64_t *len);
int shvgguf_array_len(shvgguf *g, const char *key, uint64_t *n);
int shvgguf_uints(shvgguf *g, const char *key, uint64_t *dst, uint64_t max);
int shvgguf_ints(shvgguf *g, const char *key, int64_t *dst, uint64_t max);
int shvgguf_floats(shvgguf *g, const char *key, double *dst, uint64_t max);
int shvgguf_string_at(shvgguf *g, const char *key, uint64_t i, const char **out, uint64_t *len);
/* block geometry of a ggml type: name ("?<n>" when unknown; valid until the next call on this thread) */
const char *shvgguf_type_name(uint32_t type);
int shvgguf_type_block(uint32_t type, int32_t *elems, int32_t *nbytes);   /* 0 when unknown */
int64_t shvgguf_size_of(uint32_t type, int64_t n);                        /* -1 with the error set */

/* ---- the text on either side of the token loop (host/text.hpp).  Strings the library hands out are malloc'ed, NUL-
 * terminated copies (with their length where they may hold NUL) and go back through shvtext_free. ---- */
typedef struct shvtext_tokenizer shvtext_tokenizer;
typedef struct shvtext_decoder shvtext_decoder;
void shvtext_free(void *p);
/* tokenizer.FromVocab (zimage/tokenizer/vocab.go:62): tokens by id over the byte-level alphabet, merges as "left right";
 * types (llama_token_attr numbering, one an id) or NULL; specials: names to match whole besides the types'; pre: "qwen2",
 * "" or "qwen35" */
int shvtext_tokenizer_from_vocab(const char *const *tokens, const uint64_t *token_len, int n_tokens, const char *const *merges,
                                 const uint64_t *merge_len, int n_merges, const int32_t *types, const char *const *specials,
                                 int n_specials, const char *pre, shvtext_tokenizer **out);
/* LoadTokenizer + EndOfGeneration (llm/tokenizer.go:22-68) from an open checkpoint's metadata: the stop set's ids go to
 * eog (up to eog_max of them), their count to n_eog */
int shvtext_tokenizer_from_gguf(shvgguf *g, shvtext_tokenizer **out, int32_t *eog, int eog_max, int *n_eog);
void shvtext_tokenizer_free(shvtext_tokenizer *t);
int shvtext_tokenizer_size(shvtext_tokenizer *t);
int shvtext_tokenizer_id(shvtext_tokenizer *t, const char *token, int32_t *id);   /* 1 found, 0 not */
int shvtext_encode(shvtext_tokenizer *t, const char *text, uint64_t len, int32_t **ids, int *n);
int shvtext_decode(shvtext_tokenizer *t, const int32_t *ids, int n, char **out, uint64_t *len);
/* the pre-tokenizer's pieces (zimage/tokenizer/split.go): concatenated in out, their byte lengths in piece_len */
int shvtext_split(const char *text, uint64_t len, int marks, char **out, uint64_t *out_len, int32_t **piece_len, int *n);
/* pyJSON (llm/pyjson.go:31): Python's json.dumps(x, ensure_ascii=False) of one JSON value */
int shvtext_pyjson(const char *raw, char **out);
/* ParseToolArguments (llm/chat.go:399): [{"name": ..., "value": <the JSON as it arrived>}, ...] in the object's order */
int shvtext_parse_tool_arguments(const char *s, char **out_json);
/* RenderChat (llm/chat.go:195).  request_json: {"messages": [{"role", "content" | "parts": [{"text"} | {"image": true}],
 * "reasoning", "tool_calls": [{"name", "args": [{"name", "value"}]}]}], "tools": [...], "opts": {"effort", "no_thinking",
 * "drop_thinking", "no_generation_prompt", "add_vision_id"}} -- the shape of the reference's own test cases */
int shvtext_render_chat(const char *request_json, char **out);
/* ChatDecoder (llm/chatdecode.go): tools_json is the request's tools array or NULL; thinking: the generation prompt left
 * <think> open */
int shvtext_decoder_new(const char *tools_json, int thinking, shvtext_decoder **out);
void shvtext_decoder_free(shvtext_decoder *d);
int shvtext_decoder_stop_at(shvtext_decoder *d, const char *const *seqs, const uint64_t *lens, int n);
const char *shvtext_decoder_stopped(shvtext_decoder *d, uint64_t *len);   /* valid until the next call on d */
int shvtext_decoder_write(shvtext_decoder *d, const char *piece, uint64_t len, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len);
/* calls_json: [{"name": ..., "arguments": "<a JSON object as a string>"}, ...] */
int shvtext_decoder_close(shvtext_decoder *d, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len, char **calls_json);

/* The text side of the emit loop (backend/llm.go:561-590): a sampled id becomes its bytes, whole characters (a
 * character's bytes come in several tokens routinely) go to the completion reader, and what that releases is the token's
 * delta.  finish: 0 running, 1 an end-of-generation id, 2 a stop sequence.  The tokenizer must outlive the stream. */
typedef struct shvtext_stream shvtext_stream;
int shvtext_stream_new(shvtext_tokenizer *t, const int32_t *eog, int n_eog, const char *tools_json, int thinking, shvtext_stream **out);
void shvtext_stream_free(shvtext_stream *s);
int shvtext_stream_stop_at(shvtext_stream *s, const char *const *seqs, const uint64_t *lens, int n);
int shvtext_stream_push(shvtext_stream *s, int32_t id, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len, int *finish);
const char *shvtext_stream_stopped(shvtext_stream *s, uint64_t *len);
int shvtext_stream_close(shvtext_stream *s, char **reasoning, uint64_t *r_len, char **content, uint64_t *c_len, char **calls_json);

#ifdef __cplusplus
}
#endif
#endif
