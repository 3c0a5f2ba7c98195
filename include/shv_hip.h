/*
 * shv_hip.h — C ABI of the MI355X (gfx950) backend for strix-halo-vulkan's language-model
 * token loop.  It takes the place of the reference's Vulkan shim (vk/shim.h) underneath the
 * Go-side op surface (llm/gpu_*.go): a host binding (cgo, ctypes, C++) sees opaque handles,
 * device addresses, plain sizes and POD argument blocks, and nothing else.
 *
 * Conventions
 *   - every function returns 0 on success and a negative SHV_E_* code otherwise;
 *     shv_last_error() gives the message for the calling thread (vk.Error{Op,Result},
 *     vk/engine.go:21-36, carries the same two facts).
 *   - a context owns ONE in-order HIP stream: consecutive ops are ordered as the reference's
 *     dispatches are by the barrier it records between them (vk/engine.go:853-859).
 *   - the context is not internally synchronised: one host thread at a time, as
 *     backend.Device.Do serialises every caller of the reference (backend/device.go:24-36).
 *   - device memory is not host-mapped on a discrete GPU, so Buffer.Write* / Read*
 *     (vk/engine.go:319-634) become shv_upload / shv_download on device addresses.
 *   - an op is {kind, flags, 248-byte POD block}: the analogue of MultiDispatch{Pipeline,
 *     GroupsX, GroupsY, PushConstants} with its 256-byte push block (vk/engine.go:848-860,
 *     llm/gpu.go:60-109).  Grid shapes are chosen inside the library.
 *   - values that change from token to token (sequence position, token id) are read by the
 *     kernels from device memory, so a recorded sequence is byte-identical between tokens
 *     and can be replayed (vk/engine.go:997-1081).
 */
#ifndef SHV_HIP_H
#define SHV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SHV_OK 0
#define SHV_E_INVALID (-1)   /* bad argument or shape the kernels do not cover */
#define SHV_E_HIP (-2)       /* a HIP runtime call failed                     */
#define SHV_E_NOMEM (-3)
#define SHV_E_STATE (-4)     /* call not valid in the context's current state */

#define SHV_Q4K_BLOCK 256    /* weights per GGUF Q4_K super-block */
#define SHV_Q4K_BYTES 144    /* bytes per super-block: f16 d, f16 dmin, 12 B scales, 128 B nibbles */

typedef struct shv_ctx shv_ctx;
typedef struct shv_prerecorded shv_prerecorded;

typedef struct {
    char name[128];
    char arch[32];
    int32_t compute_units;
    int32_t wave_size;
    int32_t lds_bytes_per_cu;
    int32_t clock_mhz;
    uint64_t hbm_bytes;
} shv_props;

/* ---- device, replaces shim_create_instance .. shim_create_device (vk/shim.h:84-114) ---- */
const char *shv_last_error(void);
int shv_device_count(int *out);
int shv_init(int device, shv_ctx **out);
void shv_destroy(shv_ctx *ctx);
int shv_device_props(shv_ctx *ctx, shv_props *out);   /* vk/engine.go:144-253 PhysicalDevice */
int shv_sync(shv_ctx *ctx);                           /* shim_device_wait_idle, vk/shim.h:115 */
int shv_submits(shv_ctx *ctx, uint64_t *out);         /* Device.Submits, vk/engine.go:303-308 */

/* ---- buffers, replaces shim_create_storage_buffer / shim_destroy_buffer (vk/shim.h:120-131)
 *      and the Buffer read/write family (vk/engine.go:319-634).  Upload/download block. ---- */
int shv_alloc(shv_ctx *ctx, size_t bytes, void **dptr);
int shv_free(shv_ctx *ctx, void *dptr);
int shv_upload(shv_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int shv_download(shv_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
/* shv_upload for a pass's control words and token ids (Buffer.WriteU32s on a host-visible buffer,
 * vk/engine.go:319-634, costs the reference a store; a blocking upload costs 16 us of host time here,
 * a dozen of them a speculative round): up to SHV_UPLOAD_ASYNC_MAX bytes are copied into pinned
 * staging of the library's own and handed to the stream; the call returns at once, src_host may
 * be reused, and the bytes are in place for every later op, copy or download of THIS context (work
 * elsewhere must follow a shv_sync).  Larger transfers, and all of them with SHV_UPLOAD_SYNC=1 in
 * the environment, block like shv_upload. */
#define SHV_UPLOAD_ASYNC_MAX 512
int shv_upload_async(shv_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int shv_copy(shv_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);  /* async, in order */
int shv_zero(shv_ctx *ctx, void *dst_dev, size_t bytes);                       /* Buffer.Zero*, async */
/* Pinned host memory the device can address: staging for transfers, and somewhere an op can leave a
 * small result (the arg-max's best) that the host reads after the submit's wait without a download. */
int shv_host_alloc(shv_ctx *ctx, size_t bytes, void **hptr);
int shv_host_free(shv_ctx *ctx, void *hptr);

/* ---- op argument blocks ---------------------------------------------------------------- */

enum {
    SHV_OP_GEMV_Q4K = 1,
    SHV_OP_DEQUANT_Q4K = 2,
    SHV_OP_QUANTIZE_Q4K = 3,
    SHV_OP_FILL_NORMAL = 4,
    SHV_OP_MOE_ROUTER = 5,
    SHV_OP_MOE_UP = 6,
    SHV_OP_MOE_DOWN = 7,
    SHV_OP_DN_STEP = 8,
    SHV_OP_ATTN_DECODE = 9,
    SHV_OP_EMBED = 10,
    SHV_OP_ARGMAX = 11,
    SHV_OP_ADVANCE = 12,
    SHV_OP_DEQUANT = 13,
    SHV_OP_GEMV = 14,
    SHV_OP_RING_ROWS = 15,
    SHV_OP_ROUTER_FOLD = 16,
    SHV_OP_QSA_INDEX = 17,
    SHV_OP_ARGMAX_STATIC = 18, /* shv_argmax_static as an op, so that a recorded sequence can hold it */
    SHV_OP__COUNT
};

/* prologues a Q4_K GEMV can apply to its input vector while staging it */
enum {
    SHV_PRO_NONE = 0,
    SHV_PRO_RMSNORM = 1,     /* x * rsqrt(mean(x^2)+eps) * gamma            (llm/hc.go:176-190)       */
    SHV_PRO_GATED_NORM = 2,  /* per head of head_dim: rms * gamma[head_dim] * sigmoid(z)
                                                                            (llm/deltanet.go:329-341) */
    SHV_PRO_MUL_SIGMOID = 3, /* x * sigmoid(z); with head_dim > 0, z holds [q | gate] per head and
                                the gate half is read                      (llm/attn.go:162-166,198-205) */
    SHV_PRO_RMSNORM_PAIR = 4 /* the draft head's input (llm/mtp.go:44-46): the k-wide vector is
                                [RMSNorm(x)*gamma[0..k/2) | RMSNorm(z)*gamma[k/2..k)], x and z each
                                k/2 wide with strides x_stride and z_stride                        */
};

/* y[t][r] = sum_i W[r][i] * pro(x[t])[i] (+ residual[t][r]); W is GGUF Q4_K, row-major, k%256==0.
 * The reference's CPU form is matvec over Tensor.DequantizeRow (llm/hc.go:255-264,
 * gguf/dequant.go:119-124); its GPU forms are llm_gemv.comp and llm_moe_gemv.comp.
 * Rows are grouped into sequences of seq_len consecutive tokens (seq_len 0 means one sequence
 * of n_tok).  ring_slots>0 selects ring output, the DeltaNet projection ring of
 * shaders/llm_dn_conv.comp:36-49 and llm_seq_hist.comp:17-26: row i of sequence s is written at
 * y + (slot[s]*ring_slots + (pos[s]+i) % ring_slots) * ring_stride, slot[s] = s when slot is NULL,
 * instead of y + t*y_stride.  z_ring != 0 reads the prologue's z row from the same ring
 * geometry instead (z + (slot*ring_slots + (pos+i) % ring_slots) * ring_stride) and leaves y
 * plain: the DeltaNet output projection takes its gate z from the projection ring. */
typedef struct {
    const void *w;
    const float *x;
    float *y;
    const float *residual;
    const float *gamma;
    const float *z;
    const int32_t *pos;
    const int32_t *slot;
    int32_t n, k, n_tok;
    int32_t prologue;
    int32_t head_dim;
    float eps;
    int32_t x_stride, y_stride, z_stride;
    int32_t seq_len, ring_slots, ring_stride;
    int32_t z_ring;
    float *y_flat;           /* with ring output, one row (n_tok == 1): the row is also stored here, at an
                                address that does not depend on the position, for a consumer that would
                                otherwise wait for the position word before it can ask for the row (the
                                DeltaNet output projection's gate z); NULL: not stored */
    /* The router's logits in the same launch (one to four rows, k = 4096, n = 2048, a residual): the
     * projection feeds y = residual + W pro(x) to an RMSNorm and a float32 router R (llm/moe.go:
     * 219-232), and R (gamma * y) is linear in y: it is fold[e] . [pro(x) | residual] with
     * fold [fold_rows][k + n] = [R diag(gamma) W | R diag(gamma)] made once by shv_router_fold.
     * fold_out[e] receives that product WITHOUT the norm's factor rsqrt(mean(y^2) + eps), which
     * shv_moe_up applies (its gamma argument).  residual must not alias y then.  NULL: no logits. */
    const float *fold;
    float *fold_out;
    int32_t fold_rows;
    int32_t fold_stride;     /* two to four rows: row t's products go to fold_out + t * fold_stride */
    /* The greedy sampler in the same launch (one row; the vocabulary projection of a decode step):
     * what shv_argmax does with its best / ids / pos / advance over y[0..n) is done by the block
     * of this launch that finishes last (Argmax, llm/sample.go:359-367: first maximum, NaN never
     * wins).  amax_best NULL: no arg-max. */
    int32_t *amax_best;
    int32_t *amax_ids;
    int32_t *amax_pos;
    int32_t amax_advance;
} shv_gemv_q4k_args;

/* The table shv_gemv_q4k's `fold` reads, for one layer: out [rows][k + n_embd] float32,
 * rows = n_expert + (shared_gate ? 1 : 0); out[e][k + i] = R[e][i] * gamma[i] and
 * out[e][j] = sum_i R[e][i] * gamma[i] * W[i][j] accumulated in float64, W [n_embd][k] the Q4_K
 * output projection as dequantQ4_K expands it (gguf/dequant.go:252-276), R the router's rows with
 * the shared gate as the last.  scratch: n_embd * k floats.  Made once when a graph is staged,
 * as the reference makes its dense banks then (llm/bank_q4.go:172-266). */
typedef struct {
    const float *router;
    const float *shared_gate;
    const float *gamma;
    const void *w_out;
    float *out;
    float *scratch;
    int32_t n_expert, n_embd, k;
} shv_router_fold_args;

/* ggml type numbers of the tensor types the reference's loader accepts (Dequantizable,
 * gguf/dequant.go:103-110) */
enum {
    SHV_GGML_F32 = 0, SHV_GGML_F16 = 1, SHV_GGML_Q4_1 = 3, SHV_GGML_Q5_0 = 6, SHV_GGML_Q5_1 = 7, SHV_GGML_Q8_0 = 8,
    SHV_GGML_Q4_K = 12, SHV_GGML_Q5_K = 13, SHV_GGML_Q6_K = 14, SHV_GGML_IQ4_NL = 20, SHV_GGML_BF16 = 30
};

/* n elements of any of those types to float32, bit for bit what gguf.Dequantize gives
 * (gguf/dequant.go:52-98; the arms :128-356).  n must be whole blocks of the type (32 or 256). */
typedef struct {
    const void *src;
    float *dst;
    int64_t n;
    int32_t type;
} shv_dequant_args;

/* y[t][r] = sum_i W[r][i] * pro(x[t])[i] (+ residual[t][r]) for W [n][k] row-major in any of those
 * types: the CPU path's matvec over Tensor.DequantizeRow (llm/hc.go:255-264, gguf/dequant.go:119-124)
 * for the tensors of a checkpoint that are not Q4_K.  gamma non-NULL: pro is the RMSNorm
 * x * rsqrt(mean(x^2) + eps) * gamma (llm/hc.go:176-190), which is how a vocabulary projection kept in
 * the checkpoint's own type (a Q6_K head) takes its rows; NULL: pro(x) = x.  n_tok 0 means one row;
 * rows are x_stride and y_stride floats apart (0: k and n); the weights are read once for every four
 * rows.  Q4_K weights on the token path go through shv_gemv_q4k. */
typedef struct {
    const void *w;
    const float *x;
    float *y;
    const float *residual;
    int32_t n, k;
    int32_t type;
    int32_t n_tok;
    const float *gamma;
    float eps;
    int32_t x_stride, y_stride;
} shv_gemv_args;

/* dst[i] = d*sc*q - dmin*m for every weight of `rows` rows, the reference's dequantQ4_K
 * expression term for term (gguf/dequant.go:252-276); bit-exact. */
typedef struct {
    const void *w;
    float *dst;
    int64_t rows;
    int32_t k;
} shv_dequant_q4k_args;

/* src float32 [rows][k] -> GGUF Q4_K rows, the reference's round-to-nearest quantiser
 * (llm/quantk.go:115-179, llm/sim.go:982-1060, llm/moebank.go:489-532); bit-exact. */
typedef struct {
    const float *src;
    void *dst;
    int64_t rows;
    int32_t k;
} shv_quantize_q4k_args;

/* dst[i] = mean + std * N(0,1), counter-based (seed, i): synthetic weights made in HBM.
 * half != 0 stores binary16 (round to nearest even) instead of float32. */
typedef struct {
    void *dst;
    int64_t n;
    uint64_t seed;
    float mean, std;
    int32_t half;
} shv_fill_normal_args;

/* MoE router (MoETrace.Route, llm/moe.go:219-274; shaders llm_moe_router/route.comp): per token
 * xn = RMSNorm(h)*gamma (gamma NULL: h is used as it is), logits = router*xn in float32, softmax,
 * the n_used largest probabilities in descending order (ties to the lower index), their sum
 * clamped at 2^-14, the normalised weights; weights[t][n_used] = sigmoid(shared_gate . xn)
 * (llm/moe.go:396-402).  logits is [T][n_expert+1], the last column the shared-gate logit.
 * defer_route != 0 stops after the logits (topk and weights may then be NULL) and leaves the
 * selection to shv_moe_up, which can make it from the logits in its own prologue. */
typedef struct {
    const float *h;
    const float *gamma;
    const float *router;
    const float *shared_gate;
    float *xn;
    float *logits;
    int32_t *topk;
    float *weights;
    int32_t n_tok, n_embd, n_expert, n_used;
    float eps;
    int32_t h_stride;
    int32_t defer_route;
} shv_moe_router_args;

/* Expert-gathered gate/up GEMV with SwiGLU (MoETrace.Experts/Shared, llm/moe.go:289-409;
 * llm_moe_gemv.comp MODE 0): act[t][s] = silu(Wg_e xn[t]) * (Wu_e xn[t]) for e = topk[t][s],
 * s < n_used, and for the shared expert in slot n_used.  Only the selected experts' rows are
 * read.  Banks are GGUF Q4_K: expert e's row j is row e*ffn + j, n_embd long.
 * When logits is given ([T][n_expert+1] from a router run with defer_route) every block first
 * routes its token from them exactly as the router would, and the selection is also stored to
 * topk [T][n_used] and weights [T][n_used+1] for the down projection; otherwise topk is read.
 * A pass of many rows (128 and more; SHV_MOE_GROUP_MIN) whose topk is given, with n_expert stated
 * and a `group` workspace of 2 * n_expert + 1 + T * n_used ints, is grouped by expert on the matrix
 * cores: an expert's weights are read once per 48 tokens that chose it (the prompt arm of
 * llm_moe_gemv.comp). */
typedef struct {
    const float *xn;
    int32_t *topk;
    const void *gate_exps, *up_exps;
    const void *gate_sh, *up_sh;
    float *act;
    int32_t n_tok, n_embd, n_used, ffn;
    const float *logits;
    float *weights;
    int32_t n_expert;
    /* ggml type (SHV_GGML_*) of each bank; 0 or SHV_GGML_Q4_K is Q4_K, the tuned path.  A bank in
     * another accepted type (Q8_0, Q4_1, Q5_0, Q5_1, IQ4_NL, Q5_K, Q6_K, F16, BF16) is read as the
     * checkpoint holds it (llm_moe_gemv.comp's other arms; llm/gpu_moe.go:673-688), rows as
     * Tensor.DequantizeRow forms them; the selection then comes from the router (logits NULL). */
    int32_t gate_type, up_type, gate_sh_type, up_sh_type;
    int32_t *group;          /* workspace of the grouped path, or NULL */
    int32_t no_shared_gate;  /* with logits: nonzero says the router ran without a shared_gate (it then
                                left logits[n_expert] unwritten), and weights[t][n_used] is stored as 0,
                                as the router's own selection stores it */
    int32_t act_packed;      /* grouped path only: act is left as the matrix-core operands the grouped
                                shv_moe_down reads (two binary16 parts of every value, same bytes a row)
                                instead of floats; the shv_moe_down of this pass must be the library's
                                next call on the stream, with act_packed and group_ready set too */
    const float *gamma;      /* with logits, up to four rows: xn is the row BEFORE its RMSNorm and logits are the
                                router's products without the norm's factor (shv_gemv_q4k's fold_out);
                                the kernel forms the factor from the row it stages, multiplies the row
                                by gamma and applies the factor to its own products and to the logits
                                (llm/hc.go:176-190).  NULL: xn is normalised already */
    float eps;
    const float *shared_gate; /* with gamma: the shared expert's gate vector (llm/moe.go:396-402); its weight
                                sigmoid(shared_gate . xn) is then formed here from the staged row instead of
                                read from logits[n_expert].  NULL: from the logits */
} shv_moe_up_args;

/* Down projection, weighting and combine (llm/moe.go:331-357,390-407; llm_moe_gemv.comp MODE 1 +
 * llm_moe_combine.comp): out[t] = residual[t] + sum_s weights[t][s] * (Wd_e act[t][s])
 * + weights[t][n_used] * (Wd_shared act[t][n_used]).  residual may be NULL.
 * Grouped by expert as shv_moe_up is when the caller gives n_expert, a `group` workspace of the
 * same size and `pairs`, [T][n_used+1][n_embd] floats for the products of every (token, slot)
 * before they are weighted and summed in slot order.  group_ready != 0 says that `group` already
 * holds this pass's lists (the grouped shv_moe_up of the same topk and n_tok filled it just before)
 * and spares the launch that would build them again. */
typedef struct {
    const float *act;
    const int32_t *topk;
    const float *weights;
    const void *down_exps, *down_sh;
    const float *residual;
    float *out;
    int32_t n_tok, n_embd, n_used, ffn;
    int32_t res_stride, out_stride;
    int32_t down_type, down_sh_type;  /* as in shv_moe_up_args: 0 or SHV_GGML_Q4_K, or the bank's own type */
    int32_t n_expert;        /* the grouped path: experts in the bank, */
    int32_t *group;          /* its workspace */
    float *pairs;            /* and the per-pair products; NULL keeps the per-(token, slot) kernels */
    int32_t group_ready;     /* the lists in `group` are this pass's already */
    int32_t act_packed;      /* act is what the grouped shv_moe_up left with its act_packed set (needs group_ready) */
} shv_moe_down_args;

/* Gated DeltaNet step(s) after the fused projection (DeltaNetLayer, llm/deltanet.go:266-327 and
 * deltaRule :365-403; shaders llm_dn_conv.comp + llm_dn_scan.comp): for each of n_seq sequences,
 * seq_len consecutive tokens starting at pos[s] on state slot[s] (s itself when slot is NULL):
 * depthwise causal conv (kernel 4) over the ring of fused projection rows, SiLU, L2-normalised
 * q and k per key head, g = exp(softplus(alpha+dt_bias)*A), beta = sigmoid(b), then
 * S *= g; delta = (v - S^T k)*beta; S += k delta^T; o = S^T q / sqrt(d).
 * A ring row is [q (hk*d) | k (hk*d) | v (hv*d) | z (hv*d) | alpha (hv) | beta (hv)]; positions
 * before the start of a sequence read as zero.  state is [n_slots][hv][d][d] float32 holding
 * S[i][j] at [j*d+i] (the reference's transposed layout), updated in place; out is the raw
 * attention output [n_seq*seq_len][hv*d] that the gated norm of the out projection consumes.
 * v-head h reads key head h % hk (kHeadOfV, llm/deltanet.go:412-418).
 * Rewindable passes (DeltaNetGPU.Speculate / KeepSlot, llm/gpu_deltanet.go:1091-1133): with
 * n_planes > 1 a state slot holds n_planes copies of S, state is [n_slots][n_planes][hv][d][d],
 * and plane[slot] names the committed one, which is the one read.  spec == 0 updates it in place.
 * spec != 0 leaves it untouched and stores the state after row i of the pass into plane
 * (plane[slot] + 1 + i) % n_planes, so that accepting the first k rows of the pass is
 * plane[slot] = (plane[slot] + k) % n_planes and discarding it is doing nothing; seq_len must then
 * be below n_planes.  plane NULL reads plane 0.
 * work (optional): work_floats floats of scratch, 16-byte aligned.  With at least n_seq*seq_len*
 * (2*hk*d + hv*d + 2*hv) of them a plain pass (spec == 0) of more than 16 rows goes 64 rows at a
 * time on the matrix cores (the chunked form of the same rule: q^, k^, v, log g and beta of every
 * row are prepared into work first, then each chunk is a few 64-row products and one triangular
 * solve against the state, which is read and written once per pass); results agree with the
 * row-by-row rule to float32 rounding.  With room behind those rows (their count rounded up to a
 * multiple of 4 floats) for 10 880 more floats per (sequence, chunk of 64 rows, value head), what a
 * chunk needs that does not depend on the state is formed for every chunk of the pass at once, by a
 * launch of its own, instead of inside the walk over the chunks by each of a head's eight blocks:
 * the same values bit for bit, the walk a quarter shorter.  The reference scans row by row at every pass length
 * (shaders/llm_dn_scan.comp; llm/gpu_deltanet.go:48-52 names the chunked form as not built there). */
typedef struct {
    const float *ring;
    const float *conv1d;
    const float *a;
    const float *dt_bias;
    float *state;
    float *out;
    const int32_t *pos;
    const int32_t *slot;
    int32_t n_seq, seq_len;
    int32_t n_head_k, n_head_v, head_dim, conv;
    int32_t ring_slots, ring_stride;
    float eps;
    int32_t qk_norm_max;
    const int32_t *plane;
    int32_t n_planes, spec;
    float *work;
    int64_t work_floats;
} shv_dn_step_args;

/* Gated full-attention decode over an fp16 KV cache (AttnLayerAt, llm/attn.go:162-205, and
 * attention :444-496; shaders llm_attn_pack.comp + llm_attn_wmma.comp -DSPLITK +
 * llm_attn_combine.comp).  Input is the fused projection row
 *   [ per head: q (d) | gate (d) ] x n_head, then k (n_head_kv*d), then v (n_head_kv*d).
 * For each of n_seq sequences, seq_len consecutive rows at positions pos[s]+i on cache slot
 * slot[s] (s itself when NULL): per-head RMS norm of q and k with one gamma each, NeoX rotary on
 * the first rope_dims dims from the host-built table (row p: cos[rope_dims/2] then
 * sin[rope_dims/2]; llm/gpu_attn.go:1452-1476), K and V rounded to binary16 into cell p of the
 * cache, then causal GQA softmax attention of the row over cells 0..p, split n_splits ways over
 * the cells and merged.  out is [rows][n_head*d] BEFORE the sigmoid gate, which the output
 * projection applies as its prologue.  kcache is [n_slots][max_cells][n_head_kv][d] binary16;
 * vcache holds V transposed in tiles of 32 cells, [n_slots][max_cells/32][n_head_kv][d][32] binary16
 * (four cells of one dim are one operand of the second product, a tile of one KV head is 16
 * contiguous KB).  max_cells is a multiple of 32 and both caches hold finite
 * values in every cell (zeros before a cell is written): the last tile of a sequence reads a few
 * cells past its end and weights them by zero. partial is scratch of
 * n_seq*(seq_len rounded up to even)*n_head_kv*n_splits*(n_head/n_head_kv)*(d+2) floats.  The rows of a sequence are
 * taken two at a time over one pass of the cache; with more than two rows every row's cell is
 * written first and all pairs go in one launch, each masked to its own position. */
typedef struct {
    const float *qkv;
    const float *q_norm;
    const float *k_norm;
    const float *rope;
    void *kcache;
    void *vcache;
    float *partial;
    float *out;
    const int32_t *pos;
    const int32_t *slot;
    int32_t n_seq, seq_len;
    int32_t n_head, n_head_kv, head_dim, rope_dims;
    int32_t max_cells, qkv_stride, n_splits;
    float eps;
    /* The block-sparse selection (AttnTrace.selected, llm/attn.go:423-443): row r of the pass may
     * read cell c only if bit c % 32 of mask[r * mask_stride + c / 32] is set (and c is visible at
     * all); shv_qsa_index makes it.  NULL: every visible cell. */
    const uint32_t *mask;
    int32_t mask_stride;
} shv_attn_decode_args;

/* The block-sparse indexer beside a full-attention layer (AttnTrace.indexerAt, llm/attn.go:231-421;
 * topK / topKThreshold / f2ui :588-682; shaders llm_attn_idx / score / select / selblk.comp), for
 * n_seq sequences of seq_len consecutive rows at positions pos[s]+i on slot[s]:
 *   [q (idx_heads*idx_dim) | k (idx_dim)] = w . RMSNorm(x)*gamma in float32; the raw key goes to
 *   idxcache (binary16) at the row's cell; every block of `ratio` cells the pass completes is pooled
 *   (mean), RMS-normed with k_norm, rotated at its first cell's position and kept in `pooled`; a
 *   query head is normed with q_norm and rotated at the row's position; a block's score is the sum
 *   over heads of max(0, q_h . k); a cell's value is its block's score, plus 1e9 for blocks at or
 *   after the row's own incomplete block, and the score of the block that does not exist (cell 0
 *   pooled `ratio` times, the reference's zero fill) plus 1e9 for the cells after the last whole
 *   block; of the row's visible cells the (top_k + ratio - 1) largest are taken by a radix select:
 *   everything strictly above the threshold, then cells equal to it in ascending index.
 * mask [rows][mask_stride] receives the selection, a bit a cell, for shv_attn_decode.
 * idxcache is [n_slots][max_cells][idx_dim] binary16; pooled [n_slots][max_cells/ratio + 1][idx_dim]
 * float32 (the last row is rewritten by every call); work [rows][idx_heads*idx_dim + idx_dim] and
 * score [rows][max_cells/ratio + 1] are scratch.  rope is the attention's table. */
typedef struct {
    const float *x;
    const float *gamma;
    const float *w;
    const float *q_norm;
    const float *k_norm;
    const float *rope;
    uint16_t *idxcache;
    float *pooled;
    const int32_t *pos;
    const int32_t *slot;
    float *work;
    float *score;
    uint32_t *mask;
    int32_t n_seq, seq_len, n_embd;
    int32_t idx_heads, idx_dim, top_k, ratio, rope_dims;
    int32_t max_cells, mask_stride;
    float eps;
} shv_qsa_index_args;

/* Token embedding gather (Model.Embeddings, llm/model.go:134; hc.UploadInit, llm/graph.go:1815):
 * x[t] = float32(table[id_t]) for n_tok rows, id_t = ids[pos[0]+t] when pos is given, else ids[t].
 * table is [vocab][n_embd] in ggml type `type` (SHV_GGML_*): binary16 is the fast path, any other
 * accepted type is expanded as Tensor.DequantizeRow does (llm/model.go:125-131), bit for bit.
 * An id outside [0, vocab) yields a row of NaN. */
typedef struct {
    const void *table;
    const int32_t *ids;
    const int32_t *pos;
    float *x;
    int32_t n_tok, n_embd, vocab, x_stride;
    int32_t type;
} shv_embed_args;

/* Greedy sampler (Argmax, llm/sample.go:359-367): the index of the first maximum of each row of
 * logits [n_rows][n]; NaN never wins.  best[r] receives the index.  When ids and pos are given
 * (n_rows must be 1) the index is also stored as the next token, ids[pos[0]+advance], and pos[0]
 * is advanced by `advance` (0 means 1: the rows the pass carried), so a recorded decode step can be
 * replayed back to back without the host. */
typedef struct {
    const float *logits;
    int32_t *best;
    int32_t *ids;
    int32_t *pos;
    int32_t n_rows, n, logits_stride;
    int32_t advance;
} shv_argmax_args;

/* pos[s] += delta for s < n_seq: the step of a recorded pass that does not sample. */
typedef struct {
    int32_t *pos;
    int32_t n_seq, delta;
} shv_advance_args;

/* Rows of one ring of projection rows copied into another: positions pos[0]+first ..
 * pos[0]+first+count-1 (those below zero are skipped), row p from src[(p % src_slots) * stride] to
 * dst[(p % dst_slots) * stride], n floats each.  A prompt pass of many rows keeps its DeltaNet
 * projection rows in a ring of its own, sized for the pass: the conv's three rows of history are
 * brought into it before the step, and the pass's last three rows are left in the sequence's small
 * ring after it.  (No counterpart in the reference, whose conv window lives in the layer's own
 * activation buffer, llm/gpu_deltanet.go:1046-1052.) */
typedef struct {
    const float *src;
    float *dst;
    const int32_t *pos;
    int32_t src_slots, dst_slots, stride, n;
    int32_t first, count;
} shv_ring_rows_args;

typedef struct {
    uint32_t kind;
    uint32_t flags;          /* bit 0: may overlap the previous op (MultiDispatch.Overlap) */
    uint8_t args[248];
} shv_op;

/* ---- running ops ------------------------------------------------------------------------- */

/* Enqueue one op on the context's stream and return without waiting. */
int shv_enqueue(shv_ctx *ctx, uint32_t kind, const void *args, size_t args_bytes);

/* DispatchMultiTimed / DispatchMultiMarked (vk/engine.go:893-935): run the sequence `iters`
 * times, block until done, return GPU time for the whole run in total_ns (first launch to last
 * completion, gaps included) and, if per_op_ns is not NULL (one slot per op, iters must be 1),
 * the time each op's kernels ran, from timestamps on the kernels themselves. */
int shv_dispatch_multi(shv_ctx *ctx, const shv_op *ops, int n_ops, int iters,
                       uint64_t *total_ns, uint64_t *per_op_ns);

/* NewPrerecorded / Submit / Count / Destroy (vk/engine.go:997-1086): the sequence is recorded
 * once (a HIP graph) and replayed.  submit blocks and returns GPU time; launch does not block. */
int shv_prerecord(shv_ctx *ctx, const shv_op *ops, int n_ops, shv_prerecorded **out);
int shv_prerecorded_submit(shv_ctx *ctx, shv_prerecorded *p, int iters, uint64_t *total_ns);
int shv_prerecorded_launch(shv_ctx *ctx, shv_prerecorded *p);
/* GPU time between two points of the stream for work handed over with launch (which does not block):
 * shv_stamp(i) marks the point the stream has reached, i in 0..SHV_STAMPS-1; after a wait (shv_sync,
 * a submit, a download) shv_stamp_elapsed gives the nanoseconds from stamp `from` to stamp `to`. */
#define SHV_STAMPS 4
int shv_stamp(shv_ctx *ctx, int i);
int shv_stamp_elapsed(shv_ctx *ctx, int from, int to, uint64_t *ns);
int shv_prerecorded_count(const shv_prerecorded *p);
void shv_prerecorded_destroy(shv_ctx *ctx, shv_prerecorded *p);

/* Convenience entry points: one op each, enqueued without waiting. */
int shv_gemv_q4k(shv_ctx *ctx, const shv_gemv_q4k_args *a);
int shv_dequant_q4k(shv_ctx *ctx, const shv_dequant_q4k_args *a);
int shv_dequant(shv_ctx *ctx, const shv_dequant_args *a);
int shv_gemv(shv_ctx *ctx, const shv_gemv_args *a);
int shv_quantize_q4k(shv_ctx *ctx, const shv_quantize_q4k_args *a);
int shv_fill_normal(shv_ctx *ctx, const shv_fill_normal_args *a);
int shv_moe_router(shv_ctx *ctx, const shv_moe_router_args *a);
int shv_moe_up(shv_ctx *ctx, const shv_moe_up_args *a);
int shv_moe_down(shv_ctx *ctx, const shv_moe_down_args *a);
int shv_dn_step(shv_ctx *ctx, const shv_dn_step_args *a);
int shv_attn_decode(shv_ctx *ctx, const shv_attn_decode_args *a);
int shv_embed(shv_ctx *ctx, const shv_embed_args *a);
int shv_argmax(shv_ctx *ctx, const shv_argmax_args *a);
int shv_advance(shv_ctx *ctx, const shv_advance_args *a);
int shv_ring_rows(shv_ctx *ctx, const shv_ring_rows_args *a);
int shv_router_fold(shv_ctx *ctx, const shv_router_fold_args *a);
int shv_qsa_index(shv_ctx *ctx, const shv_qsa_index_args *a);

/* shv_argmax for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * results as shv_argmax; the per-block winners and arrival counters live in a static device
 * array of the library (under 8 KB on each GPU, bound at shv_init) instead of in memory the
 * context allocated, and the call allocates and frees nothing.  At most
 * SHV_ARGMAX_STATIC_MAX_ROWS rows a call; more is refused with SHV_E_INVALID.  All calls on one
 * GPU share the array: calls that overlap on one GPU (two contexts, two streams) race. */
#define SHV_ARGMAX_STATIC_MAX_ROWS 14
int shv_argmax_static(shv_ctx *ctx, const shv_argmax_args *a);

#ifdef __cplusplus
}
#endif
#endif
