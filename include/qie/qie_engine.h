/*
 * qie_engine.h — engine-level C ABI of libqie.so: weights, KV cache,
 * prefill and hipGraph-captured decode.
 *
 * Replaces the reference's driver / step API:
 *   llm()                               layers/src/qwen_main.cu:64-417, iengine.cuh:51
 *       -> qie_prefill() (state == prefill) / qie_decode_step() (state == decode)
 *   create_new_sequence()               layers/src/iengine.cu:25-47
 *   initialize_model_buffers()          layers/src/utills.cu:4-129
 *   destroy_model_buffers()             layers/src/utills.cu:142-205
 *       -> qie_batch_create() / qie_batch_destroy()
 *   create_page_list / allocate_page_buffers / free_page_list
 *                                       layers/src/iengine.cu:73-109
 *       -> the KV cache owned by qie_batch (contiguous per (layer, kv head))
 *   load_all_weights_to_gpu_chunked()   layers/src/iengine.cu:117-223
 *       -> qie_engine_load_weights_bin()
 *   parsed_tensors / build_indexed_tensors (tensor_parser.cpp:31-165)
 *       -> qie_index_* (reference-compatible weights.bin index)
 *
 * All functions return 0 on success; qie_last_error() (qie_ops.h) has the text.
 */
#ifndef QIE_ENGINE_H
#define QIE_ENGINE_H

#include "qie_types.h"
#include "qie_ops.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qie_engine qie_engine;
typedef struct qie_comm qie_comm;
typedef struct qie_batch qie_batch;
typedef struct qie_index qie_index;

/* ------------------------------------------------------------------ index
 * Reference-compatible tensor index (tensor_parser.hh:204-210):
 * {tensor_name, shape, data_offsets (bytes, re-based into one contiguous
 * weights.bin), layer_index (-1 for globals), short_name}; lm_head.weight
 * has short_name "logits". */
int qie_index_load_meta(const char* meta_data_txt, qie_index** out);   /* meta_data.txt format */
int qie_index_synthetic(const qie_model_spec* spec, qie_index** out);  /* HF names, sorted, one shard */
int qie_index_count(const qie_index* idx);
int qie_index_get(const qie_index* idx, int i, const char** name, const char** short_name,
                  int32_t* layer, int64_t* off0, int64_t* off1, int32_t* ndim, int64_t* shape4);
int64_t qie_index_total_bytes(const qie_index* idx);
int qie_index_write_meta(const qie_index* idx, const char* path);
void qie_index_destroy(qie_index* idx);

/* ----------------------------------------------------------------- engine */
/* ------------------------------------------------------ tensor parallelism
 * One communicator per rank.  RCCL: rank 0 calls qie_comm_unique_id() and ships the
 * QIE_COMM_ID_BYTES bytes to every rank (any host channel), then every rank calls
 * qie_comm_create_rccl() with its device (blocks until all ranks joined).  Local:
 * qie_comm_create_local(world, out[world]) makes `world` ranks of ONE process on one
 * device, driven by one host thread each (test backend; engines on it run without
 * hipGraphs).  Pass the handle as qie_engine_opts.tp_comm; the engine then holds
 * only its shard and every collective call of a step must be made by
 * all ranks (prefill, decode, qie_batch_logits). */
#define QIE_COMM_ID_BYTES 128
int qie_comm_unique_id(void* id_out);
int qie_comm_create_rccl(const void* id, int32_t world, int32_t rank, int32_t device, qie_comm** out);
int qie_comm_create_local(int32_t world, qie_comm** out);
/* Peer backend: every rank's exchange buffer mapped into every rank, one
 * kernel per collective (push + per-block generation flags + rank-ordered reduce, the
 * residual add fused into the row-parallel all-reduce); graph-capturable.  Across
 * processes: qie_comm_create_peer() returns this rank's QIE_COMM_PEER_HANDLE_BYTES IPC
 * handle, the host ships all handles to every rank (handles[r] = rank r's), then
 * qie_comm_peer_connect().  Ranks of one process on one device (world <= 2: the
 * process's hardware queues must give every rank its own):
 * qie_comm_create_peer_local(world, out[world]).  A rank that waited ~10 s for a peer
 * sets the error word qie_comm_peer_error() reads (no kernel waits forever); it then stores
 * no result, the communicator stays poisoned (later exchanges return at once) and the
 * engine's next synchronising call fails. */
#define QIE_COMM_PEER_HANDLE_BYTES 128
int qie_comm_create_peer(int32_t world, int32_t rank, int32_t device, qie_comm** out, void* handle_out);
int qie_comm_peer_connect(qie_comm* c, const void* handles);
int qie_comm_create_peer_local(int32_t world, qie_comm** out);
int qie_comm_peer_error(const qie_comm* c, int32_t* err);
/* Peer backend exchange form, set identically on every rank between steps
 * (a captured decode graph keeps the form it was captured with): tagged = 1 sends
 * row-parallel exchanges of <= 131,072 elements as {generation tag, f32} words that the
 * readers poll directly (no flags, no system fences), 0 the flagged form; push = 1 (with
 * tagged) lets a batch-1 projection's GEMV epilogue write those words itself, so the
 * exchange kernel only waits and reduces.  Results are bit-identical in every form.
 * Defaults: env QIE_PEER_TAGGED / QIE_PEER_PUSH, else 1 / 1. */
int qie_comm_peer_set_mode(qie_comm* c, int32_t tagged, int32_t push);
/* x (bf16 [n]) = bf16(x + bf16(sum over ranks of part)), in place on x (part may be
 * overwritten): the exchange after a row-parallel projection */
int qie_comm_allreduce_residual_bf16(qie_comm* c, const float* part, void* x, int64_t n, void* stream);
/* Measurement: `count` row-parallel exchanges of n elements captured in one hipGraph on
 * `stream` and replayed `reps` times (after one warm replay); *us_out = microseconds per
 * exchange (hipEvents).  form 0: as the engine runs them (the current mode), 1: the flagged
 * form, 2: the flagged form with n = 0 (the synchronisation alone at the same grid).  Every
 * rank must call it with the same arguments. */
int qie_comm_time_exchange(qie_comm* c, const float* part, void* x, int64_t n, int32_t count, int32_t reps,
                           int32_t form, void* stream, float* us_out);
int qie_comm_rank(const qie_comm* c, int32_t* world, int32_t* rank);
int qie_comm_allreduce_sum_f32(qie_comm* c, float* buf, int64_t n, void* stream);
/* in place: element-wise max over ranks of u64 words (the greedy arg-max keys) */
int qie_comm_allreduce_max_u64(qie_comm* c, uint64_t* buf, int64_t n, void* stream);
void qie_comm_destroy(qie_comm* c);

typedef struct qie_engine_opts {
    int32_t device;          /* HIP device ordinal                                   */
    int32_t max_ctx;         /* RoPE table rows (reference CONTEXT_SIZE = 32786)     */
    int32_t use_graph;       /* 1: decode steps replay a captured hipGraph           */
    int32_t tp_rank, tp_size;/* informational; taken from tp_comm when it is set     */
    void* tp_comm;           /* qie_comm* (tensor parallel over its ranks) or NULL   */
    int32_t weight_fp8;      /* 1: linear weights + lm_head quantised to OCP e4m3 with
                                power-of-two row scales after loading (qie_ops.h)     */
    int32_t comm_always;     /* 1: run the exchange steps (row-parallel all-reduces, the
                                greedy key max, the logit gather) through tp_comm even at
                                world 1 — the captured-collective path on one GPU (tests) */
    int32_t prefill_fp8;     /* 1 (with weight_fp8): the prefill projections run on the
                                block-scaled fp8 MFMA (QIE_LINEAR_ACT_FP8) — activations
                                quantised per row to e4m3 before each projection, a
                                different model from the bf16-activation one (numerics flag) */
    int32_t compute_f32;     /* layered engines: 1 = every product, activation and cache row in
                                true fp32 (weights widened exactly from bf16); 0 = bf16 matrix
                                operands with fp32 accumulation, the residual stream, norms,
                                routers, scores and softmax in fp32 either way               */
    int32_t reserved[4];
} qie_engine_opts;

int qie_engine_create(const qie_model_spec* spec, const qie_engine_opts* opts, qie_engine** out);
/* Synthetic checkpoint at real shapes (no weights ship here): reference-layout
 * arena (qie_index_synthetic), every tensor filled by qie_synthetic_fill with
 * tensor_id = qie_tensor_id(name): linear weights offset 0 / scale w_scale,
 * norm weights 1 + norm_scale*u, biases bias_scale*u. */
int qie_engine_init_synthetic(qie_engine* e, uint64_t seed, float w_scale, float norm_scale,
                              float bias_scale);
/* Reference flat weights.bin + meta_data.txt index, read in chunks through a
 * pinned staging buffer (load_all_weights_to_gpu_chunked semantics). */
int qie_engine_load_weights_bin(qie_engine* e, const char* weights_bin, const char* meta_data_txt,
                                int64_t chunk_bytes);
/* Caller-owned device weights (e.g. torch tensors); not freed by qie. */
int qie_engine_set_weights(qie_engine* e, const qie_model_weights* w);
int qie_engine_weights(const qie_engine* e, qie_model_weights* out, const qie_layer_weights** layers);
int qie_engine_spec(const qie_engine* e, qie_model_spec* out);
void* qie_engine_stream(qie_engine* e);
int qie_engine_sync(qie_engine* e);
void qie_engine_destroy(qie_engine* e);

/* ------------------------------------------------------------------ batch
 * B independent sequences decoded together (weights streamed once per step).
 * KV cache [B][L][nkv][max_ctx][hd] bf16; token history [B][max_ctx]. */
int qie_batch_create(qie_engine* e, int32_t batch, int32_t max_ctx, qie_batch** out);
void qie_batch_destroy(qie_batch* b);

/* Paged KV cache with a device block table.  Replaces the
 * reference's per-sequence linked page list — create_page_list /
 * allocate_page_buffers / free_page_list (iengine.cu:73-109) walked by
 * kv_copy_layer_to_cache_prefill/decode (include_cuda.cu:165-279) and the
 * batch_metadata slots (iengine.cuh:27-37).  A pool of n_pages pages of
 * page_tokens tokens (a power of two >= 128; 0 = 128) shared by the B slots;
 * n_pages 0 = enough for every slot at max_ctx.  Pages are taken on demand by
 * qie_prefill / qie_decode* / qie_batch_set_position and returned by
 * qie_batch_release; running out of pages fails the call (-28, nothing launched).
 * Page 0 is a scratch page that idle slots write into. */
int qie_batch_create_paged(qie_engine* e, int32_t batch, int32_t max_ctx, int32_t page_tokens,
                           int32_t n_pages, qie_batch** out);
/* Ends sequence `seq`: its pages go back to the pool (paged) and the slot idles —
 * it still runs through every decode step on the scratch page, its outputs are
 * meaningless — until the next qie_prefill into it.  Any batch. */
int qie_batch_release(qie_batch* b, int32_t seq);
/* Pool state: free pages, pages per slot (host [B], may be NULL), page_tokens. */
int qie_batch_page_stats(qie_batch* b, int32_t* free_pages, int32_t* pages_per_seq, int32_t* page_tokens);
/* The n first block-table entries of `seq` (host copy); paged batches only. */
int qie_batch_block_table(qie_batch* b, int32_t seq, int32_t* host_pages, int32_t n);

/* Prefill sequence `seq` with n prompt ids (host array); writes its KV rows
 * 0..n-1, samples the first generated token (host *next_id, may be NULL) and
 * makes it the sequence's current token at position n. */
int qie_prefill(qie_batch* b, int32_t seq, const int32_t* ids, int32_t n, const qie_sampling* s,
                int32_t* next_id);
/* qie_prefill of n_seqs prompts of len ids each (host [n_seqs][len], laid end to end)
 * into slots seq0 .. seq0+n_seqs-1 in one pass: every projection GEMM runs once over
 * the n_seqs*len rows (the reference prefills one sequence per call, iengine.cu
 * prefill path; this is the batch-admission form of it).  next_ids: host [n_seqs]
 * or NULL.  Paged batches: all-or-nothing on the pool, as qie_prefill. */
int qie_prefill_batch(qie_batch* b, int32_t seq0, int32_t n_seqs, const int32_t* ids, int32_t len,
                      const qie_sampling* s, int32_t* next_ids);
/* One decode step for all B sequences (hipGraph replay when enabled);
 * next_ids: host [B] or NULL (then nothing is synchronised). */
int qie_decode_step(qie_batch* b, const qie_sampling* s, int32_t* next_ids);
/* n_steps decode steps back to back; out_ids host [n_steps][B] (may be NULL). */
int qie_decode(qie_batch* b, int32_t n_steps, const qie_sampling* s, int32_t* out_ids);
/* Last logits of every sequence: host bf16 [B][V]. */
int qie_batch_logits(qie_batch* b, void* host_out);
/* Current positions (host int32 [B]) and token history row of `seq`. */
int qie_batch_positions(qie_batch* b, int32_t* host_pos);
int qie_batch_history(qie_batch* b, int32_t seq, int32_t* host_ids, int32_t n);
/* Rewind/set sequence `seq` to position pos with current token `token`
 * (KV rows >= pos are simply overwritten later). */
int qie_batch_set_position(qie_batch* b, int32_t seq, int32_t pos, int32_t token);
/* Decode structure of the batch's steps: 0 = five launches per layer (the reference path:
 * QKV GEMV, attention, O GEMV, gate/up GEMV, down GEMV, hipGraph-captured); 1 = the whole
 * layer stack as ONE persistent launch (one workgroup per CU, weight streams running ahead of
 * the layer's dependency edges, tagged hand-offs between CUs; bit-identical outputs).  Mode 1
 * covers batch 1, bf16 weights, one device, head_dim 64 or 128 and a contiguous KV cache;
 * other batches return an error (QIE_EINVAL) naming what is not covered.  The next step
 * re-captures the decode graph.  qie_batch_decode_mode returns the current mode.  Mode 1 is
 * SLOWER on MI355X (Qwen2-7B 317.5 vs 370.9 tok/s, Qwen2-0.5B 1,065 vs 1,566: its cross-CU
 * hand-offs cost more than the kernel boundaries they replace); mode 0 is
 * the default and the measured path. */
int qie_batch_set_decode_mode(qie_batch* b, int32_t mode);
int qie_batch_decode_mode(const qie_batch* b);
/* Diagnostics of decode mode 1: enable != 0 makes the persistent step record s_memrealtime
 * stamps (100 MHz, chip-wide) at its phase boundaries, [n_cu][n_layers][12] uint64 (slots:
 * 0 layer start, 1 x gathered, 2 QKV done, 3 attention done (attention CUs), 4 attention
 * output gathered (other CUs), 5 O done, 6 x' gathered + norm, 7 gate/up done, 8 h gathered,
 * 9 down done); host_out (n >= that count) receives the last step's stamps; enable = 0
 * frees the buffer.  Changing it re-captures the decode graph. */
int qie_batch_pk_trace(qie_batch* b, int32_t enable, uint64_t* host_out, int64_t n);
/* Batch geometry: B slots, max_ctx positions per slot. */
int qie_batch_dims(const qie_batch* b, int32_t* batch, int32_t* max_ctx);
/* KV descriptor of slot `seq` for the operator tier (qie_kv_write, qie_attention with
 * sequence index 0): contiguous -> that slot's region; paged -> the pool with the
 * slot's block-table row.  Valid until the batch is destroyed. */
int qie_batch_kv_cache(const qie_batch* b, int32_t seq, qie_kv_cache* out);
/* Operator tier: make slot `seq` a live sequence holding the KV pages for positions
 * [0, n_tokens) (paged: taken from the pool, all-or-nothing; contiguous: a bounds
 * check).  allocate_page_buffers (iengine.cu:90-100) in the reference's terms. */
int qie_batch_reserve(qie_batch* b, int32_t seq, int32_t n_tokens);
/* The engine's weight arena (load_all_weights_to_gpu_chunked's d_base_out /
 * total_bytes_out, iengine.cu:117) and its RoPE tables (fp32 [rows][head_dim/2]). */
int qie_engine_arena(const qie_engine* e, void** base, int64_t* bytes);
int qie_engine_rope_tables(const qie_engine* e, const float** rope_cos, const float** rope_sin,
                           int32_t* rows);
/* Time `iters` launches of one of the decode step's kernels with hipEvents on
 * the engine stream (which: 0 = gate/up GEMV, 1 = down GEMV, 2 = QKV GEMV,
 * 3 = O GEMV, 4 = lm_head GEMV, 5 = attention; the layer GEMVs cycle through
 * layers 1..L-1 so no weight stays cache-resident; 6 = the persistent layer stack of decode
 * mode 1, all layers per launch, the sequence state restored afterwards).  Returns the average
 * microseconds per launch and the algorithmic bytes per launch. */
int qie_batch_time_kernel(qie_batch* b, int32_t which, int32_t iters, double* avg_us,
                          double* bytes);
/* One decode step run eagerly (as qie_decode_step) that also copies the residual stream
 * into host_x: bf16 [2 n_layers + 1][batch][hidden], slot 0 = the step's input row, slot
 * 2l + 1 = after layer l's attention block (O-proj + residual), 2l + 2 = after its MLP
 * block (down-proj + residual).  Parity diagnostics (tools/flip_attrib.py). */
int qie_batch_debug_step(qie_batch* b, const qie_sampling* smp, int32_t* next_ids, void* host_x);


/* ---------------------------------------------------------- layered engines
 * A model given as a per-layer program instead of the fixed Qwen decoder: every layer names its
 * mixer and its feed-forward with their own sizes and constants, so one engine serves layer
 * orders and sizes that differ from layer to layer.  The same qie_engine / qie_batch handles,
 * slots, block table and page pool as above; the step is ragged (qie_batch_step): portions of
 * prompts beside single decoded tokens in one pass.
 *
 * Mixer QIE_MIXER_LATENT_ATTENTION: queries q = W_q h laid out per head as [dim unrotated |
 * rot_dim rotated]; W_dkv h = [compressed row (kv_rank), RMS-normed with a weight | one rotated
 * key part shared by all heads]; per head k = W_uk c, v = W_uv c; rotate-half rotary on the
 * first rot_dims coordinates of the rotated parts (angle pos * rot_base^(-2i/rot_dims));
 * softmax over the last `window` positions; per-head sigmoid gate from the mixer's input;
 * W_o.  Only [c | rotated key part] is cached.  kv_from >= 0: the layer has no W_dkv and reads
 * that layer's cache rows.  The engine runs the absorbed form (W_uk folded into the query,
 * W_uv applied to the softmax-weighted sum of c), for prompts and decoding alike.
 * Feed-forward: none, dense gated SiLU, or a mixture of `experts` gated-SiLU experts with a
 * sigmoid router (fp32) whose `top` largest scores, not renormalised, scale the experts' input.
 * (Ranked by the fp32 router logits, which order the experts as the scores do but do not
 * saturate; equal logits: the lower index.)
 * Layer: y = x + g1 * rms(mixer(x)); z = y + g2 * rms(ff(y)) (scalar gains; each branch is
 * normed after it is computed, its input is the raw stream); the next layer's input is the depth-weighted sum over the embedding
 * output and every layer result so far. */
enum { QIE_MIXER_LATENT_ATTENTION = 1, QIE_MIXER_GQA = 2, QIE_MIXER_GQA_RECURRENT = 3, QIE_MIXER_MINGRU = 4,
       QIE_MIXER_CHANNEL_DELTA = 5 };
enum { QIE_FF_NONE = 0, QIE_FF_DENSE = 1, QIE_FF_MOE = 2 };
/* Which keys j <= i a query at position i sees: all of them; the last `size`; those of its own
 * block of `size` positions (blocks counted from position 0 of the sequence). */
enum { QIE_MASK_CAUSAL = 0, QIE_MASK_WINDOW = 1, QIE_MASK_CHUNK = 2 };
/* RMS norm of every query / key head over dim before rotation: none, with a weight vector
 * shared by the heads, or without one. */
enum { QIE_QKNORM_NONE = 0, QIE_QKNORM_WEIGHT = 1, QIE_QKNORM_PLAIN = 2 };
/* Rotary pairs inside the rotated coordinates: i with i + dims / 2, or 2i with 2i + 1. */
enum { QIE_ROT_HALVES = 0, QIE_ROT_INTERLEAVED = 1 };
/* Block: 0 = y = x + g * rms(branch(x)) with scalar gains (branches read the raw stream);
 * 1 = x += N_b(branch(N_a(x))) with weight vectors stored around zero (N(v) = rms(v) (1 + w))
 * before and after every branch; 2 = x += branch(N(x)) with N(v) = rms(v) (norm_offset + w) (weight
 * vectors 'l<i>.norm1|norm2', 'final.norm'; norm_offset 0: plain weights, 1: stored around zero), one
 * norm before every branch and none after.  Options of block 2 (qie_arch_desc): several residual
 * streams with learned mixing (streams), a causal convolution on the mixer's normed input
 * (canon_taps), a norm of the embedding rows (embed_norm). */
enum { QIE_BLOCK_POSTNORM_GAIN = 0, QIE_BLOCK_SANDWICH = 1, QIE_BLOCK_PRENORM = 2 };
/* Router: 0 = sigmoid scores, the `top` largest scale the experts' input; 1 = logits with a
 * bias, the `top` largest weighted by the softmax over those alone scale the experts' output. */
enum { QIE_ROUTER_SIGMOID_IN = 0, QIE_ROUTER_SOFTMAX_OUT = 1, QIE_ROUTER_SOFTMAX_ALL = 2 };
/* Router 2: scores s = softmax over ALL router outputs (`experts` experts with weights, then
 * `identity` experts whose output is their input); experts are chosen by s + correction ('l<i>.mlp.
 * correction'), only inside the `groups_keep` best of `groups` contiguous, equally sized groups of
 * outputs (a group's rank: its largest s + correction); the `top` chosen are weighted by
 * s / (sum of the chosen s + 1e-20) * route_scale, applied to the experts' outputs. */
/* Dense feed-forward: 0 = W_down (silu(W_gate h) * W_up h); 1 = W_down xielu(W_up h) with the two
 * numbers p, q of 'l<i>.mlp.act': xielu(z) = softplus(p) z^2 + z / 2 for z > 0, else
 * (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2.  Experts are always of form 0. */
/* 2 = W_down (gelu_tanh(W_gate h) * W_up h), gelu_tanh(z) = z / 2 (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))). */
enum { QIE_ACT_SILU_GATED = 0, QIE_ACT_XIELU = 1, QIE_ACT_GELU_TANH_GATED = 2 };
/* Attention weights of the visible keys: softmax of the scores, or sigmoid(score + pb_h) with a
 * number per head ('mix.pb'); a row's weights are used as they are. */
enum { QIE_WEIGHTS_SOFTMAX = 0, QIE_WEIGHTS_SIGMOID = 1 };
/* Positions in the embedding: none, or the vector with entry 2i = sin(p * 10000^(-2i / width)),
 * entry 2i + 1 = cos of the same, added to the scaled embedding row. */
enum { QIE_POS_NONE = 0, QIE_POS_SINUSOID = 1 };

/* Mixer QIE_MIXER_GQA: grouped-query softmax attention over a paged K / V cache.  q = W_q h
 * (heads x dim), k = W_k h (kv_heads x dim), v = W_v h (kv_heads x vdim); query head h reads
 * key / value head h / (heads / kv_heads).  Options, each a parameter: the q / k head norm; a
 * rotary on the first rot_dims coordinates of q and k (angle pos * rot_base^(-2i / rot_dims));
 * rot_values: the value at position j is turned by j over all vdim coordinates (same pairing,
 * angle j * rot_base^(-2m / vdim)), cached so, and a head's weighted sum at position i is turned
 * back by i; the mask; values_are_keys: no W_v, the value is the projected key as it leaves W_k
 * (before its norm; vdim == dim); dist_bias: the score loses r1_h * ln(1 + r2_h * (i - j)). */
/* Rotary frequencies scaled by their wavelength l = 2 pi / f (factor 0: no scaling): f stays where
 * l < original / high, becomes f / factor where l > original / low, and between the two, with
 * s = (original / l - low) / (high - low), (1 - s) f / factor + s f. */
typedef struct qie_rot_scaling {
    float factor, low, high, original;
} qie_rot_scaling;

typedef struct qie_gqa_desc {
    int32_t heads, kv_heads, dim, vdim;
    int32_t qk_norm;          /* QIE_QKNORM_*   */
    int32_t rot_dims;         /* even, <= dim; 0 = no rotation of q and k */
    int32_t rot_layout;       /* QIE_ROT_*      */
    int32_t rot_values;
    int32_t mask, mask_size;  /* QIE_MASK_*     */
    int32_t values_are_keys;
    int32_t dist_bias;
    float rot_base, scale;
    int32_t qk_bias;          /* 1: q and k get a bias vector after their projection ('mix.q.b', 'mix.k.b'); a key cached as
                                 the value carries its bias */
    int32_t sink;             /* 1: the softmax denominator also holds exp(sink_h), a number per head ('mix.sink') that has
                                 no key and no value                                                             */
    int32_t weights;          /* QIE_WEIGHTS_*                                               */
    int32_t slope_bias;       /* 1: the score loses 2^(-8 (h + 1) / heads) * (i - j)         */
    int32_t head_gate;        /* 1: head h's output times sigmoid(W_g x)_h ('mix.g' [heads, width]) */
    int32_t q_temp_every;     /* > 0: after its norm q is multiplied by                      */
    float q_temp_coef;        /*   1 + coef * ln(floor((pos + 1) / every) + 1)               */
    int32_t out_gate;         /* 1: the concatenated head outputs times sigmoid(W_g x), element by element
                                 ('mix.g' [heads * vdim, width])                             */
    int32_t reserved2[2];
    qie_rot_scaling rot_scaling;
} qie_gqa_desc;

/* Gated linear recurrence (the second half of QIE_MIXER_GQA_RECURRENT): per head a state
 * S [dim][vdim] in fp32 that lives in the slot, S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,
 * o_t = S_t^T q_t with q = silu(W_q h), v = W_v h and the forget gate
 * f = lower + (1 - lower) * sigmoid(W_f h + b); o is RMS-normed per head over vdim with a weight
 * vector.  A slot that starts at position 0 starts from S = 0.  The mixer's result is
 * gqa_scale * attention + rec_scale * recurrence (each after its own output projection). */
typedef struct qie_recurrent_desc {
    int32_t heads, dim, vdim;
    int32_t reserved;
} qie_recurrent_desc;

/* Mixer QIE_MIXER_MINGRU: a recurrence per channel whose update gate and candidate depend on the current input alone.  With x the
 * mixer's input: z = sigmoid(W_z x + b_z), u = W_x x + b_x (`width` channels each), candidate
 * c = u + 1/2 where u >= 0, sigmoid(u) where u < 0; per channel S_t = (1 - z_t) S_(t-1) + z_t c_t,
 * S fp32 in the slot, zero at position 0; output W_o (S_t * silu(W_g x)).  Tensors
 * 'l<i>.mix.z|z.b|x|x.b|g|o'. */
typedef struct qie_mingru_desc {
    int32_t width;
    int32_t reserved[3];
} qie_mingru_desc;

/* Mixer QIE_MIXER_CHANNEL_DELTA: gated delta rule with one decay per head and key channel.  With x the
 * mixer's input: q = W_q x, k = W_k x (kv_heads x dim), v = W_v x (heads x vdim); each passes a causal
 * convolution over time per channel ('mix.q.conv' etc. [channels, conv], last column = the current
 * token) and silu; q and k become unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q times dim^(-1/2);
 * beta = sigmoid(W_b x) per head; decay g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 x) + dt_bias)), heads x
 * dim.  Per head (query / key head h / (heads / kv_heads)), S [dim][vdim] fp32 in the slot, zero at
 * position 0: S = diag(g) S; u = beta (v - S^T k); S += k u^T; o = S^T q.  o is RMS-normed per head over
 * vdim with the weight 'mix.norm' [vdim], times sigmoid(W_g2 (W_g1 x)) (heads x vdim), then W_o.  The
 * last conv - 1 rows of q, k, v before their convolution belong to the slot's state.  rank_a / rank_g:
 * rows of W_a1 / W_g1.  Tensors 'l<i>.mix.q|q.conv|k|k.conv|v|v.conv|b|A_log|a1|a2|dt_bias|g1|g2|norm|o'. */
typedef struct qie_delta_desc {
    int32_t heads, kv_heads, dim, vdim, conv, rank_a, rank_g;
    int32_t reserved;
} qie_delta_desc;

typedef struct qie_layer_desc {
    int32_t mixer;            /* QIE_MIXER_*                                          */
    int32_t heads, dim, rot_dim, vdim, kv_rank;
    int32_t window;           /* query at position i attends keys i - window < j <= i */
    int32_t kv_from;          /* -1: own W_dkv; else the layer whose cache rows it reads */
    int32_t rot_dims;         /* rotated coordinates of a rotated part (even, <= rot_dim) */
    float rot_base, scale;
    int32_t ff_kind;          /* QIE_FF_*                                             */
    int32_t ff;               /* hidden size of the dense feed-forward / of one expert */
    int32_t experts, top;
    int32_t router;           /* QIE_ROUTER_*                                          */
    /* latent attention options: q_rank > 0: the queries come through a latent of their own,
     * q = W_uq rms(W_dq x) w ('mix.dq' [q_rank, width], 'mix.dq.norm', 'mix.uq'; no 'mix.q');
     * rot_layout QIE_ROT_*; head_gate 1: the per-head sigmoid gate 'mix.g'.  window 0: every j <= i. */
    int32_t q_rank, rot_layout, head_gate;
    qie_gqa_desc gqa;         /* QIE_MIXER_GQA, QIE_MIXER_GQA_RECURRENT                */
    qie_recurrent_desc rec;   /* QIE_MIXER_GQA_RECURRENT                               */
    float gqa_scale, rec_scale;
    qie_mingru_desc mingru;   /* QIE_MIXER_MINGRU                                      */
    int32_t ff_act;           /* QIE_ACT_* of a dense feed-forward                     */
    int32_t identity;         /* QIE_ROUTER_SOFTMAX_ALL: identity experts after the `experts` real ones */
    int32_t groups, groups_keep;
    float route_scale;
    int32_t reserved3[3];
    qie_delta_desc delta;     /* QIE_MIXER_CHANNEL_DELTA                               */
    qie_rot_scaling rot_scaling;   /* latent attention                                 */
} qie_layer_desc;

typedef struct qie_arch_desc {
    int32_t n_layers, width, vocab;
    float norm_eps;
    int32_t depth_mix;        /* 1: depth-weighted sum of all earlier results ('l<i>.dwa') */
    int32_t block;            /* QIE_BLOCK_*                                            */
    int32_t tied_head;        /* 1: the logits are taken against 'embed' (no 'head')    */
    /* layers [loop_start, loop_stop) run loop_times times in a row with the same weights (each
     * run with its own cache region and state); before every run of the group but the first
     * the embedding rows are added to the stream.  loop_times <= 1: every layer once. */
    int32_t loop_start, loop_stop, loop_times;
    int32_t pos_embed;        /* QIE_POS_*                                              */
    float embed_scale;        /* the embedding row is multiplied by it (0 is read as 1) */
    const qie_layer_desc* layers;
    /* QIE_BLOCK_PRENORM only.  streams >= 1: `streams` copies x_1 .. x_n of the residual row, all equal to
     * the embedding output at the start; sublayer q of layer i (1 mixer, 2 feed-forward) reads
     * u = sum_s in[s] x_s, computes y = sublayer(N(u)) and sets, all at once from the old rows,
     * x_t = sum_s mix[s][t] x_s + out[t] y ('l<i>.hc<q>.in|out' [streams], 'l<i>.hc<q>.mix' [streams,
     * streams]); the output norm reads the sum of the rows.  0: one row, x += y.
     * canon_taps >= 1: the mixer reads h + conv(h) instead of its normed input h, conv(h)_t = sum_j w[:, j]
     * h_(t - taps + 1 + j) per channel ('l<i>.canon1' [width, taps]); the last taps - 1 rows h belong to
     * the slot's state.  embed_norm 1: the embedding rows pass N with 'embed.norm' first. */
    int32_t streams, canon_taps, embed_norm;
    float norm_offset;
} qie_arch_desc;

int qie_engine_create_layered(const qie_arch_desc* arch, const qie_engine_opts* opts, qie_engine** out);
/* Hand the engine one checkpoint tensor (host memory, copied): dtype 0 = bf16 words, 1 = int32,
 * 2 = fp32.  Names: 'embed', 'head', 'final.norm', 'l<i>.norm1|norm2|dwa' (sandwich blocks: also
 * 'l<i>.norm1b|norm2b', all vectors of the width), 'l<i>.mix.q|dkv|dkv.norm|uk|uv|g|o' (latent
 * attention), 'l<i>.mix.q|k|v|q.norm|k.norm|r1|r2|o' (QIE_MIXER_GQA; under 'l<i>.mix.left.' when a
 * recurrence runs beside it, whose tensors are 'l<i>.mix.right.q|f|f.b|lower|v|norm|o'),
 * 'l<i>.mix.pb|g' (sigmoid weights, head gate), 'l<i>.mix.z|z.b|x|x.b|g|o' (QIE_MIXER_MINGRU),
 * 'l<i>.mix.q.b|k.b|sink' (biased, sink attention), 'l<i>.mix.dq|dq.norm|uq' (latent queries), the
 * QIE_MIXER_CHANNEL_DELTA tensors, 'embed.norm', 'l<i>.hc1|hc2.in|out|mix', 'l<i>.canon1',
 * 'l<i>.mlp.gate|up|down|act|router|router.b|correction', 'l<i>.mlp.e<j>.gate|up|down'.
 * qie_engine_finalize_weights checks every tensor the architecture needs against its shape,
 * builds the device layouts (fused projection rows, per-head transposed W_uk, experts end to
 * end) and drops the host copies. */
int qie_engine_put_tensor(qie_engine* e, const char* name, const void* host, int32_t dtype, int32_t ndim,
                          const int64_t* shape);
int qie_engine_finalize_weights(qie_engine* e);
/* One ragged step over a paged batch of a layered engine (qie_batch_create_paged; page_tokens a
 * power of two >= 16): entry i feeds counts[i] tokens (laid end to end in `tokens`) to slot
 * slots[i], continuing at the slot's position (a released or fresh slot starts at 0).  Pages are
 * taken for exactly the positions written, all-or-nothing over the whole step.  want_rows
 * (n_want indices into the step's packed rows) selects the rows whose logits are computed:
 * fp32 [n_want][vocab] to host_logits (may be NULL: they stay on the device for
 * qie_batch_step_sample). */
int qie_batch_step(qie_batch* b, int32_t n_entries, const int32_t* slots, const int32_t* counts, const int32_t* tokens,
                   int32_t n_want, const int32_t* want_rows, float* host_logits);
/* Samples one id per wanted row of the last qie_batch_step; host_ids [n_want].  Greedy
 * (top_k <= 1 or temperature <= 0): arg-max of the fp32 row, ties to the lowest id; otherwise
 * qie_sample on the rows rounded to bf16, as the sampler reads them. */
int qie_batch_step_sample(qie_batch* b, const qie_sampling* s, int32_t* host_ids);
/* Steps of at most 16 rows replay a hipGraph of their shape (rows, wanted rows, row groups),
 * captured the second time the shape is seen, when the engine was created with use_graph; every
 * per-step value (ids, slots, positions, block table, row groups) is read from device memory.
 * Instantiated graphs and replays so far: */
int qie_batch_step_graphs(qie_batch* b, int32_t* n_graphs, int64_t* n_replays);
/* Diagnostics: enable != 0 makes every following step keep the stream after each layer run (a
 * repeated layer counts every time); qie_batch_step_layers copies the last step's
 * [layer runs][rows][width] fp32 to host_out.  qie_engine_layer_runs: how many there are. */
int qie_engine_layer_runs(const qie_engine* e);
int qie_batch_keep_layers(qie_batch* b, int32_t enable);
int qie_batch_step_layers(qie_batch* b, float* host_out, int64_t n);
/* Time `iters` runs of one stage of the last step's shape (hipEvents on the engine stream):
 * which 0 = the whole layer stack, 1 = attention of `layer`, 2 = its projections (input, absorb,
 * value expansion, output), 3 = its feed-forward, 4 = its recurrence (gated scan + head norm, the
 * minGRU scan, or the delta rule's gates, scan and output norm; the slots' states of that layer run are advanced by it, so time it last).  The cache is read, not
 * advanced. */
int qie_batch_time_stage(qie_batch* b, int32_t which, int32_t layer, int32_t iters, double* avg_us);

#ifdef __cplusplus
}
#endif

#endif /* QIE_ENGINE_H */
