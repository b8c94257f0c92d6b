/*
 * yalm_hip.h — the drop-in C ABI of the MI355X (gfx950) decode engine.
 *
 * This header replaces the GPU-facing interface of the reference
 * (/root/reference/src/model.h:33-39, 70-79, 353-385 and the C++ members
 * compiled in src/infer.cu). It contains no HIP, CUDA or C++ types: every
 * entry point takes plain pointers, sizes and POD structs, so the reference's
 * own host (model.cpp, main.cpp, test.cpp) — or our C++20 mirror of it under
 * yalm_amd/host/ — binds it directly.
 *
 * Errors: every int-returning function returns YALM_OK (0) or a YALM_ERR_*
 * code; yalm_last_error() describes the last failure on the calling thread.
 * (The reference aborts on any runtime error, infer.cu:13-31; callers that
 * want that behaviour check the code and abort.)
 *
 * Threading: one decoder per stream; a decoder is not re-entrant (same as the
 * reference's InferenceState, model.h:84-190).
 */
#ifndef YALM_HIP_H
#define YALM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define YALM_OK 0
#define YALM_ERR_HIP 1         /* a HIP runtime call failed */
#define YALM_ERR_ARG 2         /* bad argument / shape */
#define YALM_ERR_UNSUPPORTED 3 /* configuration the kernels do not implement */

/* DType codes follow the reference enum order (codec.h:15-25). */
enum { YALM_F32 = 0, YALM_F16 = 1, YALM_BF16 = 2, YALM_F8E5M2 = 3 };
/* ActivationType (model.h:14-17) */
enum { YALM_GELU = 0, YALM_SILU = 1 };
/* InferenceMode (model.h:28-31) */
enum { YALM_HYDRATE_KV_CACHE = 0, YALM_OUTPUT_LOGITS = 1 };

/* Opaque stream handle; replaces cudaStream_t in init_cuda_stream (model.h:39). */
typedef struct yalm_stream_s *yalm_stream;
/* Opaque decoder: the device half of InferenceState + Model (model.h:84-190,
 * 303-327) — scratch buffers, KV caches, per-mode hipGraphs. */
typedef struct yalm_decoder_s *yalm_decoder;

/* Config (model.h:41-68). Same field meaning; MoE fields are not carried
 * because the reference GPU path asserts on MoE (infer.cu:865-867). */
typedef struct yalm_config {
	int dim, hidden_dim, head_dim, n_layers, n_heads, n_kv_heads, vocab_size, max_seq_len;
	float rope_theta;
	int rotary_dim;
	float norm_eps;
	int act;          /* YALM_GELU / YALM_SILU */
	float qkv_clip;   /* FLT_MAX when absent (model.cpp:60-61) */
	int weight_dtype; /* YALM_F32 / YALM_F16 / YALM_F8E5M2 */
} yalm_config;

/* Device pointers of one block (Block private fields, model.h:286-300). If
 * key_cache/value_cache are NULL the decoder allocates them (zeroed,
 * max_seq_len x n_kv_heads x head_dim f16 each). */
typedef struct yalm_block_weights {
	const float *rms_att, *rms_ffn;
	const void *wq, *wk, *wv, *wo, *w1, *w2, *w3;
	uint16_t *key_cache, *value_cache;
} yalm_block_weights;

/* Device pointers of the model (Model fields, model.h:303-311). wcls may equal
 * token_embedding (tied weights, model.cpp:370-377). blocks is a HOST array
 * of n_layers entries, copied by yalm_decoder_create. */
typedef struct yalm_model_weights {
	const void *token_embedding;
	const float *rms_final;
	const void *wcls;
	const yalm_block_weights *blocks;
} yalm_model_weights;

/* ---------------- device shim: replaces model.h:33-39 / infer.cu:59-90 ---------------- */
const char *yalm_last_error(void);
/* set_cuda_device (model.h:38): selects the HIP device for this thread. */
int yalm_set_device(int device);
/* upload_cuda (model.h:33): device alloc + H2D copy; returns NULL on failure. */
void *yalm_upload(const void *host, size_t size);
/* device alloc (zero-filled); returns NULL on failure. */
void *yalm_alloc(size_t size);
/* download_cuda (model.h:34): D2H copy into a caller buffer (the reference
 * allocated pinned memory and passed std::string through extern "C"). */
int yalm_download(void *host, const void *device, size_t size);
/* register_cuda_host / unregister_cuda_host (model.h:35, 37). */
int yalm_register_host(void *host, size_t size);
int yalm_unregister_host(void *host);
/* free_cuda (model.h:36). */
int yalm_free(void *device);
/* init_cuda_stream (model.h:39), with an opaque handle. */
int yalm_stream_create(yalm_stream *out);
int yalm_stream_destroy(yalm_stream s);
int yalm_stream_sync(yalm_stream s);
/* Fill n device elements of dtype with the deterministic synthetic
 * initialiser (uniform in [offset-scale, offset+scale); f32 adds offset).
 * Used to build random-weight models of real shapes in HBM without a PCIe
 * upload (bench.py). Same integer hash as the CPU oracle. */
int yalm_synth(void *device, size_t n, int dtype, uint64_t seed, float scale, float offset, yalm_stream s);

/* ---------------- decoder: replaces Model::_forward_cuda / Block::_block_cuda ---------------- */
/* Creates the device state for one sequence (InferenceState::cuda,
 * model.cpp:323-345) on stream s (NULL = a private stream). Weight pointers
 * must stay valid for the decoder's lifetime. */
int yalm_decoder_create(const yalm_config *config, const yalm_model_weights *weights, yalm_stream s,
                        yalm_decoder *out);
int yalm_decoder_destroy(yalm_decoder d);
/* Model::forward (model.cpp:396-407 -> infer.cu:1021-1039): one token through
 * every block at position pos (sliding-window/sink indices as infer.cu:1081-
 * 1083). mode YALM_OUTPUT_LOGITS also computes the final norm + logits and,
 * if logits_host != NULL, copies vocab_size floats there before returning
 * (synchronous, like the reference's OUTPUT mode). YALM_HYDRATE_KV_CACHE is
 * asynchronous. Graph-replayed after the first call per mode. */
int yalm_forward(yalm_decoder d, int token, int pos, int mode, float *logits_host);
/* Device-resident greedy decode (-t 0; sampler.cpp:27-38 first-max argmax on
 * the device): feeds `token` at `pos`, then n_steps-1 more tokens each chosen
 * by argmax of the previous step; writes the n_steps argmax tokens to
 * out_tokens (host). No host round trip per token: each token's kernels are
 * launched back to back (eagerly: measured 0.3-0.5% faster than replaying the
 * per-token graph, whose kernel count yalm_graph_kernels still reports). */
int yalm_generate_greedy(yalm_decoder d, int token, int pos, int n_steps, int *out_tokens);
/* Launch-only variant for benchmarking: enqueue n_steps greedy steps
 * continuing from the decoder's device-resident token/pos; no sync. */
int yalm_enqueue_greedy(yalm_decoder d, int n_steps);
/* Read back the device-resident next token / position after enqueue+sync. */
int yalm_device_step(yalm_decoder d, int *token, int *pos);
/* The greedy tokens produced on the device since the last yalm_generate_greedy
 * (that call's tokens, then every yalm_enqueue_greedy step, up to 65536):
 * copies min(*n_total, cap) of them to out (host) after a sync; *n_total = how many
 * were produced. Lets tensor-parallel ranks compare whole sequences (bench.py). */
int yalm_device_tokens(yalm_decoder d, int *out, int cap, int *n_total);
/* Block::block (model.cpp:213-265) for one layer, eagerly, on the decoder's
 * current activation x (the test hook for per-layer parity). */
int yalm_block(yalm_decoder d, int layer, int pos, int kv_sink, int kv_pos, int kv_len);
/* Host access to the decoder's activation x (dim floats) and logits. After a
 * YALM_HYDRATE_KV_CACHE forward of an IPC tensor-parallel decoder x is undefined
 * (that forward's last W2 partial is never exchanged: nothing reads it); after
 * yalm_block and OUTPUT forwards it is the full hidden state on every rank. */
int yalm_get_x(yalm_decoder d, float *host);
int yalm_set_x(yalm_decoder d, const float *host);
int yalm_get_logits(yalm_decoder d, float *host);
/* Average device time (ms) of one kernel of the forward, launched eagerly on
 * the decoder's stream `iters` times between HIP events (layers rotated so the
 * weights come from HBM). kernel_id: 0 = QKV GEMV, 1 = attention, 2 = Wo GEMV,
 * 3 = W1/W3 GEMV+GLU, 4 = W2 GEMV, 5 = logits GEMV, 6 = one tensor-parallel
 * exchange of x (RCCL all-reduce or IPC exchange; collective: every rank calls it
 * with the same iters), 8 = the fused attention + Wo
 * launch (yalm_decoder_attn_wo; each timed launch gets a fresh step epoch, so its
 * Wo waves wait for the heads as in a real forward; the epoch-bump launches are
 * timed separately and subtracted). Used by bench.py for the roofline of the
 * dominant kernel. */
int yalm_time_kernel(yalm_decoder d, int kernel_id, int iters, float *avg_ms);
/* The same-process streaming envelope: average ms of one pure read-only pass over
 * `bytes` of HBM (16-byte non-temporal loads, the best of a few wave geometries,
 * `iters` back-to-back launches alternating two buffers so the 256 MiB Infinity
 * Cache cannot serve them). bench.py reports a kernel's time against it so the
 * roofline fraction is also stated relative to what THIS box streams. */
int yalm_stream_envelope(size_t bytes, int iters, float *avg_ms);
/* Override the GEMV launch geometry of one weight-streaming kernel kind
 * (0 = QKV, 1 = Wo, 2 = W1/W3, 3 = W2, 4 = logits): workgroup size
 * 256|512|1024, unroll (16-byte loads in flight per lane) 2|4|8, and `gpw` =
 * workgroups per CU of the row-block kernel; 0 = automatic.
 * Drops captured graphs (re-captured on next use). Tuning/ablation hook. */
int yalm_set_gemv_config(yalm_decoder d, int kind, int threads, int unroll, int gpw);
/* Kernel launches per forward of graph `mode` (0 = HYDRATE, 1 = OUTPUT_LOGITS, 2 = the
 * device greedy step): *kernels = kernel nodes of the captured per-token hipGraph (RCCL
 * collectives count as the kernels they capture), *nodes (may be NULL) = all nodes. Test
 * and measurement hook (tensor parallelism adds no exchange launches over IPC). */
int yalm_graph_kernels(yalm_decoder d, int mode, int *kernels, int *nodes);
/* Name of kernel_id's device function (to match rocprofv3 summaries). */
const char *yalm_kernel_name(yalm_decoder d, int kernel_id);
/* 1 if this decoder's launch path runs attention and the Wo projection (+ the
 * residual add) as ONE launch (attn_wo.h: the Wo weight stream overlaps the
 * attention; replaces attn + fused_matmul_add_residuals, infer.cu:338-524, 270):
 * head_dim 128, fp16 / fp8 weights with 1, 2, 4 or 8 KB (per-rank) Wo rows, and
 * not YALM_LAUNCH_SEPARATE_ATTN_WO. 0 = two separate launches. The split-KV
 * attention output is handed to the Wo workgroups as {value, epoch} granules. */
int yalm_decoder_attn_wo(yalm_decoder d);
/* Launch-mode switches of one decoder (default 0; drops captured graphs):
 * YALM_LAUNCH_EAGER every forward launches its kernels directly instead of replaying
 * the per-token graph (profilers that mis-handle graph replay); YALM_LAUNCH_SYNC a
 * stream sync after every replay (debugging); YALM_LAUNCH_SEPARATE_ATTN_WO separate
 * attention and Wo launches where the fused one would run (A/B and tests). The
 * production library reads no environment variable. */
#define YALM_LAUNCH_EAGER 1
#define YALM_LAUNCH_SYNC 2
#define YALM_LAUNCH_SEPARATE_ATTN_WO 4
int yalm_decoder_set_launch(yalm_decoder d, int flags);
/* The fused launch's plan for a (per-rank) config when `slots` workgroups of 256
 * threads are co-resident (occupancy x CUs): returns 1 and the key splits per kv head
 * and the grid size, or 0 = separate attention and Wo launches (unsupported shape, or
 * fewer than 2 key splits fit beside the mergers and Wo workgroups while contexts can
 * exceed head mode). Pure host arithmetic: no device is touched. */
int yalm_attn_wo_plan(const yalm_config *config, int slots, int *splits, int *grid);
/* Timeline of the most recent fused attention + Wo launch (decoder created with
 * YALM_ATTN_WO_TRACE=1): 16 stamps per workgroup at [w * 16 + k]: k < 8
 * s_memrealtime (100 MHz), k + 8 the shader clock (s_memtime) at the same point (k = 0: instead the
 * workgroup's place, HW_ID | XCC_ID << 32); k = 0 start, 1 hand-off signalled (attention; 0 if this workgroup did not
 * finish a kv head) or Wo slice landed (Wo; the trace waits for it), 2 poll passed (Wo) or
 * first K/V/q loads landed (attention; the trace waits for them), 3 end; attention units:
 * 4 scores of the last chunk, 5 its softmax, 6 P.V sums combined, 7 head outputs / partials
 * issued; merger workgroups (2 and 4 read 0): 5 gather issued, 7 every partial seen. A
 * phase a workgroup never reached reads 0. Workgroups [0, *attention_workgroups) are
 * attention units and mergers, the rest Wo. */
int yalm_attn_wo_trace(yalm_decoder d, unsigned long long *host, size_t count, int *workgroups,
                       int *attention_workgroups);

/* ---------------- tensor parallelism (BASELINE config 5) ----------------
 * Megatron row/column split of one model over tp_size GPUs, one process per
 * GPU: rank r holds Wq/Wk/Wv rows of heads [r*H/N, (r+1)*H/N) (kv heads
 * likewise), Wo columns of those heads, W1/W3 rows and W2 columns
 * [r*hidden/N, (r+1)*hidden/N), Wcls rows [r*vocab/N, ..); norms and the
 * embedding are replicated. Each layer then needs two all-reduces of x
 * (after Wo and after W2), captured in the per-token graph as RCCL
 * ncclAllReduce over xGMI; the greedy argmax gathers one (value, index) pair
 * per rank. Replaces the single-device forward of model.cpp:396-407 /
 * infer.cu:1021-1128 for multi-GPU; the reference has no multi-GPU path. */
/* 128-byte RCCL unique id, created by rank 0 and shared with the other ranks
 * out of band (bench.py: torch.distributed broadcast). */
int yalm_tp_unique_id(void *id_out);
/* config: the FULL model; weights: this rank's shards as above (blocks as in
 * yalm_decoder_create, KV caches for the local kv heads or null). Collective:
 * every rank calls it concurrently (ncclCommInitRank). All yalm_forward /
 * yalm_generate_greedy calls must then be made by every rank in lockstep;
 * logits (full vocabulary) and greedy tokens are identical on all ranks. */
int yalm_decoder_create_tp(const yalm_config *config, const yalm_model_weights *weights, int tp_rank, int tp_size,
                           const void *unique_id, yalm_stream s, yalm_decoder *out);
/* The same split with an IPC one-shot exchange instead of RCCL (no NCCL
 * communicator; also runs several ranks on ONE GPU, which RCCL refuses): each
 * rank allocates its exchange buffer (yalm_tp_ipc_alloc, config = full model,
 * s = the stream its decoder will run on) and shares the YALM_TP_HANDLE_BYTES
 * rank record out of band (the buffer's hipIpcMemHandle, the GPU's UUID and the
 * stream's CU mask); every rank then passes all tp_size records (rank order)
 * and the same stream s. Ranks on one GPU whose CU masks overlap get a one-wave
 * gate launch before each exchange consumer (they could otherwise hold the CUs a
 * peer's producer needs); one GPU per rank, or disjoint CU masks
 * (yalm_stream_create_cu_part), run the production sequence without it. The
 * decoder takes ownership of own_buf (1..8 ranks). Per exchange no launch of its own:
 * the producer (the fused attention + Wo launch, the W2 GEMV, the logits GEMV,
 * the argmax) pushes each value of this rank's partial into this rank's slot of
 * EVERY rank's buffer as an 8-byte {value, tag} granule (one system-scope store:
 * the data is its own ready flag); the consumer (the next normalising GEMV)
 * waits for every rank's granules while its weight stream starts and sums them
 * in rank order, so x is identical on every rank. Past 4 ranks a collect launch
 * sums x once before the consumer. The exchange sequence numbers live in the
 * decoder's step state, so every rank must make the same calls in lockstep. */
#define YALM_TP_HANDLE_BYTES 128
#define YALM_CU_MASK_WORDS 8 /* 256 CUs */
int yalm_tp_ipc_alloc(const yalm_config *config, int tp_size, yalm_stream s, void **buf, void *handle_out);
/* A stream restricted to CU block `part` of `n_parts` (CUs [part * ncu / n_parts,
 * (part + 1) * ncu / n_parts), spread by the driver over all XCDs): n_parts rank
 * processes on ONE GPU then run on disjoint CUs like n_parts small GPUs (the
 * one-GPU rehearsal of tensor parallelism; tests/test_gpu_mistral_dims.py, bench.py
 * --rehearse). Destroy with yalm_stream_destroy. */
int yalm_stream_create_cu_part(int part, int n_parts, yalm_stream *out);
int yalm_decoder_create_tp_ipc(const yalm_config *config, const yalm_model_weights *weights, int tp_rank, int tp_size,
                               void *own_buf, const void *handles, yalm_stream s, yalm_decoder *out);
/* Device-to-device 2D copy (hipMemcpy2D): shard slicing of weights resident in HBM. */
int yalm_copy_2d(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t width, size_t height);

/* ---------------- batched prefill (MFMA): the perplexity / prompt path ----------------
 * Replaces the reference's position-by-position forward loop over a prompt
 * (main.cpp:128-200 `-m perplexity`, main.cpp:95-101 prompt hydration,
 * Model::forward per position, model.cpp:396-407) with one pass per layer
 * over all n positions: rmsnorm + QKV GEMM + RoPE + fp16 KV-cache write, causal
 * GQA attention, Wo / W1|W3 / W2 GEMMs on the f16 MFMA units.
 * Fills the KV cache rows pos0 .. pos0 + n - 1 exactly where the decoder
 * expects them, so yalm_forward / yalm_generate_greedy can continue at
 * pos0 + n. logprobs (host, n floats, may be NULL): logprobs[i] =
 * log softmax(logits at position pos0 + i)[tokens[i + 1]] for i < n - 1 (the
 * quantity main.cpp:155 sums), logprobs[n - 1] = 0. Requires f16 weights,
 * dims multiple of 128, head_dim 64 | 128 and pos0 + n <= max_seq_len
 * (the sliding window past max_seq_len stays on the decode path).
 * Synchronous. Activations are rounded to f16 for the MFMA inputs: results
 * match the decode path within the tolerance stated in tests/test_gpu_prefill.py.
 * Range guard: where the reference's f32 activations would not fit an f16 operand,
 * a layer's GLU output (W2's A operand; trained checkpoints' "massive activations")
 * is stored with an exact power-of-two scale that W2's epilogue undoes, and the pass
 * runs again; any other operand out of range (the normalised x, Q) returns
 * YALM_ERR_UNSUPPORTED (the decode path keeps them in f32). */
int yalm_prefill(yalm_decoder d, const int *tokens, int n, int pos0, float *logprobs);
/* The last yalm_prefill's passes (1 = no operand out of range) and the number of
 * layers whose GLU output ran scaled. */
int yalm_prefill_info(yalm_decoder d, int *passes, int *scaled_layers);
/* Precision form of decoder d's prefill. YALM_PREFILL_FAST (default): f16 activation
 * operands (the K / V columns' over a split [hi | lo] operand). YALM_PREFILL_SPLIT: every
 * activation operand -- the normalised x, Q, the attention probabilities P, the attention
 * output, the GLU output -- as f16 [hi | lo] pairs (~22 significant bits, the f32 the
 * reference keeps, to ~2^-22), at twice the matrix work; the perplexity bar of SURVEY §7
 * (|d log ppl| <= 1e-3) then holds on peaked models too. The CLI's
 * -m perplexity uses SPLIT, prompt hydration FAST. */
#define YALM_PREFILL_FAST 0
#define YALM_PREFILL_SPLIT 1
int yalm_set_prefill_precision(yalm_decoder d, int mode);
/* Average device time (ms) of one n-position prefill with log-probs (synthetic
 * token ids), over `iters` back-to-back runs (bench_prefill.py). */
int yalm_prefill_time(yalm_decoder d, int n, int iters, float *avg_ms);
/* Test / ablation hook: the prefill GEMM forms of decoder d (d = NULL: of the
 * yalm_gemm_f16 test hook). spec = comma-separated key:value pairs, NULL or "" = the
 * defaults: qkv|wo|glu|w2|cls|test:<128|192|256|320> force that GEMM's tile width;
 * 8p:0 the 2-phase kernel; persist:0 one workgroup per tile; skinny:0 the large tiles
 * for T <= 64 too; qkv1:0 the q and k|v GEMMs as two launches; skl:0 the skinny GEMMs'
 * weights as register loads; wnorm:0 the row norms as one workgroup per row (default:
 * one wave per row). Every GEMM form is exact against the others (tests). An
 * unknown key is YALM_ERR_ARG. */
int yalm_set_prefill_forms(yalm_decoder d, const char *spec);

/* ---------------- layer-list models: mixers and feed-forwards chosen per layer ----------------
 * A second decoder kind beside yalm_decoder, for designs whose layers differ from one
 * another: every layer names a token mixer (latent attention over a cached low-rank
 * key/value latent, a real-gated linear recurrence, a gated delta rule, softmax attention
 * over cached keys and values with a window or chunk mask, a selective state-space layer; or
 * two of them side by side on the same input) and a feed-forward (none, dense
 * GLU, routed experts with an optional shared expert, a plain two-matrix one), each with
 * its own sizes and constants. Serial blocks (block_kind = YALM_BLOCK_SERIAL): around every
 * sublayer x += norm_b(f(norm(x))) (pre_norm = 1) or x += norm_b(f(x)) (pre_norm = 0).
 * Parallel blocks (YALM_BLOCK_PARALLEL): h = norm1(x), x += ls1 * mixer(h) + ls2 * ff(h), one
 * norm read by both sublayers, each result scaled elementwise by its own vector (NULL: 1); a
 * layer of such a block that has norm2 feeds its feed-forward norm2(x) of the same x. The norms
 * are rms norms or mean-subtracting layer norms (norm_kind), both with a weight and no bias.
 * The layer array is the order the layers RUN in: a block of layers that is walked several
 * times with the same weights is passed unrolled, its entries naming the same tensors, and
 * every entry has its own caches and states; pre_add is a vector added to the stream before
 * an entry's opening norm (the per-pass vector of such a loop).
 * One yalm_seq holds ONE sequence: its position, the latent caches and the recurrent
 * and convolution states, all in HBM; yalm_seq_step appends tokens (a whole prompt, a
 * portion of one, or a single decoded token) from where the last call stopped, so the
 * logits do not depend on how a prompt was cut. Residual stream, norms, attention
 * scores, routers and everything inside a recurrence are f32; weight_dtype selects the
 * matrices: YALM_BF16 (bf16 MFMA products with f32 accumulation for portions, bf16
 * weight-streaming GEMVs for single tokens) or YALM_F32 (true f32 products).
 * Matrices are row-major [out][in]. */
enum { YALM_MIX_LATENT = 0, YALM_MIX_RGLRU = 1, YALM_MIX_DELTA = 2, YALM_MIX_ATTN = 3, YALM_MIX_SSM = 4 };
enum { YALM_FF_NONE = 0, YALM_FF_DENSE = 1, YALM_FF_MOE = 2, YALM_FF_PLAIN = 3 };
enum { YALM_NORM_RMS = 0, YALM_NORM_LAYER = 1 };
enum { YALM_BLOCK_SERIAL = 0, YALM_BLOCK_PARALLEL = 1 };
/* gated feed-forwards: y = w_down (act(w_gate x) (.) w_up x) */
enum { YALM_ACT_DEFAULT = 0, /* dense: gelu; experts and shared expert: clamp */
	   YALM_ACT_GELU = 1,  /* gelu_tanh(g) u */
	   YALM_ACT_CLAMP = 2, /* g' sigmoid(1.702 g') (u' + 1), g' = min(g, limit), u' = clamp(u, -limit, limit) */
	   YALM_ACT_SILU = 3,  /* g sigmoid(g) u */
	   YALM_ACT_RELU2 = 4  /* plain feed-forward only: w_down max(w_up x, 0)^2 */ };
/* routed experts: how the `top` experts and their weights come from the router logits */
enum { YALM_ROUTER_SOFTMAX_TOP = 0, /* softmax over all experts, best groups, top scores, weight = score * router_scale */
	   YALM_ROUTER_TOP_SOFTMAX = 1, /* the top logits (+ router_bias) win, weights = softmax over the chosen logits only */
	   YALM_ROUTER_SIGMOID_GROUPS = 2 /* scores sigmoid(logit); the choice ranks score + router_bias: a group by the sum of
	                                    its two largest, the `top` largest within the groups_keep best groups win (ties: the
	                                    lower index); weight = score * router_scale (without the bias, not renormalised) */ };
/* attn: which earlier positions j <= i a position i sees */
enum { YALM_MASK_CAUSAL = 0, /* all of them */
	   YALM_MASK_WINDOW = 1, /* i - j < mask_size */
	   YALM_MASK_CHUNK = 2 /* floor(i / mask_size) == floor(j / mask_size), chunks counted from position 0 */ };
/* attn: norm of queries and keys */
enum { YALM_QK_NONE = 0,
	   YALM_QK_HEAD_UNIT = 1, /* after the rotation, every head divided by its rms over dim, no weight */
	   YALM_QK_WHOLE = 2, /* before the rotation, rms norm over the whole projection with weights q_norm / kv_norm */
	   YALM_QK_HEAD_W = 3 /* every head rms-normed over dim, times q_norm / kv_norm [dim] shared by all heads (no rotation) */ };
/* delta: activation of the output gate */
enum { YALM_GATE_SILU = 0, YALM_GATE_SIGMOID = 1 };

typedef struct yalm_seq_layer {
	int mixer;                     /* YALM_MIX_* */
	int heads, kv_heads, dim, vdim; /* latent: heads x dim queries / keys, vdim values; delta: kv_heads x dim
	                                  queries / keys shared by heads / kv_heads value heads of vdim; attn: heads
	                                  query heads of dim, kv_heads key (dim) / value (vdim) heads, query head h
	                                  reads key/value head h / (heads / kv_heads) */
	int kv_rank, q_rank, kv_from;  /* latent: ranks; kv_from >= 0: read that layer's latent cache (no own w_in rows);
	                                  q_rank = 0: the queries are projected from the input directly */
	int rot_dim;                   /* latent with q_rank = 0: every query head is [dim plain | rot_dim rotated] entries and
	                                  w_in's last rot_dim rows give one rotated key part shared by all heads (not normed),
	                                  score = (q_plain . W_uk c + q_rot . k_rot) * attn_scale; rotation as rot_dims / rot_base
	                                  below (rot_dims <= rot_dim); mask_kind / mask_size / sink / sink_w apply */
	float attn_scale;              /* latent, attn: score = q.k * attn_scale */
	int rec_width, blocks;         /* rglru: channels, diagonal gate blocks */
	int conv;                      /* rglru, delta: taps of the causal per-channel convolution */
	int ff_kind, ff;               /* YALM_FF_*; ff: hidden size (dense, plain) or one expert's (moe) */
	int experts, top, groups, groups_keep; /* moe: top experts among the groups_keep best of `groups` groups */
	float router_scale, limit;     /* moe: weight = softmax score * router_scale; clamp of the dense / expert pair */
	int shared_ff;                 /* moe: shared expert's hidden size, 0 = none */
	float shared_limit;
	int ff_act;                    /* YALM_ACT_*: the gated pair of the dense feed-forward, of the experts and the shared expert */
	int router_kind;               /* YALM_ROUTER_* */
	/* attn */
	int mask_kind, mask_size;      /* YALM_MASK_* and its size in positions */
	int qk_norm;                   /* YALM_QK_* */
	int v_norm;                    /* 1: every value head divided by its rms over vdim (no weight) before it is cached */
	int sink;                      /* 1: the softmax has one more key without a value: exp(sink_w[h]) is added to head h's
	                                  denominator, unscaled (sink_w NULL: score 0, i.e. 1 is added) */
	int out_gate;                  /* 1: head h's output times sigmoid(w_g[h] . x), heads gate rows close w_in;
	                                  2: the concatenated heads times sigmoid(W_g x) elementwise, heads vdim gate rows close w_in */
	int rot_dims, rot_orig;        /* rotary positions on the first rot_dims entries of every query / key head, pairs
	                                  (2i, 2i + 1), frequency rot_base^(-2i / rot_dims); rot_orig: see rot_factor */
	float rot_base;
	float rot_factor, rot_fast, rot_slow; /* rot_factor > 0: frequencies rescaled between the pair that turns rot_fast
	                                  times and the pair that turns rot_slow times within rot_orig positions (f / factor
	                                  where slower, f where faster, a linear ramp between), cos and sin times
	                                  0.1 ln(rot_factor) + 1 */
	/* ssm (YALM_MIX_SSM): heads heads of vdim channels, a state of ssm_state x vdim per head, ssm_groups groups of
	   B / C vectors (head h reads group h / (heads / ssm_groups)); w_in rows [gate: heads vdim | x: heads vdim |
	   B: ssm_groups ssm_state | C: the same | step: heads]; x | B | C pass the convolution (conv taps, conv_w,
	   conv_b) and silu; dt = softplus(step + dt_bias[h]); S <- exp(-exp(a_log[h]) dt) S + dt B x^T; y = S^T C +
	   d_skip[h] x; y silu(gate) is rms-normed in norm_groups equal parts, times out_norm [heads vdim]; then w_o */
	int ssm_state, ssm_groups, norm_groups;
	/* delta: decay_rank > 0: one decay per head and key channel, g = exp(-exp(a_log[h]) softplus(w_a2 (a) + dt_bias)),
	   `a` the decay_rank decay rows of w_in (instead of heads), w_a2 [heads dim][decay_rank], dt_bias [heads dim];
	   gate_rank > 0: the output gate's logits are w_g2 (g), `g` the gate_rank gate rows of w_in (instead of heads
	   vdim), w_g2 [heads vdim][gate_rank]; gate_act: YALM_GATE_* */
	int decay_rank, gate_rank, gate_act;
	/* attn: q_temp_every > 0: the query at position p times 1 + q_temp_coef ln(floor((p + 1) / q_temp_every) + 1) */
	float q_temp_coef;
	int q_temp_every;
	/* attn: rel_rows > 0: rel[bucket(i - j)][h] is added to the scaled score of query i and key j; bucket(n) = n below
	   rel_rows / 2, else min(rel_rows - 1, rel_rows / 2 + floor(ln(n / (rel_rows / 2)) / ln(rel_max / (rel_rows / 2))
	   (rel_rows - rel_rows / 2))) (integer halves) */
	int rel_rows;
	float rel_max;
	float join_scale;              /* side != NULL: mixer result = join_scale (rms(a) join_w + rms(b) side_join_w) */
	/* f32 vectors */
	const float *norm1, *norm1b, *norm2, *norm2b; /* [width] each; norm2* unused without a feed-forward; parallel blocks: norm1 only */
	const float *ls1, *ls2;         /* parallel blocks: [width] scales of the mixer's and the feed-forward's result */
	const float *pre_add;           /* [width] added to the stream before this entry's opening norm, or NULL */
	const float *sink_w;            /* [heads], see sink */
	const float *o_bias;            /* attn: [width] bias of the output projection, or NULL */
	const float *router_bias;       /* moe: [experts] added to the router logits, or NULL */
	const float *q_norm, *kv_norm;  /* latent: [q_rank], [kv_rank]; attn with YALM_QK_WHOLE: [heads dim], [kv_heads dim] */
	const float *in_bias;           /* rglru: [2 rec_width] (gate branch, recurrent branch); attn: [rows of w_in] or NULL */
	const float *head_temp;         /* attn: [heads], score of head h times head_temp[h], or NULL */
	const float *talk;              /* attn: [heads][heads], score_h <- sum_g talk[h][g] score_g before mask and softmax, or NULL */
	const float *conv_w, *conv_b;   /* [channels][conv] (last column = current token); rglru bias [rec_width] */
	const float *gate_a, *gate_a_b, *gate_i, *gate_i_b; /* rglru: [blocks][bs][bs], [rec_width] (bs = rec_width / blocks) */
	const float *lam;               /* rglru: [rec_width] */
	const float *a_log, *dt_bias, *out_norm; /* delta: [heads], [heads] ([heads dim] with decay_rank), [vdim]; ssm: [heads], [heads], [heads vdim] */
	const float *router, *shared_sg; /* moe: [experts][width]; [width]: the shared expert times sigmoid(shared_sg . x), NULL: times 1 */
	/* matrices of weight_dtype */
	const void *w_in;  /* latent: [q_rank (+ kv_rank if own latent)][width] (query down, latent down), with q_rank = 0
	                      [heads (dim + rot_dim) + kv_rank + rot_dim][width] (queries, latent down, rotated key part);
	                      rglru: [2 rec_width][width] (gate branch, recurrent branch);
	                      delta: [2 kv_heads dim + heads vdim + (gate_rank | heads vdim) + heads + (decay_rank | heads)][width]
	                      (q, k, v, output gate, beta, decay);
	                      ssm: [2 heads vdim + 2 ssm_groups ssm_state + heads][width] (gate, x, B, C, step);
	                      attn: [heads dim + kv_heads dim + kv_heads vdim (+ heads | heads vdim if out_gate)][width] (q, k, v, gate) */
	const void *w_uq;  /* latent: [heads dim][q_rank] (unused with q_rank = 0) */
	const void *w_ukt; /* latent: [heads][kv_rank][dim], the key up-projection transposed per head */
	const void *w_uv;  /* latent: [heads vdim][kv_rank]; NULL with w_ukv: its last heads vdim rows */
	const void *w_ukv; /* latent with q_rank = 0, or NULL: [heads dim + heads vdim][kv_rank], the key and the value
	                      up-projections stacked; portions then expand the cached latents they see into per-head keys
	                      and values instead of attending over the latents */
	const void *w_o;   /* [width][heads vdim | rec_width] */
	const void *w_gate, *w_up, *w_down; /* dense: [ff][width] x2, [width][ff]; moe: the same per expert, stacked;
	                                       plain: w_down gelu(w_up x), no w_gate */
	const void *ws_gate, *ws_up, *ws_down; /* moe shared expert */
	const float *rel;              /* attn: [rel_rows][heads], see rel_rows */
	const float *d_skip;           /* ssm: [heads] */
	const float *join_w, *side_join_w; /* side != NULL: [width] each */
	const void *w_a2, *w_g2;       /* delta: see decay_rank / gate_rank */
	const struct yalm_seq_layer *side; /* HOST pointer or NULL: a second mixer that reads the same input beside this
	                                  one (its mixer fields and tensors only; no norms, no feed-forward, no side of its
	                                  own), with caches and states of its own; the two results are each rms-normed over
	                                  the width (no mean taken off) and summed, see join_scale */
} yalm_seq_layer;

typedef struct yalm_seq_config {
	int width, vocab, n_layers, max_tokens; /* n_layers: entries of the layer array (layer runs); max_tokens: positions one sequence may hold */
	float embed_scale, norm_eps;
	int weight_dtype; /* YALM_BF16 | YALM_F32 */
	int norm_kind;    /* YALM_NORM_*: every norm of the model (sublayers, final) */
	int pre_norm;     /* 1: a sublayer reads norm1 / norm2 of the stream; 0: it reads the stream itself (norm1 / norm2 unused) */
	int pos_embed;    /* 1: the interleaved sin / cos position vector (frequencies 10000^(-2i / width)) is added to the embedding */
	float logit_scale; /* logits = head . norm(x) * logit_scale */
	int block_kind;   /* YALM_BLOCK_*; parallel blocks need pre_norm = 1 */
} yalm_seq_config;

typedef struct yalm_seq_weights {
	const void *embed;       /* [vocab][width] */
	const float *final_norm; /* [width] */
	const void *head;        /* [vocab][width] */
	const yalm_seq_layer *layers; /* HOST array of n_layers entries, copied by yalm_seq_create */
	const float *embed_norm;  /* [width] or NULL: the embedding row (scaled, with its position vector) is normed
	                             with this weight before it becomes the stream */
} yalm_seq_weights;

typedef struct yalm_seq_s *yalm_seq;

int yalm_seq_create(const yalm_seq_config *config, const yalm_seq_weights *weights, yalm_stream s, yalm_seq *out);
int yalm_seq_destroy(yalm_seq q);
/* The sequence ends: recurrent and convolution states zeroed, position 0 (cache rows are
 * simply overwritten by the next sequence). */
int yalm_seq_reset(yalm_seq q);
int yalm_seq_pos(yalm_seq q, int *pos);
/* Appends n tokens at the current position. want: n_want ascending indices into tokens whose
 * logits are asked for; logits_host receives [n_want][vocab] f32 (both may be NULL / 0).
 * Synchronous when logits are asked for. */
int yalm_seq_step(yalm_seq q, const int *tokens, int n, const int *want, int n_want, float *logits_host);
/* Device-resident greedy decode, as yalm_generate_greedy: feeds `token` at the current
 * position, then n_steps - 1 more tokens, each the first-max argmax of the previous
 * step's logits, with no host round trip per token; out_tokens gets the n_steps choices. */
int yalm_seq_generate_greedy(yalm_seq q, int token, int n_steps, int *out_tokens);
/* Test hook: keep the residual stream after every layer of the next steps (on = 1), and
 * read the last step's [n_layers][n][width] f32 back. */
int yalm_seq_layer_dump(yalm_seq q, int on);
int yalm_seq_get_layers(yalm_seq q, float *host, size_t count);
/* Average device time (ms) of one n-token portion at position pos0 (synthetic token ids,
 * states left as they were found is NOT promised: call yalm_seq_reset after), over iters
 * back-to-back runs; n = 1 times the single-token path. */
int yalm_seq_time_step(yalm_seq q, int n, int pos0, int iters, float *avg_ms);

/* ---------------- test API: replaces infer.cu:890-1019 (model.h:370-384) ---------------- */
/* Host pointers in and out; synchronous. dtype selects the weight type
 * (matmul_cuda<float|half|uint8_t>). */
int yalm_matmul(float *xout, const float *x, const void *w, int n, int d, int dtype);
/* mha_cuda: xout (n_heads, head_dim), att (n_heads, max_seq_len) softmax
 * probabilities for t < kv_len. */
int yalm_mha(float *xout, float *att, const uint16_t *kb, const uint16_t *vb, const float *q, int head_dim, int kv_len,
             int max_seq_len, int n_heads, int n_kv_heads);
/* ffn_cuda: xout = W2 (act(W1 x) * W3 x). */
int yalm_ffn(float *xout, const float *x, const void *w1, const void *w2, const void *w3, int hidden_dim, int dim,
             int act, int dtype);

/* Device greedy sampling (sampler.cpp:27-38 sample_argmax: strict '>' scan, the
 * FIRST maximum wins, 0 when nothing exceeds -FLT_MAX): *out = argmax of n host
 * logits through argmax_kernel, the kernel of the -t 0 decode loop. n_shards > 1
 * runs the tensor-parallel form instead: one per-shard first max as a (value,
 * global index) pair over each n / n_shards slice, then argmax_pick_kernel. */
int yalm_argmax(const float *logits, int n, int n_shards, int *out);

/* Prefill building blocks (host pointers, synchronous):
 * c[M][N] f32 = a[M][K] f16 · w[N][K]^T f16 (the MFMA GEMM; N % 128 == 0, K % 64 == 0). */
int yalm_gemm_f16(float *c, const uint16_t *a, const uint16_t *w, int M, int N, int K);
/* Causal GQA attention of T query rows at positions pos0 .. pos0 + T - 1:
 * q [T][n_heads * head_dim] f16, kc / vc [pos0 + T][n_kv_heads * head_dim] f16,
 * o [T][n_heads * head_dim] f16 (infer.cpp:216-248 per row and head). */
int yalm_attn_prefill(uint16_t *o, const uint16_t *q, const uint16_t *kc, const uint16_t *vc, int T, int pos0,
                      int n_heads, int n_kv_heads, int head_dim);

#ifdef __cplusplus
}
#endif
#endif
