/*
 * libshainet_hip_kernels.so: C ABI of the MI355X (gfx950) attention hot path
 * of SHAInet's LlamaBlock: Q/K/V bias, Qwen3 per-head QK-RMSNorm, half-split
 * RoPE, KV-cache append and causal grouped-query attention (decode and prefill),
 * all fp32, all on the device.
 *
 * Plain pointers and ints only; every function returns an int status
 * (0 = ok) unless it mirrors a reference symbol that returns void.  A failing
 * call leaves a message for shainet_hip_last_error().
 *
 * Threading: one caller at a time per context (the reference serialises its
 * callers the same way, examples/openai_server.cr:57-62).  Work is issued on the
 * context's own HIP stream; calls that take host pointers return with the result
 * in place, calls that take device pointers are asynchronous until
 * shainet_attn_sync().
 */
#ifndef SHAINET_HIP_ATTN_H
#define SHAINET_HIP_ATTN_H

#ifdef __cplusplus
extern "C" {
#endif

#define SHAINET_HIP_OK 0
#define SHAINET_HIP_ERR_ARGUMENT 1 /* the Crystal layer raises ArgumentError */
#define SHAINET_HIP_ERR_RUNTIME 2  /* a HIP runtime call or a launch failed */
#define SHAINET_HIP_ERR_ALLOC 3    /* device allocation failed: Crystal runs GC.collect and retries (cuda.cr:124-140) */
#define SHAINET_HIP_ERR_CAPACITY 4 /* the cache cannot hold the appended rows */

#define SHAINET_HIP_MEM_HOST 0   /* q,k,v,out are host pointers; the call is synchronous */
#define SHAINET_HIP_MEM_DEVICE 1 /* q,k,v,out are device pointers; the call is asynchronous */

#define SHAINET_HIP_MAX_BATCH 64 /* sequences per shainet_attn_forward call */

/* Message of the last failing call on this thread.  Replaces the reference's
 * printf of cudaGetLastError (src/shainet/native/cuda_kernels.cu:722-725, 821-824). */
const char *shainet_hip_last_error(void);

/* 1 when a gfx950 device is visible and usable, else 0.  The counterpart of
 * CUDA.fully_available? (src/shainet/cuda.cr:63-83, 111-122, 778-780). */
int shainet_hip_available(void);

/* ---- entry points with the reference's own names and signatures ----------- */

/* Scatter the staged new rows into a [num_kv_heads, capacity, head_dim] cache
 * at start_pos.  staging = K chunks (kv-head major, each new_tokens*head_dim)
 * then V chunks, K already rotated.  Same symbol, arguments and layout as
 * src/shainet/native/cuda_kernels.cu:713-726 (bound at src/shainet/cuda.cr:838-861).
 * Runs on the default stream, like the reference. */
void kv_cache_append_f32(const float *staging, float *kc, float *vc, int new_tokens, int start_pos,
                         int num_kv_heads, int head_dim, int capacity);

/* Causal GQA attention of new_tokens rotated query rows over the device cache.
 * Same symbol, arguments and layouts as src/shainet/native/cuda_kernels.cu:808-825
 * (bound at src/shainet/cuda.cr:866-891).  `ws` is accepted and ignored: scores
 * never leave the chip.  Runs on the default stream, like the reference. */
void attention_kv_f32(const float *q, const float *kc, const float *vc, float *out, float *ws,
                      int new_tokens, int start_pos, int num_heads, int heads_per_kv, int head_dim,
                      int capacity, float scale);

/* ---- fused, batched entry points ------------------------------------------ */

typedef struct shainet_attn_ctx shainet_attn_ctx;
typedef struct shainet_kv_cache shainet_kv_cache;

/* The attention parameters of one LlamaBlock (src/shainet/transformer/llama_block.cr:10-28,
 * 73-108).  rope_freqs: NULL or head_dim/2 inverse frequencies that override
 * theta^(-2i/head_dim) (llama_block.cr:669-675).  q_norm/k_norm: NULL or a
 * weight vector with its length; a length other than head_dim is an argument
 * error, as in llama_block.cr:618.  qk_norm_eps is the block's eps (llama_block.cr:92).
 * max_positions sizes the cos/sin table (it grows on demand). */
int shainet_attn_create(shainet_attn_ctx **out, int num_heads, int num_kv_heads, int head_dim,
                        double rope_theta, const float *rope_freqs, const float *q_norm, int q_norm_len,
                        const float *k_norm, int k_norm_len, double qk_norm_eps, int max_positions);

/* Optional Q/K/V projection biases, added to the incoming rows before QK-norm
 * (llama_block.cr:257-259, 585-601).  NULL clears one.  A length that is not
 * num_heads*head_dim (q) or num_kv_heads*head_dim (k, v) is an argument error. */
int shainet_attn_set_bias(shainet_attn_ctx *ctx, const float *b_q, int b_q_len, const float *b_k,
                          int b_k_len, const float *b_v, int b_v_len);

int shainet_attn_destroy(shainet_attn_ctx *ctx);

/* Wait for everything issued on the context's stream. */
int shainet_attn_sync(shainet_attn_ctx *ctx);

/* The context's hipStream_t, for callers that enqueue their own work around it. */
void *shainet_attn_stream(shainet_attn_ctx *ctx);

/* Issue the context's work on a caller-owned hipStream_t instead (NULL = the
 * default stream, which is what the reference uses throughout).  The context's
 * own stream is kept and restored by passing the value shainet_attn_stream()
 * returned before the first call of this function. */
int shainet_attn_set_stream(shainet_attn_ctx *ctx, void *stream);

/* Copy of the inverse frequencies in use (head_dim/2 floats, host). */
int shainet_attn_inv_freq(shainet_attn_ctx *ctx, float *out);

/* A device-resident fp32 KV cache for `batch` independent sequences, each
 * [num_kv_heads, capacity, head_dim] for K and for V: the reference's device
 * layout (llama_block.cr:50-56, 497-520) with a leading sequence index.  The
 * device copy is the cache of record; there is no host mirror. */
int shainet_kv_cache_create(shainet_kv_cache **out, shainet_attn_ctx *ctx, int batch, int capacity);
int shainet_kv_cache_destroy(shainet_kv_cache *cache);

/* LlamaBlock#clear_cache! (llama_block.cr:116-122): lengths go to 0, memory is
 * kept, stale rows are overwritten before they can become visible.  seq < 0
 * clears every sequence. */
int shainet_kv_cache_clear(shainet_kv_cache *cache, int seq);

/* Drop the rows at positions >= len of one sequence (len <= its current length):
 * regenerate from an earlier point without refilling.  clear is truncate to 0. */
int shainet_kv_cache_truncate(shainet_kv_cache *cache, int seq, int len);

/* Number of cached positions of one sequence (@cache_len, llama_block.cr:48), or -1. */
int shainet_kv_cache_len(const shainet_kv_cache *cache, int seq);
int shainet_kv_cache_capacity(const shainet_kv_cache *cache);

/* Grow every sequence's capacity to at least `capacity`, keeping contents
 * (the job of ensure_gpu_cache!, llama_block.cr:497-520, without the host mirror). */
int shainet_kv_cache_reserve(shainet_kv_cache *cache, int capacity);

/* Device base pointers of the K and V arrays: [batch][num_kv_heads][capacity][head_dim]. */
float *shainet_kv_cache_k(shainet_kv_cache *cache);
float *shainet_kv_cache_v(shainet_kv_cache *cache);

/* Replace one sequence's contents with n rows per kv head, K already rotated:
 * k_rows, v_rows are [num_kv_heads][n][head_dim] (host when mem == HOST).  The
 * reference has no cache setter (its cache is private state, llama_block.cr:46-48);
 * benchmarks that start from a pre-filled cache and tests need one. */
int shainet_kv_cache_fill(shainet_kv_cache *cache, int seq, const float *k_rows, const float *v_rows, int n,
                          int mem);

/* Copy rows [pos0, pos0+n) of one kv head of one sequence to host buffers
 * ([n][head_dim] each; either may be NULL).  For tests of the cache contract. */
int shainet_kv_cache_read(shainet_kv_cache *cache, int seq, int kv_head, int pos0, int n, float *k_out,
                          float *v_out);

/* attention_cached_cpu from the projections' outputs to the head loop's output
 * (llama_block.cr:256-296), for n_seqs sequences at once, entirely on the device:
 * bias, QK-norm, RoPE with positions cache_len .. cache_len+new_tokens-1, append
 * of the rotated K rows and the V rows, causal GQA attention over the cache.
 *   seq_ids[n_seqs]     cache slots taking part, distinct (NULL = 0..n_seqs-1)
 *   new_tokens[n_seqs]  rows appended per sequence (>= 1)
 *   q   [sum new_tokens, num_heads*head_dim]      rows of sequence seq_ids[0] first
 *   k,v [sum new_tokens, num_kv_heads*head_dim]
 *   out [sum new_tokens, num_heads*head_dim]
 * Each sequence's length grows by its new_tokens.  SHAINET_HIP_ERR_CAPACITY (and
 * nothing appended) if a sequence would outgrow the capacity. */
int shainet_attn_forward(shainet_attn_ctx *ctx, shainet_kv_cache *cache, const int *seq_ids,
                         const int *new_tokens, int n_seqs, const float *q, const float *k, const float *v,
                         float *out, int mem);

/* shainet_attn_forward for decode calls, for callers that cannot allocate device memory while they
 * call it (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * this variant allocates nothing.  It has no counterpart in the reference.  Device pointers only,
 * asynchronous on the context's stream, same results as shainet_attn_forward.  What that call
 * grows on demand comes from a fixed array in device memory instead (8.06 MiB per GPU, held until
 * the process ends): 2 MiB for the rotated query rows (sum new_tokens x num_heads x head_dim
 * <= 524288 floats), 6 MiB for the split's partial results and 32 KiB of flag words (with the
 * default 256 workgroups: any batch of up to 64 sequences of head_dim <= 128).  Limits, each
 * refused with SHAINET_HIP_ERR_ARGUMENT or SHAINET_HIP_ERR_CAPACITY and a message, nothing
 * appended: head_dim a multiple of 4 up to 256; at most 32 / (num_heads / num_kv_heads) new rows per sequence
 * (the calls the split-K decode kernel takes); every position below the max_positions the
 * context was created with; sizes within the array.  All calls on one GPU share the array:
 * two calls of this entry point that overlap in time on one GPU (different contexts on
 * different streams) race; calls on one context, or one after the other, do not.
 * The address of the array on a device is looked up when a context is created on it, not in the
 * call.  Under stream capture the call may be recorded, but the recording is good for one run
 * only: the launch is planned on the host (start positions and spans are kernel arguments, the
 * cache length advances once, when the call is made), so a replay would write the same cache row
 * again.  shainet_attn_decode_step is the entry point whose recording can be replayed. */
int shainet_attn_forward_noalloc(shainet_attn_ctx *ctx, shainet_kv_cache *cache, const int *seq_ids,
                                 const int *new_tokens, int n_seqs, const float *q, const float *k, const float *v,
                                 float *out);

/* Decode steps whose launches never change, for callers that record a step once and replay it (a HIP
 * graph): one new row for each of the first n_seqs sequences of a cache, the same arithmetic as
 * shainet_attn_forward with new_tokens all 1 (LlamaBlock#attention_cached_cpu with one row,
 * llama_block.cr:246-299).  Nothing the three kernels of a step are launched with depends on how
 * many rows the cache holds: the lengths live in device memory, a one-wavefront kernel at the head
 * of each step reads them, lays out the split of the keys for the other two kernels and adds one
 * to each length.  The step allocates nothing and copies nothing; it has no counterpart in the
 * reference, whose cache length is a host integer (llama_block.cr:288-289).
 *
 * shainet_kv_cache_lengths_to_device: allocates what the steps need (first call), extends the
 *   context's cos/sin table to the cache's capacity and copies the host's lengths to the device.
 *   Call it after anything that changes the lengths on the host (shainet_attn_forward, fill,
 *   clear, truncate) or the capacity (reserve), before the next step; not while capturing.
 * shainet_attn_decode_step: q [n_seqs, num_heads*head_dim], k, v [n_seqs, num_kv_heads*head_dim],
 *   out like q; device pointers, asynchronous on the context's stream.  head_dim a multiple of 4 up to 128.
 *   A step that finds a sequence at the cache's capacity appends nothing, writes no output and
 *   leaves the lengths alone, and so do the steps after it; shainet_kv_cache_lengths_from_device
 *   (or shainet_attn_sync) then returns SHAINET_HIP_ERR_CAPACITY.
 * shainet_kv_cache_lengths_from_device: waits for the stream and copies the device's lengths
 *   back, so that shainet_kv_cache_len and the other entry points see the rows the steps appended.
 * Between the two copies the host's lengths are stale: every other entry point that reads or writes
 * them (shainet_attn_forward and its variants, fill, clear, truncate, reserve, a second
 * lengths_to_device) is refused with SHAINET_HIP_ERR_ARGUMENT and shainet_kv_cache_len returns -1;
 * after lengths_from_device a step needs lengths_to_device again.
 * A recorded step holds the addresses of the cache, of the context's cos/sin table, bias and
 * QK-norm weights: record it again after shainet_kv_cache_reserve, shainet_attn_set_bias, or a
 * call on another cache of the same context that reaches beyond the table's positions. */
int shainet_kv_cache_lengths_to_device(shainet_kv_cache *cache);
int shainet_kv_cache_lengths_from_device(shainet_kv_cache *cache);
int shainet_attn_decode_step(shainet_attn_ctx *ctx, shainet_kv_cache *cache, int n_seqs, const float *q,
                             const float *k, const float *v, float *out);

/* Copy of the rotated query rows of the last shainet_attn_forward call
 * ([sum new_tokens, num_heads*head_dim], host): lets a test check RoPE positions
 * and QK-norm of Q exactly (llama_block.cr:332-344). */
int shainet_attn_last_q_rot(shainet_attn_ctx *ctx, float *out, int rows);

/* What a shainet_attn_forward call with these sequences (cached positions start_pos[s], new rows
 * new_tokens[s]) launches for its attention step, without launching anything; needs no device.
 * plan[0] path: 0 = split-K decode kernel, 1 = MFMA prefill kernel, 2 = generic kernel;
 * plan[1] the head_dim the kernel's tiles are laid out for (64, 128 or 256: the first that holds
 * head_dim; head_dim itself on the generic path); plan[2] key chunks per row block (1 = none, > 1 adds the combine kernel);
 * plan[3] wavefront groups per workgroup (1 = four wavefronts, 2 = eight); plan[4] row blocks a
 * workgroup takes in turn (0 = one workgroup per block and chunk); plan[5] workgroups;
 * plan[6] decode: 16-key tiles per workgroup, prefill: row blocks; plan[7] workgroups per
 * compute unit the launch is held to (0 = no limit).  Lets a test name the kernel instantiation
 * it covers.  No counterpart in the reference, whose kernel has one shape (cuda_kernels.cu:808-825). */
int shainet_attn_describe_plan(int num_heads, int num_kv_heads, int head_dim, int n_seqs, const int *start_pos,
                               const int *new_tokens, int plan[8]);

/* RoPE.apply (src/shainet/transformer/rope.cr:7-33): x and out are [seq_len, head_dim] rows;
 * row r is rotated by (r + start_pos) * theta^(-2i/head_dim), half-split pairs (i, i + head_dim/2),
 * everything in fp64 on the device and rounded to fp32 once, an odd trailing column copied
 * through.  LlamaBlock does not call it (its own RoPE keeps the angle in fp32,
 * llama_block.cr:274-277); it is the stand-alone module function that spec/rope_kv_cache_spec.cr:4-27
 * pins.  mem = HOST: synchronous; DEVICE: asynchronous on the default stream. */
int shainet_rope_apply(const float *x, float *out, int seq_len, int head_dim, int start_pos, double theta, int mem);

/* ---- the attention half of a LlamaBlock, weights included ------------------
 *
 * State and behaviour of src/shainet/transformer/llama_block.cr for
 * attention_cached_cpu (246-299): x [T, d_model] (host) -> Q/K/V projections ->
 * bias, QK-norm, RoPE, append, causal GQA attention -> output projection ->
 * [T, d_model] (host), with everything between the two copies on the device.
 * Weights are row-major [in, out] as the reference keeps them (hf_loader.cr:326-329).
 * Constructor checks are those of llama_block.cr:80-89 (head_dim 0 = d_model /
 * num_heads); eps is the QK-norm eps (92).  Setters may be called at any time
 * before a forward call, as HFLoader does (hf_loader.cr:319-373); a setter after
 * rows were cached starts a new, empty cache.  Size mismatches of biases and
 * norm weights are reported by the next forward call with SHAINET_HIP_ERR_ARGUMENT,
 * where the reference raises ArgumentError (llama_block.cr:587, 618). */
typedef struct shainet_llama_attn shainet_llama_attn;
int shainet_llama_attn_create(shainet_llama_attn **out, int d_model, int num_heads, int num_kv_heads, int head_dim,
                              double eps, double rope_theta);
int shainet_llama_attn_destroy(shainet_llama_attn *layer);
int shainet_llama_attn_set_rope(shainet_llama_attn *layer, double rope_theta, const float *rope_freqs);
int shainet_llama_attn_set_qk_norm(shainet_llama_attn *layer, const float *q_norm, int q_len, const float *k_norm,
                                   int k_len);
int shainet_llama_attn_set_bias(shainet_llama_attn *layer, const float *b_q, int q_len, const float *b_k, int k_len,
                                const float *b_v, int v_len);
/* w_q [d_model, q_dim], w_k and w_v [d_model, kv_dim], w_o [q_dim, d_model], host; copied to the device (to_gpu!). */
int shainet_llama_attn_set_weights(shainet_llama_attn *layer, const float *w_q, const float *w_k, const float *w_v,
                                   const float *w_o);
/* LlamaBlock#clear_cache! (116-122) and @cache_len. */
int shainet_llama_attn_clear_cache(shainet_llama_attn *layer);
int shainet_llama_attn_cache_len(const shainet_llama_attn *layer);
/* attention_cached_cpu (246-299): x and out are host [new_tokens, d_model]; synchronous. */
int shainet_llama_attn_forward_cached(shainet_llama_attn *layer, const float *x, int new_tokens, float *out);
/* attention_full_cpu (209-243), the no-cache path of LlamaBlock#forward: the same arithmetic from
 * position 0 over the seq_len rows of x alone; @cache_len and the cached rows are left as they are. */
int shainet_llama_attn_forward_full(shainet_llama_attn *layer, const float *x, int seq_len, float *out);

/* The projection product by itself: y[rows, n] = x[rows, k] W[k, n] (+ res[rows, n]), fp32, row-major,
 * device pointers, asynchronous on `stream` (NULL = the default stream); the rows of x are
 * x_stride floats apart, y and res are dense, res may be NULL or y.  What LlamaBlock#gpu_matmul
 * dispatches (llama_block.cr:726-768: SimpleMatrix#* on the host, cuBLAS SGEMM on the device,
 * cuda.cr:237-247): up to 16 rows run the split GEMV of the decode step, more rows the MFMA
 * kernel of the prefill.  fp32 accumulation (the host path of the reference accumulates in
 * fp64, simple_matrix.cr:61-74).  The handle-less calls keep one grow-only scratch set per stream
 * (partial products of split shapes and their flag words): calls on different streams may overlap,
 * calls on one stream are ordered by it; one host thread at a time inside the call.  A kernel of
 * an earlier call on the same stream that gave up its bounded wait for partial sums is reported by
 * the next call on that stream (SHAINET_HIP_ERR_RUNTIME), which then does nothing else. */
int shainet_hip_matmul_f32(const float *x, long long x_stride, const float *w, const float *res, float *y, int rows,
                           int k, int n, void *stream);

/* ---- the whole block ---------------------------------------------------------
 *
 * LlamaBlock#forward_cached (llama_block.cr:189-196) with a dense SwiGLU
 * feed-forward: normed = norm1(x); attn = attention_cached(normed); h = x + attn;
 * out = h + ffn(norm2(h)), with RMSNorm as rms_norm.cr:18-37 (fp64 sum, root and
 * scaling), SimpleMatrix#+ as simple_matrix.cr:39-48 and SwiGLUFF#forward as
 * swiglu_ff.cr:76-91 (g / (1 + exp(-g)) * up in fp64), every step on the device.
 * Argument order follows LlamaBlock.new (llama_block.cr:71-76): eps is both the
 * RMSNorm eps and the QK-norm eps (92-94); num_kv_heads 0 = num_heads; head_dim 0
 * = d_model / num_heads.  The mixture-of-experts feed-forward (moe_experts) is not
 * covered.  Attention weights, biases, QK-norm and RoPE are set on the handle
 * shainet_llama_block_attn returns. */
typedef struct shainet_llama_block shainet_llama_block;
int shainet_llama_block_create(shainet_llama_block **out, int d_model, int num_heads, int ff_hidden, double eps,
                               double rope_theta, int num_kv_heads, int head_dim);
int shainet_llama_block_destroy(shainet_llama_block *block);
shainet_llama_attn *shainet_llama_block_attn(shainet_llama_block *block);
/* gamma of @norm1 and @norm2, host [d_model] each; null = ones (rms_norm.cr:10). */
int shainet_llama_block_set_norms(shainet_llama_block *block, const float *norm1_gamma, const float *norm2_gamma);
/* gate_proj and up_proj [d_model, ff_hidden], down_proj [ff_hidden, d_model], host, [in, out] (swiglu_ff.cr:16-18). */
int shainet_llama_block_set_ffn(shainet_llama_block *block, const float *gate_proj, const float *up_proj,
                                const float *down_proj);
int shainet_llama_block_clear_cache(shainet_llama_block *block);
int shainet_llama_block_cache_len(const shainet_llama_block *block);
/* x and out [new_tokens, d_model].  mem = SHAINET_HIP_MEM_HOST: copies in and out, synchronous;
 * SHAINET_HIP_MEM_DEVICE: device pointers, asynchronous on the block's stream. */
int shainet_llama_block_forward_cached(shainet_llama_block *block, const float *x, int new_tokens, float *out,
                                       int mem);
/* LlamaBlock#forward (179-186): the whole sequence without the cache (Network#run with use_kv_cache off). */
int shainet_llama_block_forward(shainet_llama_block *block, const float *x, int seq_len, float *out, int mem);

/* ---- the model around the blocks ----------------------------------------------
 *
 * Network#run(SimpleMatrix) with use_kv_cache for a LLaMA-family network
 * (network_run.cr:185-226): token ids -> embedding rows (embedding_layer.cr:129-153)
 * -> every block's forward_cached -> final RMSNorm (@final_norm, optional) -> last
 * row x lm_head [d_model, vocab] (1390-1404) -> + bias (221-225).  Activations and
 * logits stay on the device.  The sampling entry points work on the logits of the
 * last run: Sampler.greedy (text/sampler.cr:38-53), Sampler#apply_repetition_penalty!
 * (59-81) and the top-k selection of Sampler#sample (88-116); the temperature
 * softmax and the draw over the k survivors (118-150) stay with the caller, who
 * owns the random generator, or run on the device too with shainet_llama_model_sample, which
 * takes the uniform draw as an argument. */
typedef struct shainet_llama_model shainet_llama_model;
int shainet_llama_model_create(shainet_llama_model **out, int vocab, int d_model, int n_layers, int num_heads,
                               int num_kv_heads, int head_dim, int ff_hidden, double eps, double rope_theta);
int shainet_llama_model_destroy(shainet_llama_model *model);
int shainet_llama_model_layers(const shainet_llama_model *model);
shainet_llama_block *shainet_llama_model_block(shainet_llama_model *model, int layer);
/* host [vocab, d_model] */
int shainet_llama_model_set_embedding(shainet_llama_model *model, const float *table);
/* host [d_model]; null = the network has no final norm */
int shainet_llama_model_set_final_norm(shainet_llama_model *model, const float *gamma);
/* host [d_model, vocab] and [vocab] (null = no bias) */
int shainet_llama_model_set_lm_head(shainet_llama_model *model, const float *weights, const float *bias);
int shainet_llama_model_clear_cache(shainet_llama_model *model);
int shainet_llama_model_cache_len(const shainet_llama_model *model);
/* tokens: host ids [n_tokens], appended to every block's cache.  logits: host [vocab], or null to leave
 * them on the device (the call is then asynchronous; the sampling calls and _sync wait). */
int shainet_llama_model_run(shainet_llama_model *model, const int *tokens, int n_tokens, float *logits);
/* The same with the network's use_kv_cache switched off (network_setup.cr:32, network_run.cr:199-204:
 * LlamaBlock#forward instead of forward_cached in every block): the n_tokens rows attend among
 * themselves from position 0, every block's cache and cache length stay as they are.  The logits of
 * the last row are left for the sampling calls like those of shainet_llama_model_run. */
int shainet_llama_model_run_full(shainet_llama_model *model, const int *tokens, int n_tokens, float *logits);
int shainet_llama_model_sync(shainet_llama_model *model);
/* How a run of ONE token walks the blocks (Network#run's loop over the layers, network_run.cr:199-204,
 * each LlamaBlock#forward_cached of llama_block.cr:189-196): one launch per product, or the whole
 * stack as a single launch of one workgroup per compute unit with barriers between the phases of a
 * block and the next product's first weights requested before each barrier.  The single launch
 * needs head_dim a power of two <= 128, 1, 2, 4 or 8 query heads per kv head, d_model and ff_hidden
 * multiples of 4 and the same geometry in every block, and must have the device's compute units to
 * itself while it runs (its workgroups wait for each other; the wait is bounded and a give-up is
 * reported by the next _sync / logits read as SHAINET_HIP_ERR_RUNTIME).  AUTO (the default) is one
 * launch per product, which measured faster on the shapes tried; the variable
 * SHAINET_HIP_PERSISTENT_STEP makes AUTO the single launch where the geometry fits.  Results of
 * the two agree to rounding (different summation orders).  No counterpart in the reference. */
#define SHAINET_HIP_DECODE_AUTO 0
#define SHAINET_HIP_DECODE_PER_PRODUCT 1
#define SHAINET_HIP_DECODE_PERSISTENT 2 /* runs of one token fail when the geometry does not fit */
int shainet_llama_model_set_decode_mode(shainet_llama_model *model, int mode);
/* SHAINET_HIP_DECODE_PER_PRODUCT or SHAINET_HIP_DECODE_PERSISTENT: what a run of one token uses now */
int shainet_llama_model_decode_mode_in_use(shainet_llama_model *model);
/* Tuning aid: with SHAINET_HIP_STEP_TRACE set before the model's first single-launch step, every
 * workgroup of such a step records its 100 MHz clock at the launch's start and at up to 24 points
 * of every block (the first ten: after the x slice of the q|k|v product, then before and after
 * each of the five barriers); this copies the last step's readings, [workgroups][*per_workgroup]
 * with *per_workgroup = 1 + 24 * layers. */
int shainet_llama_model_step_trace(shainet_llama_model *model, long long *out, int capacity, int *workgroups,
                                   int *per_workgroup);
int shainet_llama_model_read_logits(shainet_llama_model *model, float *logits);
/* replace the device logits row by host values [vocab]: lets the sampling calls run on a row that
 * was computed or edited elsewhere (the reference's Sampler takes any SimpleMatrix row) */
int shainet_llama_model_write_logits(shainet_llama_model *model, const float *logits);
/* argmax over the finite logits, lowest index among equals, 0 when none is finite */
int shainet_llama_model_greedy(shainet_llama_model *model, int *token);
/* The generation loop of examples/llama_chat.cr:181-197 with greedy selection, kept on the device:
 * best = Sampler.greedy(logits); stop if best is one of stop_ids; out << best; logits = run([best]);
 * at most max_tokens times, starting from the logits of the last run.  The chosen id goes from
 * the argmax kernel to the next step's embedding lookup through device memory, so steps queue up
 * without a host round trip; the ids are looked at every 16 steps, and when a stop id turns up
 * the caches are cut back to the rows before it (the logits row is then no longer valid: run
 * again before sampling).  out: room for max_tokens ids; *n_out = ids written. */
int shainet_llama_model_generate_greedy(shainet_llama_model *model, int max_tokens, const int *stop_ids, int n_stop,
                                        int *out, int *n_out);
/* v > 0 ? v / penalty : v * penalty for each id in order (a repeated id is penalised again); ids outside
 * [0, vocab) are skipped; penalty 1.0 is a no-op */
int shainet_llama_model_repetition_penalty(shainet_llama_model *model, const int *recent_ids, int n, double penalty);
/* the k largest logits (1 <= k <= 256), NaN excluded, descending, equal values by ascending id;
 * *count = entries written (< k when fewer are eligible) */
int shainet_llama_model_topk(shainet_llama_model *model, int k, int *ids, float *vals, int *count);
/* Sampler#sample (text/sampler.cr:88-150) on the device logits, whole: the top-k selection, the softmax
 * of v / temperature over the survivors in fp64 and the inverse-CDF pick for the uniform draw r in [0, 1)
 * that the caller's random generator made (@rng.rand, sampler.cr:136); *token = 0 when no logit is
 * eligible (all NaN).  top_k in [1, 256], temperature > 0 (sampler.cr:24-25: ArgumentError otherwise). */
int shainet_llama_model_sample(shainet_llama_model *model, int top_k, double temperature, double r, int *token);

/* ---- SafeTensors and the HuggingFace loader --------------------------------------
 *
 * SHAInet::SafeTensors::File / ShardedFile (src/shainet/safetensors.cr) over
 * memory-mapped files, host only.  `path` is a .safetensors file, or a model
 * directory holding model.safetensors or model.safetensors.index.json
 * (HFLoader.open_safetensors, hf_loader.cr:14-26). */
typedef struct shainet_safetensors shainet_safetensors;
int shainet_safetensors_open(const char *path, shainet_safetensors **out);
int shainet_safetensors_close(shainet_safetensors *st);
int shainet_safetensors_count(const shainet_safetensors *st);               /* tensor_names.size */
const char *shainet_safetensors_name(const shainet_safetensors *st, int i); /* tensor_names[i] */
int shainet_safetensors_has(const shainet_safetensors *st, const char *name);  /* has_tensor? : 1 or 0 */
/* dtype as the file spells it ("F32", "BF16", ...), up to 8 shape entries, bytes of data; any of the
 * four outputs may be null */
int shainet_safetensors_info(const shainet_safetensors *st, const char *name, char dtype[8], long long shape[8],
                             int *ndim, long long *nbytes);
/* read_f32 (safetensors.cr:90-124): F32, F16, BF16 and F64 tensors as fp32; n must be the element count */
int shainet_safetensors_read_f32(const shainet_safetensors *st, const char *name, float *out, long long n);

/* config.json of a LLaMA-family model as HFLoader.load_llama_config reads it (hf_loader.cr:199-233);
 * head_dim 0 = not given (d_model / num_heads), num_experts 0 = dense. */
typedef struct {
  char model_type[32];
  int vocab_size, hidden_size, num_attention_heads, num_hidden_layers, intermediate_size, num_key_value_heads;
  int head_dim, tie_word_embeddings, num_experts;
  double rms_norm_eps, rope_theta;
  int rope_llama3; /* rope_scaling of type "llama3" present */
  double rope_factor, rope_low_freq_factor, rope_high_freq_factor;
  int rope_original_max_position_embeddings;
} shainet_hf_llama_config;
int shainet_hf_read_llama_config(const char *model_dir, shainet_hf_llama_config *cfg);
/* HFLoader.compute_rope_freqs (hf_loader.cr:235-265): writes head_dim / 2 inverse frequencies and
 * returns that count, returns 0 when the config has no llama3 scaling (the block then uses
 * theta^(-2i/d)), or minus a status code.  n = room in out. */
int shainet_hf_rope_freqs(const shainet_hf_llama_config *cfg, float *out, int n);
/* HFLoader.load_llama (hf_loader.cr:277-412) onto the device, dense models only ("llama",
 * "mistral", "qwen2", "qwen3"): every tensor goes to the GPU in its stored type and is converted
 * to fp32 and transposed to [in, out] there.  The model is ready for shainet_llama_model_run. */
int shainet_hf_load_llama(const char *model_dir, shainet_llama_model **out);

/* Kernel timing for benchmarks: while enabled, every shainet_attn_forward call
 * times its attention kernel (the split-K decode kernel, the MFMA prefill kernel
 * with its combine kernel when it has one, or the generic kernel; not the prep
 * kernel) with a pair of HIP events on the context's stream.  For the decode and
 * prefill kernels the events take the kernel's own start and end clock readings
 * (hipExtLaunchKernel), so the idle time between two kernels is not counted.  shainet_attn_profile_read waits for the stream,
 * returns the summed kernel time in milliseconds and the number of launches
 * since the last read, and resets both; shainet_attn_profile_samples does the same
 * but hands back the time of each launch (the first `capacity` of them; *launches
 * is the number there were).  No counterpart in the reference. */
int shainet_attn_profile(shainet_attn_ctx *ctx, int enable);
int shainet_attn_profile_read(shainet_attn_ctx *ctx, double *total_ms, int *launches);
int shainet_attn_profile_samples(shainet_attn_ctx *ctx, float *ms_out, int capacity, int *launches);

/* Plain streaming kernels of known size (device pointers, n floats, n % 4 == 0,
 * grid-stride over `workgroups` workgroups of 256 lanes, on `stream`): a copy
 * and a read that writes one float per workgroup into sink[workgroups].  They
 * calibrate the HBM byte counters and the reachable stream bandwidth that the
 * attention kernels are compared with.  No counterpart in the reference. */
int shainet_hip_stream_copy_f32(const float *src, float *dst, long long n, int workgroups, void *stream);
int shainet_hip_stream_read_f32(const float *src, float *sink, long long n, int workgroups, void *stream);

/* A loop of nothing but fp32 MFMAs (v_mfma_f32_32x32x2_f32, four independent accumulators
 * per wavefront): `workgroups` workgroups of 512 lanes run `iters` rounds of 16 MFMAs per
 * wavefront and write one float per lane into sink[workgroups * 512]; *flops (nullable)
 * receives the flops of the launch.  The rate it reaches is what the matrix cores sustain at
 * the clock the device holds under that load, the yardstick next to the published peak for
 * the prefill kernels.  No counterpart in the reference. */
int shainet_hip_mfma_f32_loop(float *sink, int iters, int workgroups, long long *flops, void *stream);

/* What a launch costs on the device with no work in it: `chain` kernels of `workgroups` empty
 * workgroups, one after the other on `stream`, timed from the first kernel's own first clock
 * reading to the last kernel's last one (hipExtLaunchKernel events, as the attention kernels are
 * timed); *us = the median of `reps` such chains, in microseconds.  chain = 1 is the shortest
 * kernel the device runs, chain = 2 adds one kernel boundary: the floor under every step that
 * is a prep kernel followed by an attention kernel.  Waits for the stream.  No counterpart in the
 * reference. */
int shainet_hip_launch_latency(int chain, int reps, int workgroups, float *us, void *stream);

#ifdef __cplusplus
}
#endif
#endif
