/*
 * tlhip.h — C-ABI of libtlhip.so, the MI355X (gfx950) backend that replaces tinyllama.cpp's CUDA/cuBLAS
 * backend (reference: cuda_kernels.h:104-643 + the raw cudaMalloc/cudaMemcpy/cublas* calls inlined in
 * model.cpp, gpu_initialization.cpp, weight_management.cpp, kv_cache.cpp, gpu_memory_optimization.cpp).
 *
 * Conventions
 *   - plain C: pointers and sizes only. `void* stream` is a hipStream_t (NULL = the default stream),
 *     the counterpart of the reference's `cudaStream_t stream = 0` arguments.
 *   - every function returns int: 0 = ok, non-zero = error; tl_last_error() gives the text. The C++ host
 *     layer (tinyllama.cpp_amd/host/tl_session.cpp:14-16, `check`) turns non-zero into std::runtime_error, which is the
 *     reference's convention (gpuErrchk, cuda_kernels.h:66-82). Argument-validation failures return an
 *     error instead of the reference's log-and-return-silently (cuda_kernels.cu:1335-1351).
 *   - `*_dev` pointers are device pointers BORROWED from the caller; `*_host` are host pointers borrowed
 *     for the duration of the call. tl_qweight / tl_model handles own their device memory.
 *   - one host thread per handle, no re-entrancy (the reference's threading model).
 *
 * The big difference from the reference backend: weights stay QUANTIZED on the device. The reference
 * dequantizes every GPU layer to FP32 on the host and calls cublasSgemm with N=1
 * (weight_management.cpp:199-435, cuda_kernels.cu:291-314); here raw GGUF super-blocks are uploaded once,
 * re-laid-out into 16-byte-aligned planes (tl_qweight) and consumed by block-dequant GEMV kernels.
 */
#ifndef TLHIP_H
#define TLHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml tensor type ids (reference ggml_types.h:21-42) */
enum tl_type { TL_F32 = 0, TL_Q8_0 = 8, TL_Q4_K = 12, TL_Q6_K = 14, TL_Q8_K = 15,
               TL_BF16 = 30 /* tl_model_set_tensor only: widened to F32 at upload (exact) */ };

typedef struct tl_qweight tl_qweight; /* one quantized [rows x cols] matrix resident in HBM */
typedef struct tl_model tl_model;     /* a whole model + KV cache + workspaces + decode graph */

/* ---- runtime: replaces the inline cudaSetDevice/cudaMalloc/cudaMemcpy/cudaFree/cudaStream*/
/*      cublasCreate sites (215 of them) ---------------------------------------- */
const char* tl_last_error(void);
/* hipSetDevice + sanity (gfx950 expected) + this device's address of the static no-allocation workspace
 * (tl_attention_noalloc); call once per device the process uses, with that device's ordinal */
int tl_init(int device_ordinal);
/* frees the workspaces that the operator-level entry points (tl_attention, tl_matmul_q, tl_sample_top_k_top_p) grow
 * lazily per device; optional (the process exit frees them too). Those entry points share one workspace per device:
 * calls that overlap on one device must be serialised by the caller (one host thread, as in the reference). */
int tl_shutdown(void);
int tl_device_count(int* count_out);
int tl_malloc(void** dev_out, size_t bytes);  /* cudaMalloc sites e.g. gpu_initialization.cpp:91-531 */
int tl_free(void* dev);
int tl_memset(void* dev, int value, size_t bytes, void* stream);
int tl_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream);
int tl_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream);
int tl_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
int tl_stream_create(void** stream_out);
int tl_stream_destroy(void* stream);
int tl_stream_sync(void* stream);             /* cudaStreamSynchronize, model.cpp:1085 */
int tl_device_sync(void);

/* ---- quantized weights: replaces ensure_f32_concatenated_weights_loaded (weight_management.cpp:199-435)
 *      and the BF16 embedding/lm_head uploads (gpu_initialization.cpp:182-342) --------------------- */
/* host_blocks: rows*cols/block_elems raw GGUF blocks (quantization.h:57-124), row-major by output row.
 * cols must be a multiple of 256 for the K-quants, of 32 for Q8_0 and F32. */
int tl_qweight_upload(int type, const void* host_blocks, int rows, int cols, tl_qweight** out, void* stream);
int tl_qweight_free(tl_qweight* w);
int tl_qweight_info(const tl_qweight* w, int* type, int* rows, int* cols, size_t* device_bytes);
/* Optional: keeps an expanded copy of the matrix for the batched paths (tl_matmul_q with num_tokens > 64, prefill, the
 * multi-sequence decode step): the integers as one bf16 plane + FP32 scale words, 2.375 bytes per weight, from which the
 * matrix cores are fed by LDS-DMA instead of unpacking the quantized planes in every workgroup. Results do not change by
 * a bit. The counterpart of the reference's FP32 expansion, ensure_f32_concatenated_weights_loaded
 * (weight_management.cpp:199-435; 4 bytes per weight there). tl_model_finalize does this for a model's matrices when the
 * copy is at most a quarter of the device's memory (TL_PREFILL_PLANES=0 / 1: never / always). tl_qweight_free drops it.
 * *expanded_bytes (may be NULL): device bytes of the copy (0: this format has none -- F32 / BF16 matrices). */
int tl_qweight_expand(tl_qweight* w, size_t* expanded_bytes, void* stream);

/* Bit-exact dequantization on the device (parity hook for dequantize_q4_k_m / dequantize_q6_k /
 * dequantize_q8_0_block / dequantize_q8_k, quantization.cpp:171-266, 1009-1052): rows [row0, row0+nrows)
 * -> out_dev[nrows*cols] f32. Also what lookup_embedding (model_utils.cpp:11-182) becomes for one row. */
int tl_dequantize_rows(const tl_qweight* w, int row0, int nrows, float* out_dev, void* stream);
/* quantize_fp32_to_q8_K (quantization.cpp:719-770) on the device, bit-exact: n (multiple of 256) FP32 values ->
 * n/256 GGUF Q8_K blocks of 290 B {d:f16, qs[256]:i8, bsums[16]:i16} at blocks_dev */
int tl_quantize_q8_k(const float* x_dev, size_t n, void* blocks_dev, void* stream);

/* y[rows] = W x : replaces matvec_f32_f32_cuda (cuda_kernels.h:171) / matvec_bf16_f32_cuda (:424), on the
 * quantized weights directly. FP32 accumulate; tolerance vs the reference's Kahan-double CPU dot is stated
 * in tests/test_gpu_parity.py (test_gemv_golden, test_gemv_vs_oracle_model_shapes). */
int tl_matvec_q(const tl_qweight* w, const float* x_dev, float* y_dev, void* stream);
/* Y[T][rows] = X[T][cols] W^T : replaces gemm_f32_f32_cuda / gemm_f32_to_bf16_f32_cuda via
 * smart_gemm_batch_cuda (model.cpp:2141-2249) for batched prefill. */
int tl_matmul_q(const tl_qweight* w, const float* x_dev, float* y_dev, int num_tokens, void* stream);
/* bf16 MFMAs per FP32 product in tl_matmul_q (num_tokens >= 8) and, by default, in tl_model_prefill: both operands
 * are split into bf16 planes and a product is assembled from 1 (plain bf16), 3 or 6 (default; FP32-grade) MFMAs. */
int tl_gemm_set_terms(int terms);

/* ---- glue operators (same argument meaning as the cuda_kernels.h wrappers they replace) ------- */
/* rmsnorm_vector_cuda(_optimized) cuda_kernels.h:104,569: out = x*rsqrt(mean(x^2)+max(eps,1e-5))*w
 * (the eps floor is the CPU path's, utils.cpp:666-667, which is the parity target) */
int tl_rmsnorm_vector(const float* x_dev, const float* weight_dev, float* out_dev, int n, float eps, void* stream);
/* rmsnorm_batch_cuda cuda_kernels.h:124 (plain eps, utils.cpp:640) */
int tl_rmsnorm_batch(float* out_dev, const float* in_dev, const float* weight_dev, int num_tokens, int hidden_size,
                     float eps, void* stream);
/* RoPE table of gpu_initialization.cpp:48-58, computed on the host (glibc cosf/sinf/powf, exactly as the
 * reference) and uploaded: table_dev[max_pos][head_dim/2][2] */
int tl_rope_table_upload(float* table_dev, int max_pos, int head_dim, float theta, void* stream);
/* rope_cuda cuda_kernels.h:239 */
int tl_rope(float* vec_dev, int num_heads, int head_dim, const float* freqs_cis_dev, int pos, int max_pos,
            int use_adjacent_pairing, void* stream);
/* rope_batch_cuda cuda_kernels.h:490 */
int tl_rope_batch(float* q_batch_dev, float* k_batch_dev, const float* freqs_cis_dev, int num_tokens,
                  int num_q_heads, int num_kv_heads, int head_dim, int start_pos, int max_pos,
                  int use_adjacent_pairing, void* stream);
/* update_kv_cache_cuda cuda_kernels.h:344 — cache layout [max_seq_len][num_kv_heads][head_dim] */
int tl_update_kv_cache(float* cache_base_dev, const float* kv_vector_dev, int pos, int kv_head_idx,
                       int max_seq_len, int num_kv_heads, int head_dim, void* stream);
/* update_kv_cache_batch_cuda cuda_kernels.h:537 */
int tl_update_kv_cache_batch(float* cache_base_dev, const float* kv_batch_dev, int start_pos, int num_tokens,
                             int num_kv_heads, int head_dim, int cache_max_seq_len, void* stream);
/* attention_cuda / attention_cuda_optimized cuda_kernels.h:259,607 (math of model.cpp:632-663) */
int tl_attention(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev,
                 int num_heads, int current_seq_len, int head_dim, float scale, int cache_max_seq_len,
                 int cache_num_kv_heads, void* stream);
/* tl_attention for callers that cannot allocate. No counterpart in the reference: it is for code under HIP graph
 * capture, tight serving loops and harnesses that forbid hipMalloc, where tl_attention's lazily grown workspace is not
 * an option. Same arguments, same kernels and bit-identical results; the split partials live in a static device array
 * of 64 heads x 32 splits x (128 + 4) floats (1.03 MiB, held by every GPU the library runs on until the process ends).
 * Calls hipMalloc / hipFree never; needs tl_init(device) to have run for the current device (it looks up that
 * device's copy of the array); rejects num_heads * (head_dim + 4) beyond 64 * 132 with an error. All calls on one GPU
 * share the array: calls that overlap on one GPU (two streams) race. */
int tl_attention_noalloc(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev,
                         int num_heads, int current_seq_len, int head_dim, float scale, int cache_max_seq_len,
                         int cache_num_kv_heads, void* stream);
/* sample_top_k_top_p_temperature (api.cpp:126-216) as a device operator (the reference only has it on the host):
 * logits_dev[n] is not modified; u in [0,1) is the caller's uniform variate; *id_dev = the drawn id; optional outputs
 * (NULL to skip): the candidate ids and renormalised probabilities in draw order (capacity >= min(top_k, n)) and their
 * count. Effective top_k <= 1024. */
int tl_sample_top_k_top_p(const float* logits_dev, int n, float temperature, int top_k, float top_p, float u,
                          int* id_dev, int* cand_ids_dev, float* cand_probs_dev, int* n_cand_dev, void* stream);
/* attention_batch_prefill_cuda cuda_kernels.h:498 (math of cpu_attention.cpp:91-201), causal from the cache */
int tl_attention_batch_prefill(const float* q_batch_dev, const float* k_cache_dev, const float* v_cache_dev,
                               float* out_batch_dev, int num_tokens, int start_pos, int cache_max_seq_len,
                               int num_q_heads, int num_kv_heads, int head_dim, float scale, void* stream);
/* add_residual_cuda / add_vectors_cuda / add_residual_batch_cuda cuda_kernels.h:317,329,517 */
int tl_add_residual(const float* a_dev, const float* b_dev, float* out_dev, size_t n, void* stream);
/* swiglu_cuda cuda_kernels.h:379 (decode form, model.cpp:734-735) / swiglu_batch_cuda :482
 * (batch form, cpu_batch_processor.cpp:252-256) */
int tl_swiglu(const float* gate_dev, const float* up_dev, float* out_dev, size_t n, int batch_form, void* stream);
/* lookup_embedding_cuda cuda_kernels.h:408, from the quantized table */
int tl_lookup_embedding(const tl_qweight* table, int token_id, float* out_dev, void* stream);
/* argmax + repetition penalty on the device (api.cpp:73-97,134-136): first maximal index */
int tl_argmax(const float* logits_dev, int n, int* result_dev, void* stream);

/* ---- whole-model engine: what TinyLlamaModel::forward_device (model.cpp:810-1090) + KVCache
 *      (model.h:132-230, kv_cache.cpp:10-169) + the persistent workspaces (gpu_memory_optimization.cpp:8-52)
 *      become ------------------------------------------------------------------------------------- */
typedef struct tl_model_config {
  int hidden_size, intermediate_size, num_attention_heads, num_key_value_heads, num_hidden_layers, vocab_size;
  int max_position_embeddings; /* RoPE table rows and KV cache length */
  float rms_norm_eps, rope_theta;
  int tp_rank, tp_size; /* tensor parallel shard this handle holds (1 = unsharded) */
} tl_model_config;

/* tensor kinds for tl_model_set_tensor; names are the GGUF tensor names the reference consumes
 * (weight_management.cpp:732-960) */
enum tl_tensor_kind {
  TL_T_ATTN_Q = 0, TL_T_ATTN_K, TL_T_ATTN_V, TL_T_ATTN_OUTPUT, TL_T_FFN_GATE, TL_T_FFN_UP, TL_T_FFN_DOWN,
  TL_T_ATTN_NORM, TL_T_FFN_NORM, TL_T_TOKEN_EMBD, TL_T_OUTPUT_NORM, TL_T_OUTPUT
};

int tl_model_create(const tl_model_config* cfg, tl_model** out);
int tl_model_free(tl_model* m);
/* host_data: raw GGUF tensor bytes (blocks row-major by output row). With tp_size > 1 the caller passes THIS RANK'S SHARD
 * with its local shape: attn_q/k/v, ffn_gate/up, output by rows (rank-th block of heads / intermediate columns / vocab
 * rows), attn_output/ffn_down by columns (rank-th block of input columns, a multiple of 256); token_embd and the norms
 * whole (tinyllama.cpp_amd/tp.py has the slicing). layer = -1 for globals. */
int tl_model_set_tensor(tl_model* m, int kind, int layer, int type, const void* host_data, int rows, int cols);
/* allocate KV cache + workspaces, upload the RoPE table, check every tensor is present */
int tl_model_finalize(tl_model* m);
int tl_model_reset_kv(tl_model* m); /* KVCache::clear_data (model.h:182-197) */
/* One decode step = lookup_embedding + forward_device for one token at `pos`; logits_host may be NULL.
 * next_token_host (may be NULL) receives argmax(logits) computed on the device (greedy, no penalty). */
int tl_model_decode(tl_model* m, int token_id, int pos, float* logits_host, int* next_token_host);
/* Greedy generation entirely on the device: feeds argmax back as the next input for n_steps steps starting
 * at (first_token, start_pos); writes the n_steps sampled ids. Repetition penalty as api.cpp:86-97 over the
 * last 64 ids of `history` + what is generated (penalty <= 1: off). */
int tl_model_generate_greedy(tl_model* m, int first_token, int start_pos, int n_steps, float penalty,
                             const int* history_host, int n_history, int* out_ids_host);
/* The same loop with sample_top_k_top_p_temperature (api.cpp:126-216) on the device instead of arg-max: penalty, FP64
 * softmax of (logit - max) / temperature rounded to FP32, top_k by (probability, higher id first), FP32 cumulative
 * top_p cut, renormalisation, inverse-CDF draw as std::discrete_distribution does it. temperature < 0.05 = greedy.
 * Limit: effective top_k <= 1024 ("no top-k", i.e. top_k <= 0 or >= vocab, is rejected: sample on the host). The
 * uniform variates come from a counter-based generator keyed by `seed`. */
int tl_model_generate_sampled(tl_model* m, int first_token, int start_pos, int n_steps, float penalty,
                              const int* history_host, int n_history, float temperature, int top_k, float top_p,
                              unsigned long long seed, int* out_ids_host);
/* batched prefill of T prompt tokens starting at start_pos (forward_device_batch_prefill, model.cpp:1526-1862);
 * last_logits_host[vocab] (may be NULL) = logits of the last token; all_logits_host[T][vocab] may be NULL */
int tl_model_prefill(tl_model* m, const int* tokens_host, int num_tokens, int start_pos, float* last_logits_host,
                     float* all_logits_host);
/* Batched-prefill numerics / routing of this model (no counterpart in the reference, whose GPU prefill is FP32
 * cublasSgemm or BF16 cublasGemmEx by a T >= 4 rule, model.cpp:2152-2153): terms = bf16 MFMAs per FP32 product in the
 * prefill GEMMs: 6 (default, FP32-grade, logits within the decode tolerance), 3 (~2^-17 per product), 1 (plain bf16),
 * 0 = the process-wide value of tl_gemm_set_terms; prompts shorter than min_batch (default 8) and tensor-parallel
 * shards replay the decode graph token by token. */
int tl_model_set_prefill(tl_model* m, int terms, int min_batch);
/* device pointers into the model's state, for parity tests and for hosts that keep using the operator-level
 * calls: which = 0 K cache, 1 V cache of `layer` ([max_pos][n_kv_heads_local][head_dim] f32), 2 = x (hidden) */
int tl_model_device_ptr(tl_model* m, int which, int layer, void** dev_out);
/* algorithmic bytes one decode step at position pos must move on this rank (SURVEY §8d B_tok) */
int tl_model_bytes_per_token(const tl_model* m, int pos, double* weight_bytes, double* kv_bytes);
/* device bytes of the expanded prefill planes that tl_model_finalize keeps for this model's matrices (tl_qweight_expand;
 * 0: none -- switched off, or not affordable on this device). They serve the batched paths only: a decode step never
 * reads them. */
int tl_model_prefill_planes_bytes(const tl_model* m, size_t* bytes_out);
/* Multi-sequence decode (generate_batch api.cpp:836-1142; batch_prefill_parallel :1144, batch_generation_parallel :1423;
 * forward_cpu_batch_generation model.cpp:1158-1523 / forward_device_batch_generation :1863-2114): up to max_batch
 * sequences share the weights of every step -- the projections of the B tokens are skinny GEMMs on the matrix cores, the
 * KV cache is sequence-major ([seq][max_pos][kv heads][head_dim], model.cpp:1310-1312), attention runs per token over its
 * own sequence. tl_model_batch_init (after tl_model_finalize, tp_size 1) allocates that cache; tl_model_batch_prefill
 * fills one sequence's prompt (positions start_pos..) and returns its last logits; tl_model_batch_decode is ONE step with
 * batch_generation_parallel's arguments (token, position and sequence index per active sequence; indices must be
 * distinct), returning logits [n][vocab] and/or the first-maximum ids; tl_model_batch_generate_greedy runs n_steps steps
 * with ids and positions advancing on the device: out_ids_host [n_steps][n]. No repetition penalty on this path
 * (api.cpp:993,1084). Each sequence decodes exactly as it would alone (the reference's sequential fallback,
 * api.cpp:1116-1130); its parallel path leaves the current token out of its own attention (model.cpp:1327). */
int tl_model_batch_init(tl_model* m, int max_batch);
int tl_model_batch_prefill(tl_model* m, int seq_idx, const int* tokens_host, int num_tokens, int start_pos,
                           float* last_logits_host);
/* batch_prefill_parallel (api.cpp:1144): the tokens of ALL prompts as one packed batch (token i of sequence seq_idx[i] at
 * position positions[i]; the tokens of a sequence in position order), sequence-aware attention
 * (cpu_attention.cpp:254-325), chunks of 512 tokens. last_rows[j] = index of a token whose logits [n_last][vocab] and
 * first-maximum id are returned (the last token of each prompt); n_last <= max_batch; either output may be NULL. */
int tl_model_batch_prefill_packed(tl_model* m, int n_tokens, const int* tokens_host, const int* positions_host,
                                  const int* seq_idx_host, int n_last, const int* last_rows_host, float* last_logits_host,
                                  int* last_ids_host);
int tl_model_batch_decode(tl_model* m, int n, const int* tokens_host, const int* positions_host, const int* seq_idx_host,
                          float* logits_host, int* next_tokens_host);
int tl_model_batch_generate_greedy(tl_model* m, int n, const int* first_tokens_host, const int* start_pos_host,
                                   const int* seq_idx_host, int n_steps, int* out_ids_host);
/* ---- layer-list models: a decoder described layer by layer instead of by the fixed Llama block. No counterpart in the
 *      reference (its only model is the Llama block). Such a model lives behind the same tl_model handle: tl_model_finalize,
 *      tl_model_reset_kv, tl_model_decode, tl_model_generate_greedy / _sampled, tl_model_prefill, tl_model_set_prefill
 *      (terms 1 = bf16 activations in the chunk GEMMs, 3 = FP32-grade), tl_model_device_ptr, tl_model_bytes_per_token and
 *      tl_model_free work as for a Llama model; the multi-sequence and tensor-parallel entry points refuse it. Weights are
 *      bf16 matrices [out][in] and stay bf16 in HBM; the residual stream, norms, router, scores and caches are FP32. ------ */
enum tl_mixer_kind {
  TL_MIXER_SWA = 0,         /* windowed attention over a key/value cache (softmax or sigmoid weights, optional rotation) */
  TL_MIXER_DELTA = 1,       /* gated delta rule with a decay per key channel: a recurrent state per head, no cache of keys */
  TL_MIXER_LATENT = 2,      /* attention over a cached latent: queries through a normalised latent, keys and values of all heads
                               up-projected from one normalised latent per token, plus one rotated key part shared by the heads;
                               the cache holds the latent and that part only (optionally another layer's, kv_from) */
  TL_MIXER_GDELTA = 3,      /* generalized delta rule: decay and removal rate per key channel,
                               S <- diag(w) S - (a u)(u^T S) + k v^T with the unit key u, o = S^T r */
  TL_MIXER_LINEAR = 4       /* gated linear attention whose forget gate also decides what is written (no keys):
                               q = silu(W_q h), f = l + (1 - l) sigmoid(W_f h + b), S <- diag(f) S + (1 - f) v^T, o = S^T q,
                               RMS norm per head with one plain weight [vdim] */
};
enum tl_mlp_kind {
  TL_MLP_NONE = 0,
  TL_MLP_MOE = 1,           /* routed experts (+ shared expert) */
  TL_MLP_DENSE = 2,         /* one gated unit (tl_glu_kind) */
  TL_MLP_UNIT = 3           /* W_down act(W_up h): no gate; act = tl_act_kind (shared_ff is its size) */
};
enum tl_act_kind {
  TL_ACT_NONE = 0,
  TL_ACT_XIELU = 1,         /* z > 0: P z^2 + z / 2; z <= 0: Q (e^z - 1 - z) + z / 2, with P = softplus(p), Q = 1/2 + softplus(q)
                               from the two numbers of the tensor mlp.act */
  TL_ACT_TANH = 2
};
enum tl_glu_kind {
  TL_GLU_SWISH = 0,         /* g sigmoid(act_alpha g) (u + glu_up_add), g = min(gate, limit), u = clamp(up, -limit, limit) */
  TL_GLU_RELU = 1           /* max(gate, 0) * up */
};
enum tl_block_kind {
  TL_BLOCK_POST_NORM = 0,   /* x += N1(mixer(x)); x += N2(ff(x)): the sublayers read x, the norm is on their output */
  TL_BLOCK_PARALLEL = 1,    /* h = N1(x); x += mixer(h) + ff(h): one norm, both sublayers read its output */
  TL_BLOCK_PRE_NORM = 2     /* x += mixer(N1(x)); x += ff(N2(x)): a norm in front of each sublayer */
};
enum tl_norm_kind {
  TL_NORM_RMS_ONE_PLUS = 0, /* y / sqrt(mean(y^2) + eps) * (1 + w) */
  TL_NORM_DYT = 1,          /* tanh(alpha y) * w + b: elementwise, no mean or variance (tensors <name>, <name>.alpha, <name>.b) */
  TL_NORM_LAYER = 2,        /* (y - mean) / sqrt(var + eps) * w + b, var = mean of the squared deviations (tensors <name>, <name>.b) */
  TL_NORM_RMS = 3           /* y / sqrt(mean(y^2) + eps) * w: plain weights (pre-norm blocks) */
};
enum tl_attn_weight {
  TL_ATTN_SOFTMAX = 0,      /* weights normalised over the visible keys */
  TL_ATTN_SIGMOID = 1,      /* weight of a visible key = sigmoid(score + bias[head]); not normalised */
  TL_ATTN_SOFTMAX_SINK = 2, /* softmax with one more term in the denominator: a sink of score 0 that carries no value */
  TL_ATTN_SOFTMAX_LEARNED_SINK = 3 /* the same with exp(sink[head]) as that term: a learned number per head (mix.sink) */
};
enum tl_qk_norm {
  TL_QK_NORM_NONE = 0,
  TL_QK_NORM_WHOLE = 1,     /* RMS norm over the WHOLE q and the whole k projection, plain weights (mix.q.norm, mix.k.norm) */
  TL_QK_NORM_HEAD_UNIT = 2, /* per head, after the rotation: x / sqrt(mean(x^2) + eps), no weights */
  TL_QK_NORM_HEAD_RMS = 3   /* per head (and score map): RMS norm over dim with one plain weight [dim] for all heads
                               (mix.q.norm, mix.k.norm) */
};
enum tl_route_kind {
  TL_ROUTE_TOP_LOGITS = 0,  /* the `top` largest logits (+ bias); weights = softmax over the chosen logits */
  TL_ROUTE_SOFTMAX_GROUPS = 1, /* scores = softmax over all experts; experts in `route_groups` equal groups of neighbours, a
                               group's score its best expert's, only the best `route_keep` groups can be chosen from;
                               weights = the chosen scores divided by their sum (+ 1e-20) */
  TL_ROUTE_SIGMOID_GROUPS = 2 /* scores = sigmoid(logits); choice = score + mlp.correction[expert]; a group's rank is the sum of
                               its two best choices, experts outside the best `route_keep` groups cannot be chosen; the `top`
                               best choices are taken; weights = their scores (without the correction, not normalised) */
};
typedef struct tl_layer_spec {
  int mixer;                /* tl_mixer_kind */
  int heads, kv_heads;      /* query heads, key/value heads (query head h reads head h / (heads / kv_heads)) */
  int dim, vdim;            /* per-head query/key size, value size */
  int window;               /* position i sees j with 0 <= i - j < window; <= 0: every j <= i */
  float scale;              /* score = (q . k) * scale */
  int qk_norm;              /* tl_qk_norm */
  int v_mix;                /* 1: v <- (1 - lambda) v + lambda v_first, v_first = the first such layer's values of the token */
  int mlp;                  /* tl_mlp_kind */
  int experts, top;         /* routed experts, experts per token */
  int expert_ff;            /* y = g * sigmoid(act_alpha * g) * (u + glu_up_add), g = min(gate, limit), u = clamp(up, -limit, limit) */
  float expert_limit;       /* (a limit of +infinity clamps nothing) */
  int shared_ff;            /* 0: no shared expert. TL_MLP_DENSE: the one gated unit's size, its tensors are mlp.{gate,up,down} */
  float shared_limit;
  float act_alpha;
  /* ---- everything below is zero for the plain softmax window attention of a post-norm block ---- */
  float glu_up_add;         /* added to the up projection inside the gated unit (0 or 1) */
  int block;                /* tl_block_kind */
  int weights_of;           /* 1 + index of an EARLIER layer whose tensors (mixer, feed-forward, norms) this layer uses, with a
                               cache or state of its own; 0: its own tensors. The rest of the entry must equal that layer's. */
  int keep_first;           /* TL_MIXER_SWA: keys j < keep_first stay visible beyond the window (at their true positions) */
  int attn_weight;          /* tl_attn_weight; TL_ATTN_SIGMOID reads the per-head bias mix.pb */
  int values_are_keys;      /* 1: no value projection: v = the key as projected (before rotation and norm); vdim == dim */
  int rot_dims;             /* rotary positions on the first rot_dims dimensions of each q / k head, dimension 2i paired with
                               2i + 1, angle = position * f_i, f_i = rot_base^(-2i / rot_dims); 0: no rotation */
  float rot_base;
  float rot_factor;         /* > 0: context extension by frequency blending: with d(t) = rot_dims ln(rot_original / (2 pi t)) /
                               (2 ln rot_base), lo = max(floor(d(rot_fast)), 0), hi = min(ceil(d(rot_slow)), rot_dims - 1),
                               r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1): f_i <- f_i / rot_factor r_i + f_i (1 - r_i),
                               and cos, sin are multiplied by 0.1 ln(rot_factor) + 1 */
  float rot_original, rot_fast, rot_slow;
  int conv_taps;            /* TL_MIXER_DELTA: taps of the causal convolution over time on q, k, v (each followed by silu) */
  int decay_rank, gate_rank; /* TL_MIXER_DELTA: inner sizes of the two-step decay (a1, a2) and output gate (g1, g2) projections */
  int route;                /* tl_route_kind */
  int route_groups, route_keep;
  int shared_gate;          /* 1: the shared expert's output is multiplied by sigmoid(w_sg . h) (mlp.shared.sg) */
  float q_temp_coef;        /* TL_MIXER_SWA, q_temp_every > 0: the query at position p is multiplied by */
  int q_temp_every;         /*   1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1) */
  int q_rank, kv_rank;      /* TL_MIXER_LATENT: sizes of the query latent and of the cached key/value latent */
  int rot_dim;              /* TL_MIXER_LATENT: rotated query/key dimensions per head behind the `dim` plain ones (the key's are
                               shared by all heads); rot_dims <= rot_dim of them turn */
  int kv_from;              /* TL_MIXER_LATENT: 1 + index of an EARLIER latent layer (with a projection of its own and the same
                               kv_rank, rot_dim and rotation) whose cached latent and rotated key part this layer reads; 0: its own */
  int head_gate;            /* TL_MIXER_LATENT: 1: head n's output is multiplied by sigmoid(W_g h)_n (mix.g, one row per head) */
  float decay_scale;        /* TL_MIXER_GDELTA: decay = exp(-decay_scale * sigmoid(W_w2 tanh(W_w1 h) + w0)); decay_rank = rows of w1 */
  int act;                  /* TL_MLP_UNIT: tl_act_kind */
  int glu;                  /* tl_glu_kind of the gated units (experts, shared expert, dense unit) */
  /* ---- TL_MIXER_SWA, all zero = none of it ---- */
  int score_maps;           /* 2: differential attention -- q and k hold two maps per head ([map 1 | map 2], dim each) over the
                               same values; o = a1 - lambda a2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff_init (tensors
                               mix.lq1 .. mix.lk2 [dim]), then o / rms(o) over vdim (no weight) times (1 - diff_init) */
  float diff_init;
  int out_gate;             /* 1: the concatenated heads are multiplied by sigmoid(W_g h) (mix.g [heads * vdim][width]) */
  int qkv_bias;             /* 1: q, k, v = W h + b (mix.q.b, mix.k.b, mix.v.b) */
  int qkv_conv;             /* > 0: taps of a causal convolution over time per channel of q, k, v right after the projection
                               (mix.{q,k,v}.conv [channels][taps], no activation); its last taps - 1 inputs are state */
  float score_softcap;      /* > 0: score <- cap * tanh(score / cap) */
  int dist_bias;            /* 1: score <- score - r1[head] ln(1 + r2[head] (i - j)) (mix.r1, mix.r2) */
  /* ---- TL_MIXER_DELTA ---- */
  int decay_per_head;       /* 1: one decay per head, g = exp(-exp(A_log) softplus(W_a h + dt_bias)) with mix.a [heads][width]
                               and dt_bias [heads] (decay_rank = 0); the output gate is silu(W_g h), mix.g [heads * vdim][width]
                               (gate_rank = 0) */
  /* ---- a second mixer beside the first, both reading the same input: the layer's mixer output is
          mix_scale * mixer + side_scale * side. `side` is that mixer's entry (mixer fields only: block, feed-forward and
          weights_of are the layer's). The first mixer's tensors are then l<i>.mix.left.*, the second's l<i>.mix.right.* ---- */
  const struct tl_layer_spec* side;
  float mix_scale, side_scale;
} tl_layer_spec;
typedef struct tl_stack_config {
  int width, vocab, n_layers;
  int max_positions;        /* rows of every attention layer's key/value cache */
  float norm_eps;           /* every RMS norm: x / sqrt(mean(x^2) + eps) */
  const tl_layer_spec* layers;
  int norm;                 /* tl_norm_kind of the block norms and the final norm */
  int embed_norm;           /* 1: the embedding row is normalised (tensor embed.norm) before the first layer */
  float logit_softcap;      /* > 0: logits <- cap * tanh(logits / cap) */
  float embed_scale;        /* != 0: the embedding row is multiplied by it */
  int canon_taps;           /* > 0 (pre-norm blocks): what a sublayer reads is h + conv(h), a causal convolution over time per
                               channel with so many taps (l<i>.canon1 for the mixer, l<i>.canon2 for the feed-forward,
                               [width][taps], the last column is the current token's); the last taps - 1 inputs are state */
} tl_stack_config;
/* the operators such a model is built from, callable on their own (all FP32 in and out, weights bf16 [rows][cols]):
 * Y[T][rows] = X[T][cols] W^T; terms 1 / 3 = MFMA GEMM with bf16-rounded / three-term-split activations, 0 = FP32 GEMV (T = 1) */
int tl_dense_matmul(const void* w_bf16_dev, int rows, int cols, const float* x_dev, float* y_dev, int num_tokens, int terms,
                    void* stream);
/* q [T][heads * dim] at positions start_pos.. against caches K [*][kv_heads * dim], V [*][kv_heads * vdim] that already hold
 * those positions: softmax((q . k) * scale) over the keys j with 0 <= i - j < window (window <= 0: all j <= i) */
int tl_swa_attention(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev, int num_tokens,
                     int start_pos, int heads, int kv_heads, int dim, int vdim, int window, float scale, void* stream);
/* x[t] += y[t] / sqrt(mean(y[t]^2) + eps) * (1 + weight) */
int tl_resid_rmsnorm(float* x_dev, const float* y_dev, const float* weight_dev, int num_tokens, int width, float eps, void* stream);
/* router (TL_ROUTE_TOP_LOGITS): logits = W x + bias (FP32); ids [T][top] = the largest logits first (equal: lower index), weights = softmax over them */
int tl_moe_route(const float* x_dev, int num_tokens, int width, const void* w_bf16_dev, const float* bias_dev, int experts,
                 int top, int* ids_dev, float* weights_dev, void* stream);
/* out[r][i] = g * sigmoid(alpha * g) * (u + 1), g = min(in[r][i], limit), u = clamp(in[r][ff + i], -limit, limit) */
int tl_glu_clamp(const float* gate_up_dev, int rows, int ff, float limit, float alpha, float* out_dev, void* stream);
/* tl_swa_attention with every option of the mixer: keys j < keep_first stay visible beyond the window; sigmoid != 0: the weight
 * of a visible key is sigmoid(score + head_bias_dev[head]) and is not normalised */
int tl_window_attention(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev, int num_tokens,
                        int start_pos, int heads, int kv_heads, int dim, int vdim, int window, int keep_first, float scale,
                        int sigmoid, const float* head_bias_dev, void* stream);
/* router (TL_ROUTE_SOFTMAX_GROUPS), no bias: ids [T][top] largest score first, weights = chosen scores / their sum */
int tl_moe_route_groups(const float* x_dev, int num_tokens, int width, const void* w_bf16_dev, int experts, int top, int groups,
                        int keep, int* ids_dev, float* weights_dev, void* stream);
/* out[t] = tanh(alpha x[t]) * w + b (alpha: one device float) */
int tl_dyt_norm(const float* x_dev, const float* alpha_dev, const float* weight_dev, const float* bias_dev, float* out_dev,
                int num_tokens, int width, void* stream);
/* rotary positions as tl_layer_spec describes them (rot_factor <= 0: plain frequencies), in place on x [T][heads * dim] at
 * positions start_pos.., then (unit_norm != 0) every head divided by its root mean square (eps inside the root). The
 * frequencies and the product position * frequency are double; cos and sin of its remainder in [-pi, pi] are FP32. */
int tl_rotary_heads(float* x_dev, int num_tokens, int start_pos, int heads, int dim, int rot_dims, float rot_base,
                    float rot_factor, float rot_original, float rot_fast, float rot_slow, int unit_norm, float eps, void* stream);
/* what precedes the gated delta rule, per token: p [T][ld] holds the projections q (kv_heads * dim) | k (kv_heads * dim) |
 * v (heads * vdim) | beta (heads), a [T][heads * dim] the decay's pre-activation. q, k, v pass a causal convolution over time
 * (w bf16 [channels][taps], channels = q | k | v, the last tap is the current token's; the inputs of the taps - 1 tokens before
 * this call come from history [taps - 1][channels], oldest first, which afterwards holds the last taps - 1 inputs) and silu;
 * q and k become unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q also times dim^-1/2 -> qkv [T][channels];
 * beta [T][heads] = sigmoid; g [T][heads * dim] = exp(-exp(a_log[head]) * softplus(a + dt_bias)) */
int tl_delta_prepare(const float* p_dev, int ld, const float* a_dev, int num_tokens, int heads, int kv_heads, int dim, int vdim,
                     int taps, const void* conv_bf16_dev, float* history_dev, const float* a_log_dev, const float* dt_bias_dev,
                     float* qkv_dev, float* beta_dev, float* g_dev, void* stream);
/* gated delta rule, token by token: per head h (q / k head h / (heads / kv_heads)) with state S [dim][vdim]:
 * S <- diag(g_t) S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t. q, k [T][kv_heads * dim], v, o [T][heads * vdim],
 * beta [T][heads], g [T][heads * dim]; state_dev [heads][vdim][dim] (column-major per head), updated in place */
int tl_delta_rule(const float* q_dev, const float* k_dev, const float* v_dev, const float* beta_dev, const float* g_dev,
                  float* state_dev, float* o_dev, int num_tokens, int heads, int kv_heads, int dim, int vdim, void* stream);
/* o[t][h] <- o / sqrt(mean(o^2) + eps) * w * sigmoid(gate[t][h]) per head, in place; o, gate [T][heads * vdim], w [vdim] */
int tl_gated_head_norm(float* o_dev, const float* gate_dev, const float* weight_dev, int num_tokens, int heads, int vdim,
                       float eps, void* stream);

/* tl_window_attention over caches whose rows are k_ld / v_ld floats apart (0: kv_heads * dim, kv_heads * vdim); mode is a
 * tl_attn_weight. A latent cache serves as both: keys = the whole row, values = its first vdim columns. */
int tl_window_attention_rows(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev, int num_tokens,
                             int start_pos, int heads, int kv_heads, int dim, int vdim, int k_ld, int v_ld, int window,
                             int keep_first, float scale, int mode, const float* head_bias_dev, void* stream);
/* out[t] = (x[t] - mean) / sqrt(var + eps) * w + b */
int tl_layer_norm(const float* x_dev, const float* weight_dev, const float* bias_dev, float* out_dev, int num_tokens, int width,
                  float eps, void* stream);
/* tl_dense_matmul with an activation (tl_act_kind; p, q as the kind describes them, already transformed) on the output rows
 * from act_from on */
int tl_dense_matmul_act(const void* w_bf16_dev, int rows, int cols, const float* x_dev, float* y_dev, int num_tokens, int terms,
                        int act, float act_p, float act_q, int act_from, void* stream);
/* per head g < groups: Y[t][g * y_stride + r] = sum_c W[g][r][c] X[t][g * x_stride + c], W bf16 [groups][rows][cols]; X rows
 * ldx, Y rows ldy floats apart. terms as tl_dense_matmul (0: one token, FP32) */
int tl_dense_matmul_heads(const void* w_bf16_dev, int groups, int rows, int cols, const float* x_dev, int ldx, int x_stride,
                          float* y_dev, int ldy, int y_stride, int num_tokens, int terms, void* stream);
/* generalized delta rule, token by token. p [T][ld] holds the projections r | k | v (heads * dim each) | gate (unused here) |
 * a (heads * dim), dw [T][heads * dim] the decay's pre-activation: w = exp(-decay_scale * sigmoid(dw + w0)),
 * a = sigmoid(a + a_bias), u = k / sqrt(sum k^2 + 1e-6) per head; S <- diag(w) S - (a u)(u^T S) + k v^T; o = S^T r.
 * state_dev [heads][dim (value)][dim (key)], updated in place; o [T][heads * dim]; scratch_dev: 3 * T * heads * dim + 2 * T * heads floats */
int tl_general_delta(const float* p_dev, int ld, const float* dw_dev, const float* w0_dev, const float* a_bias_dev,
                     float decay_scale, float* state_dev, float* o_dev, float* scratch_dev, int num_tokens, int heads, int dim,
                     void* stream);

/* a causal convolution over time per channel: u[t][c] = in[t][c] (+ bias[c]); out[t][c] = act(sum_j w[c][j] u[t - taps + 1 + j][c])
 * (+ u[t][c] with add_input); w bf16 [channels][taps], the last tap is the current token's; act 0: none, 1: silu. The inputs
 * before this call come from history [taps - 1][channels] (oldest first, zeros for an empty sequence), which afterwards holds
 * the last taps - 1 inputs u. out must not overlap in when num_tokens > 1. */
int tl_causal_conv(const float* in_dev, int ld_in, int channels, int taps, int num_tokens, const float* bias_dev,
                   const void* w_bf16_dev, float* history_dev, int act, int add_input, float* out_dev, int ld_out, void* stream);
/* router (TL_ROUTE_SIGMOID_GROUPS): ids [T][top] best choice first, weights = the chosen experts' sigmoid scores */
int tl_moe_route_sigmoid_groups(const float* x_dev, int num_tokens, int width, const void* w_bf16_dev,
                                const float* correction_dev, int experts, int top, int groups, int keep, int* ids_dev,
                                float* weights_dev, void* stream);
/* softmax window attention with the score options of TL_MIXER_SWA: heads of a query / key row q_hstride / k_hstride floats
 * apart (0: dim), rows ldq / k_ld / v_ld apart (0: packed); score = (q . k) scale, capped by softcap tanh(. / softcap) when
 * softcap > 0, minus r1[head] ln(1 + r2[head] (i - j)) when r1_dev is set; sink != 0: exp(sink_dev[head]) (exp(0) without
 * sink_dev) joins the denominator */
int tl_window_attention_opts(const float* q_dev, int ldq, int q_hstride, const float* k_cache_dev, int k_ld, int k_hstride,
                             const float* v_cache_dev, int v_ld, float* out_dev, int num_tokens, int start_pos, int heads,
                             int kv_heads, int dim, int vdim, int window, float scale, float softcap, const float* r1_dev,
                             const float* r2_dev, int sink, const float* sink_dev, void* stream);
/* per head, in place: o <- (o - sub_coef sub) / sqrt(mean(.^2) + eps) * w * gate_fn(gate) * out_scale; sub_dev, weight_dev
 * ([vdim], or [heads * vdim] with weight_per_head) and gate_dev (rows gate_ld apart) may be NULL; gate_act 0: sigmoid, 1: silu */
int tl_head_norm(float* o_dev, const float* sub_dev, float sub_coef, const float* gate_dev, int gate_ld, int gate_act,
                 const float* weight_dev, int weight_per_head, float out_scale, int num_tokens, int heads, int vdim, float eps,
                 void* stream);
/* gated linear attention (TL_MIXER_LINEAR), token by token: p [T][ld] = q | f (heads * dim each) | v (heads * vdim);
 * q <- silu(q), f <- lower + (1 - lower) sigmoid(f + f_bias); S <- diag(f) S + (1 - f) v^T; o = S^T q. state_dev
 * [heads][vdim][dim], updated in place; o [T][heads * vdim]; scratch_dev: 3 * T * heads * dim floats */
int tl_gated_linear_attention(const float* p_dev, int ld, const float* lower_dev, const float* f_bias_dev, float* state_dev,
                              float* o_dev, float* scratch_dev, int num_tokens, int heads, int dim, int vdim, void* stream);

int tl_model_create_stack(const tl_stack_config* cfg, tl_model** out);
/* tensors by checkpoint name: embed, embed.norm, final.norm, head, l<i>.norm1, l<i>.norm2, l<i>.mix.{q,k,v,o,q.norm,k.norm,vmix,pb},
 * l<i>.mix.{q,k,v}.conv, l<i>.mix.{b,a1,a2,g1,g2,A_log,dt_bias,norm}, l<i>.mlp.router, l<i>.mlp.router.b,
 * l<i>.mlp.e<j>.{gate,up,down}, l<i>.mlp.shared.{gate,up,down,sg}, l<i>.mlp.{gate,up,down,act,correction}, l<i>.canon{1,2},
 * l<i>.mix.{g,lq1,lk1,lq2,lk2,r1,r2,sink}, l<i>.mix.{q,k,v}.b, l<i>.mix.{f,f.b,lower,a}; with two mixers side by side
 * l<i>.mix.left.* and l<i>.mix.right.*; latent attention
 * l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,g,o}; generalized delta rule l<i>.mix.{r,k,v,g,a,a.b,w1,w2,w0,norm,o}; a Dynamic
 * Tanh norm <n> also has <n>.alpha and <n>.b, a layer norm <n>.b. type: TL_BF16 (matrices and vectors) or TL_F32 (vectors). */
int tl_model_set_tensor_named(tl_model* m, const char* name, int type, const long long* shape, int ndim, const void* host_data);
/* a prompt, or a portion of one, at positions start_pos..: logits of the token rows listed in rows_host (ascending; NULL: the
 * last token when n_rows == 1, all tokens when n_rows == num_tokens) -> logits_host[n_rows][vocab]. The cache keeps what
 * earlier calls wrote: portions may be cut anywhere. */
int tl_model_prefill_rows(tl_model* m, const int* tokens_host, int num_tokens, int start_pos, const int* rows_host, int n_rows,
                          float* logits_host);

/* tensor-parallel wiring (one process per GPU): RCCL communicator over xGMI; unique_id is the ncclUniqueId (128 bytes)
 * produced by tl_tp_unique_id on rank 0 and broadcast by the host (torch.distributed). Call tl_model_tp_init on every
 * rank before tl_model_finalize: the decode step (incl. its 2 all-reduces per layer and the logits all-gather) is
 * captured into the graph there. Replaces distributed_coordinator.cpp's MPI request routing. */
int tl_tp_unique_id(void* id_out_128);
int tl_model_tp_init(tl_model* m, const void* unique_id_128);
/* Peer-to-peer exchange for the decode step (no counterpart in the reference): the two f32[hidden] all-reduces per layer
 * and the logits all-gather of a tp_size 2..8 group as ONE small kernel each, which pushes 8-byte {value, epoch} words
 * straight into receive areas that every rank maps from every other rank (hipIpc; xGMI links between the GPUs of a
 * node) and sums what arrives in rank order. Wiring, on every rank, before tl_model_finalize:
 *   tl_model_tp_peer_export  -> this rank's 64-byte IPC handle; the host gathers the handles of all ranks (rank order)
 *   tl_model_tp_peer_import  -> maps them and runs a COLLECTIVE self-check (known sums); *ok_out = 1 if it passed here
 *   the host agrees on min(ok) over the ranks and calls tl_model_tp_peer_enable(m, agreed) on every rank.
 * Enabled: the decode step uses the peer kernels (the batched prefill's T x hidden all-reduces stay with RCCL and need
 * tl_model_tp_init; without a communicator a sharded prefill goes token by token). Every poll is bounded (5 s, or
 * TL_TP_PEER_TIMEOUT_MS): a missing rank turns into an error return of the decode / generate call, not a hang.
 * By default the exchanges are not even launches: the attn_output / ffn_down / lm_head GEMVs push their rows as they
 * finish them and collect the other ranks' rows before they end, so the sharded step has exactly the launches of the
 * unsharded one (tl_model_tp_peer_fused reports 1; TL_TP_PEER_FUSED=0 keeps one exchange kernel per all-reduce /
 * all-gather). Folded exchanges wait inside full-chip launches: ranks that SHARE a device (rehearsals) must cap the
 * launches so that all ranks fit together (TL_GEMV_CUS = CUs / ranks); with a device per rank nothing is needed. */
int tl_model_tp_peer_export(tl_model* m, void* handle_out_64);
int tl_model_tp_peer_import(tl_model* m, const void* handles_tp_x_64, int* ok_out);
int tl_model_tp_peer_enable(tl_model* m, int on);
int tl_model_tp_peer_enabled(const tl_model* m, int* on_out);
int tl_model_tp_peer_fused(const tl_model* m, int* on_out);
/* Diagnostic (no counterpart in the reference): *captured_out = 1 when the decode step replays as one hipGraph, 0 when
 * it is enqueued launch by launch (TL_NO_GRAPH=1, a shard without a communicator, or a collective that refused
 * capture). With TL_TP_SELFTEST=1 in the environment tl_model_tp_init gives a tp_size-1 model a one-rank communicator,
 * so the RCCL calls of the step and their capture can be exercised on one GPU. */
int tl_model_graph_captured(const tl_model* m, int* captured_out);
/* Diagnostic (no counterpart in the reference): the number of nodes (launches) of the captured decode step, 0 when the
 * step is not captured. A tensor-parallel shard whose exchanges ride inside its GEMVs has as many as the whole model. */
int tl_model_graph_nodes(const tl_model* m, int* nodes_out);
/* Test hook: ALL n shards of a tp_size = n model live in this process on this device (created with tp_rank = 0..n-1,
 * finalized without tl_model_tp_init); one decode step in lockstep, collectives as plain kernels. */
int tl_tp_local_group_decode(tl_model* const* shards, int n, int token_id, int pos, float* logits_host,
                             int* next_token_host);

/* the same for the batched prefill of a prompt (collectives as plain kernels); last_logits_host[vocab] may be NULL */
int tl_tp_local_group_prefill(tl_model* const* shards, int n, const int* tokens_host, int num_tokens, int start_pos,
                              float* last_logits_host);

#ifdef __cplusplus
}
#endif
#endif
