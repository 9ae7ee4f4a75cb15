/*
 * libjitnn_hip.so - MI355X (gfx950) implementation of jitNN's GGUF quantised-weight linear path.
 *
 * Plain C ABI: opaque handles, raw pointers and sizes; no C++ or torch types.  Every function returns
 * an int status (JITNN_HIP_OK or a negative JITNN_HIP_E* code) unless stated otherwise, never throws and
 * never aborts the process; jitnn_hip_last_error() gives the message of the calling thread's last failure.
 *
 * Each entry point names the reference interface it stands in for (paths relative to the reference
 * root; "core/" = jitnn-core/src/main/java/ai/beestream/jitnn/, "gguf/" =
 * jitnn-gguf/src/main/java/ai/beestream/jitnn/gguf/).
 *
 * Conventions
 *  - fmt is the ggml type id stored in GGUF files (gguf/GgmlType.java:27-65):
 *    Q4_0=2 Q4_1=3 Q8_0=8 Q4_K=12 Q5_K=13 Q6_K=14 (the quantised-linear path proper: tuned kernels), and
 *    Q5_0=6 Q5_1=7 Q2_K=10 Q3_K=11 (the other block formats the reference dequantises,
 *    core/kernels/GgufKernels.java:147-198: bit-exact dequantiser; Q5_0 and Q3_K are served by the Q8_0 / Q6_K
 *    kernels after an exact rewrite at upload, Q5_1 and Q2_K by units of their own in the batch-1 kernel - up to four
 *    rows a launch -, by tiles of their own in the one-pass kernel from five rows to 64, and by the many-row kernel beyond).
 *  - A weight is [n, k] row-major rows of k/block_values blocks, byte-for-byte as in the GGUF file
 *    (core/Tensor.java:249-278); it stays in that layout in HBM.
 *  - Activations and outputs are FP32 row-major: x [rows, k], y [rows, n], bias [n].
 *  - "_dev" entry points take device pointers and a hipStream_t passed as void* (NULL = the null stream);
 *    they only enqueue work.  Entry points without "_dev" take host pointers and are synchronous: they copy
 *    through pinned host memory and a device buffer that the library keeps per calling thread (no allocation
 *    per call once the buffers have grown to the largest call) on a stream of that thread.
 *  - Thread safety: weights are immutable after upload and may be shared by any number of threads;
 *    each call uses only its arguments and per-call stream order; the last-error string is thread-local.
 */
#ifndef JITNN_HIP_H
#define JITNN_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

#define JITNN_HIP_API __attribute__((visibility("default")))

#define JITNN_HIP_OK 0
#define JITNN_HIP_EINVAL (-1)   /* bad argument: unknown format, k not a multiple of the block, size mismatch, NULL */
#define JITNN_HIP_EDEVICE (-2)  /* a HIP runtime call failed */
#define JITNN_HIP_ENODEVICE (-3) /* no gfx950 device / library not initialised */
#define JITNN_HIP_ENOMEM (-4)
#define JITNN_HIP_EIO (-5)       /* a file cannot be read or is not a valid GGUF file (Java: IOException) */
#define JITNN_HIP_EUNSUPPORTED (-6) /* a ggml type this path has no tensor type for (Java: UnsupportedOperationException) */

#define JITNN_HIP_Q4_0 2
#define JITNN_HIP_Q4_1 3
#define JITNN_HIP_Q8_0 8
#define JITNN_HIP_Q4_K 12
#define JITNN_HIP_Q5_K 13
#define JITNN_HIP_Q6_K 14

typedef struct jitnn_hip_weight jitnn_hip_weight;

/* ---- library and device ------------------------------------------------------------------------ */

/* Selects the device and prepares the kernels; idempotent.  The counterpart of binding an optional native
 * library at start-up (core/cpu/Blas.java:59-104): on failure the caller keeps its own path. */
JITNN_HIP_API int jitnn_hip_init(int device_ordinal);

/* Device name (NUL-terminated, truncated to cap), compute units and HBM bytes. */
JITNN_HIP_API int jitnn_hip_device_info(char *name, int cap, int *compute_units, long long *hbm_bytes);

/* Message of the calling thread's last failed call; never NULL.  Failures surface in Java as
 * JitnnException("calling ... failed", cause) (core/cpu/Blas.java:195-200, core/JitnnException.java:18-25). */
JITNN_HIP_API const char *jitnn_hip_last_error(void);

JITNN_HIP_API int jitnn_hip_sync(void);

/* Frees what the library keeps for the calling thread: the staging buffers and the stream of the host-pointer entry
 * points and the scratch of the many-row path (both grow on demand and are otherwise kept until the thread ends; the
 * process's first thread keeps them until the process ends).  Waits for the device first.  The counterpart of dropping
 * a thread's derived copies (core/cpu/Gemm.java:497-515). */
JITNN_HIP_API int jitnn_hip_thread_release(void);

/* ---- block formats (no device needed) ------------------------------------------------------------ */

/* Values per block / bytes per block of a format, 0 when fmt is not one of the ten
 * (core/DType.java:75-98, gguf/GgmlType.java:113-118). */
JITNN_HIP_API int jitnn_hip_block_values(int fmt);
JITNN_HIP_API int jitnn_hip_block_bytes(int fmt);

/* Bytes an [n, k] weight takes, or JITNN_HIP_EINVAL (unknown fmt, n < 1, k < 1, k not a multiple of the block):
 * the check of Tensor.persistent (core/Tensor.java:266-276). */
JITNN_HIP_API long long jitnn_hip_weight_nbytes(int fmt, long long n, long long k);

/* ---- weights ------------------------------------------------------------------------------------ */

/* Copies raw blocks from host memory to HBM unchanged.  Stands in for the upload of a persistent
 * block-quantised storage (Tensor.quantized / Tensor.persistent, core/Tensor.java:249-278; the bytes come
 * from GgufFile.tensor / raw, gguf/GgufFile.java:329-366).  nbytes must equal jitnn_hip_weight_nbytes.
 * Two formats without kernels of their own are rewritten on the way, block by block, into a format that holds exactly
 * the same values - Q5_0 into Q8_0, Q3_K into Q6_K (every dequantised value keeps its bits) - and run on that format's
 * kernels; jitnn_hip_weight_info still reports what was uploaded.  JITNN_HIP_TRANSCODE=0 keeps them as they are. */
JITNN_HIP_API int jitnn_hip_weight_upload(int fmt, const void *blocks_host, long long nbytes, int n, int k, jitnn_hip_weight **out);

/* Wraps blocks that are already in device memory (not copied, not owned: the caller keeps them alive).
 * dev_blocks must be 16-byte aligned. */
JITNN_HIP_API int jitnn_hip_weight_wrap_dev(int fmt, const void *dev_blocks, long long nbytes, int n, int k, jitnn_hip_weight **out);

JITNN_HIP_API int jitnn_hip_weight_free(jitnn_hip_weight *w);

/* Shape and format of a weight; any out pointer may be NULL. */
JITNN_HIP_API int jitnn_hip_weight_info(const jitnn_hip_weight *w, int *fmt, int *n, int *k, long long *nbytes);

/* ---- dequantise --------------------------------------------------------------------------------- */

/* y[i] = value(w, i), i < n*k, bit-identical to the reference's per-value decode:
 * Gguf.dequantize / op gguf_dequantize (core/ops/Gguf.java:68-73,127-133), Quant.dequantize / op
 * dequantize_q8_0 (core/ops/Quant.java:53-60,137-144), Tensor.toFloatArray on block tensors
 * (core/Tensor.java:539-555). */
JITNN_HIP_API int jitnn_hip_dequantize(const jitnn_hip_weight *w, float *y_host);
JITNN_HIP_API int jitnn_hip_dequantize_dev(const jitnn_hip_weight *w, float *y_dev, void *stream);

/* ---- linear ------------------------------------------------------------------------------------- */

/* y = x W^T (+ bias): Gguf.linear (core/ops/Gguf.java:76-98; ops gguf_matvec :136-205 and
 * gguf_dequantize + matmul) and, for Q8_0, F.linearQ8 / Quant.linear (core/F.java:1049-1051,
 * core/ops/Quant.java:66-80,147-187).  rows >= 1; bias may be NULL.
 * Up to 64 rows run the GEMV kernels at FP32-grade accuracy (error ~1e-6 of the largest output): FP32 arithmetic for
 * one and two rows, FP16 hi/lo splits of the activations on the matrix cores for more - 3 to 8 rows in one launch, 9 to
 * 64 rows in one pass over the weights (rows of whole 256-value columns; else in passes of 8); more rows (prefill) run the
 * dequantise-to-LDS MFMA kernel (FP16 operands, FP32 accumulation, error < 2e-3).
 * JITNN_HIP_GEMV_MAX_ROWS in the environment moves the switch. */
JITNN_HIP_API int jitnn_hip_linear(const jitnn_hip_weight *w, const float *x_host, int rows, const float *bias_host, float *y_host);
JITNN_HIP_API int jitnn_hip_linear_dev(const jitnn_hip_weight *w, const float *x_dev, int rows, const float *bias_dev, float *y_dev, void *stream);

/* jitnn_hip_linear_dev for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, same kernels, same results;
 * where jitnn_hip_linear_dev takes the scratch of a many-row launch (FP16 activations in operand order, their row
 * scales, the partial sums of K slices) from a buffer of the calling thread that it may have to allocate or grow, this
 * entry point takes it from a fixed array of jitnn_hip_noalloc_scratch_bytes() (64 MiB) that the library holds on the
 * GPU for the life of the process, and never calls hipMalloc or hipFree.  A call that needs more scratch (roughly
 * rows * k * 2 bytes + up to 8 * rows * n * 4 bytes for launches that split K) fails with JITNN_HIP_EINVAL before
 * anything is enqueued.  Every call on a GPU shares that one array: calls that overlap in time on one GPU (different
 * streams or threads) race on it - keep them on one stream, or order them with events. */
JITNN_HIP_API int jitnn_hip_linear_noalloc_dev(const jitnn_hip_weight *w, const float *x_dev, int rows, const float *bias_dev, float *y_dev,
                                               void *stream);
JITNN_HIP_API long long jitnn_hip_noalloc_scratch_bytes(void);

/* ---- Q8_0 quantiser ----------------------------------------------------------------------------- */

/* FP32 -> Q8_0 blocks (34 bytes per 32 values) with the reference quantiser's arithmetic: F.quantizeQ8 /
 * op quantize_q8_0 (core/F.java:1039-1041, core/ops/Quant.java:42-50,102-118).  numel % 32 == 0. */
JITNN_HIP_API int jitnn_hip_quantize_q8_0(const float *x_host, long long numel, void *blocks_host);
JITNN_HIP_API int jitnn_hip_quantize_q8_0_dev(const float *x_dev, long long numel, void *blocks_dev, void *stream);

/* ---- counters ------------------------------------------------------------------------------------ */

/* Calls and tensor bytes per operator since the library was loaded (or since jitnn_hip_stats_reset), counted the way
 * the reference's telemetry counts an operator's traffic (core/engine/Telemetry.java:222-240, tensorBytes): every input and
 * output tensor once, block-quantised tensors at numel / blockValues * blockBytes - the same "algorithmic bytes" the
 * benchmark divides by time.  Operators: "linear_gemv" (up to 64 rows), "linear_mfma" (more rows), "dequantize",
 * "quantize_q8_0", "llama_decode", "llama_prefill" (the two model steps count their own linears under themselves, not
 * under the linear operators).  Writes up to cap entries and returns the number of operators; thread-safe. */
typedef struct jitnn_hip_stat {
    char name[32];
    long long calls;
    long long tensor_bytes;
} jitnn_hip_stat;
JITNN_HIP_API int jitnn_hip_stats(jitnn_hip_stat *out, int cap);
JITNN_HIP_API int jitnn_hip_stats_reset(void);

/* ---- measurement aid ---------------------------------------------------------------------------- */

/* Streams nbytes of device memory through 128-bit loads and nothing else (the result is discarded): what the
 * device gives a pure read of the same bytes, launch included.  The benchmark prints it beside the GEMV figures;
 * it has no counterpart in the reference. */
JITNN_HIP_API int jitnn_hip_probe_read_dev(const void *dev, long long nbytes, void *stream);
/* The same with the launch shape given: workgroups of 256 threads per CU (1..16), 16-byte loads in flight per lane (1, 2, 4,
 * 8, 16), non-temporal loads or not - the benchmark sweeps these to find what a read of a buffer of that size can reach.
 * jitnn_hip_probe_read_dev uses 8 workgroups per CU with one load in flight each. */
JITNN_HIP_API int jitnn_hip_probe_read_shape_dev(const void *dev, long long nbytes, int workgroups_per_cu, int loads_in_flight, int nontemporal,
                                                 void *stream);

/* ---- device memory for callers that have no HIP binding of their own (the Java side) ------------- */

JITNN_HIP_API int jitnn_hip_malloc(long long nbytes, void **dev);
JITNN_HIP_API int jitnn_hip_free(void *dev);
JITNN_HIP_API int jitnn_hip_memcpy_h2d(void *dev, const void *host, long long nbytes);
JITNN_HIP_API int jitnn_hip_memcpy_d2h(void *host, const void *dev, long long nbytes);

/* ---- GGUF files ------------------------------------------------------------------------------------ */

/* Reader of llama.cpp's model format, versions 2 and 3, with the acceptance rules of GgufFile.open
 * (gguf/GgufFile.java:100-175, parsing :428-572): magic and version, counts that must fit the file, every metadata
 * value type (arrays nested at most 64 deep), general.alignment a power of two (default 32), tensor shapes reversed
 * to outermost-first, every tensor aligned and inside the file; truncated or crafted files give JITNN_HIP_EIO.
 * Needs no device except for jitnn_hip_gguf_tensor_upload. */
typedef struct jitnn_hip_gguf jitnn_hip_gguf;

JITNN_HIP_API int jitnn_hip_gguf_open(const char *path, jitnn_hip_gguf **out);
JITNN_HIP_API int jitnn_hip_gguf_close(jitnn_hip_gguf *f);
/* version(), alignment(), dataOffset() and the sizes of tensorInfos() / metadata() (gguf/GgufFile.java:177-200). */
JITNN_HIP_API int jitnn_hip_gguf_header(const jitnn_hip_gguf *f, int *version, int *alignment, long long *data_offset, long long *tensor_count,
                                        long long *kv_count);
/* All metadata, in file order, as one JSON object in UTF-8 (metadata(), gguf/GgufFile.java:203-206): integers of any
 * width as integers (a uint64 above 2^63-1 reads as negative, as in the reference), float32/float64 as numbers with a
 * fraction or exponent, bool, string, arrays (nested arrays as nested lists).  Copies at most cap bytes including the
 * terminating NUL and returns the full length without it. */
JITNN_HIP_API long long jitnn_hip_gguf_metadata_json(const jitnn_hip_gguf *f, char *buf, long long cap);
/* Name of tensor `index` in file order (NUL-terminated, truncated to cap). */
JITNN_HIP_API int jitnn_hip_gguf_tensor_name(const jitnn_hip_gguf *f, long long index, char *name, int cap);
/* info(name) (gguf/GgufFile.java:319-326, gguf/GgufTensorInfo.java:29-39): ggml type id, shape (outermost first, up to
 * 8 axes), byte offset in the file, byte count (-1 for a type id this reader does not know).  Any out pointer may be
 * NULL.  Unknown name: JITNN_HIP_EINVAL. */
JITNN_HIP_API int jitnn_hip_gguf_tensor_info(const jitnn_hip_gguf *f, const char *name, int *ggml_type, int *ndims, long long *dims,
                                             long long *file_offset, long long *nbytes);
/* raw(name): the tensor's bytes as stored (gguf/GgufFile.java:358-366).  nbytes must be the tensor's byte count. */
JITNN_HIP_API int jitnn_hip_gguf_tensor_read(const jitnn_hip_gguf *f, const char *name, void *dst_host, long long nbytes);
/* tensor(name) for the block-quantised types of this path (gguf/GgufFile.java:329-346): the blocks go from the
 * mapped file to HBM unchanged; an n-d tensor becomes [numel / last axis, last axis].  Other types:
 * JITNN_HIP_EUNSUPPORTED. */
JITNN_HIP_API int jitnn_hip_gguf_tensor_upload(const jitnn_hip_gguf *f, const char *name, jitnn_hip_weight **out);

/* ---- Llama-style decode step on quantised weights (BASELINE config 5) ----------------------------- */

/* The reference has no quantised Llama and no KV-cache operator; the step is the composition of its operators as
 * Llama.Block.forward defines it (jitnn-nn/src/main/java/ai/beestream/jitnn/nn/models/Llama.java:167-174,209-222)
 * with every Linear replaced by the quantised linear above and attention of the one new token over an FP32
 * cache: RMSNorm (core/ops/RowNorm.java:286-306), rotary embedding in the rotate-half form
 * (core/ops/Rope.java:86-150), grouped-query attention (core/F.java:588-624, core/ops/FlashAttention.java:538-626),
 * SwiGLU (core/F.java:1159-1161), residual adds.  Activations stay in HBM for the whole step. */
typedef struct jitnn_hip_llama jitnn_hip_llama;

#define JITNN_HIP_W_ATTN_Q 0
#define JITNN_HIP_W_ATTN_K 1
#define JITNN_HIP_W_ATTN_V 2
#define JITNN_HIP_W_ATTN_O 3
#define JITNN_HIP_W_FFN_GATE 4
#define JITNN_HIP_W_FFN_UP 5
#define JITNN_HIP_W_FFN_DOWN 6
#define JITNN_HIP_W_OUTPUT 7 /* layer argument ignored */

#define JITNN_HIP_NORM_ATTN 0
#define JITNN_HIP_NORM_FFN 1
#define JITNN_HIP_NORM_OUTPUT 2 /* layer argument ignored */

/* head_dim must be 64, 128, 192 or 256; heads a multiple of kv_heads.  Allocates the KV cache
 * (2 * layers * max_ctx * kv_heads * head_dim floats) and the activation buffers. */
JITNN_HIP_API int jitnn_hip_llama_create(int layers, int d_model, int heads, int kv_heads, int head_dim, int ffn, int vocab, int max_ctx,
                                         float rms_eps, float rope_theta, jitnn_hip_llama **out);
JITNN_HIP_API int jitnn_hip_llama_free(jitnn_hip_llama *m);

/* Attaches a weight (not owned; shapes are checked: q/o [heads*head_dim, d_model] resp. [d_model, heads*head_dim],
 * k/v [kv_heads*head_dim, d_model], gate/up [ffn, d_model], down [d_model, ffn], output [vocab, d_model]). */
JITNN_HIP_API int jitnn_hip_llama_set_weight(jitnn_hip_llama *m, int layer, int which, const jitnn_hip_weight *w);
/* Copies an RMSNorm weight vector [d_model] from host memory. */
JITNN_HIP_API int jitnn_hip_llama_set_norm(jitnn_hip_llama *m, int layer, int which, const float *w_host);

/* Writes / reads `count` cache positions from pos0 of one layer: k and v are [count, kv_heads, head_dim] in host
 * memory (keys as stored, i.e. already rotated). */
JITNN_HIP_API int jitnn_hip_llama_kv_write(jitnn_hip_llama *m, int layer, int pos0, int count, const float *k_host, const float *v_host);
JITNN_HIP_API int jitnn_hip_llama_kv_read(const jitnn_hip_llama *m, int layer, int pos0, int count, float *k_host, float *v_host);

/* One token: x [d_model] is the token's embedding, pos its position (the cache must hold positions 0..pos-1);
 * appends the token's keys and values at pos and writes logits [vocab].  _dev only enqueues on the stream and
 * allocates nothing, so it can be captured into a HIP graph. */
JITNN_HIP_API int jitnn_hip_llama_decode(jitnn_hip_llama *m, const float *x_host, int pos, float *logits_host);
JITNN_HIP_API int jitnn_hip_llama_decode_dev(jitnn_hip_llama *m, const float *x_dev, int pos, float *logits_dev, void *stream);

/* Many tokens at once (the prompt): x [tokens, d_model] are the embeddings of the tokens at positions pos0 ..
 * pos0 + tokens - 1 (the cache must hold positions 0..pos0-1); every layer runs its linears on all rows (more than 64
 * rows: the matrix-core path of jitnn_hip_linear_dev), attention is causal; appends all keys and values and writes the
 * logits [vocab] of the last token (logits may be NULL).  Same arithmetic per token as jitnn_hip_llama_decode, i.e.
 * Llama.Block.forward (jitnn-nn/.../nn/models/Llama.java:209-222) on a [1, tokens, d_model] input.  The first call, and
 * any call with more tokens than every call before, allocates the model's many-token buffers (so it is not for HIP
 * graph capture). */
JITNN_HIP_API int jitnn_hip_llama_prefill(jitnn_hip_llama *m, const float *x_host, int pos0, int tokens, float *logits_host);
JITNN_HIP_API int jitnn_hip_llama_prefill_dev(jitnn_hip_llama *m, const float *x_dev, int pos0, int tokens, float *logits_dev, void *stream);

/* ---- generation loop ------------------------------------------------------------------------------------------------ */

/* Text generation from a GGUF model is jitnn-llm's Llm.generate (jitnn-llm/src/main/java/ai/beestream/jitnn/llm/Llm.java:64-93),
 * which hands the work to the third-party jitllm engine: tokenizer, embedding lookup, the layers over a KV cache, greedy
 * choice of the next token (temperature 0, Llm.java:74-76).  Here the model side of that loop runs on the quantised decode
 * step above; the tokenizer stays with the host (jitnn_amd/llm.py reads it from the file's metadata). */

/* Pairing of the rotary embedding: 0 (default) rotates pairs (i, i + head_dim / 2), 1 pairs (2i, 2i + 1) - the two forms of
 * Rope (core/ops/Rope.java:126-150, `interleaved`).  GGUF files of the "llama" architecture hold q and k weights permuted
 * for the interleaved form. */
JITNN_HIP_API int jitnn_hip_llama_set_rope_interleaved(jitnn_hip_llama *m, int interleaved);

/* The token embedding table [vocab, d_model] (token_embd.weight) in ggml type F32 (0), F16 (1) or a block format, copied
 * to HBM as it is; a token's embedding is its row, dequantised bit-exactly (F.embedding on the dequantised table). */
JITNN_HIP_API int jitnn_hip_llama_set_embedding(jitnn_hip_llama *m, int ggml_type, const void *table_host, long long nbytes);

/* x [count, d_model] = embedding rows of `count` token ids in device memory.  The ids are the caller's: one outside
 * [0, vocab) reads nothing and gives a row of NaN. */
JITNN_HIP_API int jitnn_hip_llama_embed_dev(jitnn_hip_llama *m, const int *tokens_dev, int count, float *x_dev, void *stream);

/* *token_dev = index of the largest of the model's `vocab` logits (the lowest index among equal ones). */
JITNN_HIP_API int jitnn_hip_llama_argmax_dev(jitnn_hip_llama *m, const float *logits_dev, int *token_dev, void *stream);

/* Greedy continuation of a prompt: the prompt's tokens run through the layers at positions pos0 .. (one call, as
 * jitnn_hip_llama_prefill), then tokens are chosen and fed back one at a time until max_new_tokens were produced or
 * eos_token (-1: none) was chosen.  Each new token is written to out_tokens and, when on_token is not NULL, passed to it
 * as soon as it exists.  Returns the number of tokens produced (>= 0) or a negative error code.  Synchronous. */
JITNN_HIP_API int jitnn_hip_llama_generate(jitnn_hip_llama *m, const int *prompt, int prompt_tokens, int pos0, int max_new_tokens, int eos_token,
                                           int *out_tokens, void (*on_token)(int token, void *user), void *user);

#ifdef __cplusplus
}
#endif
#endif /* JITNN_HIP_H */
