/*
 * mfq_runtime_c.h -- flat C view of the C++ host runtime (libmfq_runtime.so), for language bindings
 * and tests.  The C++ API itself is tyloquant_amd/cpp_runtime/mfq_runtime.h; the kernel-level
 * drop-in boundary is mfq_hip.h.  Every call returns 0 on success; mfq_rt_last_error() holds the
 * message of the last failure on the calling thread.  Pointers named x / y / out are device pointers.
 */
#ifndef MFQ_RUNTIME_C_H
#define MFQ_RUNTIME_C_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char *mfq_rt_last_error(void);

/* load_quant_linear (cpp_runtime/mfq_decode.cpp:9489-9771): host blob + MFQ dtype string -> device weight. */
int mfq_rt_load_quant_linear(const char *dtype, const void *blob, size_t n, void **handle);
void mfq_rt_free_quant_linear(void *handle);
int64_t mfq_rt_linear_out(void *handle);
int64_t mfq_rt_linear_neuron_len(void *handle);
/* QuantLinear::forward (cpp_runtime/mfq_decode.cpp:9209-9226): y[M, out] fp32 = x[M, K] . W^T. */
/* Grows the weight's workspace for every batch of 1 .. max_M rows: after it, mfq_rt_linear_forward of such a batch neither
 * frees nor allocates device memory (needed before capturing the call into a HIP graph). */
int mfq_rt_linear_reserve(void *handle, int max_M);
int mfq_rt_linear_forward(void *handle, const void *x, int x_dtype, int64_t ldx, int M, float *y, void *stream);
int mfq_rt_linear_dequantize(void *handle, float *out, void *stream);
/* QuantLinear::forward_swiglu / nint_matmul_geglu (cpp_runtime/mfq_decode.cpp:9228-9240, 8462-8485) on a NINT gate/up
 * tensor [2 W, K]: hidden fp16 [M, W] = act(gate x) * (up x), act = SiLU or (gelu != 0) the tanh GELU.  One launch for one
 * or two rows and for the prefill batches the block-tiled kernel takes; otherwise the matmul goes through `scratch`
 * (fp32 [M, 2 W], may be null when the fused forms apply). */
int mfq_rt_linear_forward_glu(void *handle, const void *x, int x_dtype, int64_t ldx, int M, int gelu, void *hidden,
                              float *scratch, void *stream);
/* embed_forward (cpp_runtime/mfq_decode.cpp:13929-13957) on a NINT, NINT8-0 or NVQ table: out [n_ids, K] of out_dtype
 * (MFQ_X_*), ids device int64, rows of ids outside the table are zero; NEPQ and MX tables are refused, as there.  And
 * next_token_from_hidden (:14107-14130): token[m] device int64, logits fp32 [M, out] or null; fails on a handle that does
 * not hold a NINT tensor. */
int mfq_rt_linear_embedding(void *handle, const int64_t *ids, int n_ids, void *out, int out_dtype, void *stream);
int mfq_rt_linear_argmax(void *handle, const void *x, int x_dtype, int64_t ldx, int M, int64_t *token, float *logits,
                         void *stream);
/* run_linear_check (cpp_runtime/mfq_decode.cpp:16510-16638): out6 = production_ms, production_weight_gbps,
 * payload_gbps, production_rel, production_mean_abs, production_max_abs. */
int mfq_rt_linear_check(void *handle, int M, int reps, double *out6);

/* nvq_ffn_swiglu_down (cpp_runtime/mfq_decode.cpp:8032-8071): y[M, out(down)] = down(silu(gate x) * up x) for three
 * NVQ linears loaded with mfq_rt_load_quant_linear.  The hidden rows live in buffers of this call, so it
 * allocates and synchronises the stream before returning (not capturable; the C++ API takes caller buffers). */
int mfq_rt_nvq_ffn_swiglu_down(void *gate, void *up, void *down, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                               void *stream);

/* An MFQ1 file or shard set as one record table over read-only mappings (MfqFile, cpp_runtime/mfq_decode.cpp:1294-1527;
 * open_mmap, mfq/formats/io.py:834-965).  `path` may name any shard of a set (<stem>-NNNNN-of-NNNNN.mfq).
 * tensor_overlay / expert_overlay: NULL or "" take the environment variables MFQ_TENSOR_OVERLAY / MFQ_EXPERT_OVERLAY as
 * the reference does, "-" takes none.  Records come in file order, shard after shard; `data` points into the mapping
 * and stays valid until mfq_rt_file_close.  These calls need no GPU, except mfq_rt_file_load_quant_linear, which hands
 * the mapped bytes to mfq_rt_load_quant_linear's loader. */
int mfq_rt_file_open(const char *path, const char *tensor_overlay, const char *expert_overlay, void **handle);
void mfq_rt_file_close(void *handle);
int64_t mfq_rt_file_record_count(void *handle);
int64_t mfq_rt_file_tensor_count(void *handle);
int64_t mfq_rt_file_source_count(void *handle);
const char *mfq_rt_file_arch(void *handle);
const char *mfq_rt_file_extra(void *handle, const char *key); /* JSON text of a metadata value of the first shard, or NULL */
int mfq_rt_file_record(void *handle, int64_t index, const char **name, const char **dtype, int *source,
                       const void **data, size_t *nbytes);
int mfq_rt_file_find(void *handle, const char *name, int64_t *index);
int mfq_rt_file_load_quant_linear(void *handle, const char *name, void **linear);

/* NINTM expert-wise tensors and nint_moe_ffn_forward (cpp_runtime/mfq_decode.cpp:3394-3416). */
int mfq_rt_load_nint_moe(const void *blob, size_t n, void **handle);
/* The same with the tensor's NINTMD record from an expert overlay file (MFQ_EXPERT_OVERLAY, mfq_rt_file_open): the
 * overlay's cohorts are appended and own the experts they list (load_nint_moe_cpu, cpp_runtime/mfq_decode.cpp:5752-5774). */
int mfq_rt_load_nint_moe_overlay(const void *blob, size_t n, const void *overlay, size_t overlay_n, void **handle);
void mfq_rt_free_nint_moe(void *handle);
int mfq_rt_moe_ffn_forward(void *gate_up, void *down, const void *x, int x_dtype, int64_t ldx, int T,
                           const float *router_logits, int top_k, int topk_mode, int normalize,
                           void *shared_gate_up, void *shared_down, float *out, int32_t *ids_out,
                           float *weights_out, void *stream);
/* The same with the intermediates in a caller-owned scratch object (MoeFfnScratch): after mfq_rt_moe_scratch_reserve
 * for the largest call, mfq_rt_moe_ffn_forward_scratch neither allocates nor waits for the device, so it may be recorded
 * into a HIP graph (the reference's plan / forward allocate nothing under capture either,
 * cpp_runtime/mfq_decode.cpp:2681-2708, 3008-3016).  The selected experts and their weights of the last call stay in
 * the scratch: mfq_rt_moe_scratch_topk returns their device addresses (int32 / fp32 [T, top_k]).
 * mfq_rt_moe_ffn_forward above is the convenience form: it builds and frees a scratch of its own per call and
 * therefore waits for the stream before it returns. */
int mfq_rt_moe_scratch_create(void **scratch);
void mfq_rt_moe_scratch_free(void *scratch);
int mfq_rt_moe_scratch_reserve(void *scratch, void *gate_up, void *down, int max_tokens, int top_k,
                               void *shared_gate_up, void *shared_down);
int mfq_rt_moe_scratch_topk(void *scratch, const int32_t **ids, const float **weights);
int mfq_rt_moe_ffn_forward_scratch(void *scratch, void *gate_up, void *down, const void *x, int x_dtype, int64_t ldx,
                                   int T, const float *router_logits, int top_k, int topk_mode, int normalize,
                                   void *shared_gate_up, void *shared_down, float *out, void *stream);

/* Expert residency (MoeExpertCache, cpp_runtime/mfq_decode.cpp:5941-7500): experts of the registered NINTM tensors stay
 * in pinned host memory, the GPU holds budget_bytes worth of expert slots; forward makes the route's experts resident
 * (least recently used slots are reused, one staged copy + one scatter launch) and runs the grouped matmul.
 * ids: device int32 [T, R]; out: device fp32 [T * R, out_per_expert]; stats: hits, misses, evictions, bytes, launches.
 * Sources are owned by their cache. */
int mfq_rt_moe_cache_create(int64_t budget_bytes, void **cache);
void mfq_rt_moe_cache_free(void *cache);
int mfq_rt_moe_cache_register(void *cache, const void *blob, size_t n, int minimum_slots, void **source);
int mfq_rt_moe_cache_finalize(void *cache);
int mfq_rt_moe_cache_forward(void *cache, void *source, const void *x, int x_dtype, int64_t ldx, int routed_input,
                             const int32_t *ids, int T, int R, float *out, void *stream);
int mfq_rt_moe_cache_stats(void *cache, int64_t *out5);

#ifdef __cplusplus
}
#endif
#endif
