/*
 * mfq_hip.h -- C ABI of the MI355X (gfx950) MFQ packed-weight matmul kernels.
 *
 * Every entry point is `extern "C"`, takes plain device pointers and sizes, returns an
 * int status (0 = MFQ_OK) and launches on the stream it is given without synchronising.
 * No entry point allocates device memory: weights are written into caller-owned buffers
 * whose size comes from the *_plan call, and kernels that need scratch take a workspace
 * pointer whose size comes from the matching *_workspace_bytes query.
 * mfq_hip_last_error() returns a thread-local message for the last non-zero status.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the
 * reference tree).  Activations are bf16 or fp16 row-major [M, ldx]; outputs are fp32
 * row-major [M, ldy].
 *
 * Range of the activations.  The kernels multiply in fp16 (the reference's activation type).  fp16 rows are used as
 * given.  bf16 rows of any finite magnitude are taken by
 *   - the NINT batch-1 / batch-2 kernels (GEMV, fused GLU, arg-max, MoE decode; not NINT8-48, whose plain matmul runs on
 *     the streaming matrix-core kernel from one row on) and the NINT kernel for 3 to 16 rows that keeps the activations
 *     in LDS (groups of 32 or 16 weights, K of at most eight steps of 16 groups),
 *   - the NVQ3J kernel for one and two rows with its signed table in LDS, the NVQ kernels behind a MoE decode step on an
 *     NVQ cohort (mfq_hip_nvq_gemv_pairs), the NEPQ1 one-row kernel and the NINT8-0 streaming GEMV (one row; more rows when
 *     the activation rows are not 16-byte aligned),
 *   - the stream-family (E8, d4_1024, 1-bit, NEPQ0) wave-per-neuron kernels up to 16 rows, which multiply in fp32, and
 *     the kernels of the E8 formats whose tables fit the LDS and of NVQ1-L / NVQ1-S / NPQ0-L / NPQ0-S / NEPQ0 (packed dot
 *     products for one and two rows, matrix-core products from three to 192), which take bf16 as it is,
 *   - the MXFP4 / MXFP8 kernels up to 256 rows, whose matrix-core products take bf16 as it is (the weights are exact in
 *     bf16, scale included),
 *   - every prefill kernel:
 * every K-slice of a row (the streaming GEMVs; the whole row in the NINT8-0 GEMV and the prefill kernels) is scaled by a
 * power of two before the conversion and the sums are scaled back, so a row of values near 1e-6 or 1e6 keeps the
 * accuracy of a row near 1; within one slice, elements more than about 2^20 below its largest magnitude lose bits.
 * The streaming matrix-core kernels in between (NINT outside the LDS-resident shapes, NVQ on tables too large for the
 * one-row kernel, NVQ / NEPQ / NINT8-0 from two or three rows to a few hundred) convert bf16 without scaling: there |x|
 * must not exceed 65504 (larger values saturate), and rows whose magnitudes sit below about 1e-3 lose precision to
 * fp16's subnormal range.  A per-slice scale costs those kernels a second pass over their activation fragments, which
 * already are most of their traffic.
 */
#ifndef MFQ_HIP_H
#define MFQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *mfq_stream_t; /* a hipStream_t; NULL = the default stream */

enum { MFQ_OK = 0, MFQ_ERR_INVALID = 1, MFQ_ERR_UNSUPPORTED = 2, MFQ_ERR_LAUNCH = 3, MFQ_ERR_WORKSPACE = 4 };
enum { MFQ_X_BF16 = 0, MFQ_X_F16 = 1, MFQ_X_F32 = 2 /* outputs only, where an entry point says so */ };
/* gate activation of a gated linear unit: act(gate) * up with SiLU (SwiGLU) or the tanh form of GELU (GEGLU); the
 * numbering of mfq_glu_runtime (mfq/kernels/cuda/glu.cuh:18-20) */
enum { MFQ_GLU_SILU = 0, MFQ_GLU_GELU = 1 };

const char *mfq_hip_last_error(void);
int mfq_hip_version(void);
/* The effective launch configuration as text: "cu_count=256 MFQ_GEMV_WAVES=2048 ..." -- the device's compute-unit
 * count and every tuning knob (environment variables, read once per process) consulted so far.  Benchmarks print it
 * next to their numbers.  Thread-local buffer.  No counterpart in the reference, whose MFQ_* overrides are read where
 * they are used (e.g. cpp_runtime/mfq_decode.cpp:8518-8523). */
const char *mfq_hip_config(void);
/* Measurement aid: one launch that only reads `bytes` bytes at `data` (16-byte aligned; every wave requests a
 * contiguous share with 16-byte loads, as the decode kernels do) and stores nothing but a 4-byte checksum word at
 * `sink` when it happens to match a magic value.  Benchmarks time it next to the GEMVs: what it sustains is what the
 * memory system gives a launch of that size, start-up and drain included.  No counterpart in the reference. */
int mfq_hip_read_probe(const void *data, size_t bytes, void *sink, mfq_stream_t stream);
/* Clears `bytes` bytes at `data` (4-byte aligned, a multiple of 4) with a kernel.  For hosts that must not record a
 * memset node into a captured graph; stands in for the zero-initialised outputs of the reference's host code
 * (torch::zeros, e.g. cpp_runtime/mfq_decode.cpp:2998). */
int mfq_hip_fill_zero(void *data, size_t bytes, mfq_stream_t stream);
/* Test and tuning hook: size one-block-per-CU grids for n compute units instead of the device's own count
 * (n <= 0 restores it).  Process-wide; not for production use. */
void mfq_hip_set_cu_count(int n);

/* ------------------------------------------------------------------------------------
 * NINT (neuron-anchored INT).  Device layout: row-blocks of 16 neurons; inside a block
 * the groups of a neuron are spread over 4 lanes, 4 groups per lane per 16-group step,
 * each step stored lane-interleaved so one wave load covers a contiguous span.
 * Replaces NintWeight + to_device_nint (cpp_runtime/mfq_decode.cpp:2101-2165, 2268-2293).
 * ---------------------------------------------------------------------------------- */
typedef struct mfq_nint_desc {
    int32_t bits, sub_bits, gs, out, neuron_len, ng;
    int32_t kind;       /* 1 = paired-field fast unit, 0 = natural-order generic unit */
    int32_t dwords;     /* full dwords of codes per (neuron, group) unit */
    int32_t tail_bytes; /* 0 or 1 extra byte per unit */
    int32_t ngp;        /* groups per neuron padded to a multiple of 16 */
    int32_t nsteps;     /* ngp / 16 */
    int32_t n_rowblocks;
    int64_t step_bytes;     /* bytes of one 16-group step of one row-block */
    int64_t rowblock_bytes; /* nsteps * step_bytes */
    int64_t anchors_off;    /* float ns[16*n_rowblocks] then float nm[16*n_rowblocks] */
    int64_t total_bytes;
    int64_t payload_bytes;  /* compact MFQ payload (anchors + 3 bit streams), for GB/s accounting */
} mfq_nint_desc;

/* Fills `d` for a tensor of `out` neurons of length `neuron_len`. */
int mfq_hip_nint_plan(int bits, int sub_bits, int gs, int out, int neuron_len, mfq_nint_desc *d);

/* Load-time repack: `payload` is the device copy of the NINT blob body as pack_nint wrote
 * it (mfq/formats/io.py:191-203) after the header: ns f16[out], nm f16[out], then the
 * sub_scale, sub_min and q little-endian bit streams.  `legacy_bytes` != 0 selects the
 * one-byte-per-value tail accepted by unpack_nint (mfq/formats/io.py:223-232). */
int mfq_hip_nint_repack(const mfq_nint_desc *d, const void *payload, int64_t payload_bytes,
                        int legacy_bytes, void *weight, mfq_stream_t stream);

/* Bit-exact CPU-dequantizer twin: W[out, neuron_len] fp32 with the four separate roundings
 * of nint_quant.dequantize (mfq/quantize/nint_quant.py:896-908); replaces
 * nint_dequant_full_packed_compact_bits_cuda (cpp_runtime/mfq_decode.cpp:396-404). */
int mfq_hip_nint_dequant_f32(const mfq_nint_desc *d, const void *weight, float *w_out, int64_t ld,
                             mfq_stream_t stream);

/* y[M, out] = x[M, neuron_len] . W^T, fp32 accumulate, streaming the packed weights: once for M = 1,
 * once per 16 rows on the matrix cores for larger M (needs neuron_len % 8 == 0, ldx % 8 == 0 and a
 * 16-byte aligned x; otherwise once per 4 rows on the vector ALUs).  Any M >= 1 is valid.  Replaces
 * nint_gemv_packed_ws_cuda / nint_gemv_packed_bits_ws_cuda (cpp_runtime/mfq_decode.cpp:421-435). */
int mfq_hip_nint_gemv(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                      int64_t ldx, int M, float *y, int64_t ldy, mfq_stream_t stream);

/* Decode gate/up projection with the SwiGLU fused: the tensor holds W gate neurons, then W up neurons (out = 2 W,
 * W a multiple of 16); hidden[m, c] = silu(y[m, c]) * y[m, W + c] as bf16 / fp16 (out_dtype, MFQ_X_*), y as in
 * mfq_hip_nint_gemv, M = 1 or 2.  Replaces nint_gemv_packed_swiglu_ws_cuda (cpp_runtime/mfq_decode.cpp:393-396).
 * MFQ_ERR_UNSUPPORTED for M > 2 and for profiles without a unit: run mfq_hip_nint_gemm + mfq_hip_moe_swiglu then. */
int mfq_hip_nint_gemv_swiglu(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                             int64_t ldx, int M, void *hidden, int out_dtype, int64_t ldh, mfq_stream_t stream);
/* The same with the gate activation chosen by `activation` (MFQ_GLU_*): MFQ_GLU_GELU gives
 * hidden[m, c] = gelu_tanh(y[m, c]) * y[m, W + c] and replaces nint_gemv_packed_geglu_ws_cuda /
 * nint_gemv_packed_bits_geglu_ws_cuda (cpp_runtime/mfq_decode.cpp:397-400, 448-451; called by nint_matmul_geglu
 * :8462-8485).  mfq_hip_nint_gemv_swiglu is this call with MFQ_GLU_SILU. */
int mfq_hip_nint_gemv_glu(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                          int64_t ldx, int M, void *hidden, int out_dtype, int64_t ldh, int activation,
                          mfq_stream_t stream);
/* Prefill counterpart: the gate/up projection of M activation rows with the GLU in the matmul's epilogue, for the
 * batches mfq_hip_nint_gemm runs on its block-tiled kernel in one pass over K.  hidden[m, c] = act(y[m, c]) * y[m, W + c]
 * in 16 bits (out_dtype, MFQ_X_*), y as mfq_hip_nint_gemm gives it; the [M, 2 W] fp32 intermediate is never stored.
 * Replaces nint_matmul followed by mfq_swiglu / the GeGLU kernel in FFN::forward_impl for M > 1
 * (cpp_runtime/mfq_decode.cpp:11199-11209).  workspace: mfq_hip_nint_gemm_workspace_bytes(d, M) bytes.
 * MFQ_ERR_UNSUPPORTED (nothing launched) for batches and profiles outside that kernel: run mfq_hip_nint_gemm +
 * mfq_hip_moe_glu then.  Equal to those two calls up to the rounding of the fp32 product to 16 bits. */
int mfq_hip_nint_gemm_glu(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                          int activation, void *hidden, int out_dtype, int64_t ldh, void *workspace,
                          size_t workspace_bytes, mfq_stream_t stream);

/* Decode feed-forward block in ONE launch, one activation row: hidden = act(gate x) * (up x) as fp16, y = down hidden
 * (fp32 [down.out]).  gate_up is the [2 W, H] gate/up tensor (gate rows first), down the [N, W] tensor of the same
 * NINT profile; activation is MFQ_GLU_*.  One block per compute unit, all resident; the hidden vector crosses the
 * chip behind a grid-wide barrier while the down weights are already streaming, so the second launch's ramp is gone.
 * Replaces the batch-1 branch of FFN::forward_impl, gate_up.forward_swiglu(x) followed by down.forward(act)
 * (cpp_runtime/mfq_decode.cpp:11199-11209), and its opt-in fused pair nint_ffn_gate_up_swiglu_quant_ws_cuda +
 * nint_matmul_qx (:11176-11198).  Same values as mfq_hip_nint_gemv_glu (fp16 out) + mfq_hip_nint_gemv up to the order
 * of the fp32 sums over K.  The workspace (size from the query; 0 = this pair of tensors is outside the kernel, as is
 * MFQ_ERR_UNSUPPORTED from the call: run the two launches then) holds the barrier words and the hidden vector; its
 * first 4096 bytes (one barrier flag per compute unit) must be zero before the first call
 * (mfq_hip_nint_ffn_decode_workspace_init, or any memset) and belong to the library from then on: every call advances
 * all flags by one.  Calls that share a workspace must not overlap, and a workspace stays with one device.
 * Contract of the barrier: (1) the launch needs the device to itself -- every block waits for all the others, so all
 * of them have to be running at once; the call refuses a grid that the device's real compute units cannot hold
 * (mfq_hip_set_cu_count above the device's count), but it cannot know of kernels on other streams or of other
 * processes that keep compute units busy; (2) all flags of a workspace hold the same value between calls, so a
 * workspace is used with one grid size: after mfq_hip_set_cu_count changes it, call ..._workspace_init again.
 * When the blocks do not all run at once the barrier gives up after a bounded number of polls, y is NaN and the error
 * word behind the flags is set; nothing hangs.  mfq_hip_nint_ffn_decode_status waits for the stream, returns MFQ_OK
 * when no barrier of the calls since the last check gave up, else resets the workspace and returns MFQ_ERR_LAUNCH
 * (run the two launches then).  No counterpart in the reference (it has no grid barrier). */
size_t mfq_hip_nint_ffn_decode_workspace_bytes(const mfq_nint_desc *gate_up, const mfq_nint_desc *down);
int mfq_hip_nint_ffn_decode_workspace_init(void *workspace, mfq_stream_t stream);
int mfq_hip_nint_ffn_decode_status(void *workspace, mfq_stream_t stream);
int mfq_hip_nint_ffn_decode(const mfq_nint_desc *gate_up, const void *gate_up_weight, const mfq_nint_desc *down,
                            const void *down_weight, const void *x, int x_dtype, int activation, float *y,
                            void *workspace, size_t workspace_bytes, mfq_stream_t stream);

/* Token-embedding rows from the packed table: out[n, 0:neuron_len] = row ids[n] of the dequantized tensor (the
 * values of mfq_hip_nint_dequant_f32, rounded once more to out_dtype: MFQ_X_BF16, MFQ_X_F16 or MFQ_X_F32); ids
 * outside [0, out) give a row of zeros.  ids are device int64.  Replaces
 * nint_embedding_lookup_packed_compact_cuda / nint_embedding_lookup_packed_compact_bits_cuda
 * (cpp_runtime/mfq_decode.cpp:358-365, called at :13929-13957; kernels mfq/kernels/cuda/embedding.cu:117-187). */
int mfq_hip_nint_embedding(const mfq_nint_desc *d, const void *weight, const int64_t *ids, int n_ids,
                           void *out, int out_dtype, int64_t ldo, mfq_stream_t stream);

/* Input gate of a projection: out[m, k] = x[m, k] * act(gate[m, k]) with act = SiLU (mode 0) or the logistic
 * function (mode 1), the numbering of nint_matmul_input_mul (cpp_runtime/mfq_decode.cpp:8395-8417); x, gate and out
 * are bf16 or fp16 (x_dtype) [M, K] with row strides ldx / ldg / ldo, the product is formed in fp32 and rounded once.
 * Followed by mfq_hip_nint_gemv / mfq_hip_nint_gemm on `out` it replaces nint_gemv_packed_gate_ws_cuda /
 * nint_gemv_packed_bits_gate_ws_cuda (:389-392, :488-491) for the batches mfq_hip_nint_gemv_gate leaves out, and is
 * the reference's own unfused form nint_matmul(w, x * silu(gate)) (:8415-8416). */
int mfq_hip_input_gate(const void *x, const void *gate, int x_dtype, int64_t ldx, int64_t ldg, int M, int K,
                       int mode, void *out, int64_t ldo, mfq_stream_t stream);

/* y[m, :] = (x[m, :] * act(gate[m, :])) . W^T in one launch for M = 1 or 2: the batch-1 GEMV whose waves fetch their
 * slice of the gate row next to the activations and stage the product (fp32, rounded once to x_dtype as
 * mfq_hip_input_gate rounds it).  mode as above.  MFQ_ERR_UNSUPPORTED for M > 2, rows that are not 16-byte aligned,
 * neuron_len % 8 != 0 or neurons too long for one block: run mfq_hip_input_gate + mfq_hip_nint_gemm then.  Replaces
 * nint_gemv_packed_gate_ws_cuda / nint_gemv_packed_bits_gate_ws_cuda (cpp_runtime/mfq_decode.cpp:389-392, 488-491,
 * called at :8404-8413). */
int mfq_hip_nint_gemv_gate(const mfq_nint_desc *d, const void *weight, const void *x, const void *gate,
                           int x_dtype, int64_t ldx, int64_t ldg, int M, int mode, float *y, int64_t ldy,
                           mfq_stream_t stream);

/* LM head for greedy decoding: token[m] = argmax_n y[m, n] with y as in mfq_hip_nint_gemv (equal logits go to the
 * lower index, NaN never wins, -1 when every logit is NaN).  M = 1 on NINT4-32, NINT4-24, NINT3-24 and NINT5-28
 * takes one GEMV launch whose blocks emit their winners, and a one-block final pass; other profiles and M > 1
 * run the GEMV into the logits and reduce them in two passes.  logits (float [M, ldl]) may be null; when given
 * it receives y.  token is device int64 [M].  The workspace holds the per-block winners (and the logits when
 * none are passed).  Replaces nint_gemv_packed_bits_argmax_ws_cuda (cpp_runtime/mfq_decode.cpp:464-468, called
 * at :14116-14129; reduction mfq/kernels/cuda/nint_matmul.cu:2300-2350). */
size_t mfq_hip_nint_gemv_argmax_workspace_bytes(const mfq_nint_desc *d, int M);
int mfq_hip_nint_gemv_argmax(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                             int64_t ldx, int M, float *logits, int64_t ldl, int64_t *token,
                             void *workspace, size_t workspace_bytes, mfq_stream_t stream);

/* mfq_hip_nint_gemv_argmax for callers that cannot allocate device memory or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation): the scratch is a 4 MiB device array built into the
 * library (one copy per GPU, held until the process ends).  No counterpart in the reference.  Same arguments and
 * results as mfq_hip_nint_gemv_argmax without the workspace pair; MFQ_ERR_WORKSPACE when
 * mfq_hip_nint_gemv_argmax_workspace_bytes(d, M) exceeds 4 MiB (M = 1 fits any vocabulary up to about 900k; with
 * logits passed in, far more).  Allocates nothing and frees nothing.  The first use on a device looks the array's
 * address up (hipGetSymbolAddress, which may load the code object): that must not happen while a stream is being
 * captured, so before capturing call mfq_hip_nint_gemv_argmax_static_init once per device with that device current
 * (or make one eager call); it launches nothing and is cheap to repeat.  All calls on one GPU share the array: calls
 * that overlap on one GPU (two streams, two threads) race, and so do overlapping replays of graphs that hold one. */
int mfq_hip_nint_gemv_argmax_static_init(void);
int mfq_hip_nint_gemv_argmax_static(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                                    int64_t ldx, int M, float *logits, int64_t ldl, int64_t *token,
                                    mfq_stream_t stream);

/* Any-M entry: the streaming kernels of mfq_hip_nint_gemv up to a crossover that depends on the tensor (32 to
 * 512 rows; 256 for profiles without a prefill kernel), above that a block-tiled MFMA GEMM with in-register
 * dequantization (the paired profiles and NINT5-28) or dequantize-to-fp16 + MFMA GEMM.  The workspace (size
 * from the query, 0 when none is needed) holds fp16 activations, group sums and the partial results of a split
 * over K, or, for the second case, fp16 activations and weights.  Replaces nint_mmq_f16_packed_cuda / nint_mmq_f32_packed_cuda and the dequant + cuBLAS fallback
 * (cpp_runtime/mfq_decode.cpp:480-520, 8309-8314). */
size_t mfq_hip_nint_gemm_workspace_bytes(const mfq_nint_desc *d, int M);
int mfq_hip_nint_gemm(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                      int64_t ldx, int M, float *y, int64_t ldy, void *workspace,
                      size_t workspace_bytes, mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * NINT8-0: GGML Q8_0 blocks (fp16 scale + 32 signed 8-bit codes, weight = scale * code; mfq/formats/nint8_zero.py)
 * under the dtype string "NINT8-0".  Replaces Nint8ZeroCpu + to_device_nint8_zero
 * (cpp_runtime/mfq_decode.cpp:1591-1650, 2309-2330) and the q8_zero branch of nint_matmul (:8165-8185).
 * ---------------------------------------------------------------------------------- */
typedef struct mfq_nint8z_desc {
    int32_t out, neuron_len, ng;   /* ng = neuron_len / 32 */
    int32_t reserved;
    int64_t scales_off;            /* fp16 [out][ng] */
    int64_t codes_off;             /* int8 [out][neuron_len] */
    int64_t total_bytes;
    int64_t payload_bytes;         /* out * ng * 34: the blocks of the file */
} mfq_nint8z_desc;

/* MFQ_ERR_INVALID unless neuron_len is a positive multiple of 32 (the format's rule). */
int mfq_hip_nint8z_plan(int out, int neuron_len, mfq_nint8z_desc *d);
/* `blocks` = device copy of the out * ng 34-byte blocks that follow the blob header; splits them into the
 * device layout.  Replaces the block loop of unpack_nint8_zero (cpp_runtime/mfq_decode.cpp:1640-1648). */
int mfq_hip_nint8z_repack(const mfq_nint8z_desc *d, const void *blocks, int64_t block_bytes, void *weight,
                          mfq_stream_t stream);
/* w_out[out, ld] = f32(scale) * f32(code), bit-exact with dequantize_nint8_zero (mfq/formats/nint8_zero.py:208-218)
 * and nint8_zero_dequant_cuda (cpp_runtime/mfq_decode.cpp:8180-8182). */
int mfq_hip_nint8z_dequant_f32(const mfq_nint8z_desc *d, const void *weight, float *w_out, int64_t ld,
                               mfq_stream_t stream);
/* Token-embedding rows: out[n, 0:neuron_len] = row ids[n] of mfq_hip_nint8z_dequant_f32 rounded once to out_dtype
 * (MFQ_X_BF16, MFQ_X_F16 or MFQ_X_F32); ids (device int64) outside [0, out) give a row of zeros.  Replaces
 * nint8_zero_embedding_lookup_cuda (cpp_runtime/mfq_decode.cpp:366-370, called at :13943-13947; kernel
 * mfq/kernels/cuda/embedding.cu:190-220). */
int mfq_hip_nint8z_embedding(const mfq_nint8z_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                             int out_dtype, int64_t ldo, mfq_stream_t stream);
/* mfq_hip_nvq_gemv_pairs (below) for a cohort of NINT8-0 experts that are tensors of their own: the pairs of a MoE
 * decode step in one launch, the routing table read on the device. */
int mfq_hip_nint8z_gemv_pairs(const mfq_nint8z_desc *d, const void *const *expert_weights, const int32_t *expert_slot, int E,
                              const void *x, int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                              float *y, int64_t ldy, mfq_stream_t stream);
/* y[M, out] = x[M, neuron_len] . W^T streaming the codes once per pass of up to 8 rows (fewer when the fp16
 * activations of a pass would not fit 64 KB of LDS; MFQ_ERR_UNSUPPORTED when one row does not).  Replaces
 * nint8_zero_gemv_ws_cuda / nint8_zero_mmq_ws_cuda (cpp_runtime/mfq_decode.cpp:8167-8177). */
int mfq_hip_nint8z_gemv(const mfq_nint8z_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                        int M, float *y, int64_t ldy, mfq_stream_t stream);
/* Any M: the streaming kernel up to 32 rows, above that dequantize to fp16 (power-of-two row scales) + the dense
 * fp16 MFMA GEMM in the workspace (size from the query; 0 when none is needed).  Replaces the
 * nint8_zero_dequant_cuda + matmul fallback (cpp_runtime/mfq_decode.cpp:8179-8185). */
size_t mfq_hip_nint8z_gemm_workspace_bytes(const mfq_nint8z_desc *d, int M);
int mfq_hip_nint8z_gemm(const mfq_nint8z_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                        int M, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                        mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * NVQ-JSC, D4 family (NVQ3J = d4_256, NVQ3J-512 = d4_512; plain NVQ3 maps onto the
 * analytic one-bank tables).  Replaces NvqWeight + to_device_nvq
 * (cpp_runtime/mfq_decode.cpp:4019-4150).
 * ---------------------------------------------------------------------------------- */
typedef struct mfq_nvq_desc {
    int32_t index_bits, entries, banks, out, neuron_len, ng, nvec, nsign;
    int32_t ngp, nsteps, n_rowblocks;
    int64_t step_bytes, rowblock_bytes;
    int64_t tables_off;  /* float lut[16]; uint32 bank_for_state[16]; uint8 codebooks[banks*entries*4] */
    int64_t anchors_off; /* float anchor[16*n_rowblocks] */
    int64_t total_bytes;
    int64_t payload_bytes; /* anchors + 3 streams + 64-byte JSC header + codebook banks */
} mfq_nvq_desc;

int mfq_hip_nvq_plan(int index_bits, int banks, int out, int neuron_len, mfq_nvq_desc *d);

/* `payload` = device copy of the blob from the 64-byte JSC header on (mfq/formats/nvq.py:644-716):
 * JSC header, codebook banks i8[banks, entries, 4], anchors f16[out], then the 4-bit state,
 * index_bits-bit index and 7-bit sign streams, all tensor-contiguous. */
int mfq_hip_nvq_repack(const mfq_nvq_desc *d, const void *payload, int64_t payload_bytes, void *weight,
                       mfq_stream_t stream);
/* Plain (non-JSC) NVQ3: payload starts at the anchors; `grid` is the device copy of the
 * 256-entry int8 magnitude grid [256, 4]; state doubles as the integer relative scale. */
int mfq_hip_nvq_repack_plain(const mfq_nvq_desc *d, const void *payload, int64_t payload_bytes,
                             const void *grid, void *weight, mfq_stream_t stream);

/* Bit-exact twin of dequantize_nvq_jsc (mfq/quantize/nvq_jsc.py:1053-1079); replaces
 * nvq_dequant_cuda (cpp_runtime/mfq_decode.cpp:540-546). */
int mfq_hip_nvq_dequant_f32(const mfq_nvq_desc *d, const void *weight, float *w_out, int64_t ld,
                            mfq_stream_t stream);
/* Token-embedding rows: out[n, 0:neuron_len] = row ids[n] of mfq_hip_nvq_dequant_f32 rounded once to out_dtype
 * (MFQ_X_BF16, MFQ_X_F16 or MFQ_X_F32; the reference stores fp16); ids (device int64) outside [0, out) give a row of
 * zeros (the reference leaves such rows unwritten).  Replaces nvq_embedding_lookup_cuda
 * (cpp_runtime/mfq_decode.cpp:608, called through nvq_embedding :8072-8079 at :13937-13939; kernel
 * mfq/kernels/cuda/nvq_matmul.cu:1665-1719, launch :6026-6069). */
int mfq_hip_nvq_embedding(const mfq_nvq_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                          int out_dtype, int64_t ldo, mfq_stream_t stream);
/* A MoE decode step on a cohort of NVQ experts that are tensors of their own (one descriptor, one device pointer per
 * expert in the device array expert_weights): y[p, 0:out] = W[ids[p]] . x[p (routed_input) or p / R] for every pair
 * p < T * R whose expert belongs to the cohort -- expert_slot[e] (device, [E]) = index of expert e in expert_weights, -1
 * for the experts of other cohorts and for ids outside [0, E), whose rows are left as they are.  One launch, nothing read
 * back by the host.  Replaces the NVQ arm of the grouped decode kernels, nvq_moe_mmvq_kernel
 * (mfq/kernels/cuda/nvq_matmul.cu:2588-3175; NintMoeWeight::forward's cohort loop, cpp_runtime/mfq_decode.cpp:4800-5360). */
int mfq_hip_nvq_gemv_pairs(const mfq_nvq_desc *d, const void *const *expert_weights, const int32_t *expert_slot, int E,
                           const void *x, int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                           float *y, int64_t ldy, mfq_stream_t stream);
/* Replaces nvq_gemv_ws_cuda (cpp_runtime/mfq_decode.cpp:555-559). */
int mfq_hip_nvq_gemv(const mfq_nvq_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                     int M, float *y, int64_t ldy, mfq_stream_t stream);
/* Two projections of the same activations in one launch: y[m, 0:out0] = x . W0^T, y[m, out0:out0+out1] = x . W1^T
 * (both tensors with the same neuron_len).  Up to 32 rows on tensors the signed-table kernel takes it is one launch
 * whose blocks are shared out over both tensors; otherwise the two mfq_hip_nvq_gemv calls.  Same values as those two
 * calls.  Replaces nvq_gemv_multi2_ws_cuda (called by nvq_matmul_multi2, cpp_runtime/mfq_decode.cpp:7981-8003). */
int mfq_hip_nvq_gemv_multi2(const mfq_nvq_desc *d0, const void *weight0, const mfq_nvq_desc *d1, const void *weight1,
                            const void *x, int x_dtype, int64_t ldx, int M, float *y, int64_t ldy,
                            mfq_stream_t stream);
/* Any-M entry: the streaming kernels of mfq_hip_nvq_gemv up to a crossover of 32 to 512 rows, above that a
 * block-tiled MFMA GEMM that builds the weight fragments from the codebooks (neuron_len % 8 == 0), else
 * dequantize-to-fp16 + MFMA GEMM.  Replaces nvq_mmq_* / nvq_gemm_f16_cuda / dequant + cuBLAS
 * (cpp_runtime/mfq_decode.cpp:561-575, 7928-7931). */
size_t mfq_hip_nvq_gemm_workspace_bytes(const mfq_nvq_desc *d, int M);
int mfq_hip_nvq_gemm(const mfq_nvq_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                     int M, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                     mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * NVQ payloads read in place from their bit streams: the E8 family -- NVQ2 (e8_256, plain, parity or index-parity
 * signs), NVQ2J / NVQ2J-L / NVQ2J-XL (e8_256 / e8_1024 / e8_4096 with JSC state tables and up to four banks) -- and
 * NVQ3J-L (d4_1024), whose 10-bit indices do not fit the lane-major D4 layout above.  Group size 24, 4-bit states.
 * The device weight keeps the payload's three tensor-wide streams (4-bit state, index, 7-bit sign) as they are, with
 * the tables widened in front (float lut[16], uint32 bank_for_state[16], int8 codebooks) and fp32 anchors; fields are
 * fetched by bit offset, a wave per neuron (tables of up to 64 KB -- NVQ2, NVQ2J, NVQ2J-L, one-bank NVQ2J-XL, NVQ3J-L: a wave copies its neurons' bit ranges
 * into LDS and multiplies 24 weights per lane and step, the reference's NVQ2 fast path,
 * mfq/kernels/cuda/nvq_matmul.cu:1378-1420).  Replaces the formats 2, 5, 13, 14 and 15 of unpack_nvq / NvqWeight
 * (cpp_runtime/mfq_decode.cpp:3756-4013, 4019-4150) and their nvq_gemv_ws_cuda / nvq_mmq_* / nvq_dequant_cuda calls
 * (:540-575, 7884-7931).
 * ------------------------------------------------------------------------------------ */
typedef struct mfq_nvqs_desc {
    int32_t vector_size, index_bits, entries, banks, index_parity;
    int32_t out, neuron_len, ng, nvec, nsign;
    int64_t tables_off, anchors_off, state_off, index_off, sign_off;
    int64_t total_bytes;
    int64_t payload_bytes; /* anchors + the streams */
    int32_t kind;          /* 0: the NVQ formats above; 1: NVQ1-L / NVQ1-S; 2: NPQ0-L / NPQ0-S; 3: NEPQ0-S / NEPQ0-L (see below) */
    int32_t state_bits, cb_bytes;
    float delta;
    int32_t nbank, nsuper; /* kind 3 (NEPQ0): tables in the pool, bank ids per neuron (one per 96 weights) */
} mfq_nvqs_desc;

int mfq_hip_nvqs_plan(int vector_size, int index_bits, int banks, int index_parity, int out, int neuron_len,
                      mfq_nvqs_desc *d);
/* `payload` = device copy of the blob from the 64-byte JSC header on (jsc != 0: header, int8 banks
 * [banks, entries, vector_size], fp16 anchors, streams) or from the anchors on (jsc == 0; `grid` is then the device
 * copy of the int8 magnitude grid [entries, vector_size], and the 4-bit state is the integer relative scale). */
int mfq_hip_nvqs_repack(const mfq_nvqs_desc *d, const void *payload, int64_t payload_bytes, int jsc,
                        const void *grid, void *weight, mfq_stream_t stream);
/* Bit-exact twin of dequantize_nvq_jsc (mfq/quantize/nvq_jsc.py:1053-1079) and dequantize_nvq
 * (mfq/quantize/nvq_quant.py:608-626), index-parity sign rule included. */
int mfq_hip_nvqs_dequant_f32(const mfq_nvqs_desc *d, const void *weight, float *w_out, int64_t ld,
                             mfq_stream_t stream);
/* y = x . W^T: up to 16 rows re-read the streams once per eight rows (fp32 accumulation); above that the tensor is
 * dequantized to fp16 in the workspace (size from the query, 0 up to 16 rows) and multiplied on the matrix cores. */
int mfq_hip_nvqs_gemv(const mfq_nvqs_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                      int M, float *y, int64_t ldy, mfq_stream_t stream);
/* The 1-bit families on the same descriptor and the same dequant / gemv / gemm entry points: groups of 24 weights made of
 * three 8-weight vectors, one fp16 anchor per neuron, tensor-wide streams read in place.
 *   NVQ1-L (format 1 of unpack_nvq, cpp_runtime/mfq_decode.cpp:3759, 3805-3810; mfq/formats/nvq1_l.py): 11-bit indices
 *     into a 2048-entry ternary grid (built in, or in the blob), 3- or 4-bit integer relative scale and a delta sign
 *     per group: w = anchor * scale * (code -/+ 1/8).
 *   NVQ1-S (format 8, :3769, 3811-3813; nvq1_s.py): 9-bit indices, two 512-entry ternary banks in the blob chosen by the
 *     group's delta sign, 4-bit scale, delta 5/32.
 *   NPQ0-L / NPQ0-S (formats 7 / 9, :3768-3770, 3845-3910; npq0_l.py, npq0_s.py): a vector is two 4-dimensional int8
 *     sub-vectors, first[state][index & 7] and second[state][index >> 3] (7- / 6-bit indices, 8 / 4 states); the state
 *     also selects the relative scale from an fp16 table: w = code * anchor * lut[state].
 * `body` = device copy of the blob from behind its header, shape and neuron count on: the tables (NVQ1-L with a custom
 * grid: 4096 bytes; NVQ1-S: 2048; NPQ0: 64-byte header + sub-codebooks), fp16 anchors, streams.  `grid` = device copy
 * of the built-in grid as 2048 packed uint16 (needed only for an NVQ1-L body without a table).  The host validates the
 * blob's header and table header before calling. */
#define MFQ_NVQS_NVQ1_L 1
#define MFQ_NVQS_NVQ1_S 2
#define MFQ_NVQS_NPQ0_L 3
#define MFQ_NVQS_NPQ0_S 4
int mfq_hip_nvqs_plan_lowbit(int format, int state_bits, int out, int neuron_len, mfq_nvqs_desc *d);
int mfq_hip_nvqs_repack_lowbit(const mfq_nvqs_desc *d, const void *body, int64_t body_bytes, const void *grid,
                               void *weight, mfq_stream_t stream);
/* NEPQ0-S / NEPQ0-L (profiles 0 / 1 of the NEPQ container, mfq/formats/nepq.py:95-116; formats 9 / 7 with a table pool in
 * the reference's loader, cpp_runtime/mfq_decode.cpp:4198-4260): the product form of NPQ0 on [experts * out_per_expert, K]
 * neurons with a pool of `banks` tables; one bank id byte per neuron and 96 weights picks scale LUT and sub-codebooks
 * (dequantize_nepq, nepq.py:492-521).  `body` = device copy of the blob behind its 36-byte header: tables, fp16 anchors,
 * state and index streams, bank ids.  An expert is the row range [e * out_per_expert, (e + 1) * out_per_expert) of the
 * row-range calls below, which exist for every descriptor kind: y / w_out hold nrows columns / rows. */
int mfq_hip_nvqs_plan_nepq0(int profile, int banks, int rows, int neuron_len, mfq_nvqs_desc *d);
int mfq_hip_nvqs_repack_nepq0(const mfq_nvqs_desc *d, const void *body, int64_t body_bytes, void *weight,
                              mfq_stream_t stream);
int mfq_hip_nvqs_dequant_rows_f32(const mfq_nvqs_desc *d, const void *weight, int row0, int nrows, float *w_out,
                                  int64_t ld, mfq_stream_t stream);
/* Token-embedding rows of the families on this descriptor: the contract of mfq_hip_nvq_embedding over the rows of
 * mfq_hip_nvqs_dequant_f32 (the same reference kernel, nvq_matmul.cu:1665-1719, instantiated per format by
 * launch_by_format, :3344-3371). */
int mfq_hip_nvqs_embedding(const mfq_nvqs_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                           int out_dtype, int64_t ldo, mfq_stream_t stream);
/* mfq_hip_nvq_gemv_pairs for the families on this descriptor.  Either expert_weights (one tensor of out_per_expert rows
 * per expert) or, with expert_weights null, `weight` = one tensor whose rows slot * out_per_expert ... are expert slot's
 * (the NEPQ0 streams). */
int mfq_hip_nvqs_gemv_pairs(const mfq_nvqs_desc *d, const void *const *expert_weights, const void *weight,
                            int out_per_expert, const int32_t *expert_slot, int E, const void *x, int x_dtype, int64_t ldx,
                            int routed_input, const int32_t *ids, int T, int R, float *y, int64_t ldy, mfq_stream_t stream);
int mfq_hip_nvqs_gemv_rows(const mfq_nvqs_desc *d, const void *weight, int row0, int nrows, const void *x, int x_dtype,
                           int64_t ldx, int M, float *y, int64_t ldy, mfq_stream_t stream);
/* Workspace of mfq_hip_nvqs_gemm_rows for M rows: 0 for the batches that run from the bit streams (up to 16 rows, and up
 * to 192 for the tensors whose tables and bit ranges fit the LDS), else the fp16 copies of the weights and activations. */
size_t mfq_hip_nvqs_gemm_rows_workspace_bytes(const mfq_nvqs_desc *d, int nrows, int M);
int mfq_hip_nvqs_gemm_rows(const mfq_nvqs_desc *d, const void *weight, int row0, int nrows, const void *x, int x_dtype,
                           int64_t ldx, int M, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                           mfq_stream_t stream);
size_t mfq_hip_nvqs_gemm_workspace_bytes(const mfq_nvqs_desc *d, int M);
int mfq_hip_nvqs_gemm(const mfq_nvqs_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                      int M, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                      mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * OCP MX weights of full-precision MFQ files (mfq/formats/mx.py:16-117): kind 4 = MXFP4 (E2M1 nibbles, low nibble =
 * even column, one E8M0 scale per 32 columns of a row), kind 8 = MXFP8 (E4M3FN bytes, one E8M0 scale per 128 x 128
 * block).  values / scales: device copies of the payload's two byte matrices as they lie behind its 56-byte header
 * (values [rows, cols / 2] or [rows, cols]; scales [rows, cols / 32] or [ceil(rows / 128), cols / 128]); values
 * 16-byte aligned.  Calls work on the rows [row0, row0 + nrows) -- a whole tensor, or one expert of a pool.
 * mfq_hip_mx_dequant_rows: w_out[r - row0][c] = element * scale, one fp32 multiply (MFQ_X_F32; unpack_mxfp8 /
 * dequant_mxfp4_cpu, cpp_runtime/mfq_decode.cpp:1832-1947, mxfp8_dequant_kernel, mfq/kernels/cuda/mx_matmul.cu:222-240),
 * or that rounded once more to fp16 as the reference's device copy is (MFQ_X_F16); a scale byte 255 and the E4M3FN codes
 * 0x7f / 0xff give NaN.
 * mfq_hip_mx_gemm_rows: y[M, nrows] = x[M, cols] . W^T in fp32 (mxfp8_matmul_f32, mfq_decode.cpp:8784-8802): up to 256
 * rows of x on the matrix cores from the file's bytes (the hardware's FP4 / FP8 conversions with the E8M0 scale in
 * their exponent operand, bf16 or fp16 MFMA by the activations' type; mxfp8_small_m_f32_cuda serves 1..8 rows) when x is
 * 16-byte aligned with ldx % 8 == 0 -- otherwise a wave per neuron, four rows per pass; above 256 rows an fp16 copy of
 * the rows, each relative to its largest scale, and the fp16 MFMA GEMM -- workspace of
 * mfq_hip_mx_gemm_rows_workspace_bytes.  bf16 activations of any magnitude are taken as they are (no fp16 detour). */
int mfq_hip_mx_dequant_rows(int kind, const void *values, const void *scales, int rows, int cols, int row0, int nrows,
                            int out_dtype, void *w_out, int64_t ld, mfq_stream_t stream);
size_t mfq_hip_mx_gemm_rows_workspace_bytes(int cols, int nrows, int M);
int mfq_hip_mx_gemm_rows(int kind, const void *values, const void *scales, int rows, int cols, int row0, int nrows,
                         const void *x, int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, void *workspace,
                         size_t workspace_bytes, mfq_stream_t stream);
/* mfq_hip_nvq_gemv_pairs for a native MXFP4 pool (one [experts * out_per_expert, cols] tensor, expert slot = rows
 * slot * out_per_expert ...): the pairs of a MoE decode step in one launch (the MXFP4 arm of the grouped decode path,
 * cpp_runtime/mfq_decode.cpp:4800-5360). */
int mfq_hip_mx_gemv_pairs(int kind, const void *values, const void *scales, int rows, int cols, int out_per_expert,
                          const int32_t *expert_slot, int E, const void *x, int x_dtype, int64_t ldx, int routed_input,
                          const int32_t *ids, int T, int R, float *y, int64_t ldy, mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * NEPQ1-S / NEPQ1-L (cross-expert table pool, bank id per 96 weights).  Rows are the
 * flattened [experts * out_per_expert] neurons.  Replaces NepqWeight
 * (cpp_runtime/mfq_decode.cpp:4166-4463) and the Python nepq_matmul
 * (mfq/kernels/cuda/nepq_matmul.py:215-280).
 * ---------------------------------------------------------------------------------- */
typedef struct mfq_nepq_desc {
    int32_t profile; /* 2 = NEPQ1-S, 3 = NEPQ1-L */
    int32_t state_bits, index_bits, banks, rows, neuron_len, ng, nvec, nsuper;
    int32_t ngp, nsteps, n_rowblocks, table_entries; /* u16 entries per bank: 1024 (S) / 2048 (L) */
    int64_t step_bytes, rowblock_bytes;
    int64_t tables_off;  /* uint16 table[banks * table_entries] */
    int64_t anchors_off; /* float anchor[16*n_rowblocks] */
    int64_t total_bytes;
    int64_t payload_bytes;
} mfq_nepq_desc;

int mfq_hip_nepq_plan(int profile, int banks, int rows, int neuron_len, mfq_nepq_desc *d);
/* `payload` = device copy of the blob after the 36-byte header (mfq/formats/nepq.py:368-399):
 * tables u8[banks, table_bytes], anchors f16[rows], state / index / aux bit streams, bank ids. */
int mfq_hip_nepq_repack(const mfq_nepq_desc *d, const void *payload, int64_t payload_bytes, void *weight,
                        mfq_stream_t stream);
/* Bit-exact twin of dequantize_nepq (mfq/formats/nepq.py:492-544); replaces nepq_dequant_cuda. */
int mfq_hip_nepq_dequant_f32(const mfq_nepq_desc *d, const void *weight, float *w_out, int64_t ld,
                             mfq_stream_t stream);
/* `row0`, `nrows` select one expert's neurons; replaces nepq_gemv_ws_cuda. */
int mfq_hip_nepq_gemv(const mfq_nepq_desc *d, const void *weight, int row0, int nrows, const void *x,
                      int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, mfq_stream_t stream);
/* mfq_hip_nvq_gemv_pairs for an expert-shaped NEPQ1 tensor: expert slot owns rows slot * out_per_expert ... (a multiple of
 * 16 rows per expert).  Replaces the NEPQ arm of the grouped decode kernels (nvq_matmul.cu:4210-4580). */
int mfq_hip_nepq_gemv_pairs(const mfq_nepq_desc *d, const void *weight, int out_per_expert, const int32_t *expert_slot, int E,
                            const void *x, int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                            float *y, int64_t ldy, mfq_stream_t stream);
/* Any-M entry: mfq_hip_nepq_gemv's kernels up to 32 rows, from 33 rows a block-tiled MFMA GEMM that builds the
 * weight fragments from the ternary tables; replaces nepq_mmq_ws_cuda / nepq_gemm_f16_cuda
 * (mfq/kernels/cuda/mfq_cuda.cpp:331-350). */
size_t mfq_hip_nepq_gemm_workspace_bytes(const mfq_nepq_desc *d, int nrows, int M);
int mfq_hip_nepq_gemm(const mfq_nepq_desc *d, const void *weight, int row0, int nrows, const void *x,
                      int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, void *workspace,
                      size_t workspace_bytes, mfq_stream_t stream);
/* x <- FWHT_block(x * signs) / sqrt(block), fp32 in LDS; replaces nepq_hadamard_input_cuda
 * (mfq/kernels/cuda/nepq.cu:13-55).  `signs` int8[K] (+1/-1), block a power of two <= 4096. */
int mfq_hip_nepq_hadamard(const void *x, int x_dtype, int64_t ldx, int rows, int K, int block,
                          const int8_t *signs, void *x_out, int64_t ldo, mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * MoE routing and the expert-grouped matmul ("mul_mat_id").
 * ---------------------------------------------------------------------------------- */
enum { MFQ_TOPK_SOFTMAX = 0, MFQ_TOPK_SIGMOID = 1, MFQ_TOPK_SQRT_SOFTPLUS = 2, MFQ_TOPK_DELAYED_SOFTMAX = 3 };

/* Replaces moe_topk_cuda (mfq/kernels/cuda/moe.cu:3552-3637): ids int32[T,k], weights f32[T,k];
 * tie -> lower expert id, NaN -> -FLT_MAX, bias (may be NULL) enters the selection score only. */
int mfq_hip_moe_topk(const float *logits, const float *bias, int T, int E, int k, int mode, int normalize,
                     float norm_floor, float scale, int32_t *ids, float *weights, mfq_stream_t stream);

/* Replaces moe_build_expert_map_cuda (mfq/kernels/cuda/moe.cu:3082-3130) with a parallel
 * prefix-sum bucketing.  counts[E], expert_bounds[E+1], tile_bounds[E+1], tile_experts[max_tiles],
 * ids_dst[n_pairs] (pairs grouped by expert, ascending pair index inside an expert: deterministic).
 * max_tiles >= ceil(n_pairs/tile_m) + E.  Pairs with an out-of-range expert id are dropped. */
int mfq_hip_moe_route_map(const int32_t *ids, int n_pairs, int E, int tile_m, int32_t *counts,
                          int32_t *expert_bounds, int32_t *tile_bounds, int32_t *tile_experts,
                          int max_tiles, int32_t *ids_dst, mfq_stream_t stream);

/* One cohort of experts sharing a NINT profile (NintMoePoolWeight,
 * cpp_runtime/mfq_decode.cpp:2350-2365): `weight` holds n_local * out_per_expert neurons. */
typedef struct mfq_moe_pool {
    mfq_nint_desc desc;
    const void *weight;
} mfq_moe_pool;

/* Device tables built once per NINTM tensor (initialize_nint_moe_dispatch,
 * cpp_runtime/mfq_decode.cpp:3249-3343): expert_pool[E], expert_local[E] (int32, -1 = absent). */
/* out[pair, :] = x[src(pair), :] . W[ids[pair]]^T for every (token, route) pair; src = pair when
 * routed_input != 0 (x is [T*R, K]) else pair / R (x is [T, K]).  Invalid expert ids give zero rows.
 * Replaces nint_moe_grouped_matmul_hetero_qx_cuda / _hetero_f16_cuda / _pool_ws_cuda
 * (cpp_runtime/mfq_decode.cpp:236-280; mfq/kernels/cuda/moe.cu:3971-4345). */
/* Routes of one expert are batched mfq_hip_moe_tile_m() at a time by the mapped path: build the
 * route map with that tile_m.  Pass ids_dst == NULL (and NULL tables) to run every pair on its own
 * (decode, T*R small). */
int mfq_hip_moe_tile_m(void);
int mfq_hip_moe_grouped_matmul(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                               const int32_t *expert_local, int E, int out_per_expert, int K,
                               const void *x, int x_dtype, int64_t ldx, int routed_input,
                               const int32_t *ids, int T, int R,
                               const int32_t *ids_dst, const int32_t *expert_bounds,
                               const int32_t *tile_bounds, const int32_t *tile_experts,
                               float *out, int64_t ldo, mfq_stream_t stream);

/* The same with a workspace, which lets mapped calls run the prefill kernels (the pairs of an expert in chunks of up to
 * 128 against 256 or 512 of its neurons per block; activations pre-scaled to fp16 in the workspace).  x_rows = T * R with routed_input, else T.  The size query returns 0 when the cohorts have no
 * prefill kernel; a NULL or short workspace simply keeps the streaming kernels.  No counterpart in the
 * reference, whose hetero kernels allocate their workspace through torch
 * (cpp_runtime/mfq_decode.cpp:3008-3016). */
size_t mfq_hip_moe_grouped_workspace_bytes(const mfq_moe_pool *pools, int n_pools, int K, int x_rows);
int mfq_hip_moe_grouped_matmul_ws(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                                  const int32_t *expert_local, int E, int out_per_expert, int K,
                                  const void *x, int x_dtype, int64_t ldx, int routed_input,
                                  const int32_t *ids, int T, int R,
                                  const int32_t *ids_dst, const int32_t *expert_bounds,
                                  const int32_t *tile_bounds, const int32_t *tile_experts,
                                  float *out, int64_t ldo, void *workspace, size_t workspace_bytes,
                                  mfq_stream_t stream);

/* Gate/up projection of a mapped call with the GLU in the matmul's epilogue: pools hold [2 W] neurons per expert, gate
 * rows first; hidden [T * R, ldh] (16-bit, out_dtype) receives act(gate) * up, act = MFQ_GLU_SILU or MFQ_GLU_GELU --
 * the values of mfq_hip_moe_grouped_matmul_ws followed by mfq_hip_moe_glu (the same fp32 sums through the same
 * activation), without the fp32 [T * R, 2 W] round trip.  Needs the route map and a workspace of mfq_hip_moe_grouped_workspace_bytes; MFQ_ERR_UNSUPPORTED when the
 * call cannot take the prefill kernels (a cohort without a prefill body, K % 8, an unaligned x, a short workspace): run
 * the two calls then.  Replaces NintMoeWeight::forward_glu_output / nint_moe_grouped_matmul_hetero_glu_qx_cuda
 * (cpp_runtime/mfq_decode.cpp:3073-3127), which the reference limits to 1-4 tokens; mfq_hip_moe_decode_matmul with
 * swiglu covers those. */
int mfq_hip_moe_grouped_glu_ws(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                               const int32_t *expert_local, int E, int out_per_expert, int K,
                               const void *x, int x_dtype, int64_t ldx, int routed_input,
                               const int32_t *ids, int T, int R,
                               const int32_t *ids_dst, const int32_t *expert_bounds, int activation,
                               void *hidden, int out_dtype, int64_t ldh, void *workspace,
                               size_t workspace_bytes, mfq_stream_t stream);

/* Decode form of the grouped matmul (no route map; a handful of tokens): one launch of the batch-1 GEMV over
 * rows p = t * R + r (pair p against expert ids[p]) and, when a shared tensor [out_per_expert, K] is given, rows
 * T * R + t (the shared tensor against token t).  x row of a pair: p with routed_input, else t; of a shared row:
 * T * R + t with routed_input, else t.  swiglu = 0: out is float [rows, ldo].  swiglu = 1 (SwiGLU) or 2 (GEGLU, the
 * `gelu` flag of NintMoeWeight::forward_glu_output, cpp_runtime/mfq_decode.cpp:3074-3128): out_per_expert =
 * 2 W, gate rows first, and out is bf16 / fp16 (out_dtype, MFQ_X_*) [rows, ldo] = act(gate) * up, the fusion
 * of NintMoeWeight::forward_swiglu (cpp_runtime/mfq_decode.cpp:3203-3205) and nint_gemv_packed_swiglu_ws_cuda
 * (cpp_runtime/mfq_decode.cpp:393-396) moved to the producer.  Same values as mfq_hip_moe_grouped_matmul +
 * mfq_hip_moe_swiglu and mfq_hip_nint_gemv on the shared rows, up to the order of the fp32 sums over K.
 * MFQ_ERR_UNSUPPORTED when a cohort has no batch-1 unit, the shared tensor's rows differ from out_per_expert, or
 * K is too long for one block. */
int mfq_hip_moe_decode_matmul(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                              const int32_t *expert_local, int E, int out_per_expert, int K,
                              const void *x, int x_dtype, int64_t ldx, int routed_input,
                              const int32_t *ids, int T, int R,
                              const mfq_nint_desc *shared_desc, const void *shared_weight, int swiglu,
                              void *out, int out_dtype, int64_t ldo, mfq_stream_t stream);

/* 1 when mfq_hip_moe_decode_matmul takes these cohorts (and shared tensor) at T x R pairs, else 0: the same checks
 * the launch makes (a batch-1 unit for every cohort, the block's LDS need, the row count), so that a host can pick the
 * mapped path up front, as the T <= 8 test of NintMoeWeight::forward_impl does (cpp_runtime/mfq_decode.cpp:2935-2960).
 * Pure host arithmetic; the weight pointers of `pools` are not read. */
int mfq_hip_moe_decode_capable(const mfq_moe_pool *pools, int n_pools, int out_per_expert, int K,
                               const mfq_nint_desc *shared_desc, int T, int R, int swiglu);

/* Row gather / scatter for hosts that walk a batch expert by expert (cohorts of families the grouped kernels do not
 * hold): scatter == 0: dst row i = src row index[i]; scatter != 0: dst row index[i] = src row i, i < n.  Rows of
 * row_bytes bytes (a multiple of 4), strides in bytes; index is a device array.  Stands in for the index_select /
 * index_copy_ pair of the reference's per-expert walk over a mixed-family tensor (cpp_runtime/mfq_decode.cpp:17607-17629). */
int mfq_hip_moe_move_rows(const void *src, int64_t src_stride, const int32_t *index, int n, int row_bytes, int scatter,
                          void *dst, int64_t dst_stride, mfq_stream_t stream);

/* hidden[r, c] = silu(gate_up[r, c]) * gate_up[r, W + c]  (moe_swiglu_split_cuda,
 * mfq/kernels/cuda/moe.cu:2980-2996); output fp16 (x_dtype MFQ_X_F16) or bf16. */
int mfq_hip_moe_swiglu(const float *gate_up, int64_t ld, int rows, int W, void *hidden, int out_dtype,
                       int64_t ldh, mfq_stream_t stream);
/* The same with the gate activation chosen by `activation` (MFQ_GLU_*); MFQ_GLU_GELU replaces moe_geglu_split_cuda
 * (cpp_runtime/mfq_decode.cpp:320) and gelu_mul_cuda (mfq/kernels/cuda/activation.cu:69-104). */
int mfq_hip_moe_glu(const float *gate_up, int64_t ld, int rows, int W, void *hidden, int out_dtype,
                    int64_t ldh, int activation, mfq_stream_t stream);
/* out[t, :] = sum_r w[t, r] * pair[t, r, :] (+ shared[t, :] when shared != NULL; ungated add,
 * cpp_runtime/mfq_decode.cpp:11077-11080; with gate_logits != NULL: + sigmoid(gate_logits[t]) * shared).
 * Replaces moe_weighted_reduce_cuda / moe_weighted_reduce_shared_gate_cuda. */
int mfq_hip_moe_weighted_reduce(const float *pair, const float *weights, int T, int R, int H,
                                const float *shared, const float *gate_logits, float *out,
                                mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * Expert residency (experts kept in host memory, a GPU arena of slots for the ones in use).
 * ---------------------------------------------------------------------------------- */
/* One byte range to copy: destination = device address, source_offset = offset into the staging buffer.
 * The layout of MoeCacheScatterDescriptor (cpp_runtime/moe_cache_transfer.h:9-17). */
typedef struct mfq_scatter_desc {
    uint64_t destination, source_offset, nbytes;
} mfq_scatter_desc;
/* Copies n_transfers ranges out of `staging` (a device buffer the host has just filled with one copy: expert bodies,
 * anchors, dispatch-table words, and at descriptor_offset the table of mfq_scatter_desc) to their destinations in one
 * launch; max_bytes = the largest nbytes (sizes the grid: big ranges are spread over up to 64 blocks).  Ranges whose
 * addresses and length are multiples of 16 move as 16-byte words.  Replaces moe_cache_scatter_cuda
 * (cpp_runtime/moe_cache_transfer.h:19-23, mfq/kernels/cuda/moe.cu:45-77, 3532-3550). */
int mfq_hip_cache_scatter(const void *staging, int64_t descriptor_offset, int n_transfers, int64_t max_bytes,
                          mfq_stream_t stream);

/* ------------------------------------------------------------------------------------
 * helpers shared by the GEMM paths
 * ---------------------------------------------------------------------------------- */
/* Plain fp16 x fp16 -> fp32 MFMA GEMM: y[M, N] = a[M, K] . b[N, K]^T (used after a full dequant). */
int mfq_hip_gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K,
                        float *y, int64_t ldy, mfq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MFQ_HIP_H */
