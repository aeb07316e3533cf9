// C++ host runtime of the MFQ packed-weight matmul path on MI355X.
//
// Keeps the operator surface of the reference's cpp_runtime for this path -- the dtype-string
// registry and loaders, the weight structs, nint_matmul / nvq_matmul / nepq_matmul,
// build_moe_route_plan, NintMoeWeight::forward and nint_moe_ffn_forward, and the --check-linear
// harness -- over the C ABI of libmfq_hip.so (include/mfq_hip.h).  Activations and outputs are
// plain device pointers (bf16 or fp16 in, fp32 out) instead of torch tensors; errors are
// std::runtime_error, as in the reference's loaders.
//
//   reference (cpp_runtime/mfq_decode.cpp)            here
//   NintCpu / unpack_nint            :1529-1589       parse_nint + NintWeight::from_blob (device repack)
//   NintWeight / to_device_nint      :2101-2165,2268  NintWeight
//   nint_matmul                      :8130-8315       nint_matmul
//   NvqCpu / unpack_nvq / NvqWeight  :3418-4150       parse_nvq + NvqWeight
//   nvq_matmul                       :7884-7931       nvq_matmul
//   NepqCpu / unpack_nepq            :4166-4463       parse_nepq + NepqWeight, nepq_matmul
//   unpack_nint_moe_impl / NintMoeWeight :2367-2478, 2908-3071   parse_nintm + NintMoeWeight
//   MoeRoutePlan / build_moe_route_plan  :2579-2592, 2681-2708   MoeRoutePlan / build_moe_route_plan
//   nint_moe_ffn_forward             :3394-3416       nint_moe_ffn_forward
//   is_nint_linear_dtype / load_quant_linear :9409-9420, 9489-9771   same names
//   MfqFile                          :1294-1527       MfqFile (mapped files, shard sets, tensor / expert overlays)
//   run_linear_check                 :16510-16638     run_linear_check
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/mfq_hip.h"

namespace mfq_rt {

// ---- device memory ---------------------------------------------------------------------------
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t bytes);
    ~DeviceBuffer();
    DeviceBuffer(DeviceBuffer &&o) noexcept;
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept;
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    void *get() const { return ptr_; }
    size_t size() const { return bytes_; }
    void ensure(size_t bytes);  // grow-only
    static DeviceBuffer from_host(const void *src, size_t bytes);

private:
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
};

// ---- payload headers (host side; the bit streams themselves are read on the GPU) ----------------
struct NintHeader {
    int bits, sub_bits, gs, axis, neuron_len, out, ng;
    std::vector<int64_t> shape;
    size_t body_off, body_bytes;
    bool legacy;
};
struct NvqHeader {
    std::string codebook, dtype;
    int index_bits, vector_size, banks, out, neuron_len, gs, sub_bits;
    bool jsc, index_parity;
    size_t body_off, body_bytes;
};
struct NepqHeader {
    std::string label;
    int profile, n_experts, out_per_expert, neuron_len, banks, rotation_block;
    uint64_t rotation_seed;
    size_t body_off, body_bytes;
};
struct NintmPool {
    std::vector<int32_t> expert_ids;
    std::string dtype;
    size_t payload_off, payload_bytes, runtime_off, runtime_bytes;
};
struct NintmHeader {
    int n_experts, out_per_expert, neuron_len;
    std::vector<NintmPool> pools;
};
NintHeader parse_nint(const uint8_t *blob, size_t n);
NvqHeader parse_nvq(const uint8_t *blob, size_t n);
NepqHeader parse_nepq(const uint8_t *blob, size_t n);
// allow_partial: also an expert delta (an NINTMD overlay record: magic NID2, cohorts for some experts only;
// unpack_nint_moe_delta :2484-2487)
NintmHeader parse_nintm(const uint8_t *blob, size_t n, bool allow_partial = false);

// ---- weights ------------------------------------------------------------------------------------
struct NintWeight {
    mfq_nint_desc desc{};
    DeviceBuffer data;
    std::vector<int64_t> shape;
    mutable DeviceBuffer workspace;  // grows with M, like the reference's per-weight workspaces
    int64_t out() const { return desc.out; }
    int64_t neuron_len() const { return desc.neuron_len; }
    static NintWeight from_blob(const uint8_t *blob, size_t n, mfq_stream_t stream = nullptr);
};
// NINT8-0: GGML Q8_0 blocks (Nint8ZeroCpu + to_device_nint8_zero :1591-1650, 2309-2330)
struct Nint8ZeroWeight {
    mfq_nint8z_desc desc{};
    DeviceBuffer data;
    std::vector<int64_t> shape;
    mutable DeviceBuffer workspace;
    int64_t out() const { return desc.out; }
    int64_t neuron_len() const { return desc.neuron_len; }
    static Nint8ZeroWeight from_blob(const uint8_t *blob, size_t n, mfq_stream_t stream = nullptr);
};
struct NvqWeight {
    mfq_nvq_desc desc{};     // lane-major D4 layout (d4_256, d4_512)
    mfq_nvqs_desc sdesc{};   // streams read in place (E8 family, d4_1024): `streams` set
    bool streams = false;
    DeviceBuffer data;
    std::string dtype;
    mutable DeviceBuffer workspace;
    mutable DeviceBuffer pair_tmp;  // nvq_matmul_multi2 on stream formats: one projection at a time, grow-only
    int64_t out() const { return streams ? sdesc.out : desc.out; }
    int64_t neuron_len() const { return streams ? sdesc.neuron_len : desc.neuron_len; }
    int64_t payload_bytes() const { return streams ? sdesc.payload_bytes : desc.payload_bytes; }
    int64_t total_bytes() const { return streams ? sdesc.total_bytes : desc.total_bytes; }
    // `grid256` = the built-in 256-entry int8 magnitude grid of a plain (non-JSC) tensor: [256,4] for NVQ3, [256,8] for
    // NVQ2; JSC tensors carry their codebooks
    static NvqWeight from_blob(const uint8_t *blob, size_t n, const int8_t *grid256 = nullptr,
                               mfq_stream_t stream = nullptr);
    // The 1-bit families NVQ1-L / NVQ1-S / NPQ0-L / NPQ0-S (formats 1, 8, 7, 9 of the reference's unpack_nvq,
    // cpp_runtime/mfq_decode.cpp:3759-3770, 3800-3910), on the in-place stream kernels.  `iq1s_grid` = the built-in
    // 2048-entry ternary grid as packed uint16 (2 bits per digit), needed only by an NVQ1-L blob that carries no table.
    static NvqWeight from_lowbit_blob(const std::string &dtype, const uint8_t *blob, size_t n,
                                      const uint16_t *iq1s_grid = nullptr, mfq_stream_t stream = nullptr);
};
bool is_lowbit_linear_dtype(const std::string &dtype);
// MXFP4 / MXFP8 (OCP MX payloads of full-precision MFQ files; Mxfp8Weight / Mxfp4Cpu of the reference,
// cpp_runtime/mfq_decode.cpp:1807-1918, 2060-2100): the payload's value and scale bytes, used on the device as they lie
// in the file.  A pool of experts is the same tensor with `out_per_expert` rows per expert (MXFP8: whole 128-row blocks).
struct MxWeight {
    int kind = 0;  // 4 = MXFP4, 8 = MXFP8
    int64_t rows = 0, cols = 0, out_per_expert = 0;
    std::string dtype;
    DeviceBuffer values, scales;
    mutable DeviceBuffer workspace;
    int64_t out() const { return out_per_expert; }
    int64_t neuron_len() const { return cols; }
    int64_t n_experts() const { return rows / out_per_expert; }
    int64_t payload_bytes() const;
    static MxWeight from_blob(const std::string &dtype, const uint8_t *blob, size_t n, int64_t out_per_expert = 0,
                              mfq_stream_t stream = nullptr);
};
bool is_mx_linear_dtype(const std::string &dtype);
void mx_matmul(const MxWeight &w, int expert, const void *x, int x_dtype, int64_t ldx, int M, float *y,
               mfq_stream_t stream = nullptr);
void mx_dequantize(const MxWeight &w, int expert, float *out, mfq_stream_t stream = nullptr);
struct NepqWeight {
    mfq_nepq_desc desc{};    // lane-major layout (NEPQ1-S, NEPQ1-L)
    mfq_nvqs_desc sdesc{};   // streams read in place (NEPQ0-S, NEPQ0-L: the product tables of NPQ0): `streams` set
    bool streams = false;
    DeviceBuffer data;
    std::string label;
    int n_experts = 0, out_per_expert = 0, rotation_block = 0;
    DeviceBuffer signs;  // int8 [K] when rotated
    mutable DeviceBuffer workspace, rotated;
    int64_t out() const { return out_per_expert; }
    int64_t neuron_len() const { return streams ? sdesc.neuron_len : desc.neuron_len; }
    int64_t payload_bytes() const { return streams ? sdesc.payload_bytes : desc.payload_bytes; }
    int64_t total_bytes() const { return streams ? sdesc.total_bytes : desc.total_bytes; }
    static NepqWeight from_blob(const uint8_t *blob, size_t n, const int8_t *rotation_signs = nullptr,
                                mfq_stream_t stream = nullptr);
};

// y[M, out] (fp32, row stride out) = x[M, K] (x_dtype MFQ_X_BF16 / MFQ_X_F16, row stride ldx) . W^T
void nint_matmul(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                 mfq_stream_t stream = nullptr);
// hidden fp16 [M, W] = silu(gate) * up of a [2W, K] gate/up tensor (gate rows first): one fused launch for one or two
// rows (nint_gemv_packed_swiglu_ws_cuda :393-396) and for prefill batches the block-tiled kernel takes
// (mfq_hip_nint_gemm_glu), else nint_matmul into `scratch` (fp32 [M, 2W]) + the SwiGLU kernel
void nint_matmul_swiglu(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, void *hidden,
                        float *scratch = nullptr, mfq_stream_t stream = nullptr);
// y = (x * silu(gate)) . W^T (mode 0) or (x * sigmoid(gate)) . W^T (mode 1) (nint_matmul_input_mul :8395-8417): one or
// two rows in one GEMV launch that gates its activation slices; else the gated rows are formed in `gated` (device,
// 16-bit [M, K] of the type of x; may be null for M <= 2 rows the fused launch takes) by one elementwise launch, then nint_matmul
void nint_matmul_input_mul(const NintWeight &w, const void *x, const void *gate, int x_dtype, int64_t ldx, int64_t ldg, int M,
                           int mode, void *gated, float *y, mfq_stream_t stream = nullptr);
// the same with gelu_tanh(gate) * up (nint_matmul_geglu :8462-8485)
void nint_matmul_geglu(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, void *hidden,
                       float *scratch = nullptr, mfq_stream_t stream = nullptr);
// out [n_ids, K] (out_dtype MFQ_X_BF16 / MFQ_X_F16 / MFQ_X_F32, row stride K) = rows ids[n] (device int64) of the
// dequantized table, zeros for ids outside it (embed_forward :13929-13957)
void nint_embedding(const NintWeight &w, const int64_t *ids, int n_ids, void *out, int out_dtype,
                    mfq_stream_t stream = nullptr);
// the same for the other table formats embed_forward takes: NINT8-0 (:13943-13947) and every NVQ family
// (nvq_embedding :8072-8079, called at :13937-13939)
void nint8_zero_embedding(const Nint8ZeroWeight &w, const int64_t *ids, int n_ids, void *out, int out_dtype,
                          mfq_stream_t stream = nullptr);
void nvq_embedding(const NvqWeight &w, const int64_t *ids, int n_ids, void *out, int out_dtype,
                   mfq_stream_t stream = nullptr);
// token[m] (device int64) = argmax over the neurons of x[m] . W^T, ties to the lower index; logits (fp32 [M, out],
// may be null) receives the values the arg-max was taken from (next_token_from_hidden :14107-14130)
void nint_matmul_argmax(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, int64_t *token,
                        float *logits = nullptr, mfq_stream_t stream = nullptr);
void nvq_matmul(const NvqWeight &w, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                mfq_stream_t stream = nullptr);
void nepq_matmul(const NepqWeight &w, int expert, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                 mfq_stream_t stream = nullptr);
void nint_dequantize(const NintWeight &w, float *out, mfq_stream_t stream = nullptr);
// y[M, out0 + out1] = cat(x . W0^T, x . W1^T) for two tensors that share their input (nvq_matmul_multi2 :7981-8003)
void nvq_matmul_multi2(const NvqWeight &first, const NvqWeight &second, const void *x, int x_dtype, int64_t ldx, int M,
                       float *y, mfq_stream_t stream = nullptr);
// hidden fp16 [M, W] = silu(x . Wg^T) * (x . Wu^T) for an equal-width gate/up pair (nvq_matmul_swiglu :8004-8029):
// nvq_matmul_multi2 into `scratch` (fp32 [M, 2W]) + the SwiGLU kernel
void nvq_matmul_swiglu(const NvqWeight &gate, const NvqWeight &up, const void *x, int x_dtype, int64_t ldx, int M,
                       void *hidden, float *scratch, mfq_stream_t stream = nullptr);
// y fp32 [M, down.out] = Wd . hidden with hidden = nvq_matmul_swiglu(gate, up, x) (nvq_ffn_swiglu_down :8032-8071);
// `hidden` is a fp16 [M, W] buffer and `scratch` a fp32 [M, 2W] one, both the caller's
void nvq_ffn_swiglu_down(const NvqWeight &gate, const NvqWeight &up, const NvqWeight &down, const void *x, int x_dtype,
                         int64_t ldx, int M, float *y, void *hidden, float *scratch, mfq_stream_t stream = nullptr);
void nvq_dequantize(const NvqWeight &w, float *out, mfq_stream_t stream = nullptr);
// the q8_zero branch of nint_matmul (:8165-8185) and nint8_zero_dequant_cuda
void nint8_zero_matmul(const Nint8ZeroWeight &w, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                       mfq_stream_t stream = nullptr);
void nint8_zero_dequantize(const Nint8ZeroWeight &w, float *out, mfq_stream_t stream = nullptr);
void nepq_dequantize(const NepqWeight &w, float *out, mfq_stream_t stream = nullptr);

// ---- dtype registry -------------------------------------------------------------------------------
bool is_nint_linear_dtype(const std::string &dtype);
bool is_nvq_linear_dtype(const std::string &dtype);
bool is_nepq_linear_dtype(const std::string &dtype);
enum class QuantLinearKind { Nint, Nvq, Nepq, Nint8Zero, Mx };
struct QuantLinear {
    QuantLinearKind kind;
    std::shared_ptr<NintWeight> nint;
    std::shared_ptr<Nint8ZeroWeight> nint8z;
    std::shared_ptr<NvqWeight> nvq;
    std::shared_ptr<NepqWeight> nepq;
    std::shared_ptr<MxWeight> mx;
    int64_t out() const;
    int64_t neuron_len() const;
    int64_t payload_bytes() const;
    void forward(const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream = nullptr) const;
    void dequantize(float *out, mfq_stream_t stream = nullptr) const;
    // The tensor as a token-embedding table (embed_forward :13929-13957): NINT, NINT8-0 and NVQ tables; NEPQ and MX
    // tables are refused, as there.
    void embedding(const int64_t *ids, int n_ids, void *out, int out_dtype, mfq_stream_t stream = nullptr) const;
    // Grows the weight's workspace to the largest need of any batch of 1 .. max_M rows, so that forward() of such a batch
    // neither frees nor allocates device memory: call it once before capturing forward() into a HIP graph, and before
    // sharing the weight between threads or streams (the workspace itself is still one buffer per weight: concurrent
    // forward() calls on one weight need a weight object each, or the C ABI with caller-owned workspaces).
    void reserve(int max_M) const;
};
QuantLinear load_quant_linear(const std::string &dtype, const uint8_t *blob, size_t n, mfq_stream_t stream = nullptr);

// ---- MoE ----------------------------------------------------------------------------------------
struct MoeRoutePlan {
    const int32_t *ids = nullptr;  // device int32 [tokens, routes]
    int tokens = 0, routes = 0, n_experts = 0;
    DeviceBuffer ids_dst, expert_bounds, tile_bounds, tile_experts, counts;  // grow-only; valid when has_map
    bool map_ready = false, has_map = false;
    bool mapped() const { return has_map; }
    // Sizes the tables for up to max_tokens x routes pairs over n_experts experts: building a plan of that size or
    // smaller in place then allocates nothing (HIP graph capture, serving loops).
    void reserve(int max_tokens, int routes, int n_experts);
};
// Builds the expert map only above 8 tokens, like the reference (cpp_runtime/mfq_decode.cpp:2681-2708).  The first form
// returns a new plan; the second rebuilds `plan` in place, reusing its tables (no allocation once they are large
// enough, no host synchronisation in either).
MoeRoutePlan build_moe_route_plan(const int32_t *ids, int tokens, int routes, int n_experts,
                                  mfq_stream_t stream = nullptr);
void build_moe_route_plan(MoeRoutePlan &plan, const int32_t *ids, int tokens, int routes, int n_experts,
                          mfq_stream_t stream = nullptr);

// Cuts an NVQ-family or 1-bit-family blob of parts * n neurons into `parts` blobs of n neurons each: same flags and
// tables, the rows' anchors and their share of every tensor-wide bit stream re-packed from bit 0.
std::vector<std::vector<uint8_t>> split_rows(const std::string &dtype, const uint8_t *blob, size_t n, int parts);

// A NINTM cohort of another family (NVQ, the 1-bit families, NEPQ, MXFP4).  The reference runs them inside its grouped kernels
// (cpp_runtime/mfq_decode.cpp:4800-5360); here every expert is a tensor of its own on that family's kernels and the host
// walks the experts a batch routes to -- correct, one matmul per expert hit, not a fast path.
struct MoeForeignCohort {
    std::string dtype;
    std::vector<int32_t> expert_ids;
    std::vector<uint8_t> live;          // per expert: still owned (an expert overlay may give it to a later cohort)
    std::vector<QuantLinear> linears;   // one per expert (NVQ, 1-bit families)
    std::shared_ptr<NepqWeight> nepq;   // or the cohort as one expert-shaped tensor
    std::shared_ptr<MxWeight> mx;       // or a native MXFP4 pool: one [experts * out, K] tensor, experts = row ranges
    int64_t payload_bytes() const;
    void matmul(int local, const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) const;
    void dequantize(int local, float *out, mfq_stream_t stream) const;  // [out_per_expert, K]
    // One launch over all (token, route) pairs of a decode step, the routing table read on the device
    // (mfq_hip_{nvq,nvqs,nepq,nint8z,mx}_gemv_pairs): out[p] = W[ids[p]] . x[p or p / R] for the pairs routed to this
    // cohort.  prepare_pairs builds the device tables at load; matmul_pairs returns false where they were not built
    // (NEPQ1 experts that are not whole row-blocks).  Replaces the cohort arms of the reference's grouped decode
    // kernels (mfq/kernels/cuda/nvq_matmul.cu:2588-3175, 4210-4580; cpp_runtime/mfq_decode.cpp:4800-5360).
    static constexpr int kPairsMax = 64;  // pairs up to which add_foreign takes this form
    DeviceBuffer pair_slot, pair_weights;
    void prepare_pairs(int n_experts, int out_per_expert, mfq_stream_t stream);
    bool matmul_pairs(int n_experts, int out_per_expert, const void *x, int x_dtype, int64_t ldx, bool routed_input,
                      const int32_t *ids, int T, int R, float *out, mfq_stream_t stream) const;
};

struct NintMoeWeight {
    int n_experts = 0, out_per_expert = 0, neuron_len = 0;
    std::vector<std::shared_ptr<NintWeight>> pools;
    std::vector<std::vector<int32_t>> pool_expert_ids;
    std::vector<MoeForeignCohort> foreign;  // experts the grouped kernels skip (dispatch entry -1): added by add_foreign
    mutable DeviceBuffer f_index, f_x, f_y;
    // rows of the pairs routed to foreign experts: gather, multiply, scatter into out [T*R, out_per_expert]; reads the
    // routing table on the host (synchronizes the stream)
    void add_foreign(const void *x, int x_dtype, int64_t ldx, bool routed_input, const MoeRoutePlan &route, float *out,
                     mfq_stream_t stream) const;
    DeviceBuffer expert_pool, expert_local;  // int32 [E] dispatch tables
    std::vector<mfq_moe_pool> pool_table;
    mutable DeviceBuffer workspace;  // prefill path, grown on demand (do not grow it under graph capture)
    // overlay: the NINTMD record of the same name from an expert overlay file (MfqFile::expert_overlays): its cohorts are
    // appended and own the experts they list (load_nint_moe_cpu :5752-5774)
    static NintMoeWeight from_blob(const uint8_t *blob, size_t n, mfq_stream_t stream = nullptr,
                                   const uint8_t *overlay = nullptr, size_t overlay_n = 0);
    // x: [T, K] (routed_input = false) or [T*R, K]; out: fp32 [T*R, out_per_expert]
    void forward(const void *x, int x_dtype, int64_t ldx, bool routed_input, const MoeRoutePlan &route, float *out,
                 mfq_stream_t stream = nullptr) const;
    // act(gate) * up of a gate/up tensor as fp16 [T*R, out_per_expert / 2] (NintMoeWeight::forward_glu_output,
    // cpp_runtime/mfq_decode.cpp:3073-3127): the GLU runs in the epilogue of the mapped prefill kernels; where the library
    // declines, forward() into `scratch` (fp32 [T*R, out_per_expert]) and mfq_hip_moe_glu.
    void forward_glu(const void *x, int x_dtype, int64_t ldx, bool routed_input, const MoeRoutePlan &route, bool gelu,
                     void *hidden, float *scratch, mfq_stream_t stream = nullptr) const;
    // Decode step in one launch (mfq_hip_moe_decode_matmul): rows t * R + r are the routed pairs, rows T * R + t the
    // `shared` tensor (may be null) on token t.  swiglu: out is fp16 [rows, out_per_expert / 2], else fp32
    // [rows, out_per_expert].  decode_capable() tells whether the cohorts and the shared tensor fit that kernel.
    bool decode_capable(const NintWeight *shared, int tokens = 1, int routes = 1, bool swiglu = false) const;
    void forward_decode(const void *x, int x_dtype, int64_t ldx, bool routed_input, const int32_t *ids, int T, int R,
                        const NintWeight *shared, bool swiglu, void *out, mfq_stream_t stream = nullptr) const;
};

struct MoeFfnScratch {  // caller-owned intermediates of nint_moe_ffn_forward, grown on demand
    DeviceBuffer ids, weights, gate_up, hidden, down, shared_gu, shared_h, shared_out;
    MoeRoutePlan route;  // the expert map of the last call above 8 tokens
    // Sizes every intermediate, the route tables and the tensors' own workspaces for calls of up to max_tokens tokens
    // with top_k routes: nint_moe_ffn_forward then neither allocates nor waits for the device, so that a caller may
    // capture it into a HIP graph (the reference's forward does neither under capture: cpp_runtime/mfq_decode.cpp:3008-3016).
    // Tensors with cohorts of other families keep their host walk and cannot be captured.
    void reserve(const NintMoeWeight &gate_up, const NintMoeWeight &down, int max_tokens, int top_k,
                 const NintWeight *shared_gate_up = nullptr, const NintWeight *shared_down = nullptr);
};
// out fp32 [T, hidden]; top-k ids / weights stay in `scratch`.  `shared_gate_up` / `shared_down` may be null.
// Never waits for the device; allocates only when `scratch` (see MoeFfnScratch::reserve) or a workspace must grow.
void nint_moe_ffn_forward(const NintMoeWeight &gate_up, const NintMoeWeight &down, const void *x, int x_dtype,
                          int64_t ldx, int T, const float *router_logits, int top_k, int topk_mode, bool normalize,
                          const float *router_bias, float router_scale, const NintWeight *shared_gate_up,
                          const NintWeight *shared_down, MoeFfnScratch &scratch, float *out,
                          mfq_stream_t stream = nullptr);

// ---- expert residency (MoeExpertCache, cpp_runtime/mfq_decode.cpp:5941-7500) ----------------------------------
// Experts live in pinned host memory in their device layout; a GPU arena per cohort holds `slots` of them.
// prepare() makes a set of experts resident: least recently used slots are reused, all missing bytes travel as one
// staged host-to-device copy and one mfq_hip_cache_scatter launch, which also rewrites the dispatch-table words.
struct MoeCacheStats {
    int64_t hits = 0, misses = 0, evictions = 0, bytes = 0, launches = 0;
};
class MoeExpertCache;
class MoeCachedSource {
public:
    int n_experts = 0, out_per_expert = 0, neuron_len = 0;
    NintMoeWeight weight;  // view over the arenas; valid for the experts of the last prepare()
private:
    friend class MoeExpertCache;
    struct Cohort {
        mfq_nint_desc src{};
        std::vector<int32_t> expert_ids;
        void *host = nullptr;  // pinned copy of the cohort's device layout
        size_t host_bytes = 0;
        int64_t body_bytes = 0, slot_bytes = 0;
        int minimum_slots = 1;
        std::shared_ptr<NintWeight> arena;
        std::unordered_map<int, int> slot_of;  // local expert -> slot
        std::vector<int> lru, free_slots;
    };
    std::vector<Cohort> cohorts;
    std::vector<int32_t> cohort_of, local_of;
};
class MoeExpertCache {
public:
    explicit MoeExpertCache(int64_t budget_bytes);
    ~MoeExpertCache();
    MoeExpertCache(const MoeExpertCache &) = delete;
    MoeExpertCache &operator=(const MoeExpertCache &) = delete;
    MoeCachedSource *register_source(const uint8_t *blob, size_t n, int minimum_slots = 1);
    void finalize();
    // experts: host array of ids (any order, duplicates and out-of-range ids allowed)
    void prepare(MoeCachedSource &source, const int32_t *experts, size_t count, mfq_stream_t stream = nullptr);
    // reads the route's ids back to the host, prepares, and runs the grouped matmul on the arenas
    void forward(MoeCachedSource &source, const void *x, int x_dtype, int64_t ldx, bool routed_input,
                 const MoeRoutePlan &route, float *out, mfq_stream_t stream = nullptr);
    const MoeCacheStats &stats() const { return stats_; }
    int64_t allocated_bytes() const { return allocated_bytes_; }
    bool finalized() const { return finalized_; }

private:
    int64_t budget_bytes_, allocated_bytes_ = 0;
    bool finalized_ = false;
    std::vector<std::unique_ptr<MoeCachedSource>> sources_;
    MoeCacheStats stats_;
    void *stage_host_ = nullptr;
    size_t stage_bytes_ = 0;
    DeviceBuffer stage_dev_;
};

// ---- MFQ1 container + the --check-linear harness ----------------------------------------------------
// One MFQ1 file or shard set as one record table over read-only mappings of the files (MfqFile,
// cpp_runtime/mfq_decode.cpp:1294-1527; mfq/formats/io.py:834-965 open_mmap).  A file whose header carries
// split.count > 1 must be named <stem>-NNNNN-of-NNNNN.mfq; any shard of the set may be given.  Checks and messages follow
// the reference: split metadata against the file names, one architecture / version, the tensor and record totals,
// no record twice, records ending at the file size.
struct MfqRecord {
    std::string name, dtype;
    size_t offset = 0, nbytes = 0;
    int source = 0;  // index into MfqFile::source_paths
};
struct MfqFile {
    std::string path;  // the first shard (or the file itself)
    std::vector<std::string> source_paths;
    std::string model_arch;
    uint32_t version = 0;
    std::unordered_map<std::string, std::string> extra;  // metadata of the first shard: key -> JSON text
    std::vector<MfqRecord> records;                     // file order, shard after shard
    std::unordered_map<std::string, MfqRecord> tensor_overlays, expert_overlays;
    // tensor_overlay: an unsharded MFQ1 file whose records replace records of the same name (each must exist);
    // expert_overlay: NINTMD records over NINTM records of the same name, kept aside.  Empty: the environment variables
    // MFQ_TENSOR_OVERLAY / MFQ_EXPERT_OVERLAY, as in the reference; "-" disables the lookup.
    explicit MfqFile(const std::string &path, const std::string &tensor_overlay = "", const std::string &expert_overlay = "");
    ~MfqFile() = default;
    MfqFile(const MfqFile &) = delete;
    MfqFile &operator=(const MfqFile &) = delete;
    const MfqRecord &find(const std::string &name) const;
    bool has_record(const std::string &name) const;
    const uint8_t *data(const MfqRecord &r) const;  // the record's bytes inside the mapping of its file
    size_t tensor_count() const;                    // records that are not runtime assets (__mfq_asset__/...)
    std::string read_asset_text(const std::string &name) const;  // a BLOB record as text

private:
    // A read-only file mapping that unmaps itself: the constructor throws on any malformed file, and a member that
    // cleans up after itself is released then, while ~MfqFile does not run for a half-built object.
    struct Mapping {
        const uint8_t *base = nullptr;
        size_t size = 0;
        Mapping() = default;
        Mapping(Mapping &&o) noexcept : base(o.base), size(o.size) { o.base = nullptr; o.size = 0; }
        Mapping &operator=(Mapping &&o) noexcept;
        Mapping(const Mapping &) = delete;
        Mapping &operator=(const Mapping &) = delete;
        ~Mapping();
    };
    std::vector<Mapping> maps_;
    int map_file(const std::string &source);
};
struct LinearCheckResult {
    double production_ms, production_weight_gbps, payload_gbps, production_rel, production_mean_abs, production_max_abs;
    int64_t weight_bytes, payload_bytes;
};
// Deterministic input x[i] = ((i mod 97) - 48) / 512, warm-ups, `reps` timed launches between two HIP
// events, reference = device full dequant (fp32) times x on the host in fp64.
LinearCheckResult run_linear_check(const QuantLinear &lin, int M, int reps = 200);

}  // namespace mfq_rt
