// NINT tensors at the two ends of the layer stack: token-embedding rows decoded from the packed table, and the
// LM-head GEMV that also delivers the arg-max of the logits (greedy decoding never reads the logits back).
#include <limits.h>

#include <mutex>

#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_body.hpp"

namespace mfq {

void gemv_shape(const NintK &k, int mb, int &spw, int &nwaves, int &rbw, size_t &lds_bytes);

// ---- embedding rows ----------------------------------------------------------------------------
// One thread per output element: neuron `tok` lives in row-block tok / 16 at lane (tok % 16, g % 4) of step g / 16,
// slot (g % 16) / 4.  The values are those of the bit-exact dequantizer (four separate fp32 roundings), rounded once
// more to the output type; ids outside [0, out) give a row of zeros.
__global__ __launch_bounds__(256) void nint_embedding_kernel(NintK k, const uint8_t *__restrict__ w,
                                                             const int64_t *__restrict__ ids, void *__restrict__ outp,
                                                             int out_dtype, int64_t ldo) {
    const int col = blockIdx.x * 256 + threadIdx.x;
    if (col >= k.neuron_len) return;
    const int n = blockIdx.y;
    const int64_t tok = ids[n];
    float v = 0.f;
    if (tok >= 0 && tok < k.out) {
        const int g = col / k.gs, i = col - g * k.gs;
        const int rb = static_cast<int>(tok >> 4), r = static_cast<int>(tok & 15);
        const int s = g >> 4, j = (g & 15) >> 2, lane = r + 16 * (g & 3);
        const uint8_t *sp = w + rb * k.rowblock_bytes + s * k.step_bytes;
        const uint32_t *qreg = reinterpret_cast<const uint32_t *>(sp);
        const uint8_t *treg = sp + 4 * 64 * k.dwords * 4;
        const uint8_t *sreg = treg + (k.tail ? 256 : 0);
        const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
        const uint32_t tail = k.tail ? treg[lane * 4 + j] : 0u;
        const float d_eff = __fmul_rn(anchors[tok], static_cast<float>(sreg[lane * 8 + 2 * j]));
        const float m_eff = __fmul_rn(anchors[16 * k.n_rowblocks + tok], static_cast<float>(sreg[lane * 8 + 2 * j + 1]));
        const uint32_t c = unit_code(k, qreg + (j * 64 + lane) * k.dwords, tail, i);
        v = __fsub_rn(__fmul_rn(d_eff, static_cast<float>(c)), m_eff);
    }
    const int64_t at = static_cast<int64_t>(n) * ldo + col;
    if (out_dtype == MFQ_X_F32) static_cast<float *>(outp)[at] = v;
    else static_cast<uint16_t *>(outp)[at] = out_dtype == MFQ_X_F16 ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
}

// ---- LM head: GEMV + arg-max ----------------------------------------------------------------------
// Order of the arg-max: the larger value wins, equal values go to the lower index, NaN never wins; a row without
// any finite-or-infinite winner (all NaN) yields INT_MAX from the blocks and the final kernel stores -1.
__device__ __forceinline__ void argmax_take(float &best, int &best_i, float v, int i) {
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
}
__device__ __forceinline__ void argmax_wave(float &best, int &best_i) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float v = __shfl_xor(best, off);
        const int i = __shfl_xor(best_i, off);
        argmax_take(best, best_i, v, i);
    }
}

// The batch-1 GEMV with the block's winner instead of (or besides) its 16 * rbw logits: partial sums are added in
// the order of the plain kernel, so the logits are the same floats.
template <class U, int XF16, bool RING, bool XR = false>
__global__ __launch_bounds__(1024) void nint_gemv_argmax_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                const uint16_t *__restrict__ x, float *__restrict__ logits,
                                                                float *__restrict__ block_vals,
                                                                int32_t *__restrict__ block_idxs, int spw, int rbw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[1] = {x};
    float *yr[1] = {nullptr};
    constexpr bool IN_REGS = XR && !RING && U::NPAIR <= 16;  // the plain GEMV's choice, so that the sums are the same floats
    if constexpr (IN_REGS) nint_unit_body_xreg<U, XF16, 1, false>(k, w, blockIdx.x * rbw, rbw, 0, k.out, xr, yr, spw, lds);
    else nint_unit_body<U, XF16, 1, RING, false>(k, w, blockIdx.x * rbw, rbw, 0, k.out, xr, yr, spw, lds);
    __syncthreads();
    if (threadIdx.x >= 64) return;
    const int nwaves = blockDim.x >> 6;
    const float *red = reinterpret_cast<const float *>(lds + (IN_REGS ? 0 : gemv_red_offset(nwaves, 1, spw, U::GROUP)));
    float best = -INFINITY;
    int best_i = INT_MAX;
    const int o = threadIdx.x;  // rbw <= 4 row-blocks: one lane per neuron
    if (o < rbw * 16) {
        const int r = o & 15, rbi = o >> 4;
        const int row = (blockIdx.x * rbw + rbi) * 16 + r;
        if (row < k.out) {
            float s = 0.f;
            for (int wv = 0; wv < nwaves; ++wv) s += red[(rbi * nwaves + wv) * 16 + r];
            if (logits) logits[row] = s;
            argmax_take(best, best_i, s, row);
        }
    }
    argmax_wave(best, best_i);
    if (threadIdx.x == 0) {
        block_vals[blockIdx.x] = best;
        block_idxs[blockIdx.x] = best_i;
    }
}

// Winners of `chunk` consecutive logits per block, row blockIdx.y (profiles without a fused kernel, and M > 1).
__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float *__restrict__ logits, int64_t ldl, int n, int chunk,
                                                            float *__restrict__ block_vals, int32_t *__restrict__ block_idxs,
                                                            int nb_stride) {
    __shared__ float sv[4];
    __shared__ int si[4];
    const float *row = logits + static_cast<int64_t>(blockIdx.y) * ldl;
    const int lo = blockIdx.x * chunk, hi = lo + chunk < n ? lo + chunk : n;
    float best = -INFINITY;
    int best_i = INT_MAX;
    for (int i = lo + threadIdx.x; i < hi; i += 256) argmax_take(best, best_i, row[i], i);
    argmax_wave(best, best_i);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < 4; ++wv) argmax_take(best, best_i, sv[wv], si[wv]);
        block_vals[blockIdx.y * nb_stride + blockIdx.x] = best;
        block_idxs[blockIdx.y * nb_stride + blockIdx.x] = best_i;
    }
}

__global__ __launch_bounds__(1024) void argmax_final_kernel(const float *__restrict__ block_vals,
                                                            const int32_t *__restrict__ block_idxs, int nb, int nb_stride,
                                                            int64_t *__restrict__ token) {
    __shared__ float sv[16];
    __shared__ int si[16];
    float best = -INFINITY;
    int best_i = INT_MAX;
    for (int i = threadIdx.x; i < nb; i += 1024)
        argmax_take(best, best_i, block_vals[blockIdx.x * nb_stride + i], block_idxs[blockIdx.x * nb_stride + i]);
    argmax_wave(best, best_i);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < 16; ++wv) argmax_take(best, best_i, sv[wv], si[wv]);
        token[blockIdx.x] = best_i == INT_MAX ? -1 : best_i;
    }
}

constexpr int kArgmaxChunk = 2048;  // logits per block of the unfused first stage

static int64_t argmax_slots(const mfq_nint_desc *d) {
    const int64_t chunks = ceil_div(d->out, kArgmaxChunk);
    return d->n_rowblocks > chunks ? d->n_rowblocks : chunks;
}

template <int XF16>
static int launch_gemv_argmax(const NintK &k, const uint8_t *w, const uint16_t *x, float *logits, float *vals, int32_t *idxs,
                              int &nb, hipStream_t st) {
    int spw, nwaves, rbw;
    size_t lds;
    gemv_shape(k, 1, spw, nwaves, rbw, lds);
    nb = -1;
    if (lds > 65536 || k.rowblock_bytes >= (1ll << 31)) return MFQ_OK;  // the caller takes the unfused form
    const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, rbw))), block(64 * nwaves);
    // the plain GEMV's condition for activations in registers (launch_gemv_mb)
    static const int env_xreg = tune_env("MFQ_GEMV_XREG", 1);
    const bool xreg = env_xreg != 0 && k.neuron_len % 2 == 0 && (reinterpret_cast<uintptr_t>(x) & 3) == 0;
#define MFQ_ARGMAX(UNIT, B, G)                                                                                        \
    if (k.bits == B && k.gs == G) {                                                                                   \
        if (spw * rbw <= 3 && xreg)                                                                                   \
            hipLaunchKernelGGL((nint_gemv_argmax_kernel<UNIT<B, G>, XF16, false, true>), grid, block, lds, st, k, w, x, logits, \
                               vals, idxs, spw, rbw);                                                                 \
        else if (spw * rbw <= 3)                                                                                      \
            hipLaunchKernelGGL((nint_gemv_argmax_kernel<UNIT<B, G>, XF16, false>), grid, block, lds, st, k, w, x, logits, \
                               vals, idxs, spw, rbw);                                                                 \
        else                                                                                                          \
            hipLaunchKernelGGL((nint_gemv_argmax_kernel<UNIT<B, G>, XF16, true>), grid, block, lds, st, k, w, x, logits, \
                               vals, idxs, spw, rbw);                                                                 \
        nb = static_cast<int>(grid.x);                                                                                \
        return check_launch("nint_gemv_argmax");                                                                      \
    }
    if (k.kind == 1) {
        MFQ_ARGMAX(PairedUnit, 4, 32) MFQ_ARGMAX(PairedUnit, 4, 24) MFQ_ARGMAX(PairedUnit, 3, 24)
    } else {
        // (NINT8-48 takes the unfused form: its plain GEMV runs on the matrix cores, and the logits of this call are
        // the plain GEMV's floats)
        MFQ_ARGMAX(GenericUnit, 5, 28) MFQ_ARGMAX(GenericUnit, 6, 24)
    }
#undef MFQ_ARGMAX
    return MFQ_OK;
}

// Input gate of a projection: out[m, k] = x[m, k] * act(gate[m, k]), act = SiLU (mode 0) or the logistic function
// (mode 1), computed in fp32 and rounded once to the 16-bit type of x.  Eight elements per thread (16-byte accesses)
// when the rows allow it, else one.
template <int F16, int VEC>
__global__ __launch_bounds__(256) void input_gate_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ gate,
                                                         int64_t ldx, int64_t ldg, int M, int K, int mode,
                                                         uint16_t *__restrict__ out, int64_t ldo) {
    const int per_row = (K + VEC - 1) / VEC;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(M) * per_row) return;
    const int m = static_cast<int>(idx / per_row), k0 = static_cast<int>(idx - static_cast<int64_t>(m) * per_row) * VEC;
    auto one = [&](uint16_t xv, uint16_t gv) -> uint16_t { return input_gate_value<F16>(xv, gv, mode); };
    if constexpr (VEC == 8) {
        const u32x4_t xv = *reinterpret_cast<const u32x4_t *>(x + m * ldx + k0);
        const u32x4_t gv = *reinterpret_cast<const u32x4_t *>(gate + m * ldg + k0);
        u32x4_t o;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            o[t] = one(xv[t] & 0xffffu, gv[t] & 0xffffu) | (static_cast<uint32_t>(one(xv[t] >> 16, gv[t] >> 16)) << 16);
        *reinterpret_cast<u32x4_t *>(out + m * ldo + k0) = o;
    } else {
        out[m * ldo + k0] = one(x[m * ldx + k0], gate[m * ldg + k0]);
    }
}

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_nint_embedding(const mfq_nint_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                                      int out_dtype, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight, MFQ_ERR_INVALID, "nint_embedding: null argument");
    MFQ_REQUIRE(n_ids >= 0, MFQ_ERR_INVALID, "nint_embedding: n_ids=%d", n_ids);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16 || out_dtype == MFQ_X_F32, MFQ_ERR_INVALID,
                "nint_embedding: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(ldo >= d->neuron_len, MFQ_ERR_INVALID, "nint_embedding: ldo %lld < neuron_len %d", static_cast<long long>(ldo),
                d->neuron_len);
    if (n_ids == 0) return MFQ_OK;
    MFQ_REQUIRE(ids && out, MFQ_ERR_INVALID, "nint_embedding: null ids or output");
    const NintK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const dim3 grid(static_cast<unsigned>(ceil_div(k.neuron_len, 256)));
    for (int n0 = 0; n0 < n_ids; n0 += 65535) {  // grid.y holds at most 65535 rows
        const int rows = n_ids - n0 < 65535 ? n_ids - n0 : 65535;
        const size_t esize = out_dtype == MFQ_X_F32 ? 4 : 2;
        hipLaunchKernelGGL(nint_embedding_kernel, dim3(grid.x, static_cast<unsigned>(rows)), dim3(256), 0, as_stream(stream), k,
                           w, ids + n0, static_cast<void *>(static_cast<uint8_t *>(out) + static_cast<size_t>(n0) * ldo * esize),
                           out_dtype, ldo);
    }
    return check_launch("nint_embedding");
}

extern "C" size_t mfq_hip_nint_gemv_argmax_workspace_bytes(const mfq_nint_desc *d, int M) {
    if (!d || M < 1) return 0;
    const size_t m = static_cast<size_t>(M);
    return m * static_cast<size_t>(argmax_slots(d)) * 8 + m * static_cast<size_t>(d->out) * 4;
}

extern "C" int mfq_hip_nint_gemv_argmax(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                        int M, float *logits, int64_t ldl, int64_t *token, void *workspace,
                                        size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && token && workspace, MFQ_ERR_INVALID, "nint_gemv_argmax: null argument");
    MFQ_REQUIRE(M >= 1 && M <= 65535, MFQ_ERR_INVALID, "nint_gemv_argmax: M=%d outside [1, 65535]", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemv_argmax: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len, MFQ_ERR_INVALID, "nint_gemv_argmax: ldx smaller than the tensor");
    MFQ_REQUIRE(!logits || ldl >= d->out, MFQ_ERR_INVALID, "nint_gemv_argmax: ldl smaller than the tensor");
    MFQ_REQUIRE(workspace_bytes >= mfq_hip_nint_gemv_argmax_workspace_bytes(d, M), MFQ_ERR_WORKSPACE,
                "nint_gemv_argmax: workspace %zu < %zu bytes", workspace_bytes, mfq_hip_nint_gemv_argmax_workspace_bytes(d, M));
    MFQ_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 3) == 0, MFQ_ERR_INVALID, "nint_gemv_argmax: unaligned workspace");
    const hipStream_t st = as_stream(stream);
    const NintK k = to_k(d);
    const int slots = static_cast<int>(argmax_slots(d));
    float *vals = static_cast<float *>(workspace);
    int32_t *idxs = reinterpret_cast<int32_t *>(vals + static_cast<size_t>(M) * slots);
    float *own_logits = reinterpret_cast<float *>(idxs + static_cast<size_t>(M) * slots);
    int nb = -1;
    if (M == 1) {
        const uint8_t *w = static_cast<const uint8_t *>(weight);
        const uint16_t *x16 = static_cast<const uint16_t *>(x);
        const int rc = x_dtype == MFQ_X_F16 ? launch_gemv_argmax<1>(k, w, x16, logits, vals, idxs, nb, st)
                                            : launch_gemv_argmax<0>(k, w, x16, logits, vals, idxs, nb, st);
        if (rc != MFQ_OK) return rc;
    }
    if (nb < 0) {
        float *lg = logits ? logits : own_logits;
        const int64_t ld = logits ? ldl : d->out;
        const int rc = mfq_hip_nint_gemv(d, weight, x, x_dtype, ldx, M, lg, ld, stream);
        if (rc != MFQ_OK) return rc;
        nb = static_cast<int>(ceil_div(d->out, kArgmaxChunk));
        hipLaunchKernelGGL(argmax_chunks_kernel, dim3(static_cast<unsigned>(nb), static_cast<unsigned>(M)), dim3(256), 0, st, lg,
                           ld, d->out, kArgmaxChunk, vals, idxs, slots);
        const int rc2 = check_launch("nint_argmax_chunks");
        if (rc2 != MFQ_OK) return rc2;
    }
    hipLaunchKernelGGL(argmax_final_kernel, dim3(static_cast<unsigned>(M)), dim3(1024), 0, st, vals, idxs, nb, slots, token);
    return check_launch("nint_argmax_final");
}

// ---- the same call for callers that cannot allocate ---------------------------------------------------------
// The per-block winners (and the logits, when the caller passes none) live in a file-scope device array instead of a
// caller workspace.  Each GPU holds its own copy of the array at its own address: the address is looked up once per
// device, with that device current, and only that pointer is ever handed to a kernel.
constexpr size_t kStaticScratchBytes = 4u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
std::mutex g_scratch_mu;
void *g_scratch_ptr[64] = {nullptr};

// Device address of `scratch` on the current device (0 on failure, with the error text set).
void *static_scratch() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) {
        fail(MFQ_ERR_LAUNCH, "nint_gemv_argmax_static: hipGetDevice: %s", hipGetErrorString(e));
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            fail(MFQ_ERR_LAUNCH, "nint_gemv_argmax_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int mfq_hip_nint_gemv_argmax_static_init(void) { return static_scratch() ? MFQ_OK : MFQ_ERR_LAUNCH; }

extern "C" int mfq_hip_nint_gemv_argmax_static(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype,
                                               int64_t ldx, int M, float *logits, int64_t ldl, int64_t *token,
                                               mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && token, MFQ_ERR_INVALID, "nint_gemv_argmax_static: null argument");
    MFQ_REQUIRE(M >= 1 && M <= 65535, MFQ_ERR_INVALID, "nint_gemv_argmax_static: M=%d outside [1, 65535]", M);
    const size_t need = mfq_hip_nint_gemv_argmax_workspace_bytes(d, M);
    MFQ_REQUIRE(need <= kStaticScratchBytes, MFQ_ERR_WORKSPACE,
                "nint_gemv_argmax_static: %d rows of %d logits need %zu bytes of scratch, the built-in buffer holds %zu; use "
                "mfq_hip_nint_gemv_argmax with a workspace", M, d->out, need, kStaticScratchBytes);
    void *ptr = static_scratch();
    if (!ptr) return MFQ_ERR_LAUNCH;
    // nothing in the buffer has to start at zero: every slot the final pass reads is written by this call's first stage
    return mfq_hip_nint_gemv_argmax(d, weight, x, x_dtype, ldx, M, logits, ldl, token, ptr, kStaticScratchBytes, stream);
}

extern "C" int mfq_hip_input_gate(const void *x, const void *gate, int x_dtype, int64_t ldx, int64_t ldg, int M, int K,
                                  int mode, void *out, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(x && gate && out, MFQ_ERR_INVALID, "input_gate: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "input_gate: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(M >= 1 && K >= 1 && ldx >= K && ldg >= K && ldo >= K, MFQ_ERR_INVALID, "input_gate: bad shape");
    MFQ_REQUIRE(mode == 0 || mode == 1, MFQ_ERR_INVALID, "input_gate: mode=%d (0 SiLU, 1 sigmoid)", mode);
    const uint16_t *xp = static_cast<const uint16_t *>(x), *gp = static_cast<const uint16_t *>(gate);
    uint16_t *op = static_cast<uint16_t *>(out);
    const bool vec = K % 8 == 0 && ldx % 8 == 0 && ldg % 8 == 0 && ldo % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const int64_t n = static_cast<int64_t>(M) * (vec ? K / 8 : K);
    const dim3 grid(static_cast<unsigned>(ceil_div(n, 256)));
    hipStream_t st = as_stream(stream);
    if (x_dtype == MFQ_X_F16) {
        if (vec) hipLaunchKernelGGL((input_gate_kernel<1, 8>), grid, dim3(256), 0, st, xp, gp, ldx, ldg, M, K, mode, op, ldo);
        else hipLaunchKernelGGL((input_gate_kernel<1, 1>), grid, dim3(256), 0, st, xp, gp, ldx, ldg, M, K, mode, op, ldo);
    } else {
        if (vec) hipLaunchKernelGGL((input_gate_kernel<0, 8>), grid, dim3(256), 0, st, xp, gp, ldx, ldg, M, K, mode, op, ldo);
        else hipLaunchKernelGGL((input_gate_kernel<0, 1>), grid, dim3(256), 0, st, xp, gp, ldx, ldg, M, K, mode, op, ldo);
    }
    return check_launch("input_gate");
}
