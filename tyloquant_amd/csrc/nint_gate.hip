// Batch-1/2 GEMV with the input gate of the projection fused into the activation staging:
// y = (x * act(gate)) . W^T in one launch.
#include "common.hpp"
#include "gemv_common.hpp"
#include "tune.hpp"
#include "nint_body.hpp"

namespace mfq {

void gemv_shape(const NintK &k, int mb, int &spw, int &nwaves, int &rbw, size_t &lds_bytes);

template <int MB>
__device__ __forceinline__ InputGate<MB> gate_rows(const uint16_t *gate, int64_t ldg, int M, int m0, int mode) {
    InputGate<MB> xp;
#pragma unroll
    for (int m = 0; m < MB; ++m) xp.gr[m] = m0 + m < M ? gate + static_cast<int64_t>(m0 + m) * ldg : nullptr;
    xp.mode = mode;
    return xp;
}

template <class U, int XF16, int MB>
__global__ __launch_bounds__(1024) void nint_gemv_gate_kernel(NintK k, const uint8_t *__restrict__ w,
                                                              const uint16_t *__restrict__ x, int64_t ldx,
                                                              const uint16_t *__restrict__ gate, int64_t ldg, int mode, int M,
                                                              float *__restrict__ y, int64_t ldy, int spw, int rbw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_unit_body<U, XF16, MB, true, true, InputGate<MB>>(k, w, blockIdx.x * rbw, rbw, 0, k.out, xr, yr, spw, lds, 1,
                                                           gate_rows<MB>(gate, ldg, M, blockIdx.y * MB, mode));
}

template <int XF16, int MB>
__global__ __launch_bounds__(1024) void nint_gemv_gate_generic_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                      const uint16_t *__restrict__ x, int64_t ldx,
                                                                      const uint16_t *__restrict__ gate, int64_t ldg, int mode,
                                                                      int M, float *__restrict__ y, int64_t ldy, int spw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_generic_body<XF16, MB, InputGate<MB>>(k, w, blockIdx.x, 0, k.out, xr, yr, spw, lds,
                                               gate_rows<MB>(gate, ldg, M, blockIdx.y * MB, mode));
}

template <int XF16, int MB>
static int launch_gate(const NintK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, const uint16_t *gate, int64_t ldg,
                       int mode, int M, float *y, int64_t ldy, hipStream_t st) {
    int spw, nwaves, rbw;
    size_t lds;
    gemv_shape(k, MB, spw, nwaves, rbw, lds);
    MFQ_REQUIRE(lds <= kMaxDynamicLds && k.rowblock_bytes < (1ll << 31), MFQ_ERR_UNSUPPORTED,
                "nint_gemv_gate: neuron_len %d is too long for one block", k.neuron_len);
    // the hook works on the activation chunks a wave prefetches: at most 1024 pairs per wave
    MFQ_REQUIRE(spw * 16 * (k.gs / 2) <= 256 * kXChunks, MFQ_ERR_UNSUPPORTED,
                "nint_gemv_gate: a wave's slice of %d values is beyond the prefetched chunks", spw * 16 * k.gs);
    const dim3 block(64 * nwaves);
#define MFQ_GATE_LAUNCH(KERN, GRID, ...)                                                                          \
    do {                                                                                                          \
        auto kern_ = KERN;                                                                                        \
        if (int rc_ = allow_dynamic_lds(reinterpret_cast<const void *>(kern_), lds, "nint_gemv_gate")) return rc_; \
        hipLaunchKernelGGL(kern_, GRID, block, lds, st, __VA_ARGS__);                                             \
        return check_launch("nint_gemv_gate");                                                                    \
    } while (0)
    const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, rbw)), static_cast<unsigned>(ceil_div(M, MB)));
#define MFQ_GATE_UNIT(UNIT, B, G)                                                                                 \
    if (k.bits == B && k.gs == G)                                                                                 \
        MFQ_GATE_LAUNCH((nint_gemv_gate_kernel<UNIT<B, G>, XF16, MB>), grid, k, w, x, ldx, gate, ldg, mode, M, y, ldy, spw, rbw);
    if (k.kind == 1) {
        MFQ_GATE_UNIT(PairedUnit, 4, 32) MFQ_GATE_UNIT(PairedUnit, 4, 24) MFQ_GATE_UNIT(PairedUnit, 4, 16)
        MFQ_GATE_UNIT(PairedUnit, 4, 48) MFQ_GATE_UNIT(PairedUnit, 3, 24) MFQ_GATE_UNIT(PairedUnit, 2, 16)
        MFQ_GATE_UNIT(PairedUnit, 2, 32)
        return fail(MFQ_ERR_UNSUPPORTED, "nint_gemv_gate: no paired kernel for NINT%d-%d", k.bits, k.gs);
    }
    if (mfma_generic_profile(k)) {
        MFQ_GENERIC_PROFILES(MFQ_GATE_UNIT)
    }
    const dim3 ggrid(k.n_rowblocks, static_cast<unsigned>(ceil_div(M, MB)));
    MFQ_GATE_LAUNCH((nint_gemv_gate_generic_kernel<XF16, MB>), ggrid, k, w, x, ldx, gate, ldg, mode, M, y, ldy, spw);
#undef MFQ_GATE_UNIT
#undef MFQ_GATE_LAUNCH
}

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_nint_gemv_gate(const mfq_nint_desc *d, const void *weight, const void *x, const void *gate,
                                      int x_dtype, int64_t ldx, int64_t ldg, int M, int mode, float *y, int64_t ldy,
                                      mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && gate && y, MFQ_ERR_INVALID, "nint_gemv_gate: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemv_gate: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(mode == 0 || mode == 1, MFQ_ERR_INVALID, "nint_gemv_gate: mode=%d (0 SiLU, 1 sigmoid)", mode);
    MFQ_REQUIRE(M >= 1 && ldx >= d->neuron_len && ldg >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID,
                "nint_gemv_gate: bad shape");
    const NintK k = to_k(d);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gate)) & 15) == 0 &&
                         (M == 1 || (ldx % 8 == 0 && ldg % 8 == 0));
    MFQ_REQUIRE(M <= 2 && k.neuron_len % 8 == 0 && aligned, MFQ_ERR_UNSUPPORTED,
                "nint_gemv_gate: the fused gate takes one or two 16-byte aligned rows of a multiple of 8 values");
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x), *gp = static_cast<const uint16_t *>(gate);
    hipStream_t st = as_stream(stream);
    if (x_dtype == MFQ_X_F16)
        return M == 1 ? launch_gate<1, 1>(k, w, xp, ldx, gp, ldg, mode, M, y, ldy, st)
                      : launch_gate<1, 2>(k, w, xp, ldx, gp, ldg, mode, M, y, ldy, st);
    return M == 1 ? launch_gate<0, 1>(k, w, xp, ldx, gp, ldg, mode, M, y, ldy, st)
                  : launch_gate<0, 2>(k, w, xp, ldx, gp, ldg, mode, M, y, ldy, st);
}
