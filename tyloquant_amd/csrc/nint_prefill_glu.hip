// Dense gate/up projection of a prefill batch with the GLU in the matmul's epilogue: the block-tiled prefill kernel of
// nint_prefill.hpp, each wave holding a gate row-block and the up row-block W / 16 further, storing act(gate) * up
// in 16 bits.  The [M, 2 W] fp32 intermediate (four times the bytes of the result) is never written or read back.
#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_body.hpp"
#include "nint_mfma.hpp"
#include "nint_prefill.hpp"

namespace mfq {

template <class U, int MT, int NB, int PF, int XD>
__global__ __launch_bounds__(512) void nint_prefill_glu_kernel(NintK k, const uint8_t *__restrict__ w,
                                                               const uint16_t *__restrict__ x16, int Kp,
                                                               const float *__restrict__ xscale,
                                                               const uint32_t *__restrict__ xg, int M,
                                                               uint16_t *__restrict__ hidden, int64_t ldh, GluOut glu) {
    extern __shared__ __attribute__((aligned(16))) uint16_t xt[];
    const DenseRows rows{static_cast<int>(blockIdx.y) * MT * 16, M};
    nint_prefill_body<U, MT, NB, 1, 8, DenseRows, PF, XD, true>(k, w, static_cast<int>(blockIdx.x) * 8 * (NB / 2), glu.rb_stride,
                                                                0, glu.rb_stride * 16, x16, Kp, xscale, xg, rows,
                                                                reinterpret_cast<float *>(hidden), ldh, xt, 0, k.nsteps, glu);
}

// A wave's buffer window runs from its gate row-block to the end of its up row-block.
bool nint_prefill_glu_capable(const mfq_nint_desc *d) {
    return (d->kind == 1 || (d->bits == 5 && d->gs == 28)) && d->neuron_len >= 8 && d->out % 32 == 0 &&
           (d->out / 32 + 8) * d->rowblock_bytes < (1ll << 32);
}

// x16 / xscale / xg as nint_prefill takes them; hidden [M, ldh] halves, column c = act(row c) * row W + c
int nint_prefill_glu(const mfq_nint_desc *d, const void *weight, const uint16_t *x16, int Kp, const float *xscale,
                     const uint32_t *xg, int M, void *hidden, int64_t ldh, int f16, int gelu, hipStream_t st) {
    const NintK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const int rbw = d->out / 32;  // gate row-blocks
    const GluOut glu{rbw, gelu, f16};
#define MFQ_PREFILL_GLU_CFG(UNIT, B, G, MT, PF, XD)                                                            \
    {                                                                                                          \
        const dim3 grid(static_cast<unsigned>(ceil_div(rbw, 8)), static_cast<unsigned>(ceil_div(M, MT * 16))); \
        const size_t lds = prefill_lds_bytes(MT * 16, G, (XD) == 0 ? 4 : 2);                                   \
        auto kern = nint_prefill_glu_kernel<UNIT<B, G>, MT, 2, PF, XD>;                                        \
        if (lds > 65536) {                                                                                     \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                           \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
            MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nint_prefill_glu: %s", hipGetErrorString(e));        \
        }                                                                                                      \
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, k, w, x16, Kp, xscale, xg, M,                       \
                           static_cast<uint16_t *>(hidden), ldh, glu);                                         \
        return check_launch("nint_prefill_glu");                                                               \
    }
    // the two tile shapes of nint_prefill with a gate / up pair per wave, 64 or 128 tokens: the cheaper by rounds of 256
    // blocks x tile rows, the short tile at 0.9 of the tall one's rate (its weight fragments feed half as many MFMAs)
    const double cost_tall = static_cast<double>(ceil_div(ceil_div(rbw, 8) * ceil_div(M, 128), 256)) * 128;
    const double cost_short = static_cast<double>(ceil_div(ceil_div(rbw, 8) * ceil_div(M, 64), 256)) * 64 / 0.9;
    const bool small = cost_short < cost_tall;
#define MFQ_PREFILL_GLU(UNIT, B, G)                                                                            \
    if (k.bits == B && k.gs == G) {                                                                            \
        constexpr bool dma = G % 8 == 0, dma128 = dma && prefill_lds_bytes(128, G, 4) <= 160 * 1024;           \
        if (small) MFQ_PREFILL_GLU_CFG(UNIT, B, G, 4, 4, (dma ? 0 : 4))                                        \
        MFQ_PREFILL_GLU_CFG(UNIT, B, G, 8, 4, (dma128 ? 0 : (UNIT<B, G>::D >= 5 ? 1 : 2)))                     \
    }
    if (k.kind == 1) {
        MFQ_PREFILL_GLU(PairedUnit, 4, 32) MFQ_PREFILL_GLU(PairedUnit, 4, 24) MFQ_PREFILL_GLU(PairedUnit, 4, 16)
        MFQ_PREFILL_GLU(PairedUnit, 4, 48) MFQ_PREFILL_GLU(PairedUnit, 3, 24) MFQ_PREFILL_GLU(PairedUnit, 2, 16)
        MFQ_PREFILL_GLU(PairedUnit, 2, 32)
    } else {
        MFQ_PREFILL_GLU(GenericUnit, 5, 28)
    }
#undef MFQ_PREFILL_GLU
#undef MFQ_PREFILL_GLU_CFG
    return fail(MFQ_ERR_UNSUPPORTED, "nint_prefill_glu: no kernel for NINT%d-%d", k.bits, k.gs);
}

}  // namespace mfq
