// NINT: device layout plan, load-time repack, bit-exact dequantizer and the decode GEMV.
//
// Layout (one allocation per tensor):
//   row-block rb (16 neurons) -> step s (16 groups per neuron) -> three lane-interleaved regions
//     Q: [j=0..3][lane=0..63][dwords]   codes of group 16s + 4j + (lane>>4) of neuron 16rb + (lane&15)
//     T: [lane][4 bytes]                one tail byte per j (3-bit units only)
//     S: [lane][8 bytes]                (sub_scale, sub_min) per j
//   then float ns[16*n_rowblocks], float nm[16*n_rowblocks].
// A wave therefore streams a contiguous span of HBM per step and every load instruction of the
// wave covers whole 128-byte lines.
//
// "Paired" units keep two code fields 16 bits apart in each dword (even weight in the low half,
// odd weight in the high half) so that one AND/OR turns a dword into two exact bf16 (or fp16)
// integers biased by 128 (1024), ready for a packed dot product against the natural (x[2i], x[2i+1])
// activation pairs.  The bias is removed per group with the group sum of x.
#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_body.hpp"
#include "nint_mfma.hpp"
#include "nint_prefill.hpp"

namespace mfq {

// ---- repack ----------------------------------------------------------------------------
__global__ void nint_repack_kernel(NintK k, const uint8_t *__restrict__ payload, int64_t payload_bytes, int legacy,
                                   uint8_t *__restrict__ dst) {
    const int lane = threadIdx.x;
    const int rb = blockIdx.x, s = blockIdx.y;
    const int r = lane & 15, kb = lane >> 4;
    const int row = rb * 16 + r;
    const int64_t out = k.out, ng = k.ng, gs = k.gs;
    const int64_t sub_count = out * ng, q_count = out * ng * gs;
    const int sb = legacy ? 8 : k.sub_bits, qb = legacy ? 8 : k.bits;
    const int64_t ss_bytes = (sub_count * sb + 7) / 8, q_bytes = (q_count * qb + 7) / 8;
    const uint8_t *ss_s = payload + 4 * out;
    const uint8_t *sm_s = ss_s + ss_bytes;
    const uint8_t *q_s = sm_s + ss_bytes;
    uint8_t *sp = dst + rb * k.rowblock_bytes + s * k.step_bytes;
    uint32_t *qreg = reinterpret_cast<uint32_t *>(sp);
    uint8_t *treg = sp + 4 * 64 * k.dwords * 4;
    uint8_t *sreg = treg + (k.tail ? 256 : 0);
    for (int j = 0; j < 4; ++j) {
        const int g = 16 * s + 4 * j + kb;
        const bool live = row < k.out && g < k.ng;
        uint32_t q[16];
        for (int w = 0; w < k.dwords; ++w) q[w] = 0;
        uint32_t tail = 0, ssv = 0, smv = 0;
        if (live) {
            const int64_t u = static_cast<int64_t>(row) * ng + g;
            ssv = read_bits(ss_s, u, sb, ss_bytes);
            smv = read_bits(sm_s, u, sb, ss_bytes);
            for (int i = 0; i < k.gs; ++i) {
                const uint32_t c = read_bits(q_s, u * gs + i, qb, q_bytes) & ((1u << k.bits) - 1u);
                if (k.kind == 0) {
                    const int bit = i * k.bits;
                    const int w = bit >> 5, sh = bit & 31;
                    q[w] |= c << sh;
                    if (sh + k.bits > 32) q[w + 1] |= c >> (32 - sh);
                } else if (k.bits == 3 && i >= 20) {
                    if (i == 20) tail |= c;
                    else if (i == 21) tail |= c << 3;
                    else {
                        const int h = (i == 23) ? 16 : 0;
                        q[1] |= (c & 1u) << (15 + h);
                        tail |= ((c >> 1) & 1u) << (i == 23 ? 7 : 6);
                        q[0] |= ((c >> 2) & 1u) << (15 + h);
                    }
                } else {
                    int w, b;
                    paired_pos(k.bits, i, w, b);
                    q[w] |= c << b;
                }
            }
        }
        for (int w = 0; w < k.dwords; ++w) qreg[(j * 64 + lane) * k.dwords + w] = q[w];
        if (k.tail) treg[lane * 4 + j] = static_cast<uint8_t>(tail);
        sreg[lane * 8 + 2 * j] = static_cast<uint8_t>(ssv);
        sreg[lane * 8 + 2 * j + 1] = static_cast<uint8_t>(smv);
    }
    if (s == 0 && kb == 0) {
        float *anchors = reinterpret_cast<float *>(dst + k.anchors_off);
        const uint16_t *ns16 = reinterpret_cast<const uint16_t *>(payload);
        const uint16_t *nm16 = ns16 + out;
        const int out_pad = 16 * k.n_rowblocks;
        anchors[row] = row < k.out ? f16_to_f32(ns16[row]) : 0.f;
        anchors[out_pad + row] = row < k.out ? f16_to_f32(nm16[row]) : 0.f;
    }
}

// ---- dequant (bit-exact: four separate fp32 roundings) -----------------------------------
template <typename OutT>
__global__ void nint_dequant_kernel(NintK k, const uint8_t *__restrict__ w, OutT *__restrict__ outp, int64_t ld,
                                    float *__restrict__ rowscale, int kpad) {
    const int lane = threadIdx.x;
    const int rb = blockIdx.x, s = blockIdx.y;
    const int r = lane & 15, kb = lane >> 4;
    const int row = rb * 16 + r;
    const uint8_t *sp = w + rb * k.rowblock_bytes + s * k.step_bytes;
    const uint32_t *qreg = reinterpret_cast<const uint32_t *>(sp);
    const uint8_t *treg = sp + 4 * 64 * k.dwords * 4;
    const uint8_t *sreg = treg + (k.tail ? 256 : 0);
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    const int out_pad = 16 * k.n_rowblocks;
    if (row >= k.out) return;
    const float ns = anchors[row], nm = anchors[out_pad + row];
    float inv = 1.f;
    if constexpr (sizeof(OutT) == 2) {
        // fp16 output is scaled per neuron by an exact power of two so the largest representable
        // weight of the neuron lands near 2^12; the GEMM epilogue multiplies it back.
        const float bound = ns * static_cast<float>(((1 << k.sub_bits) - 1) * ((1 << k.bits) - 1)) +
                            nm * static_cast<float>((1 << k.sub_bits) - 1);
        int e = 0;
        if (bound > 0.f) { frexpf(bound, &e); }
        inv = ldexpf(1.f, 12 - e);
        if (s == 0 && kb == 0) {
            rowscale[row] = ldexpf(1.f, e - 12);
            for (int col = k.neuron_len; col < kpad; ++col) outp[row * ld + col] = 0;  // K padding of the GEMM
        }
    }
    for (int j = 0; j < 4; ++j) {
        const int g = 16 * s + 4 * j + kb;
        if (g >= k.ng) continue;
        uint32_t q[16];
        for (int t = 0; t < k.dwords; ++t) q[t] = qreg[(j * 64 + lane) * k.dwords + t];
        const uint32_t tail = k.tail ? treg[lane * 4 + j] : 0u;
        const float ss = static_cast<float>(sreg[lane * 8 + 2 * j]);
        const float sm = static_cast<float>(sreg[lane * 8 + 2 * j + 1]);
        const float d_eff = __fmul_rn(ns, ss);
        const float m_eff = __fmul_rn(nm, sm);
        for (int i = 0; i < k.gs; ++i) {
            const int col = g * k.gs + i;
            if (col >= k.neuron_len) break;
            const float qf = static_cast<float>(unit_code(k, q, tail, i));
            const float v = __fsub_rn(__fmul_rn(d_eff, qf), m_eff);
            if constexpr (sizeof(OutT) == 2) outp[row * ld + col] = f32_to_f16_rne(v * inv);
            else outp[row * ld + col] = v;
        }
    }
}

// ---- GEMV ------------------------------------------------------------------------------
// Block shape: the waves of a block split the K steps (spw steps each, at most 16 waves) and walk
// through rbw row-blocks.  A wave takes up to three (row-block, step) items -- what the kernel variant
// without a prefetch ring holds in registers -- as long as the grid keeps about gemv_target_waves()
// waves; long neurons spend the items on K (fewer waves to reduce), short ones on row-blocks (the
// staged activations are reused).  MFQ_GEMV_SPW / MFQ_GEMV_RBW override the choice for tuning.
void gemv_shape(const NintK &k, int mb, int &spw, int &nwaves, int &rbw, size_t &lds_bytes) {
    static const int env_spw = tune_env("MFQ_GEMV_SPW", 0);
    static const int env_rbw = tune_env("MFQ_GEMV_RBW", 0);
    const int64_t items = static_cast<int64_t>(k.n_rowblocks) * k.nsteps;
    int per_wave = static_cast<int>(items / gemv_target_waves());
    per_wave = per_wave < 1 ? 1 : (per_wave > 3 ? 3 : per_wave);
    const int spw_min = static_cast<int>(ceil_div(k.nsteps, 16));
    spw = k.nsteps >= 16 ? per_wave : 1;
    if (spw < spw_min) spw = spw_min;
    if (env_spw > 0) spw = env_spw < spw_min ? spw_min : env_spw;
    if (spw > k.nsteps) spw = k.nsteps;
    nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const bool unit = k.kind == 1 || mfma_generic_profile(k);
    rbw = unit ? per_wave / spw : 1;
    if (rbw < 1) rbw = 1;
    // Between one and two blocks per compute unit some units would get two blocks and the others one: two row-blocks
    // per block then give every unit one block with both row-blocks' requests in flight at once
    // (NINT5-28 6144 x 4096: 11.0 -> 7.9 us).
    if (unit && rbw == 1 && k.n_rowblocks > gemv_cu_count() && k.n_rowblocks <= 2 * gemv_cu_count()) rbw = 2;
    if (env_rbw > 0 && unit) rbw = env_rbw;
    if (rbw > kMaxRbw) rbw = kMaxRbw;
    if (rbw > k.n_rowblocks) rbw = k.n_rowblocks;
    while (rbw > 1 && static_cast<int64_t>(rbw) * k.rowblock_bytes >= (1ll << 31)) --rbw;
    lds_bytes = gemv_lds_bytes(mb, spw, k.gs, nwaves, rbw);
}

#define MFQ_SINGLE_ARG(...) __VA_ARGS__
template <int XF16, int MB>
static int launch_gemv_mb(const NintK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                          hipStream_t st) {
    int spw, nwaves, rbw;
    size_t lds;
    gemv_shape(k, MB, spw, nwaves, rbw, lds);
    MFQ_REQUIRE(lds <= kMaxDynamicLds, MFQ_ERR_UNSUPPORTED, "nint_gemv: neuron_len %d needs %zu bytes of LDS", k.neuron_len, lds);
    MFQ_REQUIRE(k.rowblock_bytes < (1ll << 31), MFQ_ERR_UNSUPPORTED, "nint_gemv: neuron_len %d is too long", k.neuron_len);
    const dim3 block(64 * nwaves);
    // blocks that stage more than 64 KB of activations (neurons longer than about 29k) opt in to the larger LDS
#define MFQ_GEMV_LAUNCH(KERN, GRID, ...)                                                                     \
    do {                                                                                                     \
        auto kern_ = KERN;                                                                                   \
        if (int rc_ = allow_dynamic_lds(reinterpret_cast<const void *>(kern_), lds, "nint_gemv")) return rc_; \
        hipLaunchKernelGGL(kern_, GRID, block, lds, st, __VA_ARGS__);                                        \
    } while (0)
    // Waves with at most three items keep the staged activations in registers when a group's pairs fit one row of
    // lanes and the rows can be fetched pair by pair (4-byte aligned rows, even K): LDS then only holds the sums.
    static const int env_xreg = tune_env("MFQ_GEMV_XREG", 1);
    const bool xreg_rows = MB <= 2 && spw * rbw <= 3 && k.neuron_len % 2 == 0 && (M == 1 || ldx % 2 == 0) &&
                           (reinterpret_cast<uintptr_t>(x) & 3) == 0 && env_xreg != 0;
    const size_t lds_xreg = static_cast<size_t>(rbw) * nwaves * MB * 16 * 4;
#define MFQ_XREG(UNIT)                                                                                         \
    if constexpr ((MB == 1 || (MB == 2 && UNIT::CBITS != 0)) && UNIT::NPAIR <= 16) { /* two rows of NINT5-28 spill */ \
        if (xreg_rows) {                                                                                       \
            const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, rbw)), static_cast<unsigned>(ceil_div(M, MB))); \
            hipLaunchKernelGGL((nint_gemv_xreg_kernel<UNIT, XF16, MB>), grid, block, lds_xreg, st, k, w, x, ldx, M, y, ldy, \
                               spw, rbw);                                                                      \
            return check_launch("nint_gemv_xreg");                                                             \
        }                                                                                                      \
    }
#define MFQ_PAIRED(B, G)                                                                                     \
    if (k.bits == B && k.gs == G) {                                                                          \
        MFQ_XREG(MFQ_SINGLE_ARG(PairedUnit<B, G>))                                                           \
        const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, rbw)), static_cast<unsigned>(ceil_div(M, MB))); \
        if (spw * rbw <= 3)                                                                                  \
            MFQ_GEMV_LAUNCH((nint_gemv_paired_kernel<B, G, XF16, MB, false>), grid, k, w, x, ldx, M, y, ldy, spw, rbw); \
        else                                                                                                 \
            MFQ_GEMV_LAUNCH((nint_gemv_paired_kernel<B, G, XF16, MB, true>), grid, k, w, x, ldx, M, y, ldy, spw, rbw); \
        return check_launch("nint_gemv_paired");                                                             \
    }
    if (k.kind == 1) {
        MFQ_PAIRED(4, 32) MFQ_PAIRED(4, 24) MFQ_PAIRED(4, 16) MFQ_PAIRED(4, 48) MFQ_PAIRED(3, 24) MFQ_PAIRED(2, 16)
        MFQ_PAIRED(2, 32)
        return fail(MFQ_ERR_UNSUPPORTED, "nint_gemv: no paired kernel for NINT%d-%d", k.bits, k.gs);
    }
#undef MFQ_PAIRED
#define MFQ_NATURAL(UNIT, B, G)                                                                              \
    if (k.kind == 0 && k.bits == B && k.gs == G) {                                                           \
        MFQ_XREG(MFQ_SINGLE_ARG(UNIT<B, G>))                                                                 \
        const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, rbw)), static_cast<unsigned>(ceil_div(M, MB))); \
        if (spw * rbw <= 3)                                                                                  \
            MFQ_GEMV_LAUNCH((nint_gemv_natural_kernel<B, G, XF16, MB, false>), grid, k, w, x, ldx, M, y, ldy, spw, rbw); \
        else                                                                                                 \
            MFQ_GEMV_LAUNCH((nint_gemv_natural_kernel<B, G, XF16, MB, true>), grid, k, w, x, ldx, M, y, ldy, spw, rbw); \
        return check_launch("nint_gemv_natural");                                                            \
    }
    MFQ_GENERIC_PROFILES(MFQ_NATURAL)
#undef MFQ_NATURAL
    const dim3 grid(k.n_rowblocks, static_cast<unsigned>(ceil_div(M, MB)));
    MFQ_GEMV_LAUNCH((nint_gemv_generic_kernel<XF16, MB>), grid, k, w, x, ldx, M, y, ldy, spw);
#undef MFQ_GEMV_LAUNCH
    return check_launch("nint_gemv_generic");
}

// ---- small batches on the matrix cores ----------------------------------------------------
static bool mfma_eligible(const NintK &k, const void *x, int64_t ldx) {
    return (k.kind == 1 || mfma_generic_profile(k)) && k.neuron_len >= 8 && k.neuron_len % 8 == 0 && ldx % 8 == 0 &&
           (reinterpret_cast<uintptr_t>(x) & 15) == 0 && 4 * k.rowblock_bytes < (1ll << 31) &&
           (15 * ldx + k.neuron_len) * 2 < (1ll << 32);  // a tile's 16 rows through one buffer window
}

bool nint_stream_capable(const mfq_nint_desc *d) {
    const NintK k = to_k(d);
    return (k.kind == 1 || mfma_generic_profile(k)) && k.neuron_len >= 8 && k.neuron_len % 8 == 0 &&
           4 * k.rowblock_bytes < (1ll << 31);
}

template <int XF16, int NB>
static int launch_mfma_nb(const NintK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                          hipStream_t st) {
    const int64_t groups = ceil_div(k.n_rowblocks, NB);
    // Up to 16 waves per block (128 registers each) where the grid is small and K has nine to sixteen steps: a wave then
    // walks one step instead of two, and a compute unit holds twice the waves to hide each other's waits (6144 x 4096
    // at 16 rows: NINT3-24 9.8 -> 8.5 us, NINT5-28 13.5 -> 11.4 us).  Three row-blocks per wave do not fit 128 registers
    // (NINT5-28 spills and loses 18 %), longer K gains nothing.  MFQ_MFMA_WIDE = 0 keeps eight waves.
    static const int env_wide = tune_env("MFQ_MFMA_WIDE", 1);
    const bool wide = env_wide && NB <= 2 && k.nsteps > 8 && k.nsteps <= 16 && groups * ceil_div(M, 16) <= 2 * gemv_cu_count();
    int spw = static_cast<int>(ceil_div(k.nsteps, wide ? 16 : 8));
    while (spw < k.nsteps && groups * ceil_div(k.nsteps, spw) > 8192) ++spw;
    const int nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const size_t lds = static_cast<size_t>(nwaves) * NB * 1024;
    const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(ceil_div(M, 16))), block(64 * nwaves);
#define MFQ_MFMA(UNIT, B, G)                                                                                   \
    if (k.bits == B && k.gs == G) {                                                                             \
        if constexpr (NB <= 2) {                                                                                \
            if (wide) {                                                                                         \
                hipLaunchKernelGGL((nint_mfma_kernel<UNIT<B, G>, XF16, NB, 16>), grid, block, lds, st, k, w, x, ldx, M, y, \
                                   ldy, spw);                                                                   \
                return check_launch("nint_mfma");                                                               \
            }                                                                                                   \
        }                                                                                                       \
        hipLaunchKernelGGL((nint_mfma_kernel<UNIT<B, G>, XF16, NB>), grid, block, lds, st, k, w, x, ldx, M, y, ldy, \
                           spw);                                                                                \
        return check_launch("nint_mfma");                                                                       \
    }
    if (k.kind == 1) {
        MFQ_MFMA(PairedUnit, 4, 32) MFQ_MFMA(PairedUnit, 4, 24) MFQ_MFMA(PairedUnit, 4, 16) MFQ_MFMA(PairedUnit, 4, 48)
        MFQ_MFMA(PairedUnit, 3, 24) MFQ_MFMA(PairedUnit, 2, 16) MFQ_MFMA(PairedUnit, 2, 32)
    } else {
        // (twelve dwords a unit: one row-block of NINT8-48 per wave; two spill and run 1.4x slower)
        if constexpr (NB > 1) {
            if (k.bits == 8) return launch_mfma_nb<XF16, 1>(k, w, x, ldx, M, y, ldy, st);
        }
        MFQ_GENERIC_PROFILES(MFQ_MFMA)
    }
#undef MFQ_MFMA
    return fail(MFQ_ERR_UNSUPPORTED, "nint_mfma: no kernel for NINT%d-%d", k.bits, k.gs);
}

template <int XF16>
static int launch_mfma(const NintK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                       hipStream_t st) {
    // row-blocks per wave: as many as still leave about 1500 waves over all 16-row tiles (a block has at most 8 waves);
    // more row-blocks share the activation fragments, and the tiles of one row-block group re-read its weights from L2
    const int64_t wpb = (k.nsteps < 8 ? k.nsteps : 8) * ceil_div(M, 16);
    static const int env_nb = tune_env("MFQ_MFMA_NB", 0);
    if (env_nb == 4) return launch_mfma_nb<XF16, 4>(k, w, x, ldx, M, y, ldy, st);
    if (env_nb == 3) return launch_mfma_nb<XF16, 3>(k, w, x, ldx, M, y, ldy, st);
    if (env_nb == 2) return launch_mfma_nb<XF16, 2>(k, w, x, ldx, M, y, ldy, st);
    if (env_nb == 1) return launch_mfma_nb<XF16, 1>(k, w, x, ldx, M, y, ldy, st);
    // Small grids: the blocks of one launch should be one even round over the compute units.  Cost of NB row-blocks per
    // wave = rounds of blocks x NB, the larger NB on a tie (it re-reads the activations less often): 12288 x 4096 takes
    // NB = 3 (256 blocks; 15.9 -> 13.0 us for NINT3-24 at 16 rows), 6144 x 4096 NB = 2, or 3 with two tiles.
    const int64_t cus = gemv_cu_count(), tiles = ceil_div(M, 16);
    if (ceil_div(k.n_rowblocks, 4) * tiles < 2 * cus) {
        int best = 1;
        int64_t best_cost = ceil_div(static_cast<int64_t>(k.n_rowblocks) * tiles, cus);
        for (int nb = 2; nb <= 4; ++nb) {
            const int64_t cost = ceil_div(ceil_div(k.n_rowblocks, nb) * tiles, cus) * nb;
            if (cost <= best_cost) best = nb, best_cost = cost;
        }
        if (best == 4) return launch_mfma_nb<XF16, 4>(k, w, x, ldx, M, y, ldy, st);
        if (best == 3) return launch_mfma_nb<XF16, 3>(k, w, x, ldx, M, y, ldy, st);
        if (best == 2) return launch_mfma_nb<XF16, 2>(k, w, x, ldx, M, y, ldy, st);
        return launch_mfma_nb<XF16, 1>(k, w, x, ldx, M, y, ldy, st);
    }
    if (ceil_div(k.n_rowblocks, 4) * wpb >= 1536) return launch_mfma_nb<XF16, 4>(k, w, x, ldx, M, y, ldy, st);
    if (ceil_div(k.n_rowblocks, 2) * wpb >= 1536) return launch_mfma_nb<XF16, 2>(k, w, x, ldx, M, y, ldy, st);
    return launch_mfma_nb<XF16, 1>(k, w, x, ldx, M, y, ldy, st);
}

// Up to 16 rows with the activations resident in LDS (nint_mfma_resident_kernel): one block per compute unit walks its
// row-block groups.  NB as in launch_mfma: the fewest rounds of groups over the compute units, the larger NB on a tie.
static bool mfma_resident_shape(const NintK &k, int M, int &nb, int &spw, int &nwaves, size_t &lds, int &red_slots) {
    static const int on = tune_env("MFQ_MFMA_RESIDENT", 1);
    if (!on || M > 16 || k.kind != 1 || (k.gs != 32 && k.gs != 16) || k.anchors_off >= (1ll << 31)) return false;
    nwaves = k.nsteps < 8 ? k.nsteps : 8;
    spw = static_cast<int>(ceil_div(k.nsteps, nwaves));
    // one step per wave: with more (4096 x 12288 at 4 rows, three steps) the older kernel measured as fast (13.0 vs 13.9 us)
    if (spw > 1 || spw * M * 2 * k.gs > 1024) return false;  // a wave stages at most 1024 16-byte chunks
    const int64_t cus = gemv_cu_count();
    int64_t best_cost = 0;
    nb = 0;
    for (int c = 1; c <= 3; ++c) {
        const int64_t cost = ceil_div(ceil_div(k.n_rowblocks, c), cus) * c;
        if (mfma_resident_lds(nwaves, c, spw, M, k.gs) > kMaxDynamicLds) break;
        if (nb == 0 || cost <= best_cost) nb = c, best_cost = cost;
    }
    if (nb == 0) return false;
    // as many reduction areas as the block has groups, where they fit (no barrier between groups then)
    const int per_block = static_cast<int>(ceil_div(ceil_div(k.n_rowblocks, nb), cus));
    red_slots = per_block <= 4 && mfma_resident_lds(nwaves, nb, spw, M, k.gs, per_block) <= kMaxDynamicLds ? per_block : 1;
    lds = mfma_resident_lds(nwaves, nb, spw, M, k.gs, red_slots);
    return true;
}

template <int XF16>
static int launch_mfma_resident(const NintK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y,
                                int64_t ldy, int nb, int spw, int nwaves, size_t lds, int red_slots, hipStream_t st) {
    const int64_t groups = ceil_div(k.n_rowblocks, nb), cus = gemv_cu_count();
    const dim3 grid(static_cast<unsigned>(groups < cus ? groups : cus), 1), block(64 * nwaves);
#define MFQ_RES_NB(UNIT, B, G, NBV)                                                                                  \
    {                                                                                                                \
        auto kern = nint_mfma_resident_kernel<UNIT<B, G>, XF16, NBV>;                                                \
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds, "nint_mfma_resident")) return rc;  \
        hipLaunchKernelGGL(kern, grid, block, lds, st, k, w, x, ldx, M, y, ldy, spw, red_slots);                     \
        return check_launch("nint_mfma_resident");                                                                   \
    }
#define MFQ_RES(UNIT, B, G)                                                                                          \
    if (k.bits == B && k.gs == G) {                                                                                  \
        if (nb == 1) MFQ_RES_NB(UNIT, B, G, 1)                                                                       \
        if (nb == 2) MFQ_RES_NB(UNIT, B, G, 2)                                                                       \
        MFQ_RES_NB(UNIT, B, G, 3)                                                                                    \
    }
    MFQ_RES(PairedUnit, 4, 32) MFQ_RES(PairedUnit, 4, 16) MFQ_RES(PairedUnit, 2, 16) MFQ_RES(PairedUnit, 2, 32)
#undef MFQ_RES
#undef MFQ_RES_NB
    return fail(MFQ_ERR_UNSUPPORTED, "nint_mfma_resident: no kernel for NINT%d-%d", k.bits, k.gs);
}

// ---- prefill: block-tiled MFMA GEMM with in-register dequantization ---------------------------
bool nint_prefill_capable(const mfq_nint_desc *d) {
    return (d->kind == 1 || (d->bits == 5 && d->gs == 28) || (d->bits == 6 && d->gs == 24)) && d->neuron_len >= 8 &&
           4 * d->rowblock_bytes < (1ll << 31);
}
size_t nint_prefill_xg_bytes(const mfq_nint_desc *d, int M) { return static_cast<size_t>(M) * d->nsteps * 64; }

// x16 [M, Kp] fp16 (rows scaled by 1 / xscale[m], zero beyond K), xg = the rows' group sums (x_prep_groups)
// y[m][n] = sum over the splits of part[z][m][n], in split order
__global__ __launch_bounds__(256) void prefill_sum_splits_kernel(const float *__restrict__ part, int64_t ystride, int splits,
                                                                 int M, int N, float *__restrict__ y, int64_t ldy) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;  // float4 index
    const int n4 = N >> 2;
    if (i >= static_cast<int64_t>(M) * n4) return;
    const int m = static_cast<int>(i / n4), c = static_cast<int>(i - static_cast<int64_t>(m) * n4) * 4;
    float4_t acc = *reinterpret_cast<const float4_t *>(part + static_cast<int64_t>(m) * N + c);
    for (int z = 1; z < splits; ++z) acc += *reinterpret_cast<const float4_t *>(part + z * ystride + static_cast<int64_t>(m) * N + c);
    if ((ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0) {
        *reinterpret_cast<float4_t *>(y + static_cast<int64_t>(m) * ldy + c) = acc;
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) y[static_cast<int64_t>(m) * ldy + c + t] = acc[t];
    }
}

int prefill_sum_splits(const float *part, int64_t ystride, int splits, int M, int N, float *y, int64_t ldy, hipStream_t st) {
    const int64_t n4 = static_cast<int64_t>(M) * (N / 4);
    hipLaunchKernelGGL(prefill_sum_splits_kernel, dim3(static_cast<unsigned>(ceil_div(n4, 256))), dim3(256), 0, st, part,
                       ystride, splits, M, N, y, ldy);
    return check_launch("prefill_sum_splits");
}

// Splits over K of a prefill launch: grids of 64-token tiles that leave CUs idle are cut along K (up to eight
// splits) as long as every split keeps at least two steps and the neuron count allows 16-byte partial rows; the partial results go to a
// workspace and are added in split order (deterministic).  1 = no split.
int nint_prefill_splits(const mfq_nint_desc *d, int M) {
    static const int env = tune_env("MFQ_PREFILL_SPLITS", 0);
    const int64_t blocks = ceil_div(d->n_rowblocks, 16) * ceil_div(M, 64);
    if (blocks > 128 || d->out % 4) return 1;
    int splits = static_cast<int>(256 / blocks);
    if (splits > 8) splits = 8;
    if (splits > d->nsteps / 2) splits = d->nsteps / 2;
    if (env > 0) splits = env;
    if (splits <= 1) return 1;
    const int spz = static_cast<int>(ceil_div(d->nsteps, splits));
    return static_cast<int>(ceil_div(d->nsteps, spz));  // no empty split
}
size_t nint_prefill_split_bytes(const mfq_nint_desc *d, int M) {
    const int splits = nint_prefill_splits(d, M);
    return splits > 1 ? static_cast<size_t>(splits) * M * d->out * 4 : 0;
}

// part: nint_prefill_split_bytes(d, M) bytes when nint_prefill_splits(d, M) > 1
int nint_prefill(const mfq_nint_desc *d, const void *weight, const uint16_t *x16, int Kp, const float *xscale,
                 uint32_t *xg, int M, float *y, int64_t ldy, float *part, hipStream_t st) {
    const NintK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const int splits = part ? nint_prefill_splits(d, M) : 1;
    const int spz = static_cast<int>(ceil_div(k.nsteps, splits));
    const int64_t ystride = static_cast<int64_t>(M) * k.out;
    float *yk = splits > 1 ? part : y;
    const int64_t ldk = splits > 1 ? k.out : ldy;
#define MFQ_PREFILL_CFG(UNIT, B, G, MT, NB, PF, XD)                                                            \
    {                                                                                                          \
        const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, 8 * NB)),                                \
                        static_cast<unsigned>(ceil_div(M, MT * 16)), static_cast<unsigned>(splits));           \
        const size_t lds = prefill_lds_bytes(MT * 16, G, (XD) == 0 ? 4 : 2);                                   \
        auto kern = nint_prefill_kernel<UNIT<B, G>, MT, NB, 1, 8, PF, XD>;                                     \
        if (lds > 65536) {                                                                                     \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                           \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
            MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nint_prefill: %s", hipGetErrorString(e));            \
        }                                                                                                      \
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, k, w, x16, Kp, xscale, xg, M, yk, ldk, spz, ystride); \
        if (splits > 1) {                                                                                      \
            const int64_t n4 = static_cast<int64_t>(M) * (k.out / 4);                                          \
            hipLaunchKernelGGL(prefill_sum_splits_kernel, dim3(static_cast<unsigned>(ceil_div(n4, 256))), dim3(256), 0, st, \
                               part, ystride, splits, M, k.out, y, ldy);                                       \
        }                                                                                                      \
        return check_launch("nint_prefill");                                                                   \
    }
    // Block = 8 waves side by side on the neurons, each with four unit buffers per row-block (three sub-steps of
    // weights in flight).  While 64-token x 256-neuron tiles give at most one block per CU, they are used with four
    // activation tiles in flight: the time is then that of one block's walk through K, and short tiles walk fastest.
    // Beyond that, the cheaper of 128 x 256 (every dequantized fragment feeds eight MFMAs) and 64 x 384 (three
    // row-blocks per wave) by rounds of 256 blocks x tile area; the second runs at 0.97 of the first's rate per area.
    const bool small = ceil_div(k.n_rowblocks, 16) * ceil_div(M, 64) <= 256;
    const double cost_a = static_cast<double>(ceil_div(ceil_div(k.n_rowblocks, 16) * ceil_div(M, 128), 256)) * (128 * 256);
    const double cost_b = static_cast<double>(ceil_div(ceil_div(k.n_rowblocks, 24) * ceil_div(M, 64), 256)) * (64 * 384) / 0.97;
    const bool wide3 = cost_b < cost_a;
#define MFQ_PREFILL(UNIT, B, G)                                                                                       \
    if (k.bits == B && k.gs == G) {                                                                                   \
        /* XD = 0 (groups of whole 16-byte chunks): the activation tiles are copied straight into a ring of four LDS */ \
        /* buffers, as long as those fit; else they pass through registers, as many tiles in flight as registers allow */ \
        constexpr bool dma = G % 8 == 0, dma128 = dma && prefill_lds_bytes(128, G, 4) <= 160 * 1024;                  \
        if (small) MFQ_PREFILL_CFG(UNIT, B, G, 4, 2, 4, (dma ? 0 : 4))                                                \
        if constexpr (UNIT<B, G>::D <= 4) {                                                                           \
            if (wide3) MFQ_PREFILL_CFG(UNIT, B, G, 4, 3, 4, (dma ? 0 : 2))                                            \
        }                                                                                                             \
        MFQ_PREFILL_CFG(UNIT, B, G, 8, 2, 4, (dma128 ? 0 : (UNIT<B, G>::D >= 5 ? 1 : 2)))                             \
    }
    static const int env_big = tune_env("MFQ_PREFILL_BIG", 0);
    if (env_big && k.bits == 4 && k.gs == 32) {
        if (env_big == 1) MFQ_PREFILL_CFG(PairedUnit, 4, 32, 8, 3, 4, 0)
        if (env_big == 2) MFQ_PREFILL_CFG(PairedUnit, 4, 32, 8, 3, 2, 0)
    }
    if (k.kind == 1) {
        MFQ_PREFILL(PairedUnit, 4, 32) MFQ_PREFILL(PairedUnit, 4, 24) MFQ_PREFILL(PairedUnit, 4, 16)
        MFQ_PREFILL(PairedUnit, 4, 48) MFQ_PREFILL(PairedUnit, 3, 24) MFQ_PREFILL(PairedUnit, 2, 16)
        MFQ_PREFILL(PairedUnit, 2, 32)
    } else {
        MFQ_PREFILL(GenericUnit, 5, 28) MFQ_PREFILL(GenericUnit, 6, 24)
    }
#undef MFQ_PREFILL
#undef MFQ_PREFILL_CFG
    return fail(MFQ_ERR_UNSUPPORTED, "nint_prefill: no kernel for NINT%d-%d", k.bits, k.gs);
}

int nint_gemv_any(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                  int64_t ldy, hipStream_t st) {
    const NintK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    static const int valu_max = tune_env("MFQ_GEMV_VALU_MAX_M", 2);
    // two rows: the vector-ALU GEMV unpacks once and takes two dot products (10.6 vs 12.9 us on 12288x4096);
    // from three rows on the matrix-core kernel wins
    // NINT8-48: the vector-ALU bodies hold a step of twelve-dword units per row-block and spill; the matrix-core kernel
    // with one row-block per wave takes every batch from one row on (12288 x 4096: 28 us against 39)
    if ((M > valu_max || k.bits == 8) && mfma_eligible(k, x, ldx)) {
        int nb, spw, nwaves, red_slots;
        size_t lds;
        if (mfma_resident_shape(k, M, nb, spw, nwaves, lds, red_slots))
            return x_dtype == MFQ_X_F16 ? launch_mfma_resident<1>(k, w, xp, ldx, M, y, ldy, nb, spw, nwaves, lds, red_slots, st)
                                        : launch_mfma_resident<0>(k, w, xp, ldx, M, y, ldy, nb, spw, nwaves, lds, red_slots, st);
        return x_dtype == MFQ_X_F16 ? launch_mfma<1>(k, w, xp, ldx, M, y, ldy, st)
                                    : launch_mfma<0>(k, w, xp, ldx, M, y, ldy, st);
    }
    // LDS per block grows with MB; large K falls back to narrower row batches, and neurons whose one-row slice no
    // block can stage (beyond about 70k elements) go to the matrix-core kernel, whose LDS use does not depend on K.
    int mb = M >= 4 ? 4 : (M >= 2 ? 2 : 1);
    for (;;) {
        int spw, nwaves, rbw;
        size_t lds;
        gemv_shape(k, mb, spw, nwaves, rbw, lds);
        if (lds <= 65536 || mb == 1) {
            if (lds > kMaxDynamicLds && mfma_eligible(k, x, ldx))
                return x_dtype == MFQ_X_F16 ? launch_mfma<1>(k, w, xp, ldx, M, y, ldy, st)
                                            : launch_mfma<0>(k, w, xp, ldx, M, y, ldy, st);
            break;
        }
        mb >>= 1;
    }
    if (x_dtype == MFQ_X_F16) {
        if (mb == 4) return launch_gemv_mb<1, 4>(k, w, xp, ldx, M, y, ldy, st);
        if (mb == 2) return launch_gemv_mb<1, 2>(k, w, xp, ldx, M, y, ldy, st);
        return launch_gemv_mb<1, 1>(k, w, xp, ldx, M, y, ldy, st);
    }
    if (mb == 4) return launch_gemv_mb<0, 4>(k, w, xp, ldx, M, y, ldy, st);
    if (mb == 2) return launch_gemv_mb<0, 2>(k, w, xp, ldx, M, y, ldy, st);
    return launch_gemv_mb<0, 1>(k, w, xp, ldx, M, y, ldy, st);
}

int nint_dequant_f16(const mfq_nint_desc *d, const void *weight, void *w16, int64_t ld, float *rowscale, hipStream_t st) {
    const NintK k = to_k(d);
    hipLaunchKernelGGL((nint_dequant_kernel<uint16_t>), dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, st, k,
                       static_cast<const uint8_t *>(weight), static_cast<uint16_t *>(w16), ld, rowscale,
                       static_cast<int>(ld));
    return check_launch("nint_dequant_f16");
}

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_nint_plan(int bits, int sub_bits, int gs, int out, int neuron_len, mfq_nint_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nint_plan: null descriptor");
    MFQ_REQUIRE(bits >= 1 && bits <= 8, MFQ_ERR_UNSUPPORTED, "nint_plan: bits=%d outside [1,8]", bits);
    MFQ_REQUIRE(sub_bits >= 1 && sub_bits <= 8, MFQ_ERR_UNSUPPORTED, "nint_plan: sub_bits=%d outside [1,8]", sub_bits);
    MFQ_REQUIRE(gs >= 2 && gs <= 64 && gs % 2 == 0, MFQ_ERR_UNSUPPORTED, "nint_plan: groupsize=%d must be even and in [2,64]", gs);
    MFQ_REQUIRE(out > 0 && neuron_len > 0, MFQ_ERR_INVALID, "nint_plan: empty tensor %dx%d", out, neuron_len);
    d->bits = bits; d->sub_bits = sub_bits; d->gs = gs; d->out = out; d->neuron_len = neuron_len;
    d->ng = static_cast<int32_t>(ceil_div(neuron_len, gs));
    d->kind = paired_profile(bits, gs) ? 1 : 0;
    if (d->kind == 1) {
        d->dwords = bits == 3 ? 2 : gs * bits / 32;
        d->tail_bytes = bits == 3 ? 1 : 0;
    } else {
        d->dwords = static_cast<int32_t>(ceil_div(gs * bits, 32));
        d->tail_bytes = 0;
    }
    d->ngp = static_cast<int32_t>(ceil_div(d->ng, 16) * 16);
    d->nsteps = d->ngp / 16;
    d->n_rowblocks = static_cast<int32_t>(ceil_div(out, 16));
    d->step_bytes = 64ll * (16 * d->dwords + (d->tail_bytes ? 4 : 0) + 8);
    d->rowblock_bytes = d->step_bytes * d->nsteps;
    d->anchors_off = d->rowblock_bytes * d->n_rowblocks;
    d->total_bytes = d->anchors_off + 2ll * 16 * d->n_rowblocks * 4;
    const int64_t subs = static_cast<int64_t>(out) * d->ng;
    d->payload_bytes = 4ll * out + 2 * ((subs * sub_bits + 7) / 8) + (subs * gs * bits + 7) / 8;
    return MFQ_OK;
}

extern "C" int mfq_hip_nint_repack(const mfq_nint_desc *d, const void *payload, int64_t payload_bytes, int legacy_bytes,
                                   void *weight, mfq_stream_t stream) {
    MFQ_REQUIRE(d && payload && weight, MFQ_ERR_INVALID, "nint_repack: null argument");
    const int64_t subs = static_cast<int64_t>(d->out) * d->ng;
    const int64_t expect = legacy_bytes ? 4ll * d->out + 2 * subs + subs * d->gs : d->payload_bytes;
    MFQ_REQUIRE(payload_bytes == expect, MFQ_ERR_INVALID, "invalid NINT blob tail: remaining=%lld, expected=%lld",
                static_cast<long long>(payload_bytes), static_cast<long long>(expect));
    const NintK k = to_k(d);
    hipLaunchKernelGGL(nint_repack_kernel, dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(payload), payload_bytes, legacy_bytes,
                       static_cast<uint8_t *>(weight));
    return check_launch("nint_repack");
}

extern "C" int mfq_hip_nint_dequant_f32(const mfq_nint_desc *d, const void *weight, float *w_out, int64_t ld,
                                        mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && w_out, MFQ_ERR_INVALID, "nint_dequant_f32: null argument");
    MFQ_REQUIRE(ld >= d->neuron_len, MFQ_ERR_INVALID, "nint_dequant_f32: ld %lld < neuron_len %d",
                static_cast<long long>(ld), d->neuron_len);
    const NintK k = to_k(d);
    hipLaunchKernelGGL((nint_dequant_kernel<float>), dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(weight), w_out, ld, static_cast<float *>(nullptr), 0);
    return check_launch("nint_dequant_f32");
}

template <int XF16, int MB>
static int launch_gemv_swiglu(const NintK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, uint16_t *hidden,
                              int out_f16, int64_t ldh, hipStream_t st) {
    // a block takes a gate and an up row-block; its waves split the K steps, at most three (row-block, step) items each
    // without the prefetch ring
    const int nwaves = k.nsteps < 16 ? k.nsteps : 16;
    const int spw = static_cast<int>(ceil_div(k.nsteps, nwaves));
    const bool ring = 2 * spw > 3;
    const size_t lds = gemv_lds_bytes(MB, spw, k.gs, nwaves, 2);
    MFQ_REQUIRE(lds <= kMaxDynamicLds, MFQ_ERR_UNSUPPORTED, "nint_gemv_swiglu: neuron_len %d needs %zu bytes of LDS", k.neuron_len, lds);
    const dim3 grid(static_cast<unsigned>(k.n_rowblocks / 2), static_cast<unsigned>(ceil_div(M, MB))), block(64 * nwaves);
#define MFQ_SWIGLU_LAUNCH(KERN)                                                                                       \
    do {                                                                                                              \
        auto kern_ = KERN;                                                                                            \
        if (int rc_ = allow_dynamic_lds(reinterpret_cast<const void *>(kern_), lds, "nint_gemv_swiglu")) return rc_;  \
        hipLaunchKernelGGL(kern_, grid, block, lds, st, k, w, x, ldx, M, hidden, out_f16, ldh, spw);                  \
    } while (0)
    static const int env_xreg = tune_env("MFQ_GEMV_XREG", 1);
    const bool xreg = env_xreg != 0 && k.neuron_len % 2 == 0 && ldx % 2 == 0 && (reinterpret_cast<uintptr_t>(x) & 3) == 0;
#define MFQ_SWIGLU(UNIT, B, G)                                                                                        \
    if (k.bits == B && k.gs == G) {                                                                                   \
        if (ring) MFQ_SWIGLU_LAUNCH((nint_gemv_swiglu_kernel<UNIT<B, G>, XF16, MB, true>));                           \
        else if (xreg) MFQ_SWIGLU_LAUNCH((nint_gemv_swiglu_kernel<UNIT<B, G>, XF16, MB, false, true>));               \
        else MFQ_SWIGLU_LAUNCH((nint_gemv_swiglu_kernel<UNIT<B, G>, XF16, MB, false>));                               \
        return check_launch("nint_gemv_swiglu");                                                                      \
    }
    if (k.kind == 1) {
        MFQ_SWIGLU(PairedUnit, 4, 32) MFQ_SWIGLU(PairedUnit, 4, 24) MFQ_SWIGLU(PairedUnit, 4, 16) MFQ_SWIGLU(PairedUnit, 4, 48)
        MFQ_SWIGLU(PairedUnit, 3, 24) MFQ_SWIGLU(PairedUnit, 2, 16) MFQ_SWIGLU(PairedUnit, 2, 32)
    } else {
        MFQ_GENERIC_PROFILES(MFQ_SWIGLU)
    }
#undef MFQ_SWIGLU
#undef MFQ_SWIGLU_LAUNCH
    return fail(MFQ_ERR_UNSUPPORTED, "nint_gemv_swiglu: no fused kernel for NINT%d-%d", k.bits, k.gs);
}

extern "C" int mfq_hip_nint_gemv_glu(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                     int M, void *hidden, int out_dtype, int64_t ldh, int activation, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && hidden, MFQ_ERR_INVALID, "nint_gemv_swiglu: null argument");
    MFQ_REQUIRE(activation == MFQ_GLU_SILU || activation == MFQ_GLU_GELU, MFQ_ERR_INVALID, "nint_gemv_glu: activation=%d", activation);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemv_swiglu: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemv_swiglu: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(M >= 1 && M <= 2, MFQ_ERR_UNSUPPORTED, "nint_gemv_swiglu: M=%d (the fused kernel takes one or two rows)", M);
    MFQ_REQUIRE(d->out % 32 == 0, MFQ_ERR_UNSUPPORTED, "nint_gemv_swiglu: %d rows are not two halves of whole row-blocks", d->out);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldh >= d->out / 2, MFQ_ERR_INVALID, "nint_gemv_swiglu: ldx/ldh smaller than the tensor");
    const NintK k = to_k(d);
    MFQ_REQUIRE(k.kind == 1 || mfma_generic_profile(k), MFQ_ERR_UNSUPPORTED, "nint_gemv_swiglu: no fused kernel for NINT%d-%d",
                k.bits, k.gs);
    MFQ_REQUIRE(static_cast<int64_t>(k.n_rowblocks / 2) * k.rowblock_bytes < (1ll << 31), MFQ_ERR_UNSUPPORTED,
                "nint_gemv_swiglu: tensor too large for one window");
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    uint16_t *h = static_cast<uint16_t *>(hidden);
    const int f16 = (out_dtype == MFQ_X_F16 ? 1 : 0) | (activation == MFQ_GLU_GELU ? 2 : 0);  // the kernel's output mode
    hipStream_t st = as_stream(stream);
    // two rows per block while their staged activations fit the LDS, else one row per block
    const int nwaves = k.nsteps < 16 ? k.nsteps : 16;
    const bool pair = M == 2 && gemv_lds_bytes(2, static_cast<int>(ceil_div(k.nsteps, nwaves)), k.gs, nwaves, 2) <= 65536;
    if (x_dtype == MFQ_X_F16)
        return pair ? launch_gemv_swiglu<1, 2>(k, w, xp, ldx, M, h, f16, ldh, st)
                    : launch_gemv_swiglu<1, 1>(k, w, xp, ldx, M, h, f16, ldh, st);
    return pair ? launch_gemv_swiglu<0, 2>(k, w, xp, ldx, M, h, f16, ldh, st)
                : launch_gemv_swiglu<0, 1>(k, w, xp, ldx, M, h, f16, ldh, st);
}

extern "C" int mfq_hip_nint_gemv_swiglu(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                        int M, void *hidden, int out_dtype, int64_t ldh, mfq_stream_t stream) {
    return mfq_hip_nint_gemv_glu(d, weight, x, x_dtype, ldx, M, hidden, out_dtype, ldh, MFQ_GLU_SILU, stream);
}

extern "C" int mfq_hip_nint_gemv(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                 int M, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nint_gemv: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nint_gemv: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemv: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nint_gemv: ldx/ldy smaller than the tensor");
    return nint_gemv_any(d, weight, x, x_dtype, ldx, M, y, ldy, as_stream(stream));
}
