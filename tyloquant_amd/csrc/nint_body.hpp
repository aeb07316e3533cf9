// NINT decode GEMV bodies, shared by the dense kernels and the expert-grouped (MoE) kernels.
//
// Unpack trick.  A paired unit keeps, in each dword, the code of an even weight in the low half
// and of the following odd weight in the high half, at the same offset.  OR-ing a field that sits
// at mantissa offset o of each half into the fp16 constant 1024.0 gives the exact fp16 pair
// (1024 + 2^o * c_even, 1024 + 2^o * c_odd) without shifting it down, and one packed dot product
// (v_dot2_f32_f16) multiplies the pair with the matching activations.  The activations of a pair
// whose field sits at offset o are staged multiplied by 2^-o (exact in fp16), so every product is
// 1024 * x' + c * x and one accumulator per group suffices; the 1024 bias leaves through T_g, the
// 1024-weighted sum of the staged activations that the staging step precomputes and the
// accumulator starts from:
//     sum_i c_i x_i = sum_pairs (1024 + 2^o c) . x'  -  T_g,   T_g = 1024 * sum_pairs (x'_2i + x'_2i+1)
// Ten mantissa bits hold two 4-bit fields, three 3-bit fields or two 2-bit fields (more with one
// shift), so a dword of codes costs one shift plus one AND-OR and one dot2 per pair.
#pragma once
#include "common.hpp"
#include "gemv_common.hpp"

namespace mfq {

struct NintK {  // what kernels need of mfq_nint_desc, passed by value
    int bits, sub_bits, gs, out, neuron_len, ng, kind, dwords, tail, nsteps, n_rowblocks;
    int64_t step_bytes, rowblock_bytes, anchors_off;
};

inline NintK to_k(const mfq_nint_desc *d) {
    NintK k;
    k.bits = d->bits; k.sub_bits = d->sub_bits; k.gs = d->gs; k.out = d->out; k.neuron_len = d->neuron_len;
    k.ng = d->ng; k.kind = d->kind; k.dwords = d->dwords; k.tail = d->tail_bytes; k.nsteps = d->nsteps;
    k.n_rowblocks = d->n_rowblocks; k.step_bytes = d->step_bytes; k.rowblock_bytes = d->rowblock_bytes;
    k.anchors_off = d->anchors_off;
    return k;
}

inline bool paired_profile(int bits, int gs) {
    if (bits == 4) return gs == 16 || gs == 24 || gs == 32 || gs == 48;
    if (bits == 2) return gs == 16 || gs == 32;
    if (bits == 3) return gs == 24;
    return false;
}

// ---- field placement shared by repack and dequant ----------------------------------------
// Position of weight i inside a paired unit: word index (dwords == tail word) and bit offset;
// 3-bit weights 22 and 23 are split over spare bits and are handled by the callers.
__device__ __forceinline__ void paired_pos(int bits, int i, int &word, int &bit) {
    const int per_half = (bits == 3) ? 5 : 16 / bits;
    const int per_word = 2 * per_half;
    word = i / per_word;
    const int r = i - word * per_word;
    bit = (r >> 1) * bits + ((r & 1) << 4);
}

__device__ __forceinline__ uint32_t unit_code(const NintK &k, const uint32_t *q, uint32_t tail, int i) {
    if (k.kind == 0) {
        const int bit = i * k.bits;
        const int w = bit >> 5, sh = bit & 31;
        uint64_t v = q[w];
        if (w + 1 < k.dwords) v |= static_cast<uint64_t>(q[w + 1]) << 32;
        return static_cast<uint32_t>(v >> sh) & ((1u << k.bits) - 1u);
    }
    if (k.bits == 3 && i >= 20) {
        if (i == 20) return tail & 7u;
        if (i == 21) return (tail >> 3) & 7u;
        const int h = (i == 23) ? 16 : 0;
        return ((q[1] >> (15 + h)) & 1u) | (((tail >> (i == 23 ? 7 : 6)) & 1u) << 1) | (((q[0] >> (15 + h)) & 1u) << 2);
    }
    int w, b;
    paired_pos(k.bits, i, w, b);
    return (q[w] >> b) & ((1u << k.bits) - 1u);
}

// natural-order profiles with a unit of their own (GEMV, streaming and prefill kernels)
// (NINT5 (5,28), NINT6 (6,24) and NINT8 (8,48): the production profiles outside the paired layouts, FORMATS.md:73-79)
inline bool mfma_generic_profile(const NintK &k) {
    return k.kind == 0 && ((k.bits == 5 && k.gs == 28) || (k.bits == 6 && k.gs == 24) || (k.bits == 8 && k.gs == 48));
}
#define MFQ_GENERIC_PROFILES(X) X(GenericUnit, 5, 28) X(GenericUnit, 6, 24) X(GenericUnit, 8, 48)

constexpr uint32_t kMagicH2 = 0x64006400u;  // (1024.0, 1024.0) in fp16
constexpr int kMaxRbw = 4;                  // row-blocks one wave may walk through

template <int BITS, int GS>
struct PairedUnit {
    static constexpr int D = (BITS == 3) ? 2 : GS * BITS / 32;
    static constexpr bool TAIL = (BITS == 3);
    static constexpr int GROUP = GS, NPAIR = GS / 2, CBITS = BITS;
    // mantissa offset class of pair i of a group (pair i = weights 2i, 2i+1): 4- and 2-bit fields
    // alternate between offset 0 and BITS; 3-bit pairs sit at offsets 0,3,6,0,3 | 0,3,6,0,3 | 0,0
    __device__ static __forceinline__ constexpr int cls(int i) {
        if constexpr (BITS == 3) return static_cast<int>((0x49124u >> (2 * i)) & 3u);
        else return i & 1;
    }
    struct Bias {
        static constexpr bool SCALED = true;
        __device__ static __forceinline__ float bw(int) { return 1024.f; }
        // 2^(-BITS * class): built in the exponent field
        __device__ static __forceinline__ float xscale(int pos, int t) {
            return __uint_as_float(0x3f800000u - (static_cast<uint32_t>(BITS * cls(BITS == 3 ? pos + t : t)) << 23));
        }
        __device__ static __forceinline__ float inv_xscale(int i) {
            return __uint_as_float(0x3f800000u + (static_cast<uint32_t>(BITS * cls(i)) << 23));
        }
        // the scale of pair i of a group, whatever its position in a chunk
        __device__ static __forceinline__ float pair_scale(int i) {
            return __uint_as_float(0x3f800000u - (static_cast<uint32_t>(BITS * cls(i)) << 23));
        }
    };

    // v[i] = fp16 pair (1024 + 2^o * code_2i, 1024 + 2^o * code_2i+1) of pair i of the group, o = BITS * cls(i)
    __device__ static __forceinline__ void unpack(const uint32_t (&q)[D], uint32_t tail, uint32_t (&v)[GS / 2]) {
        const uint32_t magic = kMagicH2;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const uint32_t hi = q[d] >> 8;
                v[4 * d] = and_or(q[d], 0x000F000Fu, magic);
                v[4 * d + 1] = and_or(q[d], 0x00F000F0u, magic);
                v[4 * d + 2] = and_or(hi, 0x000F000Fu, magic);
                v[4 * d + 3] = and_or(hi, 0x00F000F0u, magic);
            }
        } else if constexpr (BITS == 2) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t a = q[d] >> (8 * h), b = q[d] >> (8 * h + 4);
                    v[8 * d + 4 * h] = and_or(a, 0x00030003u, magic);
                    v[8 * d + 4 * h + 1] = and_or(a, 0x000C000Cu, magic);
                    v[8 * d + 4 * h + 2] = and_or(b, 0x00030003u, magic);
                    v[8 * d + 4 * h + 3] = and_or(b, 0x000C000Cu, magic);
                }
            }
        } else {
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                const uint32_t hi = q[d] >> 9;
                v[5 * d] = and_or(q[d], 0x00070007u, magic);
                v[5 * d + 1] = and_or(q[d], 0x00380038u, magic);
                v[5 * d + 2] = and_or(q[d], 0x01C001C0u, magic);
                v[5 * d + 3] = and_or(hi, 0x00070007u, magic);
                v[5 * d + 4] = and_or(hi, 0x00380038u, magic);
            }
            // weights 20, 21 live in the tail byte; 22, 23 in its top bits and the spare bits 15 / 31
            v[10] = (tail & 7u) | ((tail & 0x38u) << 13) | magic;
            uint32_t b = and_or(q[1] >> 15, 0x00010001u, magic);
            b = and_or(q[0] >> 13, 0x00040004u, b);
            b |= ((tail >> 6) & 1u) << 1;
            b |= ((tail >> 7) & 1u) << 17;
            v[11] = b;
        }
    }

    // acc[m] += sum over the pairs of the group of (1024 + 2^o * code) . x'_m; xs = the group's GS/2 staged
    // fp16 pairs of activation row 0 in LDS, row m sits mstride dwords further.  Each pair is unpacked
    // once for all rows.
    template <int MB>
    __device__ static __forceinline__ void dot(const uint32_t (&q)[D], uint32_t tail, const uint32_t *xs, int mstride,
                                               float (&acc)[MB]) {
        uint32_t v[GS / 2];
        unpack(q, tail, v);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
#pragma unroll
            for (int c = 0; c < GS / 8; ++c) {
                const u32x4_t x = *reinterpret_cast<const u32x4_t *>(xs + m * mstride + 4 * c);
                acc[m] = dot2h(v[4 * c], x.x, acc[m]);
                acc[m] = dot2h(v[4 * c + 1], x.y, acc[m]);
                acc[m] = dot2h(v[4 * c + 2], x.z, acc[m]);
                acc[m] = dot2h(v[4 * c + 3], x.w, acc[m]);
            }
        }
    }
    // the same against activations already in registers (x[i] = staged pair i of the group)
    __device__ static __forceinline__ float dot_regs(const uint32_t (&q)[D], uint32_t tail, const uint32_t (&x)[GS / 2], float acc) {
        uint32_t v[GS / 2];
        unpack(q, tail, v);
#pragma unroll
        for (int i = 0; i < GS / 2; ++i) acc = dot2h(v[i], x[i], acc);
        return acc;
    }
};

// Natural-order unit of any (bits <= 8, even groupsize): ceil(GS * BITS / 32) dwords, code i at bit i * BITS.
// unpack() yields the same (1024 + code) fp16 pairs as the paired units (offset class 0 throughout), padded
// with zero codes up to a multiple of 8 weights.
template <int BITS, int GS>
struct GenericUnit {
    static constexpr int D = (GS * BITS + 31) / 32;
    static constexpr bool TAIL = false;
    static constexpr int GROUP = GS, NPAIR = ((GS + 7) / 8) * 4, CBITS = 0;
    static_assert(BITS <= 8 && GS % 2 == 0, "natural-order units hold an even number of codes of at most 8 bits");
    __device__ static __forceinline__ constexpr int cls(int) { return 0; }
    struct Bias {  // every pair is (1024 + code): unscaled activations, T_g = 1024 * X_g
        static constexpr bool SCALED = false;
        __device__ static __forceinline__ float bw(int) { return 1024.f; }
        __device__ static __forceinline__ float xscale(int, int) { return 1.f; }
        __device__ static __forceinline__ float inv_xscale(int) { return 1.f; }
        __device__ static __forceinline__ float pair_scale(int) { return 1.f; }
    };
    __device__ static __forceinline__ uint32_t code(const uint32_t (&q)[D], int i) {
        const int bit = i * BITS, wi = bit >> 5, sh = bit & 31;
        uint32_t c = q[wi] >> sh;
        if (sh + BITS > 32) c |= q[wi + 1] << (32 - sh);
        return c & ((1u << BITS) - 1u);
    }
    // Pair p = the 2 * BITS bits from bit 2 * p * BITS: extracted (through a funnel shift when they straddle two
    // dwords), a shift-or copies the second code to bit 16, one AND-OR drops the rest and adds the magic exponent.
    __device__ static __forceinline__ void unpack(const uint32_t (&q)[D], uint32_t, uint32_t (&v)[NPAIR]) {
        constexpr uint32_t M = (1u << BITS) - 1u;
        if constexpr (BITS == 8) {  // bytes: one byte permute drops a pair into the mantissas of (1024, 1024)
#pragma unroll
            for (int p = 0; p < NPAIR; ++p)
                v[p] = 2 * p >= GS ? kMagicH2 : __builtin_amdgcn_perm(q[p / 2], kMagicH2, (p & 1) ? 0x03070106u : 0x03050104u);
            return;
        }
#pragma unroll
        for (int p = 0; p < NPAIR; ++p) {
            if (2 * p >= GS) {
                v[p] = kMagicH2;
                continue;
            }
            const int bit = 2 * p * BITS, wi = bit >> 5, sh = bit & 31;
            uint32_t win = q[wi] >> sh;
            if (sh + 2 * BITS > 32) win = __builtin_amdgcn_alignbit(q[wi + 1], q[wi], sh);
            win &= (1u << (2 * BITS)) - 1u;  // with the shift: one bit-field extract
            v[p] = and_or((win << (16 - BITS)) | win, M | (M << 16), kMagicH2);
        }
    }
    // acc[m] += sum over the pairs of the group of (1024 + code) . x_m; xs = the group's GS/2 staged fp16 pairs
    // of activation row 0 in LDS (8-byte aligned when GS/2 is even), row m sits mstride dwords further.
    template <int MB>
    __device__ static __forceinline__ void dot(const uint32_t (&q)[D], uint32_t, const uint32_t *xs, int mstride,
                                               float (&acc)[MB]) {
        static_assert(GS % 4 == 0, "the staged pairs of a group are read two at a time");
        uint32_t v[NPAIR];
        unpack(q, 0u, v);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
#pragma unroll
            for (int c = 0; c < GS / 4; ++c) {
                const u32x2_t x = *reinterpret_cast<const u32x2_t *>(xs + m * mstride + 2 * c);
                acc[m] = dot2h(v[2 * c], x.x, acc[m]);
                acc[m] = dot2h(v[2 * c + 1], x.y, acc[m]);
            }
        }
    }
};

// Requests one step (16 groups of the row-block's 16 neurons) at window offset `off`; lane_q / lane_t /
// lane_s are the lane's byte offsets inside the step's code, tail and scale regions.
template <int D, bool TAIL>
__device__ __forceinline__ void nint_load_step(__amdgpu_buffer_rsrc_t win, uint32_t off, int lane,
                                               uint32_t (&q)[4][D], uint32_t &tails, u32x2_t &sc) {
#pragma unroll
    for (int j = 0; j < 4; ++j) load_unit_win<D>(win, off + (j * 64 + lane) * (D * 4), q[j]);
    tails = 0;
    if constexpr (TAIL) tails = __builtin_amdgcn_raw_buffer_load_b32(win, off + 1024 * D + lane * 4, 0, 2);
    sc = __builtin_amdgcn_raw_buffer_load_b64(win, off + 1024 * D + (TAIL ? 256 : 0) + lane * 8, 0, 2);
}

// SERIAL: keep the four units of the step apart in the instruction schedule (one unit's unpacked pairs and staged
// activations live at a time), for kernels that hold other buffers in flight next to the step.
template <class U, int MB, bool SERIAL = false>
__device__ __forceinline__ void nint_compute_step(const uint32_t (&q)[4][U::D], uint32_t tails, u32x2_t sc, int lg0,
                                                  const uint32_t *xs, const float *xsum, int npairs, int ngl,
                                                  float (&accS)[MB], float (&accM)[MB]) {
    constexpr int GS = U::GROUP;
    if constexpr (MB == 1 && U::CBITS != 0 && !SERIAL) {
        // one row: the staged pairs of unit j + 1 are read from LDS while unit j is unpacked and multiplied, so that
        // the read latency is paid once per step, not once per unit
        uint32_t xa[GS / 2], xb[GS / 2];
        float2 sa, sb2;
        auto fetch = [&](int j, uint32_t (&xr_)[GS / 2], float2 &st) {
            const int lg = lg0 + 4 * j;
#pragma unroll
            for (int c = 0; c < GS / 8; ++c) {
                const u32x4_t x = *reinterpret_cast<const u32x4_t *>(xs + lg * (GS / 2) + 4 * c);
                xr_[4 * c] = x.x; xr_[4 * c + 1] = x.y; xr_[4 * c + 2] = x.z; xr_[4 * c + 3] = x.w;
            }
            st = *reinterpret_cast<const float2 *>(xsum + lg * 2);
        };
        auto unit = [&](int j, const uint32_t (&xr_)[GS / 2], float2 st) {
            const uint32_t scw = (j < 2) ? sc.x : sc.y;
            const float ss = ubyte_f32(scw, 2 * (j & 1)), sm = ubyte_f32(scw, 2 * (j & 1) + 1);
            const float a = U::dot_regs(q[j], (tails >> (8 * j)) & 0xffu, xr_, st.y);
            accS[0] = fmaf(ss, a, accS[0]);
            accM[0] = fmaf(sm, st.x, accM[0]);
        };
        fetch(0, xa, sa);
        fetch(1, xb, sb2);
        unit(0, xa, sa);
        fetch(2, xa, sa);
        unit(1, xb, sb2);
        fetch(3, xb, sb2);
        unit(2, xa, sa);
        unit(3, xb, sb2);
        return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int lg = lg0 + 4 * j;
        const uint32_t scw = (j < 2) ? sc.x : sc.y;
        const float ss = ubyte_f32(scw, 2 * (j & 1));
        const float sm = ubyte_f32(scw, 2 * (j & 1) + 1);
        const uint32_t tail = (tails >> (8 * j)) & 0xffu;
        float a[MB], xg[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float2 xt = *reinterpret_cast<const float2 *>(xsum + (m * ngl + lg) * 2);
            xg[m] = xt.x;
            a[m] = xt.y;  // -T_g
        }
        U::template dot<MB>(q[j], tail, xs + lg * (GS / 2), npairs, a);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            accS[m] = fmaf(ss, a[m], accS[m]);
            accM[m] = fmaf(sm, xg[m], accM[m]);
        }
        if constexpr (SERIAL) __builtin_amdgcn_sched_barrier(0);
    }
}

// ---- activations in registers ----------------------------------------------------------------------------------
// For the batch-1 kernels without a ring the staged activations never touch LDS.  A unit is the group of lane (r, kb);
// the 16 lanes of a DPP row (same kb) all need the same GS/2 activation pairs, so lane r of the row keeps pair r of the
// row's group in one register and every dot product fetches its pair with a row broadcast
// (v_dot2c_f32_f16_dpp ... row_newbcast:i).  Per item a lane holds, for each unit j, the pair register, X_g and -T_g.
template <int MB>
struct XItem {
    uint32_t x[MB][4];   // staged fp16 pair r of group (step, j, kb), times the pair's class scale
    float xg[MB][4];     // X_g of that group (every lane of the row holds the row's total)
    float nt[MB][4];     // -T_g
};

// acc += dot(x pair I + t of the row, w[t]) for t = 0..3; one statement, so that nothing is scheduled between them.
// On this target the result of a dot instruction may feed the accumulator of the same instruction at once, but any
// other reader has to stay three issue slots behind it, and the compiler cannot see into the statement: LAST appends
// those slots, and the caller sets it on the block whose result is read next.
template <int I, bool LAST>
__device__ __forceinline__ float dot2_bcast4(float acc, uint32_t x, uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
    if constexpr (LAST)
        asm("v_dot2c_f32_f16_dpp %0, %1, %2 row_newbcast:%6 row_mask:0xf bank_mask:0xf\n\t"
            "v_dot2c_f32_f16_dpp %0, %1, %3 row_newbcast:%7 row_mask:0xf bank_mask:0xf\n\t"
            "v_dot2c_f32_f16_dpp %0, %1, %4 row_newbcast:%8 row_mask:0xf bank_mask:0xf\n\t"
            "v_dot2c_f32_f16_dpp %0, %1, %5 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 2"
            : "+v"(acc)
            : "v"(x), "v"(w0), "v"(w1), "v"(w2), "v"(w3), "n"(I), "n"(I + 1), "n"(I + 2), "n"(I + 3));
    else
        asm("v_dot2c_f32_f16_dpp %0, %1, %2 row_newbcast:%6 row_mask:0xf bank_mask:0xf\n\t"
            "v_dot2c_f32_f16_dpp %0, %1, %3 row_newbcast:%7 row_mask:0xf bank_mask:0xf\n\t"
            "v_dot2c_f32_f16_dpp %0, %1, %4 row_newbcast:%8 row_mask:0xf bank_mask:0xf\n\t"
            "v_dot2c_f32_f16_dpp %0, %1, %5 row_newbcast:%9 row_mask:0xf bank_mask:0xf"
            : "+v"(acc)
            : "v"(x), "v"(w0), "v"(w1), "v"(w2), "v"(w3), "n"(I), "n"(I + 1), "n"(I + 2), "n"(I + 3));
    return acc;
}

// A register that a vector-ALU instruction has just written may be read through DPP only two issue slots later, and the
// compiler, which cannot see the DPP reads inside dot2_bcast4, is free to sink the instruction that produces an
// activation register right in front of them.  Every register that goes into dot2_bcast4 as x passes through here
// once after it is computed: the statement counts as its last writer and carries the two slots.
__device__ __forceinline__ void dpp_source_ready(uint32_t &a, uint32_t &b, uint32_t &c, uint32_t &d) {
    asm volatile("s_nop 1" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// sum over the 16 lanes of a DPP row, left in every lane of the row
__device__ __forceinline__ float row_allsum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true));  // row_ror:8
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true));  // row_ror:4
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xF, 0xF, true));  // row_ror:2
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xF, 0xF, true));  // row_ror:1
    return v;
}

template <class U, int MB>
__device__ __forceinline__ void nint_compute_step_xreg(const uint32_t (&q)[4][U::D], uint32_t tails, u32x2_t sc,
                                                       const XItem<MB> &xi, float (&accS)[MB], float (&accM)[MB]) {
    constexpr int NP = U::NPAIR;
    static_assert(NP % 4 == 0 && NP <= 16, "a row of 16 lanes holds the pairs of one group");
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t scw = (j < 2) ? sc.x : sc.y;
        const float ss = ubyte_f32(scw, 2 * (j & 1)), sm = ubyte_f32(scw, 2 * (j & 1) + 1);
        uint32_t v[NP];
        U::unpack(q[j], (tails >> (8 * j)) & 0xffu, v);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float a = xi.nt[m][j];
            a = dot2_bcast4<0, NP == 4>(a, xi.x[m][j], v[0], v[1], v[2], v[3]);
            if constexpr (NP > 4) a = dot2_bcast4<4, NP == 8>(a, xi.x[m][j], v[4], v[5], v[6], v[7]);
            if constexpr (NP > 8) a = dot2_bcast4<8, NP == 12>(a, xi.x[m][j], v[8], v[9], v[10], v[11]);
            if constexpr (NP > 12) a = dot2_bcast4<12, true>(a, xi.x[m][j], v[12], v[13], v[14], v[15]);
            accS[m] = fmaf(ss, a, accS[m]);
            accM[m] = fmaf(sm, xi.xg[m][j], accM[m]);
        }
    }
}

// Requests the raw activation pairs of one item (K step `step`): lane (r, kb) asks for pair r of group 16 step + 4 j + kb
// of every row through the row's range-checked window (lanes beyond the group's pairs and pairs beyond K read zeros).
template <class U, int MB>
__device__ __forceinline__ void xreg_issue(const __amdgpu_buffer_rsrc_t (&wx)[MB], int step, bool live, int lane,
                                           uint32_t (&raw)[MB][4]) {
    constexpr int P = U::GROUP / 2;
    const int r = lane & 15, kb = lane >> 4;
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t off = (static_cast<uint32_t>((step * 16 + 4 * j + kb) * P + r)) * 4u;
            raw[m][j] = __builtin_amdgcn_raw_buffer_load_b32(wx[m], (live && r < P) ? off : kNoStep, 0, 0);
        }
}

// Converts what xreg_issue fetched: fp16 pairs times sc[m] (the wave's power of two for the row) and the pair's class
// scale, and the two group sums, spread over each row of lanes.
template <class U, int XF16, int MB>
__device__ __forceinline__ void xreg_stage(const uint32_t (&raw)[MB][4], const float (&sc)[MB], int lane, XItem<MB> &xi) {
    const int r = lane & 15;
    const float cs = U::Bias::pair_scale(r), ci = U::Bias::inv_xscale(r);
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t h;
            if constexpr (XF16) h = scale_h2(raw[m][j], cs);
            else h = to_h2_scaled(raw[m][j], sc[m] * cs);
            xi.x[m][j] = h;
            const float ps = dot2h(h, 0x3c003c00u, 0.f);
            xi.xg[m][j] = row_allsum(ps * ci);
            xi.nt[m][j] = -row_allsum(ps * U::Bias::bw(r));
        }
#pragma unroll
    for (int m = 0; m < MB; ++m) dpp_source_ready(xi.x[m][0], xi.x[m][1], xi.x[m][2], xi.x[m][3]);
}

// One block = `rbw` consecutive 16-neuron row-blocks starting at `rb0` of the tensor at `w`; its waves
// split the K steps, `spw` steps per wave, and every wave walks through its K-slice of each row-block
// in turn, so the slice of the activations is staged once for all of them.  xr / yr name the MB
// activation and output rows (see flush_rows for row_base).
// The activations are requested first, then the anchors and the first three steps, and each later
// step three steps ahead into a ring of register buffers: loads retire in order and every weight load
// is an unconditional window load, so the staging waits for the activations only and the unpack of a
// step only for that step.  RING = false is the variant for waves with at most three steps in all, which
// never requests more.
// rb_step: distance, in row-blocks, between the block's row-blocks (1 = consecutive).  FLUSH = false leaves the
// partial sums parked (see park_rows; the reduction area starts at gemv_red_offset dwords) for the caller to
// combine after a block barrier.
__device__ __forceinline__ int gemv_red_offset(int nwaves, int mb, int spw, int gs) {
    return nwaves * (mb * (spw * 16 * (gs / 2) + 2 * spw * 16));
}

template <class U, int XF16, int MB, bool RING = true, bool FLUSH = true, class XP = NoXPre>
__device__ __forceinline__ void nint_unit_body(const NintK &k, const uint8_t *__restrict__ w, int rb0, int rbw,
                                               int row_base, int out_rows, const uint16_t *const (&xr)[MB],
                                               float *const (&yr)[MB], int spw, uint32_t *lds, int rb_step = 1,
                                               XP xp = XP()) {
    constexpr int D = U::D, GS = U::GROUP;
    const int lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;         // steps of this wave in each row-block
    const int nrb = min(rbw, (k.n_rowblocks - 1 - rb0) / rb_step + 1);  // row-blocks of this block
    const int ngl = spw * 16, npairs = ngl * (GS / 2);
    uint32_t *xs = lds + wave * (MB * (npairs + 2 * ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    float *red = reinterpret_cast<float *>(lds + nwaves * (MB * (npairs + 2 * ngl)));
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes) * rb_step;

    XRegs<MB> xg;
    stage_x_issue<MB>(xr, k.neuron_len, s0 * 16 * GS, npairs, lane, xg);
    xp.template issue<MB>(k.neuron_len, s0 * 16 * GS, npairs, lane);
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    float ns[kMaxRbw], nm[kMaxRbw];
#pragma unroll
    for (int i = 0; i < kMaxRbw; ++i) {
        const int rb = min(rb0 + i * rb_step, k.n_rowblocks - 1);
        ns[i] = anchors[rb * 16 + r];
        nm[i] = anchors[16 * k.n_rowblocks + rb * 16 + r];
    }
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb0) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);

    // issue cursor (row-block, step) three items ahead of the compute cursor; both are wave-uniform
    int irb = 0, is = 0;
#define MFQ_ISSUE(Q, T, C)                                                        \
    {                                                                             \
        const uint32_t off = (irb < nrb && n > 0) ? irb * rbb + is * sb : kNoStep; \
        nint_load_step<D, U::TAIL>(win, off, lane, Q, T, C);                      \
        if (++is >= n) { is = 0; ++irb; }                                         \
    }
    uint32_t q0[4][D], q1[4][D], q2[4][D], t0, t1, t2;
    u32x2_t c0, c1, c2;
    MFQ_ISSUE(q0, t0, c0)
    MFQ_ISSUE(q1, t1, c1)
    MFQ_ISSUE(q2, t2, c2)
    float xinv[MB];  // bf16 rows are staged times a per-wave power of two; the sums are scaled back when they are parked
    xp.template finish<XF16, MB>(xg);
    stage_x<XF16, MB, typename U::Bias, true>(xr, k.neuron_len, s0 * 16 * GS, npairs, GS, ngl, xs, xsum, lane, xg, xinv);

    float accS[MB], accM[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) accS[m] = accM[m] = 0.f;
    int crb = 0, cs = 0;
#define MFQ_COMPUTE(Q, T, C)                                                                              \
    {                                                                                                     \
        nint_compute_step<U, MB>(Q, T, C, cs * 16 + kb, xs, xsum, npairs, ngl, accS, accM);               \
        if (++cs >= n) {                                                                                  \
            float a_s = ns[0], a_m = nm[0];                                                               \
            _Pragma("unroll") for (int i = 1; i < kMaxRbw; ++i) if (crb == i) { a_s = ns[i]; a_m = nm[i]; } \
            float v[MB];                                                                                  \
            _Pragma("unroll") for (int m = 0; m < MB; ++m) {                                              \
                v[m] = (a_s * accS[m] - a_m * accM[m]) * xinv[m];                                         \
                accS[m] = accM[m] = 0.f;                                                                  \
            }                                                                                             \
            park_rows<MB>(v, red, crb * nwaves + wave, lane);                                             \
            cs = 0;                                                                                       \
            ++crb;                                                                                        \
        }                                                                                                 \
    }
    const int items = nrb * n;
    if (n <= 0) {  // a wave beyond the last step still owes its (zero) partial sums
        float z[MB];
        for (int i = 0; i < nrb; ++i) {
#pragma unroll
            for (int m = 0; m < MB; ++m) z[m] = 0.f;
            park_rows<MB>(z, red, i * nwaves + wave, lane);
        }
    } else if constexpr (!RING) {  // at most 3 items: everything is already requested
        MFQ_COMPUTE(q0, t0, c0)
        if (items > 1) MFQ_COMPUTE(q1, t1, c1)
        if (items > 2) MFQ_COMPUTE(q2, t2, c2)
    } else {
        uint32_t q3[4][D], t3;
        u32x2_t c3;
        for (int t = 0; t < items; t += 4) {
            MFQ_ISSUE(q3, t3, c3)
            MFQ_COMPUTE(q0, t0, c0)
            MFQ_ISSUE(q0, t0, c0)
            if (t + 1 < items) MFQ_COMPUTE(q1, t1, c1)
            MFQ_ISSUE(q1, t1, c1)
            if (t + 2 < items) MFQ_COMPUTE(q2, t2, c2)
            MFQ_ISSUE(q2, t2, c2)
            if (t + 3 < items) MFQ_COMPUTE(q3, t3, c3)
        }
    }
#undef MFQ_ISSUE
#undef MFQ_COMPUTE
    if constexpr (FLUSH) flush_rows<MB>(red, nwaves, nrb, rb0, row_base, out_rows, yr);
}

// The same block decomposition for waves with at most three items and activations in registers (see XItem): no LDS
// in the walk, the only shared memory is the cross-wave reduction area at the start of `lds`.  Needs rows that are
// 4-byte aligned and an even K (the caller checks); K need not be a multiple of the group size.
template <class U, int XF16, int MB, bool FLUSH = true>
__device__ __forceinline__ void nint_unit_body_xreg(const NintK &k, const uint8_t *__restrict__ w, int rb0, int rbw,
                                                    int row_base, int out_rows, const uint16_t *const (&xr)[MB],
                                                    float *const (&yr)[MB], int spw, uint32_t *lds, int rb_step = 1) {
    constexpr int D = U::D;
    const int lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int r = lane & 15;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;                         // steps of this wave in each row-block
    const int nrb = min(rbw, (k.n_rowblocks - 1 - rb0) / rb_step + 1);  // row-blocks of this block
    float *red = reinterpret_cast<float *>(lds);
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes) * rb_step;
    const int items = n > 0 ? nrb * n : 0;  // <= 3

    // item t = (row-block t / n, step t % n); requests in order of use: activations, anchors, weights
    __amdgpu_buffer_rsrc_t wx[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m)
        wx[m] = wave_window(reinterpret_cast<const uint8_t *>(xr[m]), xr[m] ? static_cast<uint32_t>(k.neuron_len) * 2u : 0u);
    int irb_[3], is_[3];
#pragma unroll
    for (int t = 0; t < 3; ++t) {
        irb_[t] = n > 0 ? t / n : 0;
        is_[t] = t - irb_[t] * n;
    }
    // activations are requested and staged once per step: set u = step u of the wave (item t reads set t % n)
    uint32_t raw[3][MB][4];
#pragma unroll
    for (int u = 0; u < 3; ++u) xreg_issue<U, MB>(wx, s0 + u, u < n, lane, raw[u]);
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    float ns[3], nm[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int rb = min(rb0 + i * rb_step, k.n_rowblocks - 1);
        ns[i] = anchors[rb * 16 + r];
        nm[i] = anchors[16 * k.n_rowblocks + rb * 16 + r];
    }
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb0) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);
    uint32_t q[3][4][D], tl[3];
    u32x2_t sc[3];
#pragma unroll
    for (int t = 0; t < 3; ++t)
        nint_load_step<D, U::TAIL>(win, t < items ? irb_[t] * rbb + is_[t] * sb : kNoStep, lane, q[t], tl[t], sc[t]);

    // bf16 rows: one power of two per wave and row brings the slice near 2^12
    float xs_[MB], xinv[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        xs_[m] = xinv[m] = 1.f;
        if constexpr (!XF16) {
            uint32_t mx = 0;
#pragma unroll
            for (int t = 0; t < 3; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j) mx = absmax_bf16(mx, raw[t][m][j]);
            xs_[m] = slice_scale(wave_max_u32(mx), xinv[m]);
        }
    }
    float accS[MB], accM[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) accS[m] = accM[m] = 0.f;
    if (items <= 0) {  // a wave beyond the last step still owes its (zero) partial sums
        float z[MB];
        for (int i = 0; i < nrb; ++i) {
#pragma unroll
            for (int m = 0; m < MB; ++m) z[m] = 0.f;
            park_rows<MB>(z, red, i * nwaves + wave, lane);
        }
    } else {
        // a wave with one step walks row-blocks with the same staged set; with two or three steps item t is step t
        XItem<MB> xi;
        xreg_stage<U, XF16, MB>(raw[0], xs_, lane, xi);
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            if (t < items) {
                if (t > 0 && n > 1) xreg_stage<U, XF16, MB>(raw[t], xs_, lane, xi);
                nint_compute_step_xreg<U, MB>(q[t], tl[t], sc[t], xi, accS, accM);
                if (is_[t] == n - 1) {
                    float a_s = ns[0], a_m = nm[0];
#pragma unroll
                    for (int i = 1; i < 3; ++i)
                        if (irb_[t] == i) { a_s = ns[i]; a_m = nm[i]; }
                    float v[MB];
#pragma unroll
                    for (int m = 0; m < MB; ++m) {
                        v[m] = (a_s * accS[m] - a_m * accM[m]) * xinv[m];
                        accS[m] = accM[m] = 0.f;
                    }
                    park_rows<MB>(v, red, irb_[t] * nwaves + wave, lane);
                }
            }
        }
    }
    if constexpr (FLUSH) flush_rows<MB>(red, nwaves, nrb, rb0, row_base, out_rows, yr);
}

template <int BITS, int GS, int XF16, int MB, bool RING = true>
__device__ __forceinline__ void nint_paired_body(const NintK &k, const uint8_t *__restrict__ w, int rb0, int rbw,
                                                 int row_base, int out_rows, const uint16_t *const (&xr)[MB],
                                                 float *const (&yr)[MB], int spw, uint32_t *lds) {
    nint_unit_body<PairedUnit<BITS, GS>, XF16, MB, RING>(k, w, rb0, rbw, row_base, out_rows, xr, yr, spw, lds);
}

// Any (bits, gs): natural-order units, one code at a time in fp32.
template <int XF16, int MB, class XP = NoXPre>
__device__ __forceinline__ void nint_generic_body(const NintK &k, const uint8_t *__restrict__ w, int rb, int row_base,
                                                  int out_rows, const uint16_t *const (&xr)[MB], float *const (&yr)[MB],
                                                  int spw, uint32_t *lds, XP xp = XP()) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int s0 = wave * spw;
    const int s1 = min(k.nsteps, s0 + spw);
    const int gs = k.gs, ngl = spw * 16, npairs = ngl * gs / 2;
    uint32_t *xs = lds + wave * (MB * (npairs + 2 * ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    float *red = reinterpret_cast<float *>(lds + nwaves * (MB * (npairs + 2 * ngl)));
    XRegs<MB> xg;
    stage_x_issue<MB>(xr, k.neuron_len, s0 * 16 * gs, npairs, lane, xg);
    xp.template issue<MB>(k.neuron_len, s0 * 16 * gs, npairs, lane);
    float xinv[MB];
    xp.template finish<XF16, MB>(xg);
    stage_x<XF16, MB, PlainBias, true>(xr, k.neuron_len, s0 * 16 * gs, npairs, gs, ngl, xs, xsum, lane, xg, xinv);
    const uint16_t *xh = reinterpret_cast<const uint16_t *>(xs);

    const int r = lane & 15, kb = lane >> 4;
    const uint8_t *base = w + static_cast<int64_t>(rb) * k.rowblock_bytes;
    const uint32_t cmask = (1u << k.bits) - 1u;
    float accS[MB], accM[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) accS[m] = accM[m] = 0.f;
    for (int s = s0; s < s1; ++s) {
        const uint8_t *sp = base + s * k.step_bytes;
        const uint8_t *sreg = sp + 1024 * k.dwords;
        for (int j = 0; j < 4; ++j) {
            const int lg = (s - s0) * 16 + 4 * j + kb;
            const uint32_t *q = reinterpret_cast<const uint32_t *>(sp) + (j * 64 + lane) * k.dwords;
            const float ss = static_cast<float>(sreg[lane * 8 + 2 * j]);
            const float sm = static_cast<float>(sreg[lane * 8 + 2 * j + 1]);
            float raw[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) raw[m] = 0.f;
            for (int i = 0; i < gs; ++i) {
                const int bit = i * k.bits;
                const int wi = bit >> 5, sh = bit & 31;
                uint64_t v = q[wi];
                if (wi + 1 < k.dwords) v |= static_cast<uint64_t>(q[wi + 1]) << 32;
                const float c = static_cast<float>(static_cast<uint32_t>(v >> sh) & cmask);
#pragma unroll
                for (int m = 0; m < MB; ++m) raw[m] = fmaf(c, f16_to_f32(xh[2 * (m * npairs) + lg * gs + i]), raw[m]);
            }
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                accS[m] = fmaf(ss, raw[m], accS[m]);
                accM[m] = fmaf(sm, xsum[(m * ngl + lg) * 2], accM[m]);
            }
        }
    }
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    const float ns = anchors[rb * 16 + r], nm = anchors[16 * k.n_rowblocks + rb * 16 + r];
    float v[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = (ns * accS[m] - nm * accM[m]) * xinv[m];
    finish_rows<MB>(v, red, wave, nwaves, lane, rb, row_base, out_rows, yr);
}

// Dense wrappers: block (rb, m-chunk).
template <int BITS, int GS, int XF16, int MB, bool RING>
__global__ __launch_bounds__(1024) void nint_gemv_paired_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                float *__restrict__ y, int64_t ldy, int spw, int rbw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_paired_body<BITS, GS, XF16, MB, RING>(k, w, blockIdx.x * rbw, rbw, 0, k.out, xr, yr, spw, lds);
}

// the same for waves with at most three items: activations in registers, LDS only for the cross-wave sums
template <class U, int XF16, int MB>
__global__ __launch_bounds__(1024) void nint_gemv_xreg_kernel(NintK k, const uint8_t *__restrict__ w,
                                                              const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                              float *__restrict__ y, int64_t ldy, int spw, int rbw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_unit_body_xreg<U, XF16, MB>(k, w, blockIdx.x * rbw, rbw, 0, k.out, xr, yr, spw, lds);
}

// natural-order profiles with a unit of their own
template <int BITS, int GS, int XF16, int MB, bool RING>
__global__ __launch_bounds__(1024) void nint_gemv_natural_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                 const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                 float *__restrict__ y, int64_t ldy, int spw, int rbw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_unit_body<GenericUnit<BITS, GS>, XF16, MB, RING>(k, w, blockIdx.x * rbw, rbw, 0, k.out, xr, yr, spw, lds);
}

// Gate/up GEMV with the SwiGLU fused: the tensor holds the W gate neurons, then the W up neurons.  Block
// blockIdx.x takes row-block blockIdx.x of each half and stores hidden[m][16 * blockIdx.x + r] = act(gate) * up
// as fp16 (bit 0 of out_f16) or bf16, act = SiLU or (bit 1 of out_f16) GELU.
template <class U, int XF16, int MB, bool RING, bool XR = false>
__global__ __launch_bounds__(1024) void nint_gemv_swiglu_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                uint16_t *__restrict__ hidden, int out_f16, int64_t ldh,
                                                                int spw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, static_cast<float *>(nullptr), 0, M, blockIdx.y * MB, xr, yr);
    const int half_rb = k.n_rowblocks / 2;
    constexpr bool IN_REGS = XR && !RING && U::NPAIR <= 16 && (MB == 1 || U::CBITS != 0);  // see nint_unit_body_xreg
    if constexpr (IN_REGS) nint_unit_body_xreg<U, XF16, MB, false>(k, w, blockIdx.x, 2, 0, k.out, xr, yr, spw, lds, half_rb);
    else nint_unit_body<U, XF16, MB, RING, false>(k, w, blockIdx.x, 2, 0, k.out, xr, yr, spw, lds, half_rb);
    __syncthreads();
    const int nwaves = blockDim.x >> 6;
    const float *red = reinterpret_cast<const float *>(lds + (IN_REGS ? 0 : gemv_red_offset(nwaves, MB, spw, U::GROUP)));
    for (int o = threadIdx.x; o < MB * 16; o += blockDim.x) {
        const int r = o & 15, m = o >> 4;
        const int row = blockIdx.y * MB + m;
        if (row >= M) continue;
        float g = 0.f, u = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) {
            g += red[(wv * MB + m) * 16 + r];
            u += red[((nwaves + wv) * MB + m) * 16 + r];
        }
        const float v = glu_value(g, u, out_f16 & 2);
        hidden[static_cast<int64_t>(row) * ldh + blockIdx.x * 16 + r] = (out_f16 & 1) ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
    }
}

template <int XF16, int MB>
__global__ __launch_bounds__(1024) void nint_gemv_generic_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                 const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                 float *__restrict__ y, int64_t ldy, int spw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_generic_body<XF16, MB>(k, w, blockIdx.x, 0, k.out, xr, yr, spw, lds);
}

}  // namespace mfq
