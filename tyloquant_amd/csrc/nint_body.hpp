// NINT decode GEMV bodies, shared by the dense kernels and the expert-grouped (MoE) kernels.
//
// Unpack trick.  A paired unit keeps, in each dword, the code of an even weight in the low half
// and of the following odd weight in the high half, at the same offset.  OR-ing a field that sits
// at mantissa offset o of each half into the fp16 constant 1024.0 gives the exact fp16 pair
// (1024 + 2^o * c_even, 1024 + 2^o * c_odd) without shifting it down, and one packed dot product
// (v_dot2_f32_f16) multiplies the pair with the matching activations.  Fields at different offsets
// go to different accumulators ("classes") that are rescaled by 2^-o once per group; the 1024 bias
// leaves through T_g, the bias-weighted activation sum that the staging step precomputes:
//     sum_i c_i x_i = sum_classes acc_class * 2^-o  -  T_g,   T_g = sum_pairs (x_2i + x_2i+1) * 1024 * 2^-o(i)
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

constexpr uint32_t kMagicH2 = 0x64006400u;  // (1024.0, 1024.0) in fp16

template <int BITS, int GS>
struct PairedUnit {
    static constexpr int D = (BITS == 3) ? 2 : GS * BITS / 32;
    static constexpr bool TAIL = (BITS == 3);
    static constexpr int NCLS = (BITS == 3) ? 3 : 2;
    // reciprocal field scale of class c
    __device__ static __forceinline__ constexpr float inv_scale(int c) {
        return BITS == 4 ? (c ? 1.f / 16.f : 1.f) : BITS == 2 ? (c ? 0.25f : 1.f) : (c == 0 ? 1.f : c == 1 ? 0.125f : 1.f / 64.f);
    }
    // class of pair i of a group (pair i = weights 2i, 2i+1)
    __device__ static __forceinline__ int cls(int i) {
        if constexpr (BITS == 3) return i < 10 ? static_cast<int>((0x10210u >> (4 * (i % 5))) & 3u) : 0;  // offsets 0,3,6,0,3
        else return i & 1;
    }
    struct Bias {
        __device__ static __forceinline__ float bw(int i) { return 1024.f * inv_scale(cls(i)); }
    };

    // acc[m][c] += sum over the pairs of class c of (1024 + scale_c * code) . x_m; xs = the group's GS/2 fp16
    // pairs of activation row 0 in LDS, row m sits mstride dwords further.  Each pair is unpacked once for all rows.
    template <int MB>
    __device__ static __forceinline__ void dot(const uint32_t (&q)[D], uint32_t tail, const uint32_t *xs, int mstride,
                                               float (&acc)[MB][NCLS]) {
        const uint32_t magic = kMagicH2;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const uint32_t hi = q[d] >> 8;
                const uint32_t v0 = and_or(q[d], 0x000F000Fu, magic), v1 = and_or(q[d], 0x00F000F0u, magic);
                const uint32_t v2 = and_or(hi, 0x000F000Fu, magic), v3 = and_or(hi, 0x00F000F0u, magic);
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const u32x4_t x = *reinterpret_cast<const u32x4_t *>(xs + m * mstride + 4 * d);
                    acc[m][0] = dot2h(v0, x.x, acc[m][0]);
                    acc[m][1] = dot2h(v1, x.y, acc[m][1]);
                    acc[m][0] = dot2h(v2, x.z, acc[m][0]);
                    acc[m][1] = dot2h(v3, x.w, acc[m][1]);
                }
            }
        } else if constexpr (BITS == 2) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t a = q[d] >> (8 * h), b = q[d] >> (8 * h + 4);
                    const uint32_t v0 = and_or(a, 0x00030003u, magic), v1 = and_or(a, 0x000C000Cu, magic);
                    const uint32_t v2 = and_or(b, 0x00030003u, magic), v3 = and_or(b, 0x000C000Cu, magic);
#pragma unroll
                    for (int m = 0; m < MB; ++m) {
                        const u32x4_t x = *reinterpret_cast<const u32x4_t *>(xs + m * mstride + 8 * d + 4 * h);
                        acc[m][0] = dot2h(v0, x.x, acc[m][0]);
                        acc[m][1] = dot2h(v1, x.y, acc[m][1]);
                        acc[m][0] = dot2h(v2, x.z, acc[m][0]);
                        acc[m][1] = dot2h(v3, x.w, acc[m][1]);
                    }
                }
            }
        } else {
            uint32_t v[12];
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
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const uint32_t *xp = xs + m * mstride;
                const u32x4_t x0 = *reinterpret_cast<const u32x4_t *>(xp);
                const u32x4_t x1 = *reinterpret_cast<const u32x4_t *>(xp + 4);
                const u32x4_t x2 = *reinterpret_cast<const u32x4_t *>(xp + 8);
                const uint32_t xv[12] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w, x2.x, x2.y, x2.z, x2.w};
#pragma unroll
                for (int i = 0; i < 12; ++i) {
                    const int p5 = i % 5;
                    const int c = i < 10 ? (p5 == 2 ? 2 : ((p5 == 1 || p5 == 4) ? 1 : 0)) : 0;   // offsets 0,3,6,0,3 | 0,0
                    acc[m][c] = dot2h(v[i], xv[i], acc[m][c]);
                }
            }
        }
    }
};

template <int D, bool TAIL>
__device__ __forceinline__ void nint_load_step(const uint8_t *__restrict__ sp, int lane, uint32_t (&q)[4][D],
                                               uint32_t &tails, u32x2_t &sc) {
#pragma unroll
    for (int j = 0; j < 4; ++j) load_unit<D>(reinterpret_cast<const uint32_t *>(sp) + (j * 64 + lane) * D, q[j]);
    tails = 0;
    if constexpr (TAIL) tails = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sp + 1024 * D) + lane);
    sc = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(sp + 1024 * D + (TAIL ? 256 : 0)) + lane);
}

template <int BITS, int GS, int MB>
__device__ __forceinline__ void nint_compute_step(const uint32_t (&q)[4][PairedUnit<BITS, GS>::D], uint32_t tails,
                                                  u32x2_t sc, int lg0, const uint32_t *xs, const float *xsum,
                                                  int npairs, int ngl, float (&accS)[MB], float (&accM)[MB]) {
    using U = PairedUnit<BITS, GS>;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int lg = lg0 + 4 * j;
        const uint32_t scw = (j < 2) ? sc.x : sc.y;
        const float ss = ubyte_f32(scw, 2 * (j & 1));
        const float sm = ubyte_f32(scw, 2 * (j & 1) + 1);
        const uint32_t tail = (tails >> (8 * j)) & 0xffu;
        float a[MB][U::NCLS];
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int c = 0; c < U::NCLS; ++c) a[m][c] = 0.f;
        U::template dot<MB>(q[j], tail, xs + lg * (GS / 2), npairs, a);
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float2 xt = *reinterpret_cast<const float2 *>(xsum + (m * ngl + lg) * 2);
            float raw = a[m][0] - xt.y;
#pragma unroll
            for (int c = 1; c < U::NCLS; ++c) raw = fmaf(a[m][c], U::inv_scale(c), raw);
            accS[m] = fmaf(ss, raw, accS[m]);
            accM[m] = fmaf(sm, xt.x, accM[m]);
        }
    }
}

// One block = one 16-neuron row-block `rb` of the tensor at `w`; its waves split the steps, `spw`
// steps per wave.  xr / yr name the MB activation and output rows (see finish_rows for row_base).
// The anchors and the first steps' weights are requested before the activations are staged, and
// each later step is requested three steps ahead into a ring of register buffers, so HBM latency
// overlaps the LDS staging and the unpack arithmetic.
template <int BITS, int GS, int XF16, int MB>
__device__ __forceinline__ void nint_paired_body(const NintK &k, const uint8_t *__restrict__ w, int rb, int row_base,
                                                 int out_rows, const uint16_t *const (&xr)[MB], float *const (&yr)[MB],
                                                 int spw, uint32_t *lds) {
    using U = PairedUnit<BITS, GS>;
    constexpr int D = U::D;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int s1 = min(k.nsteps, s0 + spw);
    const int ngl = spw * 16, npairs = ngl * (GS / 2);
    uint32_t *xs = lds + wave * (MB * (npairs + 2 * ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    float *red = reinterpret_cast<float *>(lds + nwaves * (MB * (npairs + 2 * ngl)));
    const int sb = static_cast<int>(k.step_bytes);
    const uint8_t *base = w + static_cast<int64_t>(rb) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb;
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    const float ns = anchors[rb * 16 + r], nm = anchors[16 * k.n_rowblocks + rb * 16 + r];

    // four register buffers in a ring: three steps are in flight while one is being unpacked
    uint32_t q0[4][D], q1[4][D], q2[4][D], q3[4][D], t0 = 0, t1 = 0, t2 = 0, t3 = 0;
    u32x2_t c0 = {0u, 0u}, c1 = c0, c2 = c0, c3 = c0;
    const int n = s1 - s0;
    if (n > 0) nint_load_step<D, U::TAIL>(base, lane, q0, t0, c0);
    if (n > 1) nint_load_step<D, U::TAIL>(base + sb, lane, q1, t1, c1);
    if (n > 2) nint_load_step<D, U::TAIL>(base + 2 * sb, lane, q2, t2, c2);
    stage_x<XF16, MB, typename U::Bias>(xr, k.neuron_len, s0 * 16 * GS, npairs, GS, ngl, xs, xsum, lane);

    float accS[MB], accM[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) accS[m] = accM[m] = 0.f;
    for (int i = 0; i < n; i += 4) {
        if (i + 3 < n) nint_load_step<D, U::TAIL>(base + (i + 3) * sb, lane, q3, t3, c3);
        nint_compute_step<BITS, GS, MB>(q0, t0, c0, i * 16 + kb, xs, xsum, npairs, ngl, accS, accM);
        if (i + 1 >= n) break;
        if (i + 4 < n) nint_load_step<D, U::TAIL>(base + (i + 4) * sb, lane, q0, t0, c0);
        nint_compute_step<BITS, GS, MB>(q1, t1, c1, (i + 1) * 16 + kb, xs, xsum, npairs, ngl, accS, accM);
        if (i + 2 >= n) break;
        if (i + 5 < n) nint_load_step<D, U::TAIL>(base + (i + 5) * sb, lane, q1, t1, c1);
        nint_compute_step<BITS, GS, MB>(q2, t2, c2, (i + 2) * 16 + kb, xs, xsum, npairs, ngl, accS, accM);
        if (i + 3 >= n) break;
        if (i + 6 < n) nint_load_step<D, U::TAIL>(base + (i + 6) * sb, lane, q2, t2, c2);
        nint_compute_step<BITS, GS, MB>(q3, t3, c3, (i + 3) * 16 + kb, xs, xsum, npairs, ngl, accS, accM);
    }
    float v[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = ns * accS[m] - nm * accM[m];
    finish_rows<MB>(v, red, wave, nwaves, lane, rb, row_base, out_rows, yr);
}

// Any (bits, gs): natural-order units, one code at a time in fp32.
template <int XF16, int MB>
__device__ __forceinline__ void nint_generic_body(const NintK &k, const uint8_t *__restrict__ w, int rb, int row_base,
                                                  int out_rows, const uint16_t *const (&xr)[MB], float *const (&yr)[MB],
                                                  int spw, uint32_t *lds) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int s0 = wave * spw;
    const int s1 = min(k.nsteps, s0 + spw);
    const int gs = k.gs, ngl = spw * 16, npairs = ngl * gs / 2;
    uint32_t *xs = lds + wave * (MB * (npairs + 2 * ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    float *red = reinterpret_cast<float *>(lds + nwaves * (MB * (npairs + 2 * ngl)));
    stage_x<XF16, MB, PlainBias>(xr, k.neuron_len, s0 * 16 * gs, npairs, gs, ngl, xs, xsum, lane);
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
    for (int m = 0; m < MB; ++m) v[m] = ns * accS[m] - nm * accM[m];
    finish_rows<MB>(v, red, wave, nwaves, lane, rb, row_base, out_rows, yr);
}

// Dense wrappers: block (rb, m-chunk).
template <int BITS, int GS, int XF16, int MB>
__global__ __launch_bounds__(1024) void nint_gemv_paired_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                float *__restrict__ y, int64_t ldy, int spw) {
    extern __shared__ uint32_t lds[];
    const uint16_t *xr[MB];
    float *yr[MB];
    dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
    nint_paired_body<BITS, GS, XF16, MB>(k, w, blockIdx.x, 0, k.out, xr, yr, spw, lds);
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
