// NINT decode GEMV bodies, shared by the dense kernels and the expert-grouped (MoE) kernels.
#pragma once
#include "common.hpp"
#include "gemv_common.hpp"

namespace mfq {

struct NintK {  // what kernels need of mfq_nint_desc, passed by value
    int bits, sub_bits, gs, out, neuron_len, ng, kind, dwords, tail, nsteps, n_rowblocks;
    int64_t step_bytes, rowblock_bytes, anchors_off;
};

template <int BITS, int GS, int XF16>
struct PairedUnit {
    static constexpr int D = (BITS == 3) ? 2 : GS * BITS / 32;
    static constexpr bool TAIL = (BITS == 3);
    static constexpr uint32_t MAGIC = XF16 ? 0x64006400u : 0x43004300u;
    static constexpr float BIAS = XF16 ? 1024.f : 128.f;
    static constexpr uint32_t FMASK = ((1u << BITS) - 1u) * 0x00010001u;
    // sum_i (BIAS + code_i) * x_i over the group, xs = GS/2 activation pairs in LDS
    __device__ static __forceinline__ float dot(const uint32_t (&q)[D], uint32_t tail, const uint32_t *xs) {
        float acc = 0.f;
        if constexpr (BITS == 3) {
#pragma unroll
            for (int d = 0; d < 2; ++d) {
#pragma unroll
                for (int p = 0; p < 5; ++p) {
                    const uint32_t v = ((q[d] >> (3 * p)) & FMASK) | MAGIC;
                    acc = dot2<XF16>(v, xs[5 * d + p], acc);
                }
            }
            const uint32_t a = ((tail & 7u) | MAGIC) | ((tail & 0x38u) << 13);
            acc = dot2<XF16>(a, xs[10], acc);
            uint32_t b = ((q[1] >> 15) & 0x00010001u) | MAGIC;
            b |= (q[0] >> 13) & 0x00040004u;
            b |= ((tail >> 6) & 1u) << 1;
            b |= ((tail >> 7) & 1u) << 17;
            acc = dot2<XF16>(b, xs[11], acc);
        } else {
            constexpr int PER = 16 / BITS;
#pragma unroll
            for (int d = 0; d < D; ++d) {
#pragma unroll
                for (int p = 0; p < PER; ++p) {
                    const uint32_t v = ((q[d] >> (BITS * p)) & FMASK) | MAGIC;
                    acc = dot2<XF16>(v, xs[PER * d + p], acc);
                }
            }
        }
        return acc;
    }
};

// One block = one 16-neuron row-block `rb` of the tensor at `w`; its waves split the steps, `spw`
// steps per wave.  xr / yr name the MB activation and output rows (see finish_rows for row_base).
template <int BITS, int GS, int XF16, int MB>
__device__ __forceinline__ void nint_paired_body(const NintK &k, const uint8_t *__restrict__ w, int rb, int row_base,
                                                 int out_rows, const uint16_t *const (&xr)[MB], float *const (&yr)[MB],
                                                 int spw, uint32_t *lds) {
    using U = PairedUnit<BITS, GS, XF16>;
    constexpr int D = U::D;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int s0 = wave * spw;
    const int s1 = min(k.nsteps, s0 + spw);
    const int ngl = spw * 16, npairs = ngl * (GS / 2);
    uint32_t *xs = lds + wave * (MB * (npairs + ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    stage_x<XF16, MB>(xr, k.neuron_len, s0 * 16 * GS, npairs, GS, ngl, xs, xsum, lane);

    const int r = lane & 15, kb = lane >> 4;
    const uint8_t *base = w + static_cast<int64_t>(rb) * k.rowblock_bytes;
    float accS[MB], accM[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) accS[m] = accM[m] = 0.f;
    for (int s = s0; s < s1; ++s) {
        const uint8_t *sp = base + s * k.step_bytes;
        uint32_t q[4][D];
#pragma unroll
        for (int j = 0; j < 4; ++j) load_unit<D>(reinterpret_cast<const uint32_t *>(sp) + (j * 64 + lane) * D, q[j]);
        uint32_t tails = 0;
        if constexpr (U::TAIL) tails = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sp + 1024 * D) + lane);
        const u32x2_t sc = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(sp + 1024 * D + (U::TAIL ? 256 : 0)) + lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int lg = (s - s0) * 16 + 4 * j + kb;
            const uint32_t scw = (j < 2) ? sc.x : sc.y;
            const float ss = ubyte_f32(scw, 2 * (j & 1));
            const float sm = ubyte_f32(scw, 2 * (j & 1) + 1);
            const uint32_t tail = (tails >> (8 * j)) & 0xffu;
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const float raw = U::dot(q[j], tail, xs + m * npairs + lg * (GS / 2));
                const float xg = xsum[m * ngl + lg];
                accS[m] = fmaf(ss, fmaf(-U::BIAS, xg, raw), accS[m]);
                accM[m] = fmaf(sm, xg, accM[m]);
            }
        }
    }
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    const float ns = anchors[rb * 16 + r], nm = anchors[16 * k.n_rowblocks + rb * 16 + r];
    float v[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = ns * accS[m] - nm * accM[m];
    finish_rows<MB>(v, reinterpret_cast<float *>(lds), wave, nwaves, lane, rb, row_base, out_rows, yr);
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
    uint32_t *xs = lds + wave * (MB * (npairs + ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    stage_x<XF16, MB>(xr, k.neuron_len, s0 * 16 * gs, npairs, gs, ngl, xs, xsum, lane);
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
                for (int m = 0; m < MB; ++m) raw[m] = fmaf(c, x_to_f32<XF16>(xh[2 * (m * npairs) + lg * gs + i]), raw[m]);
            }
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                accS[m] = fmaf(ss, raw[m], accS[m]);
                accM[m] = fmaf(sm, xsum[m * ngl + lg], accM[m]);
            }
        }
    }
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    const float ns = anchors[rb * 16 + r], nm = anchors[16 * k.n_rowblocks + rb * 16 + r];
    float v[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = ns * accS[m] - nm * accM[m];
    finish_rows<MB>(v, reinterpret_cast<float *>(lds), wave, nwaves, lane, rb, row_base, out_rows, yr);
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
