// Pieces shared by the decode GEMV kernels of every format: unit loads, the wave-private LDS
// staging of the activation slice with its per-group sums, and the final reductions.
#pragma once
#include <stdlib.h>

#include "common.hpp"

namespace mfq {

template <int D>
__device__ __forceinline__ void load_unit(const uint32_t *__restrict__ p, uint32_t (&q)[D]) {
    if constexpr (D % 4 == 0) {
#pragma unroll
        for (int i = 0; i < D / 4; ++i) {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p) + i);
            q[4 * i] = v.x; q[4 * i + 1] = v.y; q[4 * i + 2] = v.z; q[4 * i + 3] = v.w;
        }
    } else if constexpr (D % 2 == 0) {
#pragma unroll
        for (int i = 0; i < D / 2; ++i) {
            const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(p) + i);
            q[2 * i] = v.x; q[2 * i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < D; ++i) q[i] = __builtin_nontemporal_load(p + i);
    }
}

// Order LDS traffic between the lanes of one wave (the staged activations are wave-private, so no
// block barrier is needed).
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The kernels compute on fp16 pairs: bf16 activations are converted while they are staged (exact
// inside fp16's normal range; round-toward-zero saturates at 65504 instead of producing inf).
template <int XF16>
__device__ __forceinline__ uint32_t to_h2(uint32_t pair) {
    if constexpr (XF16) return pair;
    else {
        const float lo = __uint_as_float(pair << 16), hi = __uint_as_float(pair & 0xffff0000u);
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
    }
}

__device__ __forceinline__ float dot2h(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), acc, false);
}

// (a & mask) | orv in one VALU op; mask must be wave-uniform.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(orv));
    return r;
}

// sum over the 4 lanes of a quad with DPP row operations
__device__ __forceinline__ float quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

struct PlainBias {  // formats whose unpack needs no per-pair bias weights
    __device__ static __forceinline__ float bw(int) { return 0.f; }
};

// Stage the wave's K-slice of the MB activation rows xr[m] (null = absent row) into its private
// LDS region as fp16 (x[2i], x[2i+1]) pairs, zero beyond K.  Next to it, per group g, two floats:
// X_g = sum of x over the group and T_g = sum over its pairs i of (x[2i] + x[2i+1]) * BW::bw(i)
// (the bias the unpack trick adds to the dot product).  npairs is a multiple of 8; xs is 16-byte
// aligned.
template <int XF16, int MB, class BW>
__device__ __forceinline__ void stage_x(const uint16_t *const (&xr)[MB], int K, int k0, int npairs, int gs, int ngl,
                                        uint32_t *xs, float *xsum, int lane) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const uint16_t *p = xr[m];
        const bool vec = p && (reinterpret_cast<uintptr_t>(p) & 15) == 0;
        for (int i = lane * 4; i < npairs; i += 256) {
            const int kk = k0 + 2 * i;
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (vec && kk + 8 <= K) {
                v = *reinterpret_cast<const u32x4_t *>(p + kk);
            } else if (p) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    uint32_t lo = 0, hi = 0;
                    if (kk + 2 * t < K) lo = p[kk + 2 * t];
                    if (kk + 2 * t + 1 < K) hi = p[kk + 2 * t + 1];
                    v[t] = lo | (hi << 16);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) v[t] = to_h2<XF16>(v[t]);
            *reinterpret_cast<u32x4_t *>(xs + m * npairs + i) = v;
        }
    }
    wave_sync();
    const int hp = gs / 2, quarter = (hp + 3) / 4, part = lane & 3;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        for (int g0 = 0; g0 < ngl; g0 += 16) {
            const int g = g0 + (lane >> 2);
            float sx = 0.f, st = 0.f;
            const int i1 = min(hp, (part + 1) * quarter);
            for (int i = part * quarter; i < i1; ++i) {
                const float ps = dot2h(xs[m * npairs + g * hp + i], 0x3c003c00u, 0.f);
                sx += ps;
                st = fmaf(ps, BW::bw(i), st);
            }
            sx = quad_sum(sx);
            st = quad_sum(st);
            if (part == 0) {
                xsum[(m * ngl + g) * 2] = sx;
                xsum[(m * ngl + g) * 2 + 1] = st;
            }
        }
    }
    wave_sync();
}

// Reduce the K-split (4 lanes inside the wave, then the waves of the block through `red`, a region
// of nwaves * MB * 16 floats that nothing else uses, in a fixed order) and store neuron
// `rb*16 + r - row_base` of each output row yr[m] (null = absent row).
template <int MB>
__device__ __forceinline__ void finish_rows(float (&v)[MB], float *red, int wave, int nwaves, int lane, int rb,
                                            int row_base, int out_rows, float *const (&yr)[MB]) {
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = reduce_kb4(v[m]);
    if (lane < 16) {
#pragma unroll
        for (int m = 0; m < MB; ++m) red[(wave * MB + m) * 16 + lane] = v[m];
    }
    __syncthreads();
    if (wave == 0) {
        const int r = lane & 15;
        const int row = rb * 16 + r - row_base;
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            if ((lane >> 4) == (m & 3)) {
                float s = 0.f;
                for (int wv = 0; wv < nwaves; ++wv) s += red[(wv * MB + m) * 16 + r];
                if (yr[m] && row >= 0 && row < out_rows) yr[m][row] = s;
            }
        }
    }
}

// Waves a decode GEMV launch aims for (the K-split per row-block follows from it); MFQ_GEMV_WAVES
// overrides the default for tuning.
inline int gemv_target_waves() {
    static const int v = [] {
        const char *e = getenv("MFQ_GEMV_WAVES");
        const int n = e ? atoi(e) : 0;
        return n > 0 ? n : 6144;
    }();
    return v;
}

// LDS bytes of a GEMV block: per wave MB * steps_per_wave * 16 groups * (gs/2 pairs + 2 sums) dwords,
// plus the cross-wave reduction area.
inline size_t gemv_lds_bytes(int mb, int spw, int gs, int nwaves) {
    return (static_cast<size_t>(mb) * spw * 16 * (gs / 2 + 2) * nwaves + static_cast<size_t>(nwaves) * mb * 16) * 4;
}

// Dense activations: rows m0 .. m0+MB-1 of x[M, ldx] / y[M, ldy].
template <int MB>
__device__ __forceinline__ void dense_rows(const uint16_t *x, int64_t ldx, float *y, int64_t ldy, int M, int m0,
                                           const uint16_t *(&xr)[MB], float *(&yr)[MB]) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const bool ok = m0 + m < M;
        xr[m] = ok ? x + static_cast<int64_t>(m0 + m) * ldx : nullptr;
        yr[m] = ok ? y + static_cast<int64_t>(m0 + m) * ldy : nullptr;
    }
}

}  // namespace mfq
