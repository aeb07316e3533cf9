// Pieces shared by the decode GEMV kernels of every format: unit loads, the wave-private LDS
// staging of the activation slice with its per-group sums, and the final reductions.
#pragma once
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

// Stage the wave's K-slice of the MB activation rows xr[m] (null = absent row) into its private
// LDS region as (x[2i], x[2i+1]) pairs, zero beyond K, with the per-group sums next to it.
template <int XF16, int MB>
__device__ __forceinline__ void stage_x(const uint16_t *const (&xr)[MB], int K, int k0, int npairs, int gs, int ngl,
                                        uint32_t *xs, float *xsum, int lane) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const uint16_t *p = xr[m];
        for (int i = lane; i < npairs; i += 64) {
            const int kk = k0 + 2 * i;
            uint32_t lo = 0, hi = 0;
            if (p && kk < K) lo = p[kk];
            if (p && kk + 1 < K) hi = p[kk + 1];
            xs[m * npairs + i] = lo | (hi << 16);
        }
    }
    __syncthreads();
    const int hp = gs / 2;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        for (int g = lane; g < ngl; g += 64) {
            float s = 0.f;
            for (int i = 0; i < hp; ++i) s = dot2<XF16>(xs[m * npairs + g * hp + i], ones_pair<XF16>(), s);
            xsum[m * ngl + g] = s;
        }
    }
    __syncthreads();
}

// Reduce the K-split (4 lanes inside the wave, then the waves of the block through LDS, in a fixed
// order) and store neuron `rb*16 + r - row_base` of each output row yr[m] (null = absent row).
template <int MB>
__device__ __forceinline__ void finish_rows(float (&v)[MB], float *red, int wave, int nwaves, int lane, int rb,
                                            int row_base, int out_rows, float *const (&yr)[MB]) {
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = reduce_kb4(v[m]);
    __syncthreads();  // everyone is done with the staged x: the region is reused for the cross-wave sums
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
