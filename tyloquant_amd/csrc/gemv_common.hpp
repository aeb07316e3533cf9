// Pieces shared by the decode GEMV kernels of every format: unit loads, the wave-private LDS
// staging of the activation slice with its per-group sums, and the final reductions.
#pragma once
#include <stdlib.h>

#include "common.hpp"
#include "tune.hpp"

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

// Range-checked window over the bytes one wave streams.  Loads through it are unconditional
// instructions: an offset at or beyond `bytes` returns zeros and moves no data, so the prefetch of a
// step that does not exist needs no branch and the compiler can count outstanding loads exactly.
// `base` and `bytes` must be the same in every lane of the wave.
constexpr uint32_t kNoStep = 0x80000000u;  // an offset outside every window
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_window(const uint8_t *base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    const uint64_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(a)));
    const uint64_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(a >> 32)));
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>((hi << 32) | lo), 0,
                                             __builtin_amdgcn_readfirstlane(static_cast<int>(bytes)), 0x00020000);
}

// POLICY = 2: non-temporal (weights streamed once, decode); 0: cached (weights re-read by other blocks, prefill)
template <int D, int POLICY = 2>
__device__ __forceinline__ void load_unit_win(__amdgpu_buffer_rsrc_t win, uint32_t off, uint32_t (&q)[D]) {
    if constexpr (D % 4 == 0) {
#pragma unroll
        for (int i = 0; i < D / 4; ++i) {
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(win, off + 16 * i, 0, POLICY);
            q[4 * i] = v.x; q[4 * i + 1] = v.y; q[4 * i + 2] = v.z; q[4 * i + 3] = v.w;
        }
    } else if constexpr (D % 2 == 0) {
#pragma unroll
        for (int i = 0; i < D / 2; ++i) {
            const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(win, off + 8 * i, 0, POLICY);
            q[2 * i] = v.x; q[2 * i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < D; ++i) q[i] = __builtin_amdgcn_raw_buffer_load_b32(win, off + 4 * i, 0, POLICY);
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

// Staging policy.  xscale(pos, t): power of two by which pair pos + t of a group is multiplied
// while it is staged (pos = first pair of a 4-pair chunk); inv_xscale(i) its reciprocal for pair i;
// bw(i): weight of the staged pair sum in T_g.
struct PlainBias {  // formats whose unpack needs neither
    static constexpr bool SCALED = false;
    __device__ static __forceinline__ float bw(int) { return 0.f; }
    __device__ static __forceinline__ float xscale(int, int) { return 1.f; }
    __device__ static __forceinline__ float inv_xscale(int) { return 1.f; }
};

// staged fp16 pair times a power of two
__device__ __forceinline__ uint32_t scale_h2(uint32_t pair, float s) {
    const _Float16 h = static_cast<_Float16>(s);
    const half2_t v = __builtin_bit_cast(half2_t, pair) * half2_t{h, h};
    return __builtin_bit_cast(uint32_t, v);
}

// Activation chunks a lane may hold in registers while the first weight loads are in flight.
constexpr int kXChunks = 4;
template <int MB>
struct XRegs {
    u32x4_t v[MB][kXChunks];
    bool on;
};

// First half of the staging: request the wave's K-slice of the activation rows into registers.  Issued
// before the weight loads so that (loads retiring in order) the staging never waits for weights.  Only the
// common case is prefetched -- aligned rows, K % 8 == 0, at most 256 * kXChunks pairs, MB <= 2; anything
// else is fetched by stage_x itself.
template <int MB>
__device__ __forceinline__ void stage_x_issue(const uint16_t *const (&xr)[MB], int K, int k0, int npairs, int lane,
                                              XRegs<MB> &xg) {
    bool ok = MB <= 2 && npairs <= 256 * kXChunks && K % 8 == 0;  // K % 8: no 8-element chunk straddles the end
#pragma unroll
    for (int m = 0; m < MB; ++m) ok = ok && (reinterpret_cast<uintptr_t>(xr[m]) & 15) == 0;
    xg.on = ok;
    if (ok) {
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            // range-checked window over the row (empty for an absent row): a chunk outside the slice or the row is an
            // out-of-range offset that returns zeros, so nothing here depends on the loaded data and the weight requests
            // that follow go out without waiting for the activations
            const __amdgpu_buffer_rsrc_t wx =
                wave_window(reinterpret_cast<const uint8_t *>(xr[m]), xr[m] ? static_cast<uint32_t>(K) * 2u : 0u);
#pragma unroll
            for (int c = 0; c < kXChunks; ++c) {
                const int i = lane * 4 + c * 256;
                const bool in = i < npairs && k0 + 2 * i + 8 <= K;
                xg.v[m][c] = __builtin_amdgcn_raw_buffer_load_b128(wx, in ? static_cast<uint32_t>(k0 + 2 * i) * 2u : kNoStep, 0, 0);
            }
        }
    }
}

// Hook between the request of the activation slice and its staging: nothing (the plain GEMV) ...
struct NoXPre {
    template <int MB>
    __device__ __forceinline__ void issue(int, int, int, int) {}
    template <int XF16, int MB>
    __device__ __forceinline__ void finish(XRegs<MB> &) {}
};
// ... or the input gate of a projection: the rows' gate slices are requested right after the activations (same
// chunks, so the weight requests that follow still wait for nothing) and x * act(gate) replaces the activations in
// their registers -- input_gate_value, the rounding of the separate elementwise launch -- before they are staged.
// Needs the prefetched case of stage_x_issue (the launch checks it): MB <= 2, aligned rows, K % 8 == 0.
template <int MB>
struct InputGate {
    const uint16_t *gr[MB];
    int mode;
    u32x4_t g[MB][kXChunks];
    template <int MBX>
    __device__ __forceinline__ void issue(int K, int k0, int npairs, int lane) {
        static_assert(MBX == MB, "one gate row per activation row");
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const __amdgpu_buffer_rsrc_t wg =
                wave_window(reinterpret_cast<const uint8_t *>(gr[m]), gr[m] ? static_cast<uint32_t>(K) * 2u : 0u);
#pragma unroll
            for (int c = 0; c < kXChunks; ++c) {
                const int i = lane * 4 + c * 256;
                const bool in = i < npairs && k0 + 2 * i + 8 <= K;
                g[m][c] = __builtin_amdgcn_raw_buffer_load_b128(wg, in ? static_cast<uint32_t>(k0 + 2 * i) * 2u : kNoStep, 0, 0);
            }
        }
    }
    template <int XF16, int MBX>
    __device__ __forceinline__ void finish(XRegs<MB> &xg) {
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int c = 0; c < kXChunks; ++c)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint32_t xv = xg.v[m][c][t], gv = g[m][c][t];
                    xg.v[m][c][t] = input_gate_value<XF16>(xv & 0xffffu, gv & 0xffffu, mode) |
                                    (static_cast<uint32_t>(input_gate_value<XF16>(xv >> 16, gv >> 16, mode)) << 16);
                }
    }
};

// Largest bf16 magnitudes (bit patterns without the sign) seen so far in the low and the high halves, kept as a packed
// pair of 16-bit maxima: one AND and one packed max per dword.
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t absmax_bf16(uint32_t m, uint32_t pair) {
    const u16x2_t a = __builtin_bit_cast(u16x2_t, m), b = __builtin_bit_cast(u16x2_t, pair & 0x7fff7fffu);
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}

// Power of two that brings the wave's slice of a bf16 row to a largest magnitude near 2^12, as an fp32 bit pattern
// (`mx` = largest magnitude pattern over the slice, the same in every lane); 1.0 for an all-zero or non-finite slice.
// The reciprocal is exact and comes back through `inv`.
__device__ __forceinline__ float slice_scale(uint32_t mx, float &inv) {
    const uint32_t e = mx >> 7;  // biased exponent of the largest magnitude
    if (e == 0u || e == 255u) {
        inv = 1.f;
        return 1.f;
    }
    const uint32_t field = min(266u - e, 253u);  // 2^(139 - e), capped so that the reciprocal stays normal
    inv = __uint_as_float((254u - field) << 23);
    return __uint_as_float(field << 23);
}

// Largest 16-bit half over the whole wave of the packed pairs absmax_bf16 collects: four DPP steps spread the maximum
// over each row of 16 lanes, the four rows meet in scalar registers -- no LDS round trips.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t packed) {
    int v = static_cast<int>(max(packed & 0xffffu, packed >> 16));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));  // row_half_mirror
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));  // row_mirror
    const int a = max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16));
    const int b = max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48));
    return static_cast<uint32_t>(max(a, b));
}

// bf16 pair times a power of two, as an fp16 pair
__device__ __forceinline__ uint32_t to_h2_scaled(uint32_t pair, float s) {
    const float lo = __uint_as_float(pair << 16) * s, hi = __uint_as_float(pair & 0xffff0000u) * s;
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}

// Stage the wave's K-slice of the MB activation rows xr[m] (null = absent row) into its private
// LDS region as fp16 (x[2i], x[2i+1]) pairs times BW::xscale, zero beyond K.  Next to it, per group
// g, two floats: X_g = sum of x over the group and -T_g, T_g = sum over its pairs i of the staged
// pair sum times BW::bw(i) (the bias the unpack trick adds to the dot product).  npairs is a multiple
// of 8; xs is 16-byte aligned.  `xg` = what stage_x_issue requested.
// SCALE (bf16 rows only): the slice of every row is first multiplied by the power of two that brings its largest
// magnitude near 2^12, so that rows of any magnitude keep their bits inside fp16's range; xinv[m] receives the
// reciprocal, which the caller multiplies into the sums it forms from this slice (1 without SCALE or for fp16 rows).
template <int XF16, int MB, class BW, bool SCALE = false>
__device__ __forceinline__ void stage_x(const uint16_t *const (&xr)[MB], int K, int k0, int npairs, int gs, int ngl,
                                        uint32_t *xs, float *xsum, int lane, const XRegs<MB> &xg, float *xinv = nullptr) {
    constexpr bool RESCALE = SCALE && !XF16;
    float sc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) sc[m] = 1.f;
    if (xg.on) {
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            if constexpr (RESCALE) {
                uint32_t mx = 0;
#pragma unroll
                for (int c = 0; c < kXChunks; ++c)
#pragma unroll
                    for (int t = 0; t < 4; ++t) mx = absmax_bf16(mx, xg.v[m][c][t]);
                float inv;
                sc[m] = slice_scale(wave_max_u32(mx), inv);
                if (xinv) xinv[m] = inv;
            } else if (xinv) {
                xinv[m] = 1.f;
            }
#pragma unroll
            for (int c = 0; c < kXChunks; ++c) {
                const int i = lane * 4 + c * 256;
                u32x4_t v = xg.v[m][c];
#pragma unroll
                for (int t = 0; t < 4; ++t) v[t] = RESCALE ? to_h2_scaled(v[t], sc[m]) : to_h2<XF16>(v[t]);
                if constexpr (BW::SCALED) {
                    const int pos = i % (gs / 2);
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[t] = scale_h2(v[t], BW::xscale(pos, t));
                }
                if (i < npairs) *reinterpret_cast<u32x4_t *>(xs + m * npairs + i) = v;
            }
        }
    } else {
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const uint16_t *p = xr[m];
            const bool vec = p && (reinterpret_cast<uintptr_t>(p) & 15) == 0;
            auto fetch = [&](int i) {
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
                return v;
            };
            if constexpr (RESCALE) {  // a first pass over the slice for its largest magnitude
                uint32_t mx = 0;
                for (int i = lane * 4; i < npairs; i += 256) {
                    const u32x4_t v = fetch(i);
#pragma unroll
                    for (int t = 0; t < 4; ++t) mx = absmax_bf16(mx, v[t]);
                }
                float inv;
                sc[m] = slice_scale(wave_max_u32(mx), inv);
                if (xinv) xinv[m] = inv;
            } else if (xinv) {
                xinv[m] = 1.f;
            }
            for (int i = lane * 4; i < npairs; i += 256) {
                u32x4_t v = fetch(i);
#pragma unroll
                for (int t = 0; t < 4; ++t) v[t] = RESCALE ? to_h2_scaled(v[t], sc[m]) : to_h2<XF16>(v[t]);
                if constexpr (BW::SCALED) {
                    const int pos = i % (gs / 2);
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[t] = scale_h2(v[t], BW::xscale(pos, t));
                }
                *reinterpret_cast<u32x4_t *>(xs + m * npairs + i) = v;
            }
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
                sx = fmaf(ps, BW::inv_xscale(i), sx);
                st = fmaf(ps, BW::bw(i), st);
            }
            sx = quad_sum(sx);
            st = quad_sum(st);
            if (part == 0) {
                xsum[(m * ngl + g) * 2] = sx;
                xsum[(m * ngl + g) * 2 + 1] = -st;
            }
        }
    }
    wave_sync();
}

// Output reduction.  park_rows: reduce the K-split of the 4 lanes of a neuron and leave the wave's
// partial sums of one 16-neuron row-block in `red` slot (rbi * nwaves + wave).  flush_rows: after a
// block barrier, add the waves' partials in a fixed order and store neuron (rb0 + rbi) * 16 + r -
// row_base of each output row yr[m] (null = absent row).  `red` holds rbw * nwaves * MB * 16 floats
// that nothing else uses.
template <int MB>
__device__ __forceinline__ void park_rows(float (&v)[MB], float *red, int slot, int lane) {
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = reduce_kb4(v[m]);
    if (lane < 16) {
#pragma unroll
        for (int m = 0; m < MB; ++m) red[(slot * MB + m) * 16 + lane] = v[m];
    }
}

template <int MB>
__device__ __forceinline__ void flush_rows(const float *red, int nwaves, int rbw, int rb0, int row_base, int out_rows,
                                           float *const (&yr)[MB]) {
    __syncthreads();
    for (int o = threadIdx.x; o < rbw * MB * 16; o += blockDim.x) {
        const int r = o & 15, m = (o >> 4) % MB, rbi = (o >> 4) / MB;
        float s = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) s += red[((rbi * nwaves + wv) * MB + m) * 16 + r];
        const int row = (rb0 + rbi) * 16 + r - row_base;
        float *dst = nullptr;
#pragma unroll
        for (int mm = 0; mm < MB; ++mm)
            if (mm == m) dst = yr[mm];
        if (dst && row >= 0 && row < out_rows) dst[row] = s;
    }
}

template <int MB>
__device__ __forceinline__ void finish_rows(float (&v)[MB], float *red, int wave, int nwaves, int lane, int rb,
                                            int row_base, int out_rows, float *const (&yr)[MB]) {
    park_rows<MB>(v, red, wave, lane);
    flush_rows<MB>(red, nwaves, 1, rb, row_base, out_rows, yr);
}

// Fewest waves a decode GEMV launch aims for before a wave is given more than one step;
// MFQ_GEMV_WAVES overrides the default for tuning.
inline int gemv_target_waves() {
    static const int v = [] {
        const int n = tune_env("MFQ_GEMV_WAVES", 2048);
        return n > 0 ? n : 2048;
    }();
    return v;
}

// Compute units a one-block-per-CU grid is sized for: the device's own count (mfq_hip_set_cu_count overrides it, so
// that a test can walk the row-blocks-per-block variants on small tensors).
inline int gemv_cu_count() { return device_cu_count(); }

// LDS bytes of a GEMV block: per wave MB * steps_per_wave * 16 groups * (gs/2 pairs + 2 sums) dwords,
// plus the cross-wave reduction area of rbw row-blocks.
inline size_t gemv_lds_bytes(int mb, int spw, int gs, int nwaves, int rbw = 1) {
    return (static_cast<size_t>(mb) * spw * 16 * (gs / 2 + 2) * nwaves + static_cast<size_t>(rbw) * nwaves * mb * 16) * 4;
}

// One launch over the (token, route) pairs of a MoE decode step on a cohort whose kernels know nothing of experts:
// block row p = blockIdx.y multiplies the tensor of expert ids[p] with activation row p (routed input) or p / R into
// output row p.  slot[e] = index of expert e among the cohort's experts, -1 for an expert of another cohort (and ids
// outside [0, E)): such blocks leave at once, before any barrier.  weights: one device pointer per expert of the cohort
// (experts that are tensors of their own), or null for a cohort that is one expert-shaped tensor.  ids = null: a dense call.
struct PairSel {
    const int32_t *ids, *slot;
    const uint8_t *const *weights;
    int E, R, routed_input;
};

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

// Rows of a block: dense_rows, or the pair blockIdx.y of a PairSel launch (one row per block).  False: the pair belongs
// to another cohort.  `w` is replaced by the expert's tensor where the cohort has one per expert; `local` = its index.
template <int MB>
__device__ __forceinline__ bool select_rows(const PairSel &sel, const uint8_t *&w, int &local, const uint16_t *x, int64_t ldx,
                                            float *y, int64_t ldy, int M, const uint16_t *(&xr)[MB], float *(&yr)[MB]) {
    local = 0;
    if (!sel.ids) {
        dense_rows<MB>(x, ldx, y, ldy, M, blockIdx.y * MB, xr, yr);
        return true;
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        xr[m] = nullptr;
        yr[m] = nullptr;
    }
    const int p = blockIdx.y;
    const int e = sel.ids[p];
    const int l = (e >= 0 && e < sel.E) ? sel.slot[e] : -1;
    if (l < 0) return false;
    local = l;
    if (sel.weights) w = sel.weights[l];
    xr[0] = x + static_cast<int64_t>(sel.routed_input ? p : p / sel.R) * ldx;
    yr[0] = y + static_cast<int64_t>(p) * ldy;
    return true;
}

}  // namespace mfq
