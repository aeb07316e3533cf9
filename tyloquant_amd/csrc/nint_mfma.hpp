// NINT small-batch matmul on the matrix cores: up to 16 activation rows against packed weights
// streamed once, for the price of a batch-1 GEMV.
//
// One v_mfma_f32_16x16x32_f16 multiplies a 16-token x 32-k activation fragment with a 32-k x 16-neuron
// weight fragment.  In the R16 layout lane (r, kb) of a wave holds, per unit, the codes of one group
// of neuron r; dword/pair order is the natural weight order, so fragment m of unit j is weights
// 8m .. 8m+7 of group 4j + kb -- exactly the 8 k-values the B operand wants from lane r + 16 kb -- and
// the matching A operand of lane (token, kb) is 16 contiguous bytes of that token's activations.
// The same AND-OR that feeds the GEMV gives (1024 + 2^o c) pairs; one packed fp16 FMA per pair turns
// them into sub_scale * c / 64 (an exact small integer multiple of 1/64 for sub-scales up to 6 bits),
// so groups with different sub-scales accumulate in one fp32 MFMA accumulator and only the neuron
// anchors are applied afterwards.  The minimum term sum_g sub_min_g * X_g (X_g = a token's activation
// sum over group g) is one more MFMA per step: sub_min bytes as fp16 against X_g split into two fp16
// halves.  A wave walks NB consecutive row-blocks with the same activation fragments.
#pragma once
#include "nint_body.hpp"

namespace mfq {

// 8 activations of the lane's token from k position kpos as fp16, zero at and beyond K.  K % 8 == 0;
// kpos is a multiple of 8 (ALIGN8) or of 4, in which case the fragment may straddle K by 4 elements.
typedef u32x4_t __attribute__((aligned(4))) u32x4_a4_t;
template <int XF16, bool ALIGN8>
__device__ __forceinline__ u32x4_t load_xfrag(const uint16_t *__restrict__ xrow, int kpos, int K) {
    const int kc = min(kpos, K - 8);
    u32x4_t v;
    if constexpr (ALIGN8) v = *reinterpret_cast<const u32x4_t *>(xrow + kc);
    else v = *reinterpret_cast<const u32x4_a4_t *>(xrow + kc);
#pragma unroll
    for (int t = 0; t < 4; ++t) v[t] = to_h2<XF16>(v[t]);
    if constexpr (!ALIGN8) {
        if (kpos + 4 == K) v = u32x4_t{v.z, v.w, 0u, 0u};
    }
    if (kpos >= K) v = u32x4_t{0u, 0u, 0u, 0u};
    return v;
}
// The same in two halves for a software pipeline: the request (clamped address, 16 raw bytes) and, when the value is
// needed, the conversion to fp16 and the zeroing at and beyond K.
template <bool ALIGN8>
__device__ __forceinline__ u32x4_t load_xfrag_raw(const uint16_t *__restrict__ xrow, int kpos, int K) {
    const int kc = max(0, min(kpos, K - 8));
    if constexpr (ALIGN8) return *reinterpret_cast<const u32x4_t *>(xrow + kc);
    else return *reinterpret_cast<const u32x4_a4_t *>(xrow + kc);
}
template <int XF16, bool ALIGN8>
__device__ __forceinline__ u32x4_t xfrag_finish(u32x4_t v, int kpos, int K) {
#pragma unroll
    for (int t = 0; t < 4; ++t) v[t] = to_h2<XF16>(v[t]);
    if constexpr (!ALIGN8) {
        if (kpos + 4 == K) v = u32x4_t{v.z, v.w, 0u, 0u};
    }
    if (kpos >= K) v = u32x4_t{0u, 0u, 0u, 0u};
    return v;
}

__device__ __forceinline__ half2_t pk_h2(float lo, float hi) {
    return __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}

__device__ __forceinline__ half2_t h2_fma(uint32_t a, half2_t b, half2_t c) {
    return __builtin_elementwise_fma(__builtin_bit_cast(half2_t, a), b, c);
}

__device__ __forceinline__ float4_t mfma16(u32x4_t a, u32x4_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0,
                                                  0);
}

// Adds the waves' partial tiles left in `red` (layout of nint_mfma_body) after a block barrier and stores
// y[m0 + token][rb0 * 16 + neuron] for the tokens below M and the neurons below out_rows.
template <int NB>
__device__ __forceinline__ void mfma_store_dense(const float *red, int rb0, int m0, int M, int out_rows,
                                                 float *__restrict__ y, int64_t ldy) {
    __syncthreads();
    const int nwaves = blockDim.x >> 6;
    for (int o = threadIdx.x; o < NB * 256; o += blockDim.x) {
        const int rr = o & 15, t = (o >> 4) & 15, nb = o >> 8;
        const int slot = (nb * 4 + (t & 3)) * 64 + rr + 16 * (t >> 2);
        float s = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) s += red[wv * NB * 256 + slot];
        const int row = (rb0 + nb) * 16 + rr;
        if (m0 + t < M && row < out_rows) y[static_cast<int64_t>(m0 + t) * ldy + row] = s;
    }
}

// Block = the row-blocks [rb0, min(rb0 + NB, rb_end)); its waves split the K steps (spw each).  xrow: the
// activation row of token (lane & 15) of this 16-token tile (any valid row for an absent token).
// Leaves, in `red`, the wave's partial results: red[((wave * NB + nb) * 4 + v) * 64 + lane] =
// partial y[token 4 * (lane >> 4) + v][neuron (rb0 + nb) * 16 + (lane & 15)]; the caller adds the waves
// after a barrier.
template <class U, int XF16, int NB>
__device__ __forceinline__ void nint_mfma_body(const NintK &k, const uint8_t *__restrict__ w, int rb0, int rb_end,
                                               const uint16_t *__restrict__ xrow, int spw, float *red) {
    constexpr int D = U::D, GS = U::GROUP, NM = U::NPAIR / 4, BITS = U::CBITS;
    constexpr int NCLS = BITS == 0 ? 1 : (BITS == 3 ? 3 : 2);
    constexpr bool ALIGN8 = GS % 8 == 0;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;
    const int nrb = min(NB, rb_end - rb0);
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    float ns[NB], nm[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int rb = min(rb0 + i, k.n_rowblocks - 1);
        ns[i] = anchors[rb * 16 + r] * 64.f;
        nm[i] = anchors[16 * k.n_rowblocks + rb * 16 + r];
    }
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb0) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);
    float4_t accS[NB], accM[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) accS[i] = accM[i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // One step of register buffers per row-block, refilled unit by unit: as soon as unit j of step s is unpacked, unit j
    // of step s + 1 is requested into the same registers, so the weight stream runs most of a step ahead of the unpack
    // without a second set of buffers.  Requests past the wave's last step are out-of-range offsets that move no data.
    uint32_t q[NB][4][D], tails[NB], tailsn[NB];
    u32x2_t sc[NB], scn[NB];
    auto unit_off = [&](int i, int s, int j) -> uint32_t {
        return i < nrb && s < n ? i * rbb + s * sb + (j * 64 + lane) * (D * 4) : kNoStep;
    };
    auto scale_load = [&](int s, uint32_t (&tt)[NB], u32x2_t (&ss)[NB]) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const uint32_t off = i < nrb && s < n ? i * rbb + s * sb + 1024 * D : kNoStep;
            tt[i] = 0;
            if constexpr (U::TAIL) tt[i] = __builtin_amdgcn_raw_buffer_load_b32(win, off + lane * 4, 0, 2);
            ss[i] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (U::TAIL ? 256 : 0) + lane * 8, 0, 2);
        }
    };
    scale_load(0, tails, sc);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < NB; ++i) load_unit_win<D>(win, unit_off(i, 0, j), q[i][j]);
    // Activation fragments run two units ahead of their use and are requested before the weight refill of the unit:
    // loads retire in order, so a fragment waits for the refills issued before it -- three units old by then -- and
    // never for the one just issued.
    auto xfrags = [&](int it, u32x4_t (&dst)[NM]) {  // fragments of unit it (= 4 * step + j) of the wave's K-slice
        const int kpos = (s0 + (it >> 2)) * 16 * GS + kb * GS + 4 * (it & 3) * GS;
#pragma unroll
        for (int m = 0; m < NM; ++m) dst[m] = load_xfrag_raw<ALIGN8>(xrow, kpos + 8 * m, k.neuron_len);
    };
    u32x4_t a1[NM], a2[NM];
    xfrags(0, a1);
    xfrags(1, a2);
    for (int s = 0; s < n; ++s) {
        scale_load(s + 1, tailsn, scn);
        float xsum[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x4_t a[NM];
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                a[m] = xfrag_finish<XF16, ALIGN8>(a1[m], (s0 + s) * 16 * GS + kb * GS + 4 * j * GS + 8 * m, k.neuron_len);
                a1[m] = a2[m];
            }
            xfrags(4 * s + j + 2, a2);
            float xs = 0.f;
#pragma unroll
            for (int m = 0; m < NM; ++m)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (8 * m + 2 * t < GS) xs = dot2h(a[m][t], 0x3c003c00u, xs);  // the last fragment may reach past the group
            xsum[j] = xs;
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                // fragment scale S = sub_scale / 64 / 2^o and bias C = -1024 S, both from the fp16 pair 1024 + sub_scale
                // (the byte dropped into the mantissa of 1024.0) with one exact packed FMA each
                const uint32_t scw = (j < 2) ? sc[i].x : sc[i].y;
                const uint32_t sel = 0x03000100u | ((4u + 2u * (j & 1)) << 16) | (4u + 2u * (j & 1));
                const half2_t X = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(scw, kMagicH2, sel));
                half2_t S[NCLS], C[NCLS];
#pragma unroll
                for (int c = 0; c < NCLS; ++c) {
                    const _Float16 f = static_cast<_Float16>(1.f / static_cast<float>(64 << (BITS * c)));
                    const _Float16 g = static_cast<_Float16>(1024.f / static_cast<float>(64 << (BITS * c)));
                    const _Float16 h = static_cast<_Float16>(1024.f * 1024.f / static_cast<float>(64 << (BITS * c)));
                    S[c] = __builtin_elementwise_fma(X, half2_t{f, f}, half2_t{-g, -g});
                    C[c] = __builtin_elementwise_fma(X, half2_t{-g, -g}, half2_t{h, h});
                }
                uint32_t v[U::NPAIR];
                U::unpack(q[i][j], (tails[i] >> (8 * j)) & 0xffu, v);
                load_unit_win<D>(win, unit_off(i, s + 1, j), q[i][j]);
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    u32x4_t b;
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        b[t] = __builtin_bit_cast(uint32_t, h2_fma(v[4 * m + t], S[U::cls(4 * m + t)], C[U::cls(4 * m + t)]));
                    accS[i] = mfma16(a[m], b, accS[i]);
                }
            }
        }
        // minimum term: slots 0..3 of the lane's 8 k-values = X_g high halves, 4..7 = low halves
        u32x4_t ax;
        {
            half2_t hi[2], lo[2];
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                hi[p] = pk_h2(xsum[2 * p], xsum[2 * p + 1]);
                lo[p] = pk_h2(xsum[2 * p] - static_cast<float>(hi[p].x), xsum[2 * p + 1] - static_cast<float>(hi[p].y));
            }
            ax = u32x4_t{__builtin_bit_cast(uint32_t, hi[0]), __builtin_bit_cast(uint32_t, hi[1]),
                         __builtin_bit_cast(uint32_t, lo[0]), __builtin_bit_cast(uint32_t, lo[1])};
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const half2_t m01 = pk_h2(ubyte_f32(sc[i].x, 1), ubyte_f32(sc[i].x, 3));
            const half2_t m23 = pk_h2(ubyte_f32(sc[i].y, 1), ubyte_f32(sc[i].y, 3));
            const uint32_t b01 = __builtin_bit_cast(uint32_t, m01), b23 = __builtin_bit_cast(uint32_t, m23);
            accM[i] = mfma16(ax, u32x4_t{b01, b23, b01, b23}, accM[i]);
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            tails[i] = tailsn[i];
            sc[i] = scn[i];
        }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * NB + i) * 4 + v) * 64 + lane] = ns[i] * accS[i][v] - nm[i] * accM[i][v];
}

// Dense wrapper: block (row-block group, 16-token tile).
template <class U, int XF16, int NB, int MAXW = 8>
__global__ __launch_bounds__(64 * MAXW) void nint_mfma_kernel(NintK k, const uint8_t *__restrict__ w,
                                                         const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                         float *__restrict__ y, int64_t ldy, int spw) {
    extern __shared__ uint32_t lds[];
    float *red = reinterpret_cast<float *>(lds);
    const int rb0 = blockIdx.x * NB, m0 = blockIdx.y * 16;
    const int tok = min(m0 + static_cast<int>(threadIdx.x & 15), M - 1);
    nint_mfma_body<U, XF16, NB>(k, w, rb0, k.n_rowblocks, x + static_cast<int64_t>(tok) * ldx, spw, red);
    mfma_store_dense<NB>(red, rb0, m0, M, k.out, y, ldy);
}

}  // namespace mfq
