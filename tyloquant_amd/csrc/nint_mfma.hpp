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
// The same request through a buffer window over all activation rows (xoff = byte offset of the lane's row in it);
// live = false moves no data.
// With fragments on 8-element boundaries (K % 8 == 0) no address is clamped: a fragment at or beyond K is zeroed by
// xfrag_finish whatever was read (the next row's first elements, or nothing past the end of the window), so the
// fragments of a unit are one address register and immediate offsets.
template <bool ALIGN8>
__device__ __forceinline__ u32x4_t load_xfrag_win(__amdgpu_buffer_rsrc_t xwin, uint32_t xoff, int kpos, int m, int K, bool live) {
    if constexpr (ALIGN8) {
        const uint32_t base = live ? xoff + static_cast<uint32_t>(kpos) * 2u : kNoStep;
        return __builtin_amdgcn_raw_buffer_load_b128(xwin, base + 16u * m, 0, 0);
    } else {
        const int kc = max(0, min(kpos + 8 * m, K - 8));
        return __builtin_amdgcn_raw_buffer_load_b128(xwin, live ? xoff + static_cast<uint32_t>(kc) * 2u : kNoStep, 0, 0);
    }
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

// xfrag_finish for a bf16 row that is multiplied by a power of two on the way to fp16 (see slice_scale)
template <int XF16, bool ALIGN8>
__device__ __forceinline__ u32x4_t xfrag_finish_scaled(u32x4_t v, int kpos, int K, float scale) {
#pragma unroll
    for (int t = 0; t < 4; ++t) v[t] = XF16 ? v[t] : to_h2_scaled(v[t], scale);
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

// Block = the row-blocks [rb0, min(rb0 + NB, rb_end)); its waves split the K steps (spw each).  xwin: a buffer
// window over the activation rows, xoff: byte offset in it of the row of token (lane & 15) of this 16-token tile, or
// kNoStep for an absent token: its lanes then request nothing and multiply zeros (the fragments are what a compute
// unit moves most of -- 16 KB per wave and step against 4.6 KB of NINT4 weights -- so a tile of four rows asks for a
// quarter of them).
// Leaves, in `red`, the wave's partial results: red[((wave * NB + nb) * 4 + v) * 64 + lane] =
// partial y[token 4 * (lane >> 4) + v][neuron (rb0 + nb) * 16 + (lane & 15)]; the caller adds the waves
// after a barrier.
// AH: units by which the activation fragments run ahead of their use (4 = a whole step; 2 where the registers of a
// wave do not hold a step's fragments beside NB row-blocks of weights).
template <class U, int NB, int MAXW>
constexpr int mfma_x_ahead() {
    return (MAXW > 8 || (U::NPAIR / 4 > 4 && NB > 2)) ? 2 : 4;
}
template <class U, int XF16, int NB, int AH = 4>
__device__ __forceinline__ void nint_mfma_body(const NintK &k, const uint8_t *__restrict__ w, int rb0, int rb_end,
                                               __amdgpu_buffer_rsrc_t xwin, uint32_t xoff, int spw, float *red) {
    static_assert(AH == 2 || AH == 4, "the unit loop is unrolled four times");
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
    // Activation fragments run a whole step ahead of their use, in the registers of the unit they replace, and are
    // requested before the weights of their unit (the first step's before anything else): loads retire in order, so a
    // fragment requested behind weights waits for those weights, and one requested only two units ahead -- as an earlier
    // version did -- costs a round trip to memory per unit (12288 x 4096 at 4 rows: 20.7 us against the 12 us of one row).
    auto xfrags = [&](int u, u32x4_t (&dst)[NM]) {  // fragments of unit u (= 4 * step + j) of the wave's K-slice
        const int kpos = (s0 + (u >> 2)) * 16 * GS + kb * GS + 4 * (u & 3) * GS;
#pragma unroll
        for (int m = 0; m < NM; ++m) dst[m] = load_xfrag_win<ALIGN8>(xwin, xoff, kpos, m, k.neuron_len, (u >> 2) < n);
    };
    u32x4_t ax[AH][NM];
#pragma unroll
    for (int j = 0; j < AH; ++j) xfrags(j, ax[j]);
    scale_load(0, tails, sc);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < NB; ++i) load_unit_win<D>(win, unit_off(i, 0, j), q[i][j]);
    for (int s = 0; s < n; ++s) {
        scale_load(s + 1, tailsn, scn);
        float xsum[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x4_t a[NM];
#pragma unroll
            for (int m = 0; m < NM; ++m)
                a[m] = xfrag_finish<XF16, ALIGN8>(ax[j % AH][m], (s0 + s) * 16 * GS + kb * GS + 4 * j * GS + 8 * m, k.neuron_len);
            xfrags(4 * s + j + AH, ax[j % AH]);
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
    const int tok = m0 + static_cast<int>(threadIdx.x & 15);
    // the tile's 16 rows through one window from its first row on (at most 15 ldx + K elements)
    const __amdgpu_buffer_rsrc_t xwin =
        wave_window(reinterpret_cast<const uint8_t *>(x + static_cast<int64_t>(m0) * ldx),
                    static_cast<uint32_t>((static_cast<int64_t>(min(16, M - m0) - 1) * ldx + k.neuron_len) * 2));
    nint_mfma_body<U, XF16, NB, mfma_x_ahead<U, NB, MAXW>()>(
        k, w, rb0, k.n_rowblocks, xwin, tok < M ? static_cast<uint32_t>(static_cast<int64_t>(tok - m0) * ldx * 2) : kNoStep, spw, red);
    mfma_store_dense<NB>(red, rb0, m0, M, k.out, y, ldy);
}


// ---- up to 16 rows with the activations resident in LDS ---------------------------------------------------------------
// What a compute unit moves most of in nint_mfma_kernel is activation fragments: 16 KB per wave and K step against 4.6 KB
// of NINT4 weights, fetched again for every row-block group through the same path as the weights, and a grid of one
// block per group runs in two rounds where a compute unit holds one block (24576 x 4096 NINT4-32 at 4 rows: 18.7 us
// against the 12 us of one row).  Here one block per compute unit walks all its row-block groups; every wave converts
// its K-slice of the tile's rows once, into its own corner of the LDS (fp16; bf16 rows times the power of two that
// brings the wave's slice of a row near 2^10, the way the one-row kernels do, the partial sums scaled back), and reads the
// fragments of a unit from there while the weights of the next item stream in.  Measured on that tensor: 17.1 us at 3
// to 8 rows, 19.7 us at 16 (22.3 before); what is left over one row's time is the vector-ALU work of the unpack, which
// two waves per SIMD cannot hide behind each other the way the one-row kernel's four do, and the start (2.8 us until
// the first wave has staged its slice).  Taken when a wave owns one K step (K <= 8 steps; with more steps per wave the
// older kernel is as fast), groups of 32 or 16 weights (a 64-lane request then covers whole rows of a step), K % 8 == 0,
// the rows of the tile inside one 4 GiB window and the packed tensor inside another.
// LDS map: [red: red_slots * nwaves * NB * 256 f32][xinv: nwaves * 16 f32][chunk-row maxima and token scales: nwaves * 48 u32]
//          [fragments: nwaves * spw * rows * (32 GS + 16) bytes, a row of a step padded by 16 bytes]
template <class U>
constexpr int mfma_resident_row_bytes() { return 32 * U::GROUP + 16; }
// Largest 16-bit half of the packed pairs absmax_bf16 collects, over lanes 0 .. 31 (lo) and 32 .. 63 (hi)
__device__ __forceinline__ void half_wave_max_u32(uint32_t packed, uint32_t &lo, uint32_t &hi) {
    int v = static_cast<int>(max(packed & 0xffffu, packed >> 16));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true));  // row_half_mirror
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true));  // row_mirror
    lo = static_cast<uint32_t>(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)));
    hi = static_cast<uint32_t>(max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}
inline size_t mfma_resident_lds(int nwaves, int nb, int spw, int rows, int gs, int red_slots = 1) {
    return static_cast<size_t>(nwaves) * (red_slots * nb * 1024 + 256) + static_cast<size_t>(nwaves) * spw * rows * (32 * gs + 16);
}

template <class U, int XF16, int NB>
__global__ __launch_bounds__(512) void nint_mfma_resident_kernel(NintK k, const uint8_t *__restrict__ w,
                                                                 const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                 float *__restrict__ y, int64_t ldy, int spw,
                                                                 int red_slots) {
    constexpr int D = U::D, GS = U::GROUP, NM = U::NPAIR / 4, BITS = U::CBITS;
    constexpr int NCLS = BITS == 0 ? 1 : (BITS == 3 ? 3 : 2);
    constexpr int STEPK = 16 * GS, CPS = STEPK / 8, ROWB = mfma_resident_row_bytes<U>();
    static_assert(GS % 8 == 0, "groups of whole 16-byte chunks");
    extern __shared__ uint32_t lds[];
    const int lane = threadIdx.x & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int r = lane & 15, kb = lane >> 4;
    const int m0 = static_cast<int>(blockIdx.y) * 16, mt = min(16, M - m0);
    const int s0 = wave * spw;
    const int n = max(0, min(k.nsteps, s0 + spw) - s0);  // steps of this wave
    float *red = reinterpret_cast<float *>(lds);  // red_slots areas of nwaves * NB * 256 floats: the groups of a batch
    const int red_floats = nwaves * NB * 256;
    float *xinv = red + red_slots * red_floats + wave * 16;
    uint32_t *rowmax = reinterpret_cast<uint32_t *>(red + red_slots * red_floats + nwaves * 16) + wave * 48;
    uint8_t *xs = reinterpret_cast<uint8_t *>(red + red_slots * red_floats + nwaves * 64) + static_cast<size_t>(wave) * spw * mt * ROWB;
    typedef __attribute__((address_space(3))) const u32x4_t *lds_u32x4_ptr;
    const uint32_t xs_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)xs));

    // ---- requests, in order of use: the wave's slice of the rows, then its first item ------------------------------
    const __amdgpu_buffer_rsrc_t xwin =
        wave_window(reinterpret_cast<const uint8_t *>(x + static_cast<int64_t>(m0) * ldx),
                    static_cast<uint32_t>((static_cast<int64_t>(mt - 1) * ldx + k.neuron_len) * 2));
    // Request i of a lane is chunk c = lane % CPS of chunk-row rho = RPI * i + lane / CPS (chunk-row = step * mt +
    // token; RPI = 64 / CPS chunk-rows per request); the slice has spw * mt chunk-rows, at most 16 requests.
    constexpr int RPI = 64 / CPS;
    static_assert(CPS * RPI == 64, "a request covers whole chunk-rows");
    const int nrows = spw * mt, nreq = (nrows + RPI - 1) / RPI;
    const int c = lane & (CPS - 1), sub = lane / CPS;
    const uint32_t ldx2 = static_cast<uint32_t>(ldx) * 2u;
    u32x4_t raw[16];
    int row_of[16];  // token of the chunk, -1 = none
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int rho = RPI * i + sub;
        const int ls = (rho >= mt ? 1 : 0) + (rho >= 2 * mt ? 1 : 0) + (rho >= 3 * mt ? 1 : 0);
        const int t = rho - ls * mt;
        const int kpos = (s0 + ls) * STEPK + 8 * c;
        const bool ok = rho < nrows && ls < n && kpos < k.neuron_len;
        // (32-bit arithmetic: the launcher checks that the tile's rows span less than 4 GiB)
        raw[i] = __builtin_amdgcn_raw_buffer_load_b128(
            xwin, ok ? (static_cast<uint32_t>(t) * ldx2 + static_cast<uint32_t>(kpos) * 2u) : kNoStep, 0, 0);
        row_of[i] = rho < nrows ? t : -1;
    }
    const __amdgpu_buffer_rsrc_t win = wave_window(w, static_cast<uint32_t>(k.anchors_off));
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const int ngroups = (k.n_rowblocks + NB - 1) / NB;
    auto unit_off = [&](int g, int s, int i, int j) -> uint32_t {
        return g < ngroups && g * NB + i < k.n_rowblocks && s < n
                   ? static_cast<uint32_t>(g * NB + i) * rbb + static_cast<uint32_t>(s0 + s) * sb + (j * 64 + lane) * (D * 4)
                   : kNoStep;
    };
    uint32_t q[NB][4][D], tails[NB], tailsn[NB];
    u32x2_t sc[NB], scn[NB];
    auto scale_load = [&](int g, int s, uint32_t (&tt)[NB], u32x2_t (&ss)[NB]) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const uint32_t off = g < ngroups && g * NB + i < k.n_rowblocks && s < n
                                     ? static_cast<uint32_t>(g * NB + i) * rbb + static_cast<uint32_t>(s0 + s) * sb + 1024 * D
                                     : kNoStep;
            tt[i] = 0;
            if constexpr (U::TAIL) tt[i] = __builtin_amdgcn_raw_buffer_load_b32(win, off + lane * 4, 0, 2);
            ss[i] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (U::TAIL ? 256 : 0) + lane * 8, 0, 2);
        }
    };
    const int g_first = blockIdx.x, g_step = gridDim.x;
    scale_load(g_first, 0, tails, sc);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < NB; ++i) load_unit_win<D>(win, unit_off(g_first, 0, i, j), q[i][j]);

    // ---- the slice as fp16 in LDS ---------------------------------------------------------------------------------
    // bf16 rows: one power of two per (wave, token).  A chunk-row is a whole or a half wave of one request, so its largest
    // magnitude is a reduction over those lanes; the chunk-rows' maxima go through a 32-entry table in LDS, lanes
    // 0 .. 15 fold the steps of their token.  Requests past the slice (i >= nreq, the same for the whole wave) are skipped.
    if constexpr (!XF16) {
        uint32_t mine = 0;  // lane L keeps the maximum of chunk-row L (L < 32)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if (i < nreq) {
                uint32_t mx = 0;
#pragma unroll
                for (int t = 0; t < 4; ++t) mx = absmax_bf16(mx, raw[i][t]);
                uint32_t lo, hi;
                half_wave_max_u32(mx, lo, hi);
                if constexpr (RPI == 1) {
                    mine = lane == i ? max(lo, hi) : mine;
                } else {
                    mine = lane == 2 * i ? lo : (lane == 2 * i + 1 ? hi : mine);
                }
            }
        }
        if (lane < 32) rowmax[lane] = mine;   // chunk-rows past the slice hold zeros
        uint32_t tm = 0;
        if (lane < 16) {
#pragma unroll
            for (int ls = 0; ls < 4; ++ls)
                if (ls < spw && lane < mt) tm = max(tm, rowmax[ls * mt + lane]);
        }
        // Two binary orders below the one-row kernels' 2^12: the sum of a group's activations goes into the minimum
        // term's matrix product as two fp16 halves, so 32 elements of one sign must stay below 2 * 65504.
        float inv = 1.f;
        const float scl = slice_scale(tm, inv) * 0.25f;
        if (lane < 16) {
            rowmax[32 + lane] = __float_as_uint(scl);
            xinv[lane] = inv * 4.f;
        }
    } else {
        if (lane < 16) xinv[lane] = 1.f;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        if (i < nreq) {
            const float scl = XF16 || row_of[i] < 0 ? 1.f : __uint_as_float(rowmax[32 + row_of[i]]);
            u32x4_t v = raw[i];
#pragma unroll
            for (int t = 0; t < 4; ++t) v[t] = XF16 ? v[t] : to_h2_scaled(v[t], scl);
            if (row_of[i] >= 0) *reinterpret_cast<u32x4_t *>(xs + (RPI * i + sub) * ROWB + 16 * c) = v;
        }
    }
    // token 4 kb + v of the tile is row v of the lane's accumulators
    float xi[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) xi[v] = 4 * kb + v < mt ? xinv[4 * kb + v] : 0.f;
    const uint32_t arow = xs_lds + static_cast<uint32_t>(min(r, mt - 1) * ROWB + kb * GS * 2);  // the lane's token, its group of a unit
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    int slot = 0;  // groups of the current batch whose partial tiles wait in red
    for (int g = g_first; g < ngroups; g += g_step) {
        const int rb0 = g * NB;
        float ns[NB], nm[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int rb = min(rb0 + i, k.n_rowblocks - 1);
            ns[i] = anchors[rb * 16 + r] * 64.f;
            nm[i] = anchors[16 * k.n_rowblocks + rb * 16 + r];
        }
        float4_t accS[NB], accM[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) accS[i] = accM[i] = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < n; ++s) {
            // the item after this one: the next step of the group, or the first step of the block's next group
            const int gn = s + 1 < n ? g : g + g_step, sn = s + 1 < n ? s + 1 : 0;
            scale_load(gn, sn, tailsn, scn);
            float xsum[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x4_t a[NM];
#pragma unroll
                for (int m = 0; m < NM; ++m)
                    a[m] = *reinterpret_cast<lds_u32x4_ptr>(arow + static_cast<uint32_t>(s * mt * ROWB + 4 * j * GS * 2 + 16 * m));
                float xs_ = 0.f;
#pragma unroll
                for (int m = 0; m < NM; ++m)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (8 * m + 2 * t < GS) xs_ = dot2h(a[m][t], 0x3c003c00u, xs_);
                xsum[j] = xs_;
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const uint32_t scw = (j < 2) ? sc[i].x : sc[i].y;
                    const uint32_t sel = 0x03000100u | ((4u + 2u * (j & 1)) << 16) | (4u + 2u * (j & 1));
                    const half2_t X = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(scw, kMagicH2, sel));
                    half2_t S[NCLS], C[NCLS];
#pragma unroll
                    for (int c = 0; c < NCLS; ++c) {
                        const _Float16 f = static_cast<_Float16>(1.f / static_cast<float>(64 << (BITS * c)));
                        const _Float16 gg = static_cast<_Float16>(1024.f / static_cast<float>(64 << (BITS * c)));
                        const _Float16 h = static_cast<_Float16>(1024.f * 1024.f / static_cast<float>(64 << (BITS * c)));
                        S[c] = __builtin_elementwise_fma(X, half2_t{f, f}, half2_t{-gg, -gg});
                        C[c] = __builtin_elementwise_fma(X, half2_t{-gg, -gg}, half2_t{h, h});
                    }
                    uint32_t v[U::NPAIR];
                    U::unpack(q[i][j], (tails[i] >> (8 * j)) & 0xffu, v);
                    load_unit_win<D>(win, unit_off(gn, sn, i, j), q[i][j]);
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
            for (int v = 0; v < 4; ++v)
                red[slot * red_floats + ((wave * NB + i) * 4 + v) * 64 + lane] = (ns[i] * accS[i][v] - nm[i] * accM[i][v]) * xi[v];
        // The waves meet once per batch of red_slots groups (where the LDS holds a block's groups side by side, once per
        // launch): a barrier per group leaves every wave idle until the slowest has walked its item.
        ++slot;
        if (slot == red_slots || g + g_step >= ngroups) {
            for (int b = 0; b < slot; ++b)  // barrier, sum over the waves, store
                mfma_store_dense<NB>(red + b * red_floats, (g - (slot - 1 - b) * g_step) * NB, m0, M, k.out, y, ldy);
            __syncthreads();                // before the next batch's partial tiles land in red
            slot = 0;
        }
    }
}

}  // namespace mfq
