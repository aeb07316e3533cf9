// NINT prefill matmul: a block-tiled MFMA GEMM whose B operand is dequantized in registers.
//
// Block = 4 waves as WM (tokens) x 4/WM (neurons); a wave owns MT*16 tokens x NB*16 neurons and, like the
// small-batch kernel (nint_mfma.hpp), reads its weight units straight from HBM in the R16 layout, turns
// each dword of codes into an fp16 fragment (sub_scale * code / 64) with one AND-OR and one packed FMA
// per pair, and feeds v_mfma_f32_16x16x32_f16.  The activation tile (already fp16, see x_prep) of one
// sub-step -- the 4 * GS k-values of units j of a step -- is staged in LDS (double-buffered) once per block and
// shared by the waves; weights never touch LDS.  After the K loop the minimum term sum_g sub_min_g X_g runs as a
// short second loop (one MFMA per step and tile against precomputed group sums), then
//     y = xscale[token] * (64 * neuron_scale * S1 - neuron_min * S2).
#pragma once
#include "nint_mfma.hpp"

namespace mfq {

// xg: the group sums x_prep leaves, [token][step][kb] x 16 bytes (see gemm.hip).
template <class U, int MT, int NB, int WM, int NW>
__global__ __launch_bounds__(64 * NW) void nint_prefill_kernel(NintK k, const uint8_t *__restrict__ w,
                                                           const uint16_t *__restrict__ x16, int Kp,
                                                           const float *__restrict__ xscale,
                                                           const uint32_t *__restrict__ xg, int M,
                                                           float *__restrict__ y, int64_t ldy) {
    constexpr int D = U::D, GS = U::GROUP, NM = U::NPAIR / 4, BITS = U::CBITS;
    constexpr int NCLS = BITS == 0 ? 1 : (BITS == 3 ? 3 : 2);
    constexpr int WN = NW / WM;                // waves along the neurons
    constexpr int NT = 64 * NW;                // threads
    constexpr int BM = WM * MT * 16;           // tokens per block
    constexpr int ROW = 4 * GS + 8;            // LDS row stride in halves (16 bytes of padding)
    constexpr int CHUNKS = 4 * GS / 8;         // 16-byte chunks per tile row
    constexpr int PER_THREAD = (BM * CHUNKS + NT - 1) / NT;
    extern __shared__ __attribute__((aligned(16))) uint16_t xt[];  // two buffers of [BM][ROW]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int r = lane & 15, kb = lane >> 4;
    const int tok0 = blockIdx.y * BM;
    const int rb0 = (blockIdx.x * WN + wn) * NB;
    const int nrb = max(0, min(NB, k.n_rowblocks - rb0));
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(min(rb0, k.n_rowblocks - 1)) * k.rowblock_bytes, nrb * rbb);

    float4_t acc[MT][NB];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // global -> register copy of the activation tile of sub-step `it` (chunk c of a row = 8 halves at k0 + 8 c)
    u32x4_t xr[PER_THREAD];
    auto xload = [&](int it) {
        const int k0 = it * 4 * GS;
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int c = min(tid + NT * p, BM * CHUNKS - 1);
            const int row = c / CHUNKS, ch = c - row * CHUNKS;
            const int m = min(tok0 + row, M - 1);
            const int kk = k0 + 8 * ch;
            const int kc = min(kk, Kp - 8);
            u32x4_t v = *reinterpret_cast<const u32x4_t *>(x16 + static_cast<int64_t>(m) * Kp + kc);
            if (kk >= Kp) v = u32x4_t{0u, 0u, 0u, 0u};
            xr[p] = v;
        }
    };
    auto xstore = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int c = tid + NT * p;
            const int row = c / CHUNKS, ch = c - row * CHUNKS;
            if (c < BM * CHUNKS) *reinterpret_cast<u32x4_t *>(xt + buf * (BM * ROW) + row * ROW + 8 * ch) = xr[p];
        }
    };

    uint32_t q[NB][D], qn[NB][D], tails[NB], tailsn[NB];
    u32x2_t sc[NB], scn[NB];
    auto wload = [&](int it, uint32_t (&qq)[NB][D]) {
        const int s = it >> 2, j = it & 3;
#pragma unroll
        for (int b = 0; b < NB; ++b)
            load_unit_win<D, 0>(win, b < nrb && s < k.nsteps ? b * rbb + s * sb + (j * 64 + lane) * (D * 4) : kNoStep, qq[b]);
    };
    auto sload = [&](int s, uint32_t (&tt)[NB], u32x2_t (&ss)[NB]) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t off = b < nrb && s < k.nsteps ? b * rbb + s * sb + 1024 * D : kNoStep;
            tt[b] = 0;
            if constexpr (U::TAIL) tt[b] = __builtin_amdgcn_raw_buffer_load_b32(win, off + lane * 4, 0, 0);
            ss[b] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (U::TAIL ? 256 : 0) + lane * 8, 0, 0);
        }
    };

    xload(0);
    wload(0, q);
    sload(0, tails, sc);
    xstore(0);
    __syncthreads();
    for (int s = 0; s < k.nsteps; ++s) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int it = 4 * s + j;
        xload(it + 1);  // past the end: clamped addresses, zeros
        if (j & 1) wload(it + 1, q);
        else wload(it + 1, qn);
        if (j == 3) sload(s + 1, tailsn, scn);

        // fragment scale S = sub_scale / 64 / 2^o and bias C = -1024 S, both from the fp16 pair 1024 + sub_scale
        // (the byte dropped into the mantissa of 1024.0) with one exact packed FMA each
        half2_t S[NB][NCLS], C[NB][NCLS];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t scw = (j < 2) ? sc[b].x : sc[b].y;
            const uint32_t sel = 0x03000100u | ((4u + 2u * (j & 1)) << 16) | (4u + 2u * (j & 1));
            const half2_t X = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(scw, kMagicH2, sel));
#pragma unroll
            for (int c = 0; c < NCLS; ++c) {
                const _Float16 f = static_cast<_Float16>(1.f / static_cast<float>(64 << (BITS * c)));
                const _Float16 g = static_cast<_Float16>(1024.f / static_cast<float>(64 << (BITS * c)));
                S[b][c] = __builtin_elementwise_fma(X, half2_t{f, f}, half2_t{-g, -g});
                const _Float16 h = static_cast<_Float16>(1024.f * 1024.f / static_cast<float>(64 << (BITS * c)));
                C[b][c] = __builtin_elementwise_fma(X, half2_t{-g, -g}, half2_t{h, h});
            }
        }
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            u32x4_t af[MT];
#pragma unroll
            for (int a = 0; a < MT; ++a)
                af[a] = *reinterpret_cast<const u32x4_t *>(xt + (j & 1) * (BM * ROW) + ((wm * MT + a) * 16 + r) * ROW + kb * GS + 8 * m);
            // all weight fragments of this k-slice first, then the MFMAs back to back: while one wave's MFMAs run,
            // the other wave of the SIMD unpacks
            u32x4_t bf[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                uint32_t v[U::NPAIR];
                U::unpack((j & 1) ? qn[b] : q[b], (tails[b] >> (8 * j)) & 0xffu, v);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    bf[b][t] = __builtin_bit_cast(uint32_t, h2_fma(v[4 * m + t], S[b][U::cls(4 * m + t)], C[b][U::cls(4 * m + t)]));
            }
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int a = 0; a < MT; ++a) acc[a][b] = mfma16(af[a], bf[b], acc[a][b]);
        }
        xstore((j + 1) & 1);  // the other buffer: nobody reads it during this sub-step
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (j == 3) {
                tails[b] = tailsn[b];
                sc[b] = scn[b];
            }
        }
        __syncthreads();
      }
    }

    // minimum term and epilogue
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    float ns[NB], nm[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int rb = min(rb0 + b, k.n_rowblocks - 1);
        ns[b] = anchors[rb * 16 + r] * 64.f;
        nm[b] = anchors[16 * k.n_rowblocks + rb * 16 + r];
    }
    // sum_g sub_min_g X_g: one MFMA per step and tile, operands of step s + 1 requested while step s multiplies
    float4_t accM[MT][NB];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) accM[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
    int64_t xgrow[MT];
#pragma unroll
    for (int a = 0; a < MT; ++a)
        xgrow[a] = static_cast<int64_t>(min(tok0 + (wm * MT + a) * 16 + r, M - 1)) * k.nsteps * 16 + kb * 4;
    u32x4_t ax[MT], axn[MT];
    auto gload = [&](int s, u32x4_t (&dst)[MT]) {
        const int sc_ = min(s, k.nsteps - 1);
#pragma unroll
        for (int a = 0; a < MT; ++a) dst[a] = *reinterpret_cast<const u32x4_t *>(xg + xgrow[a] + sc_ * 16);
    };
    sload(0, tails, sc);
    gload(0, ax);
    for (int s = 0; s < k.nsteps; ++s) {
        sload(s + 1, tailsn, scn);
        gload(s + 1, axn);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const half2_t m01 = pk_h2(ubyte_f32(sc[b].x, 1), ubyte_f32(sc[b].x, 3));
            const half2_t m23 = pk_h2(ubyte_f32(sc[b].y, 1), ubyte_f32(sc[b].y, 3));
            const uint32_t b01 = __builtin_bit_cast(uint32_t, m01), b23 = __builtin_bit_cast(uint32_t, m23);
            const u32x4_t bfm = u32x4_t{b01, b23, b01, b23};
#pragma unroll
            for (int a = 0; a < MT; ++a) accM[a][b] = mfma16(ax[a], bfm, accM[a][b]);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) sc[b] = scn[b];
#pragma unroll
        for (int a = 0; a < MT; ++a) ax[a] = axn[a];
    }
#pragma unroll
    for (int a = 0; a < MT; ++a) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int m = tok0 + (wm * MT + a) * 16 + 4 * kb + v;
            if (m >= M) continue;
            const float xs = xscale[m];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int row = (rb0 + b) * 16 + r;
                if (row < k.out) y[static_cast<int64_t>(m) * ldy + row] = xs * (ns[b] * acc[a][b][v] - nm[b] * accM[a][b][v]);
            }
        }
    }
}

}  // namespace mfq
