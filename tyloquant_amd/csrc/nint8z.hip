// NINT8-0: the GGML Q8_0 block layout under an MFQ dtype label -- blocks of one fp16 scale and 32 signed 8-bit codes,
// weight = scale * code (mfq/formats/nint8_zero.py:1-10).
//
// Device layout: the blocks of the file (34 bytes, which no aligned load can walk) are split at load time into
//   scales: fp16 [out][ng]          (ng = neuron_len / 32; the format requires a multiple of 32)
//   codes:  int8 [out][neuron_len]  (row-major: a wave reads 1 KB of one row per step, 16 codes per lane)
// Small batches: a wave owns a row at a time; the activations of the pass (up to MB rows) sit in LDS as fp16 next to
// their sums over 16-element chunks.  A code byte c becomes the fp16 value 1024 + (c ^ 0x80) = c + 1152 by dropping it
// into the mantissa of 1024.0 (one byte permute per pair), so a lane's 16 codes cost 8 permutes and 8 dot2 per
// activation row, and 1152 times the chunk sum comes off afterwards; the block scale multiplies the chunk's result.
// Larger batches dequantize once to fp16 rows with a power-of-two row scale and run the dense fp16 GEMM.
#include "common.hpp"
#include "nint_mfma.hpp"

namespace mfq {

struct N8zK {
    int out, neuron_len, ng;
    int64_t scales_off, codes_off;
};
static N8zK to_k(const mfq_nint8z_desc *d) {
    N8zK k;
    k.out = d->out; k.neuron_len = d->neuron_len; k.ng = d->ng; k.scales_off = d->scales_off; k.codes_off = d->codes_off;
    return k;
}

// one thread per 34-byte block of the payload
__global__ __launch_bounds__(256) void nint8z_repack_kernel(N8zK k, const uint8_t *__restrict__ blocks, uint8_t *__restrict__ dst) {
    const int64_t b = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (b >= static_cast<int64_t>(k.out) * k.ng) return;
    const uint8_t *src = blocks + b * 34;
    reinterpret_cast<uint16_t *>(dst + k.scales_off)[b] = static_cast<uint16_t>(src[0] | (src[1] << 8));
    uint32_t *q = reinterpret_cast<uint32_t *>(dst + k.codes_off) + b * 8;
#pragma unroll
    for (int t = 0; t < 8; ++t)
        q[t] = src[2 + 4 * t] | (src[3 + 4 * t] << 8) | (src[4 + 4 * t] << 16) | (static_cast<uint32_t>(src[5 + 4 * t]) << 24);
}

// fl(f32(scale) * f32(code)): the product of an 11-bit and an 8-bit significand is exact in fp32
__global__ __launch_bounds__(256) void nint8z_dequant_f32_kernel(N8zK k, const uint8_t *__restrict__ w, float *__restrict__ outp,
                                                                 int64_t ld) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= static_cast<int64_t>(k.out) * k.neuron_len) return;
    const int row = static_cast<int>(i / k.neuron_len), col = static_cast<int>(i - static_cast<int64_t>(row) * k.neuron_len);
    const float s = f16_to_f32(reinterpret_cast<const uint16_t *>(w + k.scales_off)[static_cast<int64_t>(row) * k.ng + (col >> 5)]);
    const int c = reinterpret_cast<const int8_t *>(w + k.codes_off)[i];
    outp[row * ld + col] = __fmul_rn(s, static_cast<float>(c));
}

// Embedding rows: out[n, col] = fl(scale * code) of neuron ids[n], rounded once more to the output type; ids outside
// [0, out) give a row of zeros.
__global__ __launch_bounds__(256) void nint8z_embedding_kernel(N8zK k, const uint8_t *__restrict__ w,
                                                               const int64_t *__restrict__ ids, void *__restrict__ outp,
                                                               int out_dtype, int64_t ldo) {
    const int col = blockIdx.x * 256 + threadIdx.x;
    if (col >= k.neuron_len) return;
    const int n = blockIdx.y;
    const int64_t tok = ids[n];
    float v = 0.f;
    if (tok >= 0 && tok < k.out) {
        const float s = f16_to_f32(reinterpret_cast<const uint16_t *>(w + k.scales_off)[tok * k.ng + (col >> 5)]);
        const int c = reinterpret_cast<const int8_t *>(w + k.codes_off)[(tok * k.ng + (col >> 5)) * 32 + (col & 31)];
        v = __fmul_rn(s, static_cast<float>(c));
    }
    store_rounded(outp, static_cast<int64_t>(n) * ldo + col, v, out_dtype);
}

// fp16 rows for the dense GEMM: block = one row; values times 2^(12 - e), e = exponent of the row's largest
// |scale| * 127, so that they stay below 4096; rowscale[row] = 2^(e - 12); columns up to kpad are zero
__global__ __launch_bounds__(256) void nint8z_dequant_f16_kernel(N8zK k, const uint8_t *__restrict__ w, uint16_t *__restrict__ outp,
                                                                 int64_t ld, float *__restrict__ rowscale, int kpad) {
    __shared__ float smax[256];
    const int row = blockIdx.x, tid = threadIdx.x;
    const uint16_t *sc = reinterpret_cast<const uint16_t *>(w + k.scales_off) + static_cast<int64_t>(row) * k.ng;
    float m = 0.f;
    for (int g = tid; g < k.ng; g += 256) {
        const float s = fabsf(f16_to_f32(sc[g]));
        if (s == s && s <= 65504.f) m = fmaxf(m, s);  // a NaN or infinite scale does not set the range
    }
    smax[tid] = m;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if (tid < st) smax[tid] = fmaxf(smax[tid], smax[tid + st]);
        __syncthreads();
    }
    int e = 0;
    const float bound = smax[0] * 127.f;
    if (bound > 0.f) frexpf(bound, &e);
    const float inv = ldexpf(1.f, 12 - e);
    if (tid == 0) rowscale[row] = ldexpf(1.f, e - 12);
    const int8_t *q = reinterpret_cast<const int8_t *>(w + k.codes_off) + static_cast<int64_t>(row) * k.neuron_len;
    for (int col = tid; col < kpad; col += 256) {
        float v = 0.f;
        if (col < k.neuron_len) v = f16_to_f32(sc[col >> 5]) * static_cast<float>(q[col]) * inv;
        outp[row * ld + col] = f32_to_f16_rne(v);
    }
}

// ---- small batches -----------------------------------------------------------------------------------------------
// Block = 4 waves, RW rows per wave in turn; activation rows m0 .. m0 + MB - 1 of the pass.  LDS: fp16 x [MB][K], then
// float chunk sums [MB][K / 16].
template <int XF16, int MB>
__global__ __launch_bounds__(256) void nint8z_gemv_kernel(N8zK k, const uint8_t *__restrict__ w_in, const uint16_t *__restrict__ x_in,
                                                          int64_t ldx, int M_in, float *__restrict__ y_in, int64_t ldy, int rw,
                                                          PairSel sel) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint8_t *w = w_in;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = blockIdx.y * MB;
    if (sel.ids) {  // a pair of a MoE decode step: one row, the expert's own tensor
        const uint16_t *xr[1];
        float *yr[1];
        int local;
        if (!select_rows<1>(sel, w, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    const int K = k.neuron_len;
    uint16_t *xh = reinterpret_cast<uint16_t *>(lds);
    float *xsum = reinterpret_cast<float *>(lds + MB * K / 2);
    const bool vec = ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;  // 16-byte chunks (K is a multiple of 32)
    const int cpr = K / 8;
    // bf16 rows: each row times the power of two that brings its largest magnitude near 2^12 (rows of any magnitude stay
    // inside fp16's range); the sums are scaled back when they are stored
    __shared__ uint32_t rowmax[MB];
    float rs[MB], rinv[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) rs[m] = rinv[m] = 1.f;
    // one row of up to 8192 values in 16-byte chunks: the chunks stay in registers between the maximum and the conversion
    constexpr int HELD = 4;
    const bool held = MB == 1 && !XF16 && vec && cpr <= HELD * 256;
    u32x4_t keep[HELD];
    if (held) {
        if (tid == 0) rowmax[0] = 0u;
        __syncthreads();
        const uint16_t *xrow = x + static_cast<int64_t>(min(m0, M - 1)) * ldx;
        uint32_t mx = 0;
#pragma unroll
        for (int j = 0; j < HELD; ++j) {
            const int c = tid + 256 * j;
            keep[j] = c < cpr ? *reinterpret_cast<const u32x4_t *>(xrow + 8 * c) : u32x4_t{0u, 0u, 0u, 0u};
            mx = absmax_bf16(absmax_bf16(absmax_bf16(absmax_bf16(mx, keep[j].x), keep[j].y), keep[j].z), keep[j].w);
        }
        const uint32_t wm = wave_max_u32(mx);
        if (lane == 0) atomicMax(&rowmax[0], wm);
        __syncthreads();
        rs[0] = slice_scale(rowmax[0], rinv[0]);
#pragma unroll
        for (int j = 0; j < HELD; ++j) {
            const int c = tid + 256 * j;
            if (c < cpr)
                *reinterpret_cast<u32x4_t *>(xh + 8 * c) = u32x4_t{to_h2_scaled(keep[j].x, rs[0]), to_h2_scaled(keep[j].y, rs[0]),
                                                                   to_h2_scaled(keep[j].z, rs[0]), to_h2_scaled(keep[j].w, rs[0])};
        }
    } else if constexpr (!XF16) {
        if (tid < MB) rowmax[tid] = 0u;
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const uint16_t *xrow = x + static_cast<int64_t>(min(m0 + m, M - 1)) * ldx;
            uint32_t mx = 0;
            if (vec) {
                for (int c = tid; c < cpr; c += 256) {
                    const u32x4_t v = *reinterpret_cast<const u32x4_t *>(xrow + 8 * c);
                    mx = absmax_bf16(absmax_bf16(absmax_bf16(absmax_bf16(mx, v.x), v.y), v.z), v.w);
                }
            } else {
                for (int c = tid; c < K; c += 256) mx = absmax_bf16(mx, xrow[c]);
            }
            const uint32_t wm = wave_max_u32(mx);
            if (lane == 0) atomicMax(&rowmax[m], wm);
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MB; ++m) rs[m] = slice_scale(rowmax[m], rinv[m]);
    }
    if (held) {
        // staged above
    } else if (vec) {
        for (int i = tid; i < MB * cpr; i += 256) {
            const int m = i / cpr, c = i - m * cpr;
            const int row = min(m0 + m, M - 1);
            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(x + static_cast<int64_t>(row) * ldx + 8 * c);
            uint32_t h[4] = {v.x, v.y, v.z, v.w};
            if constexpr (!XF16) {
                float sc = rs[0];
#pragma unroll
                for (int mm = 1; mm < MB; ++mm)
                    if (m == mm) sc = rs[mm];
#pragma unroll
                for (int t = 0; t < 4; ++t) h[t] = to_h2_scaled(h[t], sc);
            }
            *reinterpret_cast<u32x4_t *>(xh + m * K + 8 * c) = u32x4_t{h[0], h[1], h[2], h[3]};
        }
    } else {
        for (int i = tid; i < MB * K; i += 256) {
            const int m = i / K, c = i - m * K;
            const int row = min(m0 + m, M - 1);
            const uint16_t v = x[static_cast<int64_t>(row) * ldx + c];
            float sc = rs[0];
#pragma unroll
            for (int mm = 1; mm < MB; ++mm)
                if (m == mm) sc = rs[mm];
            xh[i] = XF16 ? v : f32_to_f16_rne(bf16_to_f32(v) * sc);
        }
    }
    __syncthreads();
    for (int i = tid; i < MB * (K / 16); i += 256) {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(xh) + i * 8;
        float s = 0.f;
#pragma unroll
        for (int t = 0; t < 8; ++t) s = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, p[t]), half2_t{1, 1}, s, false);
        xsum[i] = s;
    }
    __syncthreads();
    const uint16_t *scales = reinterpret_cast<const uint16_t *>(w + k.scales_off);
    const uint8_t *codes = w + k.codes_off;
    const int row_first = (blockIdx.x * 4 + wave) * rw;
    for (int ri = 0; ri < rw; ++ri) {
        const int row = row_first + ri;  // wave-uniform
        if (row >= k.out) break;
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.f;
        for (int c0 = 0; c0 < K; c0 += 1024) {
            const int col = c0 + lane * 16;
            if (col < K) {
                const u32x4_t q = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(codes + static_cast<int64_t>(row) * K + col));
                const float s = f16_to_f32(scales[static_cast<int64_t>(row) * k.ng + (col >> 5)]);
                uint32_t pr[8];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint32_t u = q[t] ^ 0x80808080u;
                    pr[2 * t] = __builtin_amdgcn_perm(u, 0x64006400u, 0x03050104u);
                    pr[2 * t + 1] = __builtin_amdgcn_perm(u, 0x64006400u, 0x03070106u);
                }
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const u32x4_t xa = *reinterpret_cast<const u32x4_t *>(xh + m * K + col);
                    const u32x4_t xb = *reinterpret_cast<const u32x4_t *>(xh + m * K + col + 8);
                    // plain scalars: a bit cast of a vector element taken in place reads the vector's first element
                    const uint32_t xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
                    float r = 0.f;
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        r = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, pr[t]), __builtin_bit_cast(half2_t, xv[t]), r, false);
                    acc[m] = fmaf(s, fmaf(-1152.f, xsum[m * (K / 16) + (col >> 4)], r), acc[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float v = acc[m];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0 && m0 + m < M) y[static_cast<int64_t>(m0 + m) * ldy + row] = v * rinv[m];
        }
    }
}

// ---- 2 .. 32 rows on the matrix cores ------------------------------------------------------------------------------
// One MFMA (16 tokens x 16 neurons x 32 k) covers exactly one Q8_0 block of each of its 16 neurons: the codes enter as
// exact fp16 integers (byte -> mantissa of 1024, minus 1152), the product sum of the block comes out of an accumulator
// that starts at zero, and the block's scale multiplies it in fp32 -- the arithmetic of the reference's
// dequantize-then-multiply up to the order of the fp32 additions.  A block of the grid owns RPB row-blocks of 16 neurons
// and a 16-row tile of the activations; its waves split K in chunks of eight blocks (256 values): a wave requests the
// chunk's codes and scales of all its row-blocks, then the activation fragments (32 registers, shared by the
// row-blocks).  A code load takes 16 bytes per lane -- 64 contiguous bytes of a neuron, two blocks -- and one lane swap
// per register between the wave's halves sorts them into one block per fragment (an MFMA does not care which of its
// 32 k slots holds which k as long as both operands agree).  LDS: waves * RPB * 1 KB for the final sum over the waves.
template <int XF16, int RPB>
__global__ __launch_bounds__(1024) void nint8z_tile_kernel(N8zK k, const uint8_t *__restrict__ w, const uint16_t *__restrict__ x,
                                                           int64_t ldx, int M, float *__restrict__ y, int64_t ldy) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    float *red = reinterpret_cast<float *>(lds);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = blockDim.x >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const int K = k.neuron_len, nchunks = (k.ng + 7) / 8;
    const int rb0 = static_cast<int>(blockIdx.x) * RPB, m0 = static_cast<int>(blockIdx.y) * 16;
    const uint16_t *xrow = x + static_cast<int64_t>(min(m0 + n, M - 1)) * ldx;
    const uint16_t *scales = reinterpret_cast<const uint16_t *>(w + k.scales_off);
    const uint8_t *codes = w + k.codes_off;
    float4_t acc[RPB];
#pragma unroll
    for (int i = 0; i < RPB; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    // k position of the lane's eight values inside a block: the two lane halves trade code halves (below), which
    // leaves lanes kb = 0 .. 3 with bytes 0-7, 16-23, 8-15, 24-31 of the block
    const int koff = kb == 0 ? 0 : kb == 1 ? 16 : kb == 2 ? 8 : 24;
    for (int c = wave; c < nchunks; c += nwaves) {
        // requests: codes and scales (8 fp16 = 16 bytes) of every row-block, then the activations.  A code load is 16
        // bytes per lane, 64 contiguous bytes per neuron: lanes kb = 0, 1 take block 2 p of the chunk, kb = 2, 3 block
        // 2 p + 1.
        u32x4_t q[RPB][4];
        u32x4_t sc[RPB];
#pragma unroll
        for (int i = 0; i < RPB; ++i) {
            const int row = min((rb0 + i) * 16 + n, k.out - 1);
            const uint8_t *cp = codes + static_cast<int64_t>(row) * K + 256 * c + 16 * kb;
#pragma unroll
            for (int p = 0; p < 4; ++p)
                q[i][p] = 8 * c + 2 * p + (kb >> 1) < k.ng ? __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(cp + 64 * p))
                                                            : u32x4_t{0u, 0u, 0u, 0u};
            // a row's scales are 2 ng bytes apart: 16-byte aligned chunks when ng is a multiple of 8, else two-byte reads
            const uint16_t *sp = scales + static_cast<int64_t>(row) * k.ng + 8 * c;
            if ((k.ng & 7) == 0) {
                sc[i] = *reinterpret_cast<const u32x4_t *>(sp);
            } else {
                uint32_t h[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) h[j] = 8 * c + j < k.ng ? sp[j] : 0u;
                sc[i] = u32x4_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
            }
        }
        u32x4_t a[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = load_xfrag_raw<true>(xrow, 256 * c + 32 * j + koff, K);
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = xfrag_finish<XF16, true>(a[j], 256 * c + 32 * j + koff, K);
#pragma unroll
        for (int i = 0; i < RPB; ++i) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                // lanes 32-63 give their low halves (block 2 p + 1) for the high halves of lanes 0-31 (block 2 p): the
                // first pair of registers then holds block 2 p in all four lane groups, the second block 2 p + 1
                const auto s0 = __builtin_amdgcn_permlane32_swap(q[i][p].x, q[i][p].z, false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(q[i][p].y, q[i][p].w, false, false);
                const uint32_t cw[2][2] = {{s0[0], s1[0]}, {s0[1], s1[1]}};
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int j = 2 * p + h;
                    const uint32_t u0 = cw[h][0] ^ 0x80808080u, u1 = cw[h][1] ^ 0x80808080u;
                    const half2_t off = half2_t{static_cast<_Float16>(-1152.f), static_cast<_Float16>(-1152.f)};
                    u32x4_t b;
                    b[0] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(u0, 0x64006400u, 0x03050104u)) + off);
                    b[1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(u0, 0x64006400u, 0x03070106u)) + off);
                    b[2] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(u1, 0x64006400u, 0x03050104u)) + off);
                    b[3] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(u1, 0x64006400u, 0x03070106u)) + off);
                    const float4_t part = mfma16(a[j], b, float4_t{0.f, 0.f, 0.f, 0.f});
                    const uint32_t sw = p == 0 ? sc[i].x : p == 1 ? sc[i].y : p == 2 ? sc[i].z : sc[i].w;
                    const float s = f16_to_f32(static_cast<uint16_t>(h ? sw >> 16 : sw & 0xffffu));
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[i][v] = fmaf(s, part[v], acc[i][v]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RPB; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * RPB + i) * 4 + v) * 64 + lane] = acc[i][v];
    __syncthreads();
    for (int o = tid; o < RPB * 256; o += blockDim.x) {
        const int rr = o & 15, t = (o >> 4) & 15, nb = o >> 8;
        const int slot = (nb * 4 + (t & 3)) * 64 + rr + 16 * (t >> 2);
        float sum = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) sum += red[wv * RPB * 256 + slot];
        const int row = (rb0 + nb) * 16 + rr;
        if (m0 + t < M && row < k.out) y[static_cast<int64_t>(m0 + t) * ldy + row] = sum;
    }
}

int gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, const float *sa,
                const float *sb, float *y, int64_t ldy, hipStream_t st, float *part = nullptr);
float *dequant_gemm_part(float *wscale, int N, int K, int M);
int x_prep(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, hipStream_t st);
size_t dequant_gemm_workspace(int N, int K, int M);
void dequant_gemm_carve(void *ws, int N, int K, int M, uint16_t *&x16, float *&xscale, uint16_t *&w16, float *&wscale,
                        int &Kp);

// activation rows per pass: the most of 8, 4, 2, 1 whose fp16 rows and chunk sums fit 64 KB of LDS; 0 = none does
static int nint8z_rows_per_pass(int K, int M) {
    for (int mb = 8; mb >= 1; mb >>= 1)
        if (mb <= (M > 4 ? 8 : (M > 2 ? 4 : (M > 1 ? 2 : 1))) && static_cast<size_t>(mb) * K * 2 + static_cast<size_t>(mb) * (K / 16) * 4 <= 65536)
            return mb;
    return 0;
}

template <int XF16>
static int nint8z_gemv_launch(const N8zK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                              hipStream_t st) {
    const int mb = nint8z_rows_per_pass(k.neuron_len, M);
    MFQ_REQUIRE(mb > 0, MFQ_ERR_UNSUPPORTED, "nint8z_gemv: neuron_len %d does not fit the LDS", k.neuron_len);
    // rows per wave: as many as leave about four blocks per CU (one or two activation rows) or two (more: a block's
    // staged activations then serve twice the weight rows)
    int rw = k.out / (4 * (M <= 2 ? 1024 : 512));
    if (rw < 1) rw = 1;
    const dim3 grid(static_cast<unsigned>(ceil_div(k.out, 4 * rw)), static_cast<unsigned>(ceil_div(M, mb)));
    const size_t lds = static_cast<size_t>(mb) * k.neuron_len * 2 + static_cast<size_t>(mb) * (k.neuron_len / 16) * 4;
#define MFQ_N8Z(MB)                                                                                                  \
    if (mb == MB) hipLaunchKernelGGL((nint8z_gemv_kernel<XF16, MB>), grid, dim3(256), lds, st, k, w, x, ldx, M, y, ldy, rw, PairSel{});
    MFQ_N8Z(8) MFQ_N8Z(4) MFQ_N8Z(2) MFQ_N8Z(1)
#undef MFQ_N8Z
    return check_launch("nint8z_gemv");
}

// the same kernel, one row per block row, over the pairs of a MoE decode step (see PairSel)
template <int XF16>
static int nint8z_launch_pairs(const N8zK &k, const uint16_t *x, int64_t ldx, int n_pairs, float *y, int64_t ldy, const PairSel &sel,
                               hipStream_t st) {
    MFQ_REQUIRE(nint8z_rows_per_pass(k.neuron_len, 1) > 0, MFQ_ERR_UNSUPPORTED, "nint8z_gemv_pairs: neuron_len %d does not fit the LDS",
                k.neuron_len);
    int rw = k.out / 1024;  // about four blocks per compute unit and pair
    if (rw < 1) rw = 1;
    const dim3 grid(static_cast<unsigned>(ceil_div(k.out, 4 * rw)), static_cast<unsigned>(n_pairs));
    const size_t lds = static_cast<size_t>(k.neuron_len) * 2 + static_cast<size_t>(k.neuron_len / 16) * 4;
    hipLaunchKernelGGL((nint8z_gemv_kernel<XF16, 1>), grid, dim3(256), lds, st, k, static_cast<const uint8_t *>(nullptr), x, ldx, n_pairs,
                       y, ldy, rw, sel);
    return check_launch("nint8z_gemv_pairs");
}

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_nint8z_plan(int out, int neuron_len, mfq_nint8z_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nint8z_plan: null descriptor");
    MFQ_REQUIRE(out > 0, MFQ_ERR_INVALID, "nint8z_plan: empty tensor");
    MFQ_REQUIRE(neuron_len > 0 && neuron_len % 32 == 0, MFQ_ERR_INVALID, "NINT8-0 neuron_len must be a positive multiple of 32");
    d->out = out; d->neuron_len = neuron_len; d->ng = neuron_len / 32;
    d->scales_off = 0;
    const int64_t sb = static_cast<int64_t>(out) * d->ng * 2;
    d->codes_off = (sb + 255) / 256 * 256;
    d->total_bytes = d->codes_off + static_cast<int64_t>(out) * neuron_len;
    d->payload_bytes = static_cast<int64_t>(out) * d->ng * 34;
    return MFQ_OK;
}

extern "C" int mfq_hip_nint8z_repack(const mfq_nint8z_desc *d, const void *blocks, int64_t block_bytes, void *weight,
                                     mfq_stream_t stream) {
    MFQ_REQUIRE(d && blocks && weight, MFQ_ERR_INVALID, "nint8z_repack: null argument");
    MFQ_REQUIRE(block_bytes == d->payload_bytes, MFQ_ERR_INVALID, "invalid NINT8-0 block bytes: got %lld, expected %lld",
                static_cast<long long>(block_bytes), static_cast<long long>(d->payload_bytes));
    const N8zK k = to_k(d);
    const int64_t n = static_cast<int64_t>(k.out) * k.ng;
    hipLaunchKernelGGL(nint8z_repack_kernel, dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(blocks), static_cast<uint8_t *>(weight));
    return check_launch("nint8z_repack");
}

extern "C" int mfq_hip_nint8z_gemv_pairs(const mfq_nint8z_desc *d, const void *const *expert_weights, const int32_t *expert_slot,
                                         int E, const void *x, int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T,
                                         int R, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && expert_weights && expert_slot && x && ids && y, MFQ_ERR_INVALID, "nint8z_gemv_pairs: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint8z_gemv_pairs: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(T >= 0 && R >= 1 && E >= 1, MFQ_ERR_INVALID, "nint8z_gemv_pairs: T=%d R=%d E=%d", T, R, E);
    MFQ_REQUIRE(static_cast<int64_t>(T) * R <= 65535, MFQ_ERR_UNSUPPORTED, "nint8z_gemv_pairs: %lld pairs (at most 65535 per launch)",
                static_cast<long long>(T) * R);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nint8z_gemv_pairs: ldx/ldy smaller than the tensor");
    if (T == 0) return MFQ_OK;
    const PairSel sel{ids, expert_slot, reinterpret_cast<const uint8_t *const *>(expert_weights), E, R, routed_input ? 1 : 0};
    const N8zK k = to_k(d);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    return x_dtype == MFQ_X_F16 ? nint8z_launch_pairs<1>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream))
                                : nint8z_launch_pairs<0>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream));
}

extern "C" int mfq_hip_nint8z_embedding(const mfq_nint8z_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                                        int out_dtype, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight, MFQ_ERR_INVALID, "nint8z_embedding: null argument");
    MFQ_REQUIRE(n_ids >= 0, MFQ_ERR_INVALID, "nint8z_embedding: n_ids=%d", n_ids);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16 || out_dtype == MFQ_X_F32, MFQ_ERR_INVALID,
                "nint8z_embedding: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(ldo >= d->neuron_len, MFQ_ERR_INVALID, "nint8z_embedding: ldo %lld < neuron_len %d", static_cast<long long>(ldo),
                d->neuron_len);
    if (n_ids == 0) return MFQ_OK;
    MFQ_REQUIRE(ids && out, MFQ_ERR_INVALID, "nint8z_embedding: null ids or output");
    const N8zK k = to_k(d);
    const size_t esize = out_dtype == MFQ_X_F32 ? 4 : 2;
    for (int n0 = 0; n0 < n_ids; n0 += 65535) {  // the grid's second dimension holds 65535 rows
        const int rows = n_ids - n0 < 65535 ? n_ids - n0 : 65535;
        hipLaunchKernelGGL(nint8z_embedding_kernel, dim3(static_cast<unsigned>(ceil_div(k.neuron_len, 256)), static_cast<unsigned>(rows)),
                           dim3(256), 0, as_stream(stream), k, static_cast<const uint8_t *>(weight), ids + n0,
                           static_cast<void *>(static_cast<uint8_t *>(out) + static_cast<size_t>(n0) * ldo * esize), out_dtype, ldo);
    }
    return check_launch("nint8z_embedding");
}

extern "C" int mfq_hip_nint8z_dequant_f32(const mfq_nint8z_desc *d, const void *weight, float *w_out, int64_t ld,
                                          mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && w_out, MFQ_ERR_INVALID, "nint8z_dequant_f32: null argument");
    MFQ_REQUIRE(ld >= d->neuron_len, MFQ_ERR_INVALID, "nint8z_dequant_f32: ld smaller than neuron_len");
    const N8zK k = to_k(d);
    const int64_t n = static_cast<int64_t>(k.out) * k.neuron_len;
    hipLaunchKernelGGL(nint8z_dequant_f32_kernel, dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0, as_stream(stream),
                       k, static_cast<const uint8_t *>(weight), w_out, ld);
    return check_launch("nint8z_dequant_f32");
}

template <int XF16>
static int nint8z_tile_launch(const N8zK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                              hipStream_t st) {
    // row-blocks per block: one block per compute unit where that takes at most four; up to 16 waves over the chunks of K
    const int nrb = static_cast<int>(ceil_div(k.out, 16)), nchunks = (k.ng + 7) / 8;
    int rpb = static_cast<int>(ceil_div(nrb, gemv_cu_count()));
    rpb = rpb > 4 ? 4 : rpb;
    const int nwaves = nchunks < 16 ? nchunks : 16;
    const dim3 grid(static_cast<unsigned>(ceil_div(nrb, rpb)), static_cast<unsigned>(ceil_div(M, 16))), block(64 * nwaves);
    const size_t lds = static_cast<size_t>(nwaves) * rpb * 1024;
#define MFQ_N8Z_TILE(R) \
    if (rpb == R) hipLaunchKernelGGL((nint8z_tile_kernel<XF16, R>), grid, block, lds, st, k, w, x, ldx, M, y, ldy);
    MFQ_N8Z_TILE(1) MFQ_N8Z_TILE(2) MFQ_N8Z_TILE(3) MFQ_N8Z_TILE(4)
#undef MFQ_N8Z_TILE
    return check_launch("nint8z_tile");
}

static int nint8z_gemv_any(const mfq_nint8z_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                           float *y, int64_t ldy, hipStream_t st) {
    const N8zK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    // from two rows on: the matrix cores, where the activation rows allow 16-byte reads.  Two rows on the vector ALUs
    // take 8.8 / 16.7 / 29.6 us on 4096 x 4096 / 12288 x 4096 / 4096 x 12288 against 7.6 / 17.7 / 17.8 us here
    // (MFQ_N8Z_TILE_MIN_M for tuning)
    static const int tile_min = tune_env("MFQ_N8Z_TILE_MIN_M", 2);
    if (M >= tile_min && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && k.neuron_len % 8 == 0)
        return x_dtype == MFQ_X_F16 ? nint8z_tile_launch<1>(k, w, xp, ldx, M, y, ldy, st)
                                    : nint8z_tile_launch<0>(k, w, xp, ldx, M, y, ldy, st);
    return x_dtype == MFQ_X_F16 ? nint8z_gemv_launch<1>(k, w, xp, ldx, M, y, ldy, st)
                                : nint8z_gemv_launch<0>(k, w, xp, ldx, M, y, ldy, st);
}

extern "C" int mfq_hip_nint8z_gemv(const mfq_nint8z_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                   int M, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nint8z_gemv: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nint8z_gemv: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint8z_gemv: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nint8z_gemv: ldx/ldy smaller than the tensor");
    return nint8z_gemv_any(d, weight, x, x_dtype, ldx, M, y, ldy, as_stream(stream));
}

// rows up to which the weights are re-streamed (8 rows per pass) rather than dequantized for the dense GEMM
static constexpr int kN8zStreamMaxM = 32;
static bool nint8z_streams(const mfq_nint8z_desc *d, int M) {
    return M <= kN8zStreamMaxM && nint8z_rows_per_pass(d->neuron_len, M) > 0;
}

extern "C" size_t mfq_hip_nint8z_gemm_workspace_bytes(const mfq_nint8z_desc *d, int M) {
    if (!d || M < 1 || nint8z_streams(d, M)) return 0;
    return dequant_gemm_workspace(d->out, d->neuron_len, M);
}

extern "C" int mfq_hip_nint8z_gemm(const mfq_nint8z_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                   int M, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                                   mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nint8z_gemm: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nint8z_gemm: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint8z_gemm: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nint8z_gemm: ldx/ldy smaller than the tensor");
    hipStream_t st = as_stream(stream);
    if (nint8z_streams(d, M)) return nint8z_gemv_any(d, weight, x, x_dtype, ldx, M, y, ldy, st);
    const size_t need = dequant_gemm_workspace(d->out, d->neuron_len, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nint8z_gemm: workspace %zu < %zu bytes",
                workspace_bytes, need);
    uint16_t *x16, *w16;
    float *xscale, *wscale;
    int Kp;
    dequant_gemm_carve(workspace, d->out, d->neuron_len, M, x16, xscale, w16, wscale, Kp);
    int rc = x_prep(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, st);
    if (rc) return rc;
    const N8zK k = to_k(d);
    hipLaunchKernelGGL(nint8z_dequant_f16_kernel, dim3(static_cast<unsigned>(k.out)), dim3(256), 0, st, k,
                       static_cast<const uint8_t *>(weight), w16, static_cast<int64_t>(Kp), wscale, Kp);
    rc = check_launch("nint8z_dequant_f16");
    if (rc) return rc;
    return gemm_f16_nt(x16, Kp, w16, Kp, M, d->out, Kp, xscale, wscale, y, ldy, st, dequant_gemm_part(wscale, d->out, d->neuron_len, M));
}
