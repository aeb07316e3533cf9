// NVQ-JSC, D4 family (4-dim magnitude vectors, 8/9-bit indices, 7-bit parity sign masks per
// 8 weights, 4-bit joint scale/codebook state per 24 weights).
//
// Device layout: same row-block / step / lane interleave as NINT.  One (neuron, group) unit is three
// dwords made of six 16-bit fields F(t) = idx_t << 7 | nib_t << 3, one per 4-dim vector: nib_t is the vector's four
// sign bits (the parity bit of the 7-bit mask is worked out at load time), so F(t) & 0xfff8 is the byte offset of
// the vector in a table of (entry, sign nibble) -> four signed fp16 values:
//   a = F(0) | F(1) << 16
//   b = F(2) | F(3) << 16
//   c = F(4) | state >> 3 | (F(5) >> 3) << 16 | (state & 7) << 29      (rotl(c, 6) & 0x78 = 8 * state)
// Step = Q [j][lane][a, b] then C [lane][c of j = 0..3].  The tensor tail holds
//   float lut[16]; uint32 bank_for_state[16]; int8 codebooks[banks][entries][4]; float anchor[].
// In the GEMV the codebook banks (as ready-made activation-typed pairs), a 128-entry table that
// expands a sign mask (with its parity bit) into XOR masks, and the scale LUT all stay in LDS; the small-batch
// matrix-core kernel keeps the signed table (banks * entries * 16 vectors of 8 bytes) in LDS instead.
#include <type_traits>

#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_prefill.hpp"

namespace mfq {

struct NvqK {
    int ib, entries, banks, out, neuron_len, ng, nvec, nsign, nsteps, n_rowblocks;
    int64_t step_bytes, rowblock_bytes, tables_off, anchors_off;
};

static NvqK to_k(const mfq_nvq_desc *d) {
    NvqK k;
    k.ib = d->index_bits; k.entries = d->entries; k.banks = d->banks; k.out = d->out; k.neuron_len = d->neuron_len;
    k.ng = d->ng; k.nvec = d->nvec; k.nsign = d->nsign; k.nsteps = d->nsteps; k.n_rowblocks = d->n_rowblocks;
    k.step_bytes = d->step_bytes; k.rowblock_bytes = d->rowblock_bytes; k.tables_off = d->tables_off;
    k.anchors_off = d->anchors_off;
    return k;
}

__device__ __forceinline__ uint32_t parity8(uint32_t m7) { return m7 | ((__popc(m7) & 1u) << 7); }

// ---- repack ----------------------------------------------------------------------------
// `body` points at the anchors; `lut_src` is the fp16 LUT of the JSC header or null (plain NVQ:
// lut[s] = s); `bank_src` the 16 state->bank bytes or null (all zero); `cb_src` the int8 banks.
__global__ void nvq_repack_kernel(NvqK k, const uint8_t *__restrict__ body, int64_t body_bytes,
                                  const uint16_t *__restrict__ lut_src, const uint8_t *__restrict__ bank_src,
                                  const int8_t *__restrict__ cb_src, uint8_t *__restrict__ dst) {
    const int lane = threadIdx.x;
    const int rb = blockIdx.x, s = blockIdx.y;
    const int r = lane & 15, kb = lane >> 4;
    const int row = rb * 16 + r;
    const int64_t out = k.out;
    const int64_t st_bytes = (out * k.ng * 4 + 7) / 8, ix_bytes = (out * k.nvec * k.ib + 7) / 8,
                  sg_bytes = (out * k.nsign * 7 + 7) / 8;
    const uint8_t *st_s = body + 2 * out;
    const uint8_t *ix_s = st_s + st_bytes;
    const uint8_t *sg_s = ix_s + ix_bytes;
    uint8_t *sp = dst + rb * k.rowblock_bytes + s * k.step_bytes;
    uint32_t *qreg = reinterpret_cast<uint32_t *>(sp);
    uint32_t *creg = reinterpret_cast<uint32_t *>(sp + 2048);
    for (int j = 0; j < 4; ++j) {
        const int g = 16 * s + 4 * j + kb;
        uint32_t d0 = 0, d1 = 0, h = 0;
        if (row < k.out && g < k.ng) {
            uint32_t idx[6], m[3];
            for (int t = 0; t < 6; ++t) {
                const int v = 6 * g + t;
                idx[t] = v < k.nvec ? read_bits(ix_s, static_cast<int64_t>(row) * k.nvec + v, k.ib, ix_bytes) : 0u;
            }
            for (int t = 0; t < 3; ++t) {
                const int u = 3 * g + t;
                m[t] = u < k.nsign ? read_bits(sg_s, static_cast<int64_t>(row) * k.nsign + u, 7, sg_bytes) : 0u;
            }
            const uint32_t state = read_bits(st_s, static_cast<int64_t>(row) * k.ng + g, 4, st_bytes);
            uint32_t f[6];
            for (int t = 0; t < 3; ++t) {
                const uint32_t m8 = parity8(m[t]);
                f[2 * t] = (idx[2 * t] << 7) | ((m8 & 15u) << 3);
                f[2 * t + 1] = (idx[2 * t + 1] << 7) | ((m8 >> 4) << 3);
            }
            d0 = f[0] | (f[1] << 16);
            d1 = f[2] | (f[3] << 16);
            h = f[4] | (state >> 3) | ((f[5] >> 3) << 16) | ((state & 7u) << 29);
        }
        qreg[(j * 64 + lane) * 2] = d0;
        qreg[(j * 64 + lane) * 2 + 1] = d1;
        creg[lane * 4 + j] = h;
    }
    if (s == 0 && kb == 0) {
        float *anchors = reinterpret_cast<float *>(dst + k.anchors_off);
        anchors[row] = row < k.out ? f16_to_f32(reinterpret_cast<const uint16_t *>(body)[row]) : 0.f;
    }
    if (rb == 0 && s == 0) {
        float *lut = reinterpret_cast<float *>(dst + k.tables_off);
        uint32_t *bfs = reinterpret_cast<uint32_t *>(lut + 16);
        int8_t *cb = reinterpret_cast<int8_t *>(bfs + 16);
        if (lane < 16) {
            lut[lane] = lut_src ? f16_to_f32(lut_src[lane]) : static_cast<float>(lane);
            bfs[lane] = bank_src ? bank_src[lane] : 0u;
        }
        const int n = k.banks * k.entries * 4;
        for (int i = lane; i < n; i += 64) cb[i] = cb_src[i];
    }
}

struct NvqUnit {
    uint32_t idx[6], mask[3], state;
};
__device__ __forceinline__ NvqUnit nvq_decode(uint32_t a, uint32_t b, uint32_t c) {
    NvqUnit u;
    const uint32_t f[6] = {a & 0xffffu, a >> 16, b & 0xffffu, b >> 16, c & 0xffffu, (c >> 13) & 0xfff8u};
#pragma unroll
    for (int t = 0; t < 6; ++t) u.idx[t] = f[t] >> 7;
#pragma unroll
    for (int m = 0; m < 3; ++m) u.mask[m] = (((f[2 * m] >> 3) & 15u) | (((f[2 * m + 1] >> 3) & 15u) << 4)) & 127u;
    u.state = (__builtin_rotateleft32(c, 6) >> 3) & 15u;
    return u;
}

// ---- dequant: f32(mag * sign) * fl(anchor * lut[state]) ------------------------------------
template <typename OutT>
__global__ void nvq_dequant_kernel(NvqK k, const uint8_t *__restrict__ w, OutT *__restrict__ outp, int64_t ld,
                                   float *__restrict__ rowscale, int kpad) {
    const int lane = threadIdx.x;
    const int rb = blockIdx.x, s = blockIdx.y;
    const int r = lane & 15, kb = lane >> 4;
    const int row = rb * 16 + r;
    if (row >= k.out) return;
    const uint8_t *sp = w + rb * k.rowblock_bytes + s * k.step_bytes;
    const uint32_t *qreg = reinterpret_cast<const uint32_t *>(sp);
    const uint32_t *creg = reinterpret_cast<const uint32_t *>(sp + 2048);
    const float *lut = reinterpret_cast<const float *>(w + k.tables_off);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cb = reinterpret_cast<const int8_t *>(bfs + 16);
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[row];
    float inv = 1.f;
    if constexpr (sizeof(OutT) == 2) {
        float lmax = 0.f;
        for (int i = 0; i < 16; ++i) lmax = fmaxf(lmax, lut[i]);
        const float bound = anchor * lmax * 127.f;
        int e = 0;
        if (bound > 0.f) frexpf(bound, &e);
        inv = ldexpf(1.f, 12 - e);
        if (s == 0 && kb == 0) {
            rowscale[row] = ldexpf(1.f, e - 12);
            for (int col = k.neuron_len; col < kpad; ++col) outp[row * ld + col] = 0;
        }
    }
    for (int j = 0; j < 4; ++j) {
        const int g = 16 * s + 4 * j + kb;
        if (g >= k.ng) continue;
        const NvqUnit u = nvq_decode(qreg[(j * 64 + lane) * 2], qreg[(j * 64 + lane) * 2 + 1], creg[lane * 4 + j]);
        const float scale = __fmul_rn(anchor, lut[u.state]);
        const int8_t *bank = cb + static_cast<int64_t>(bfs[u.state]) * k.entries * 4;
        for (int i = 0; i < 24; ++i) {
            const int col = g * 24 + i;
            if (col >= k.neuron_len) break;
            const int mag = bank[u.idx[i >> 2] * 4 + (i & 3)];
            const uint32_t m8 = parity8(u.mask[i >> 3]);
            const float sv = ((m8 >> (i & 7)) & 1u) ? -static_cast<float>(mag) : static_cast<float>(mag);
            const float v = __fmul_rn(sv, scale);
            if constexpr (sizeof(OutT) == 2) outp[row * ld + col] = f32_to_f16_rne(v * inv);
            else outp[row * ld + col] = v;
        }
    }
}

// ---- embedding rows: row ids[n] of the dequantized table, rounded once more to the output type -------------
// One thread per group of 24 weights: a wave takes four steps of the neuron (16 groups each).  Group g of neuron
// `tok` lives in row-block tok / 16, step g / 16, unit slot (g % 16) / 4 of lane (tok % 16) + 16 * (g % 4).  ids outside
// [0, out) give a row of zeros.
__global__ __launch_bounds__(64) void nvq_embedding_kernel(NvqK k, const uint8_t *__restrict__ w,
                                                           const int64_t *__restrict__ ids, void *__restrict__ outp,
                                                           int out_dtype, int64_t ldo) {
    const int s = blockIdx.x * 4 + (threadIdx.x >> 4), slot = threadIdx.x & 15;
    const int j = slot >> 2, kb = slot & 3;
    const int g = 16 * s + 4 * j + kb;
    if (s >= k.nsteps || g >= k.ng) return;
    const int n = blockIdx.y;
    const int64_t tok = ids[n];
    const int64_t at = static_cast<int64_t>(n) * ldo + g * 24;
    const int ncol = min(24, k.neuron_len - g * 24);
    if (tok < 0 || tok >= k.out) {
        for (int i = 0; i < ncol; ++i) store_rounded(outp, at + i, 0.f, out_dtype);
        return;
    }
    const int rb = static_cast<int>(tok >> 4), lane = static_cast<int>(tok & 15) + 16 * kb;
    const uint8_t *sp = w + rb * k.rowblock_bytes + s * k.step_bytes;
    const uint32_t *qreg = reinterpret_cast<const uint32_t *>(sp);
    const uint32_t *creg = reinterpret_cast<const uint32_t *>(sp + 2048);
    const float *lut = reinterpret_cast<const float *>(w + k.tables_off);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cb = reinterpret_cast<const int8_t *>(bfs + 16);
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[tok];
    const NvqUnit u = nvq_decode(qreg[(j * 64 + lane) * 2], qreg[(j * 64 + lane) * 2 + 1], creg[lane * 4 + j]);
    const float scale = __fmul_rn(anchor, lut[u.state]);
    const int8_t *bank = cb + static_cast<int64_t>(bfs[u.state]) * k.entries * 4;
    for (int i = 0; i < ncol; ++i) {
        const int mag = bank[u.idx[i >> 2] * 4 + (i & 3)];
        const uint32_t m8 = parity8(u.mask[i >> 3]);
        const float sv = ((m8 >> (i & 7)) & 1u) ? -static_cast<float>(mag) : static_cast<float>(mag);
        store_rounded(outp, at + i, __fmul_rn(sv, scale), out_dtype);
    }
}

// ---- GEMV ------------------------------------------------------------------------------
// LDS map (dwords): [codebook pairs: banks*entries*2][sign xor table: 128*4][lut: 16][bank: 16][x staging ...]
template <int XF16, int MB>
__global__ __launch_bounds__(1024) void nvq_gemv_kernel(NvqK k, const uint8_t *__restrict__ w_in,
                                                        const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                        float *__restrict__ y, int64_t ldy, int spw, PairSel sel) {
    extern __shared__ uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int rb = blockIdx.x;
    const uint16_t *xr[MB];
    float *yr[MB];
    const uint8_t *w = w_in;
    int local;
    if (!select_rows<MB>(sel, w, local, x, ldx, y, ldy, M, xr, yr)) return;
    const int ncb = k.banks * k.entries;
    uint32_t *cbp = lds;                 // 2 dwords per entry: (m0, m1), (m2, m3) as fp16 pairs
    uint32_t *sgx = cbp + 2 * ncb;       // 4 dwords per 7-bit mask
    float *lutf = reinterpret_cast<float *>(sgx + 512);
    uint32_t *bankoff = reinterpret_cast<uint32_t *>(lutf + 16);
    uint32_t *xbase = bankoff + 16;
    {
        const float *lut = reinterpret_cast<const float *>(w + k.tables_off);
        const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
        const uint32_t *cb = bfs + 16;  // 4 int8 magnitudes per entry
        for (int i = tid; i < ncb; i += blockDim.x) {
            const uint32_t e = cb[i];
            uint32_t h[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float f = static_cast<float>((e >> (8 * t)) & 0xffu);
                h[t] = f32_to_f16_rne(f);
            }
            cbp[2 * i] = h[0] | (h[1] << 16);
            cbp[2 * i + 1] = h[2] | (h[3] << 16);
        }
        for (int i = tid; i < 128; i += blockDim.x) {
            const uint32_t m8 = parity8(i);
#pragma unroll
            for (int p = 0; p < 4; ++p)
                sgx[4 * i + p] = (((m8 >> (2 * p)) & 1u) << 15) | (((m8 >> (2 * p + 1)) & 1u) << 31);
        }
        if (tid < 16) {
            lutf[tid] = lut[tid];
            bankoff[tid] = bfs[tid] * k.entries * 2;
        }
    }
    const int s0 = wave * spw;
    const int s1 = min(k.nsteps, s0 + spw);
    const int ngl = spw * 16, npairs = ngl * 12;
    uint32_t *xs = xbase + wave * (MB * (npairs + 2 * ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    float *red = reinterpret_cast<float *>(xbase + nwaves * (MB * (npairs + 2 * ngl)));
    const uint8_t *base = w + static_cast<int64_t>(rb) * k.rowblock_bytes;
    struct Step {
        u32x2_t q[4];
        u32x4_t cc;
    };
    auto load_step = [&](int s, Step &st) {
        const uint8_t *sp = base + s * k.step_bytes;
#pragma unroll
        for (int j = 0; j < 4; ++j) st.q[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t *>(sp) + j * 64 + lane);
        st.cc = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(sp + 2048) + lane);
    };
    Step cur, nxt;
    XRegs<MB> xg;
    stage_x_issue<MB>(xr, k.neuron_len, s0 * 16 * 24, npairs, lane, xg);
    if (s0 < s1) load_step(s0, cur);
    float xinv[MB];  // bf16 rows are staged times a per-wave power of two; the sums are scaled back below
    stage_x<XF16, MB, PlainBias, true>(xr, k.neuron_len, s0 * 16 * 24, npairs, 24, ngl, xs, xsum, lane, xg, xinv);
    __syncthreads();  // the LDS tables were filled by the whole block

    const int r = lane & 15, kb = lane >> 4;
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.f;
    for (int s = s0; s < s1; ++s) {
        if (s + 1 < s1) load_step(s + 1, nxt);
        const u32x2_t *q = cur.q;
        const u32x4_t cc = cur.cc;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int lg = (s - s0) * 16 + 4 * j + kb;
            const NvqUnit un = nvq_decode(q[j].x, q[j].y, cc[j]);
            const uint32_t state = un.state;
            const uint32_t *bank = cbp + bankoff[state];
            const float sc = lutf[state];
            const uint32_t(&mk)[3] = un.mask;
            const uint32_t(&ix)[6] = un.idx;
            float raw[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) raw[m] = 0.f;
#pragma unroll
            for (int v = 0; v < 3; ++v) {
                const u32x4_t sx = *reinterpret_cast<const u32x4_t *>(sgx + 4 * mk[v]);
                const u32x2_t c0 = *reinterpret_cast<const u32x2_t *>(bank + 2 * ix[2 * v]);
                const u32x2_t c1 = *reinterpret_cast<const u32x2_t *>(bank + 2 * ix[2 * v + 1]);
                const uint32_t w0 = c0.x ^ sx.x, w1 = c0.y ^ sx.y, w2 = c1.x ^ sx.z, w3 = c1.y ^ sx.w;
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const uint32_t *xp = xs + m * npairs + lg * 12 + 4 * v;
                    raw[m] = dot2h(w0, xp[0], raw[m]);
                    raw[m] = dot2h(w1, xp[1], raw[m]);
                    raw[m] = dot2h(w2, xp[2], raw[m]);
                    raw[m] = dot2h(w3, xp[3], raw[m]);
                }
            }
#pragma unroll
            for (int m = 0; m < MB; ++m) acc[m] = fmaf(sc, raw[m], acc[m]);
        }
        if (s + 1 < s1) cur = nxt;
    }
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[rb * 16 + r];
    float v[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) v[m] = anchor * acc[m] * xinv[m];
    finish_rows<MB>(v, red, wave, nwaves, lane, rb, 0, k.out, yr);
}

// ---- matrix-core path: up to 16 activation rows per streamed pass ----------------------------------
// Same scheme as the NINT kernel (nint_mfma.hpp): lane (r, kb) holds the unit of group 4j + kb of neuron r,
// fragment m of a unit is its weights 8m .. 8m+7 = two codebook vectors and one sign mask.  The magnitudes
// come from LDS as fp16 pairs, get their sign bits XOR-ed in and are multiplied by the group's scale-LUT
// entry in fp16 (one rounding of mag * lut, relative error below 2^-12); the neuron anchor is applied to
// the fp32 accumulator.  Codes of padding groups are zero (not zero weights), so the activation fragments
// read as zero at and beyond K.
// LDS map (dwords): [codebook pairs: banks*entries*2][sign xor table: 512][lut pairs: 16][bank offset: 16][red]
// PAIRS: the launch runs over the pairs of a MoE decode step (see PairSel); the tile's one bf16 row is scaled per wave
// by the power of two that brings its K-slice near 2^12 (rows of any magnitude), as in the one-row kernels.
template <int XF16, int NB, bool PAIRS = false>
__global__ __launch_bounds__(512) void nvq_mfma_kernel(NvqK k, const uint8_t *__restrict__ w_in,
                                                       const uint16_t *__restrict__ x_in, int64_t ldx, int M_in,
                                                       float *__restrict__ y_in, int64_t ldy, int spw, PairSel sel) {
    extern __shared__ uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint8_t *w = w_in;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = blockIdx.y * 16;
    if constexpr (PAIRS) {  // a tile of one row, the expert's own tensor
        const uint16_t *xr[1];
        float *yr[1];
        int local;
        if (!select_rows<1>(sel, w, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    const int ncb = k.banks * k.entries;
    uint32_t *cbp = lds;
    uint32_t *sgx = cbp + 2 * ncb;
    uint32_t *luth = sgx + 512;
    uint32_t *bankoff = luth + 16;
    float *red = reinterpret_cast<float *>(bankoff + 16);
    {
        const float *lut = reinterpret_cast<const float *>(w + k.tables_off);
        const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
        const uint32_t *cb = bfs + 16;  // 4 int8 magnitudes per entry
        for (int i = tid; i < ncb; i += blockDim.x) {
            const uint32_t e = cb[i];
            uint32_t h[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) h[t] = f32_to_f16_rne(static_cast<float>((e >> (8 * t)) & 0xffu));
            cbp[2 * i] = h[0] | (h[1] << 16);
            cbp[2 * i + 1] = h[2] | (h[3] << 16);
        }
        for (int i = tid; i < 128; i += blockDim.x) {
            const uint32_t m8 = parity8(i);
#pragma unroll
            for (int p = 0; p < 4; ++p)
                sgx[4 * i + p] = (((m8 >> (2 * p)) & 1u) << 15) | (((m8 >> (2 * p + 1)) & 1u) << 31);
        }
        if (tid < 16) {
            const uint32_t h = f32_to_f16_rne(lut[tid]);  // the LUT is fp16 in the payload: exact
            luth[tid] = h | (h << 16);
            bankoff[tid] = bfs[tid] * k.entries * 2;
        }
    }
    const int rb0 = blockIdx.x * NB;
    const int tok = min(m0 + (lane & 15), M - 1);
    const uint16_t *xrow = x + static_cast<int64_t>(tok) * ldx;
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;
    const int nrb = min(NB, k.n_rowblocks - rb0);
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    float anchor[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
        anchor[i] = reinterpret_cast<const float *>(w + k.anchors_off)[min(rb0 + i, k.n_rowblocks - 1) * 16 + r];
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb0) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);
    float4_t acc[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    float xscale = 1.f, xinv = 1.f;
    if constexpr (PAIRS && !XF16) {  // largest magnitude of the wave's K-slice of the row (K is a multiple of 8)
        uint32_t mx = 0;
        const int k0 = s0 * 16 * 24, k1 = min(k.neuron_len, (s0 + max(n, 0)) * 16 * 24);
        for (int c = k0 + 8 * lane; c < k1; c += 512) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(x + c);
            mx = absmax_bf16(absmax_bf16(absmax_bf16(absmax_bf16(mx, v.x), v.y), v.z), v.w);
        }
        xscale = slice_scale(wave_max_u32(mx), xinv);
    }
    __syncthreads();  // tables

    if constexpr (NB <= 2) {
        // Software pipeline as in nint_mfma_body: a row-block's four unit buffers are refilled unit by unit for the next
        // step, and the activation fragments run two units ahead and are requested before that refill.
        u32x2_t q[NB][4];
        u32x4_t hh[NB], hhn[NB];
        auto unit_off = [&](int i, int s, int j) -> uint32_t {
            return i < nrb && s < n ? i * rbb + s * sb + (j * 64 + lane) * 8 : kNoStep;
        };
        auto hload = [&](int s, u32x4_t (&h)[NB]) {
#pragma unroll
            for (int i = 0; i < NB; ++i)
                h[i] = __builtin_amdgcn_raw_buffer_load_b128(win, i < nrb && s < n ? i * rbb + s * sb + 2048 + lane * 16 : kNoStep, 0, 2);
        };
        auto xfrags = [&](int it, u32x4_t (&dst)[3]) {
            const int kpos = (s0 + (it >> 2)) * 16 * 24 + kb * 24 + 4 * (it & 3) * 24;
#pragma unroll
            for (int m = 0; m < 3; ++m) dst[m] = load_xfrag_raw<true>(xrow, kpos + 8 * m, k.neuron_len);
        };
        hload(0, hh);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i) q[i][j] = __builtin_amdgcn_raw_buffer_load_b64(win, unit_off(i, 0, j), 0, 2);
        u32x4_t a1[3], a2[3];
        xfrags(0, a1);
        xfrags(1, a2);
        for (int s = 0; s < n; ++s) {
            hload(s + 1, hhn);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x4_t a[3];
#pragma unroll
                for (int m = 0; m < 3; ++m) {
                    if constexpr (PAIRS)
                        a[m] = xfrag_finish_scaled<XF16, true>(a1[m], (s0 + s) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len, xscale);
                    else
                        a[m] = xfrag_finish<XF16, true>(a1[m], (s0 + s) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len);
                    a1[m] = a2[m];
                }
                xfrags(4 * s + j + 2, a2);
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const NvqUnit un = nvq_decode(q[i][j].x, q[i][j].y, hh[i][j]);
                    q[i][j] = __builtin_amdgcn_raw_buffer_load_b64(win, unit_off(i, s + 1, j), 0, 2);
                    const uint32_t state = un.state;
                    const uint32_t *bank = cbp + bankoff[state];
                    const half2_t sc = __builtin_bit_cast(half2_t, luth[state]);
                    const uint32_t(&mk)[3] = un.mask;
                    const uint32_t(&ix)[6] = un.idx;
#pragma unroll
                    for (int m = 0; m < 3; ++m) {
                        const u32x4_t sx = *reinterpret_cast<const u32x4_t *>(sgx + 4 * mk[m]);
                        const u32x2_t c0 = *reinterpret_cast<const u32x2_t *>(bank + 2 * ix[2 * m]);
                        const u32x2_t c1 = *reinterpret_cast<const u32x2_t *>(bank + 2 * ix[2 * m + 1]);
                        const uint32_t wv[4] = {c0.x ^ sx.x, c0.y ^ sx.y, c1.x ^ sx.z, c1.y ^ sx.w};
                        u32x4_t b;
#pragma unroll
                        for (int t = 0; t < 4; ++t) b[t] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, wv[t]) * sc);
                        acc[i] = mfma16(a[m], b, acc[i]);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < NB; ++i) hh[i] = hhn[i];
        }
    } else {  // four row-blocks per wave: the plain loop is faster (measured on 17408x5120)
        for (int s = 0; s < n; ++s) {
            u32x2_t q[NB][4];
            u32x4_t hh[NB];
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const uint32_t off = i < nrb ? i * rbb + s * sb : kNoStep;
#pragma unroll
                for (int j = 0; j < 4; ++j) q[i][j] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (j * 64 + lane) * 8, 0, 2);
                hh[i] = __builtin_amdgcn_raw_buffer_load_b128(win, off + 2048 + lane * 16, 0, 2);
            }
            const int kbase = (s0 + s) * 16 * 24 + kb * 24;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x4_t a[3];
#pragma unroll
                for (int m = 0; m < 3; ++m) a[m] = load_xfrag<XF16, true>(xrow, kbase + 4 * j * 24 + 8 * m, k.neuron_len);
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const NvqUnit un = nvq_decode(q[i][j].x, q[i][j].y, hh[i][j]);
                    const uint32_t state = un.state;
                    const uint32_t *bank = cbp + bankoff[state];
                    const half2_t sc = __builtin_bit_cast(half2_t, luth[state]);
                    const uint32_t(&mk)[3] = un.mask;
                    const uint32_t(&ix)[6] = un.idx;
#pragma unroll
                    for (int m = 0; m < 3; ++m) {
                        const u32x4_t sx = *reinterpret_cast<const u32x4_t *>(sgx + 4 * mk[m]);
                        const u32x2_t c0 = *reinterpret_cast<const u32x2_t *>(bank + 2 * ix[2 * m]);
                        const u32x2_t c1 = *reinterpret_cast<const u32x2_t *>(bank + 2 * ix[2 * m + 1]);
                        const uint32_t wv[4] = {c0.x ^ sx.x, c0.y ^ sx.y, c1.x ^ sx.z, c1.y ^ sx.w};
                        u32x4_t b;
#pragma unroll
                        for (int t = 0; t < 4; ++t) b[t] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, wv[t]) * sc);
                        acc[i] = mfma16(a[m], b, acc[i]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * NB + i) * 4 + v) * 64 + lane] = anchor[i] * acc[i][v] * xinv;
    mfma_store_dense<NB>(red, rb0, m0, M, k.out, y, ldy);
}

// ---- 16-row tiles with the signed table in LDS ---------------------------------------------------
// Up to 16 activation rows per block (blockIdx.y = tile), one block per CU: a block owns up to RPB consecutive row-blocks, its waves split the K
// steps.  The table maps (bank, entry, sign nibble) to the four signed fp16 magnitudes of a vector, so a fragment is
// two 8-byte LDS reads at byte offsets that sit ready-made in the unit's fields, and one packed multiply per pair by
// the state's scale; no sign table, no XOR, no index arithmetic.  A wave keeps the activation fragments of its current
// step in registers (requested before any weights) and walks (step, row-block) items through a ring of RING unit
// buffers: the only loads inside the walk are weights, each requested RING items before its use, so the waits are
// for weights alone and the first request wave covers most of a block's share.
// LDS map (bytes): [signed table: banks*entries*128][state table: 16 x {lut pair, bank base}][red: waves * 1024]
// [codebook entries as fp16 pairs: banks*entries*8]
typedef const __attribute__((address_space(3))) u32x2_t *lds_u32x2_ptr;
struct NvqSecond {  // the second tensor of a two-projection launch; blocks0 = grid.x when there is none
    NvqK k;
    const uint8_t *w;
    int blocks0, col;
};
template <int XF16, int RPB, int RING, bool ONE>
__global__ __launch_bounds__(1024) void nvq_signed_kernel(NvqK k_first, const uint8_t *__restrict__ w_first,
                                                          const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                          float *__restrict__ y_first, int64_t ldy, int spw, NvqSecond s2) {
    // blocks from s2.blocks0 on belong to a second tensor of the same neuron length (same activations), whose
    // outputs follow the first tensor's in each row of y
    const bool second = static_cast<int>(blockIdx.x) >= s2.blocks0;
    const NvqK &k = second ? s2.k : k_first;
    const uint8_t *__restrict__ w = second ? s2.w : w_first;
    float *__restrict__ y = y_first + (second ? s2.col : 0);
    const int bx = static_cast<int>(blockIdx.x) - (second ? s2.blocks0 : 0);
    // item (step ls, row-block i) lives in ring[i % RING]: the ring depth divides the row-blocks of a step
    static_assert(ONE ? RING <= RPB : RPB % RING == 0, "ring slots are chosen at compile time");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ncb = k.banks * k.entries;
    uint32_t *stab = lds + ncb * 32;
    float *red = reinterpret_cast<float *>(stab + 32);
    // LDS byte address of the signed table (0 unless something else is placed first)
    const uint32_t lds_base = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint32_t *)lds));

    const int rb_first = bx * RPB;
    const int nrb = min(RPB, k.n_rowblocks - rb_first);  // row-blocks of this block
    const int m0 = static_cast<int>(blockIdx.y) * 16;  // the block's 16-row tile
    const int tok = min(m0 + static_cast<int>(lane & 15), M - 1);
    const uint16_t *xrow = x + static_cast<int64_t>(tok) * ldx;
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;  // may be <= 0: the wave only takes part in the barriers
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb_first) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);

    struct Item {
        u32x2_t q[4];
        u32x4_t c;
    };
    Item ring[RING];
    auto wload = [&](int ls, int i, Item &it) {  // step s0 + ls of row-block rb_first + i; zeros when there is none
        const uint32_t off = ls < n && i < nrb ? i * rbb + ls * sb : kNoStep;
#pragma unroll
        for (int j = 0; j < 4; ++j) it.q[j] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (j * 64 + lane) * 8, 0, 2);
        it.c = __builtin_amdgcn_raw_buffer_load_b128(win, off + 2048 + lane * 16, 0, 2);
    };
    u32x4_t xf[4][3];
    auto xload = [&](int ls) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int m = 0; m < 3; ++m)
                xf[j][m] = load_xfrag_raw<true>(xrow, (s0 + ls) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len);
    };
    auto xfinish = [&](int ls) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int m = 0; m < 3; ++m)
                xf[j][m] = xfrag_finish<XF16, true>(xf[j][m], (s0 + ls) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len);
    };
    // Everything a wave reads from global memory outside the walk is requested first, in the order of its use, so that
    // no wait has to cover weight requests issued later (loads return in order): the raw codebook entries (at most
    // four per thread: blocks have at least four waves), the state tables, the anchors, the activation fragments.
    const float *lut = reinterpret_cast<const float *>(w + k.tables_off);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const uint32_t *cb = bfs + 16;  // 4 int8 magnitudes per entry
    uint32_t craw[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) craw[t] = cb[min(tid + t * static_cast<int>(blockDim.x), ncb - 1)];
    const float lutv = lut[tid & 15];
    const uint32_t bankv = bfs[tid & 15];
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);

    // the first RING items: every wave requests its first item before any wave requests its second, so that the first
    // items of all waves come back first (requests are served roughly in the order the CU issued them)
    if (n > 0) xload(0);
#pragma unroll
    for (int t = 0; t < RING; ++t) {
        if (n > 0) wload(t / RPB, t % RPB, ring[t]);
        if (t + 1 < RING) __builtin_amdgcn_s_barrier();
    }
    // the entries as two fp16 pairs each, converted once (ncb x 8 bytes behind the reduction area)
    u32x2_t *cbh = reinterpret_cast<u32x2_t *>(red + (blockDim.x >> 6) * 256);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (tid + t * static_cast<int>(blockDim.x) < ncb) {
            uint32_t h[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) h[b] = f32_to_f16_rne(static_cast<float>((craw[t] >> (8 * b)) & 0xffu));
            cbh[tid + t * blockDim.x] = u32x2_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
        }
    }
    if (tid < 16) {
        const uint32_t h = f32_to_f16_rne(lutv);  // the LUT is fp16 in the payload: exact
        stab[2 * tid] = h | (h << 16);
        stab[2 * tid + 1] = lds_base + bankv * k.entries * 128;
    }
    __syncthreads();  // raw entries
    // chunk c = 16 bytes = the vectors of sign nibbles 2 * (c & 7) and 2 * (c & 7) + 1 of entry c >> 3
    for (int c = tid; c < ncb * 8; c += blockDim.x) {
        const u32x2_t e = cbh[c >> 3];
        const uint32_t p0 = e.x, p1 = e.y;
        const uint32_t n0 = 2u * (c & 7), n1 = n0 + 1u;
        u32x4_t v;
        v.x = p0 ^ (((n0 & 1u) << 15) | ((n0 & 2u) << 30));
        v.y = p1 ^ (((n0 & 4u) << 13) | ((n0 & 8u) << 28));
        v.z = p0 ^ (((n1 & 1u) << 15) | ((n1 & 2u) << 30));
        v.w = p1 ^ (((n1 & 4u) << 13) | ((n1 & 8u) << 28));
        *reinterpret_cast<u32x4_t *>(lds + 4 * c) = v;
    }
    const uint32_t stab_base = lds_base + ncb * 128;
    __syncthreads();  // tables

    // one item = the four units of a (step, row-block); its registers are refilled unit by unit, as soon as each is
    // read, from byte offset noff of the window (kNoStep: nothing left to request)
    auto process = [&](Item &it, uint32_t noff, bool refill, float4_t &acc) {
        const u32x4_t uc4 = it.c;
        if (refill) it.c = __builtin_amdgcn_raw_buffer_load_b128(win, noff + 2048 + lane * 16, 0, 2);
        // the state entries of the four units first: one LDS round trip for the item instead of one per unit
        const uint32_t ucv[4] = {uc4.x, uc4.y, uc4.z, uc4.w};
        u32x2_t stv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            stv[j] = *reinterpret_cast<lds_u32x2_ptr>(stab_base + (__builtin_rotateleft32(ucv[j], 6) & 0x78u));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t ua = it.q[j].x, ub = it.q[j].y, uc = ucv[j];
            if (refill) it.q[j] = __builtin_amdgcn_raw_buffer_load_b64(win, noff + (j * 64 + lane) * 8, 0, 2);
            const u32x2_t st = stv[j];
            const half2_t sc = __builtin_bit_cast(half2_t, st.x);
            const uint32_t off[6] = {and_or(ua, 0xfff8u, st.y), and_or(ua >> 16, 0xfff8u, st.y),
                                     and_or(ub, 0xfff8u, st.y), and_or(ub >> 16, 0xfff8u, st.y),
                                     and_or(uc, 0xfff8u, st.y), and_or(uc >> 13, 0xfff8u, st.y)};
#pragma unroll
            for (int m = 0; m < 3; ++m) {
                const u32x2_t c0 = *reinterpret_cast<lds_u32x2_ptr>(off[2 * m]);
                const u32x2_t c1 = *reinterpret_cast<lds_u32x2_ptr>(off[2 * m + 1]);
                const uint32_t wv[4] = {c0.x, c0.y, c1.x, c1.y};
                u32x4_t b;
#pragma unroll
                for (int t = 0; t < 4; ++t) b[t] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, wv[t]) * sc);
                acc = mfma16(xf[j][m], b, acc);
            }
        }
    };
    auto store = [&](int i, const float4_t &acc) {  // adds the waves' partial sums of row-block i; block-uniform
        const float av = anchors[(rb_first + i) * 16 + r];
#pragma unroll
        for (int v = 0; v < 4; ++v) red[(wave * 4 + v) * 64 + lane] = av * acc[v];
        mfma_store_dense<1>(red, rb_first + i, m0, M, k.out, y, ldy);
        __syncthreads();
    };
    if constexpr (ONE) {  // one step per wave: the ring may have any depth up to RPB
        float4_t acc[RPB];
#pragma unroll
        for (int i = 0; i < RPB; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
        if (n > 0) {
            xfinish(0);
#pragma unroll
            for (int i = 0; i < RPB; ++i)
                process(ring[i % RING], i + RING < nrb ? (i + RING) * rbb : kNoStep, i + RING < RPB, acc[i]);
        }
#pragma unroll
        for (int i = 0; i < RPB; ++i)
            if (i < nrb) store(i, acc[i]);
    } else {
        float4_t acc[RPB];
#pragma unroll
        for (int i = 0; i < RPB; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int ls = 0; ls < n; ++ls) {
            if (ls > 0) xload(ls);
            xfinish(ls);
#pragma unroll
            for (int i = 0; i < RPB; ++i) {
                const int nls = ls + (i + RING) / RPB, ni = (i + RING) % RPB;
                process(ring[i % RING], nls < n && ni < nrb ? ni * rbb + nls * sb : kNoStep, true, acc[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < RPB; ++i)
            if (i < nrb) store(i, acc[i]);
    }
}

// ---- one or two rows with the signed table in LDS and the activations in registers ------------------------------
// The block frame of nvq_signed_kernel (one block per compute unit with RPB consecutive row-blocks, its waves split the
// K steps, SPW steps per wave) for one or two activation rows, on the vector ALUs: a unit (24 weights of the neuron of
// lane (r, kb)) is six 8-byte reads of signed fp16 vectors out of the LDS table and twelve packed dot products whose
// activation pair comes out of another lane's register -- the 16 lanes of a DPP row share a group, lane r of the row
// keeps pair r of it (12 pairs) and v_dot2c_f32_f16_dpp ... row_newbcast:i fetches pair i.  So the activations of a
// step are four registers per row instead of 48 registers of matrix-core fragments, the unit's scale is one multiply
// of its dot product, and the registers that frees hold a whole item's 24 gathers at once: an item costs two LDS round
// trips (states, then all vectors) instead of eight.
// Items are walked row-block by row-block (steps inside), item (row-block i, step ls) in ring slot (i % DEPTH) * SPW +
// ls, each slot refilled -- after the last read of what it holds -- with the same step DEPTH row-blocks further on.
// What bounds the kernel is the LDS: 128 KB of table writes (1.3 us at the 64 bytes a cycle a compute unit's LDS
// takes) and 28 LDS instructions an item (24 of them 8-byte gathers at random addresses, about 7 cycles each against 4
// without bank conflicts) -- on 17408 x 5120, 70 items a block, 6.5 us of LDS time after a table that stands at
// 3.4 us, in a launch of 11.1 us.  A compute unit also keeps only about 64 memory requests in flight, whatever their
// size, hands their data back in the order they were issued whichever wave they are for, and a wave whose request does
// not fit waits at the request: asking for more than one item per wave before the tables stand only delays the waves
// that have to build them (tables at 4.8 us with two items ahead, at 7.1 us with four).
// LDS map (bytes): [signed table: banks*entries*128][state table: 16 x {lut f32, bank base}][red: RPB * waves * MB * 16 f32]
// [anchors: RPB * 16 f32][raw codebook entries as fp16 pairs: banks*entries*8]
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}
template <int XF16, int MB, int SPW>
__global__ __launch_bounds__(1024) void nvq_bcast_kernel(NvqK k_first, const uint8_t *__restrict__ w_first,
                                                         const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                         float *__restrict__ y_first, int64_t ldy, int rpb, NvqSecond s2) {
    // DEPTH row-blocks of the wave's steps are in flight in the walk, PRE of them requested before the tables are built
    // (17408 x 5120, DEPTH/PRE: 2/1 13.7 us, 2/2 14.3, 3/1 14.5, 4/2 15.5, 1/1 14.7)
    constexpr int DEPTH = SPW <= 2 ? 2 : 1, RING = SPW * DEPTH;
    constexpr int PRE = 1;
    const bool second = static_cast<int>(blockIdx.x) >= s2.blocks0;
    const NvqK &k = second ? s2.k : k_first;
    const uint8_t *__restrict__ w = second ? s2.w : w_first;
    float *__restrict__ y = y_first + (second ? s2.col : 0);
    const int bx = static_cast<int>(blockIdx.x) - (second ? s2.blocks0 : 0);
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ncb = k.banks * k.entries;
    uint32_t *stab = lds + ncb * 32;
    float *red = reinterpret_cast<float *>(stab + 32);
    const uint32_t lds_base = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint32_t *)lds));

    const int rb_first = bx * rpb;
    const int nrb = min(rpb, k.n_rowblocks - rb_first);
    const int m0 = static_cast<int>(blockIdx.y) * MB;
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * SPW;
    const int n = min(k.nsteps, s0 + SPW) - s0;  // steps of this wave, may be <= 0
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb_first) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);
    struct Item {
        u32x2_t q[4];
        u32x4_t c;
    };
    Item ring[RING];
    auto wload = [&](int ls, int i, Item &it) {  // step s0 + ls of row-block rb_first + i; zeros when there is none
        const uint32_t off = ls < n && i < nrb ? i * rbb + ls * sb : kNoStep;
#pragma unroll
        for (int j = 0; j < 4; ++j) it.q[j] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (j * 64 + lane) * 8, 0, 2);
        it.c = __builtin_amdgcn_raw_buffer_load_b128(win, off + 2048 + lane * 16, 0, 2);
    };
    // A compute unit hands back what its waves asked for in the order they asked, whichever wave it is for.  The first
    // wave of the block therefore asks for everything the tables are made of (codebook entries, state table, anchors)
    // before any wave asks for weights: fetched by all waves, each wave's share would arrive behind the weights the
    // waves launched before it have requested, and the tables -- which every wave waits for -- with the last of them.
    const uint8_t *tb = w + k.tables_off;
    u32x4_t craw[4] = {};   // wave 0: entries 4 * (t * 64 + lane) .. + 3, four int8 magnitudes each
    uint32_t lutv = 0, bankv = 0;
    u32x2_t anc_v = {0, 0};
    if (wave == 0) {
        const __amdgpu_buffer_rsrc_t wt = wave_window(tb, 128u + static_cast<uint32_t>(ncb) * 4u);
#pragma unroll
        for (int t = 0; t < 4; ++t) craw[t] = __builtin_amdgcn_raw_buffer_load_b128(wt, 128u + static_cast<uint32_t>(t * 64 + lane) * 16u, 0, 0);
        lutv = __builtin_amdgcn_raw_buffer_load_b32(wt, lane < 16 ? lane * 4u : kNoStep, 0, 0);
        bankv = __builtin_amdgcn_raw_buffer_load_b32(wt, lane < 16 ? 64u + lane * 4u : kNoStep, 0, 0);
        const __amdgpu_buffer_rsrc_t wa = wave_window(w + k.anchors_off + static_cast<int64_t>(rb_first) * 64, static_cast<uint32_t>(nrb) * 64u);
        anc_v = __builtin_amdgcn_raw_buffer_load_b64(wa, lane * 8u, 0, 0);
    }
    // activations: lane (r, kb) asks for pair r (of 12) of group 16 (s0 + ls) + 4 j + kb of every row
    uint32_t xraw[MB][SPW][4];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const bool row_ok = m0 + m < M;
        const __amdgpu_buffer_rsrc_t wx = wave_window(reinterpret_cast<const uint8_t *>(x + static_cast<int64_t>(row_ok ? m0 + m : 0) * ldx),
                                                      row_ok ? static_cast<uint32_t>(k.neuron_len) * 2u : 0u);
#pragma unroll
        for (int ls = 0; ls < SPW; ++ls)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t off = static_cast<uint32_t>(((s0 + ls) * 16 + 4 * j + kb) * 12 + r) * 4u;
                xraw[m][ls][j] = __builtin_amdgcn_raw_buffer_load_b32(wx, (ls < n && r < 12) ? off : kNoStep, 0, 0);
            }
    }
    // the first PRE row-blocks' items go out now, the rest of the ring once the tables stand
#pragma unroll
    for (int d = 0; d < PRE; ++d)
#pragma unroll
        for (int ls = 0; ls < SPW; ++ls) wload(ls, d, ring[d * SPW + ls]);
    // tables: the entries as two fp16 pairs each, then the signed table (see nvq_signed_kernel); the anchors wait in LDS
    // because a global load inside the walk would have to wait for every weight request before it
    float *anc = red + rpb * nwaves * MB * 16;  // rpb * 16 anchors
    u32x2_t *cbh = reinterpret_cast<u32x2_t *>(anc + rpb * 16);
    if (wave == 0) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int e0 = 4 * (t * 64 + lane);
            if (e0 < ncb) {
                const uint32_t cr[4] = {craw[t].x, craw[t].y, craw[t].z, craw[t].w};
                uint32_t h[4][4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int b = 0; b < 4; ++b) h[e][b] = f32_to_f16_rne(static_cast<float>((cr[e] >> (8 * b)) & 0xffu));
                u32x4_t *dst = reinterpret_cast<u32x4_t *>(cbh + e0);
                dst[0] = u32x4_t{h[0][0] | (h[0][1] << 16), h[0][2] | (h[0][3] << 16), h[1][0] | (h[1][1] << 16), h[1][2] | (h[1][3] << 16)};
                dst[1] = u32x4_t{h[2][0] | (h[2][1] << 16), h[2][2] | (h[2][3] << 16), h[3][0] | (h[3][1] << 16), h[3][2] | (h[3][3] << 16)};
            }
        }
        if (lane < 16) {
            stab[2 * lane] = lutv;
            stab[2 * lane + 1] = lds_base + bankv * k.entries * 128;
        }
        if (lane * 2 < nrb * 16) *reinterpret_cast<u32x2_t *>(anc + lane * 2) = anc_v;
    }
    __syncthreads();  // raw entries
    for (int c = tid; c < ncb * 8; c += blockDim.x) {
        const u32x2_t e = cbh[c >> 3];
        const uint32_t p0 = e.x, p1 = e.y;
        const uint32_t n0 = 2u * (c & 7), n1 = n0 + 1u;
        u32x4_t v;
        v.x = p0 ^ (((n0 & 1u) << 15) | ((n0 & 2u) << 30));
        v.y = p1 ^ (((n0 & 4u) << 13) | ((n0 & 8u) << 28));
        v.z = p0 ^ (((n1 & 1u) << 15) | ((n1 & 2u) << 30));
        v.w = p1 ^ (((n1 & 4u) << 13) | ((n1 & 8u) << 28));
        *reinterpret_cast<u32x4_t *>(lds + 4 * c) = v;
    }
    const uint32_t stab_base = lds_base + ncb * 128;
    __syncthreads();  // tables
#pragma unroll
    for (int d = PRE; d < DEPTH; ++d)
#pragma unroll
        for (int ls = 0; ls < SPW; ++ls) wload(ls, d, ring[d * SPW + ls]);
    // the activation pairs as fp16 (bf16 rows: times the wave's power of two that brings its slice near 2^12)
    uint32_t xh[MB][SPW][4];
    float xinv[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float sc = 1.f;
        xinv[m] = 1.f;
        if constexpr (!XF16) {
            uint32_t mx = 0;
#pragma unroll
            for (int ls = 0; ls < SPW; ++ls)
#pragma unroll
                for (int j = 0; j < 4; ++j) mx = absmax_bf16(mx, xraw[m][ls][j]);
            sc = slice_scale(wave_max_u32(mx), xinv[m]);
        }
#pragma unroll
        for (int ls = 0; ls < SPW; ++ls)
#pragma unroll
            for (int j = 0; j < 4; ++j) xh[m][ls][j] = XF16 ? xraw[m][ls][j] : to_h2_scaled(xraw[m][ls][j], sc);
#pragma unroll
        for (int ls = 0; ls < SPW; ++ls) dpp_source_ready(xh[m][ls][0], xh[m][ls][1], xh[m][ls][2], xh[m][ls][3]);
    }

    // one item: the states of its four units, then all 24 vectors at once, then the dot products
    auto process = [&](Item &it, uint32_t noff, const uint32_t (&xs)[MB][SPW][4], auto LS, float (&acc)[MB]) {
        constexpr int ls = decltype(LS)::value;  // compile time: the pair register goes into the dot products as it is
        // The slot is refilled only after the last use of what it holds: requested any earlier, the new values would need
        // registers of their own and a copy into the slot, and that copy would wait for the request it came from.
        const uint32_t ucv[4] = {it.c.x, it.c.y, it.c.z, it.c.w};
        u32x2_t stv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            stv[j] = *reinterpret_cast<lds_u32x2_ptr>(stab_base + (__builtin_rotateleft32(ucv[j], 6) & 0x78u));
        // GB units' vectors are gathered at once (all four where the registers allow it)
        constexpr int GB = (SPW == 1) ? 4 : 2;
#pragma unroll
        for (int j0 = 0; j0 < 4; j0 += GB) {
            u32x2_t vec[GB][6];
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                const int j = j0 + g;
                const uint32_t ua = it.q[j].x, ub = it.q[j].y, uc = ucv[j];
                const uint32_t base = stv[j].y;
                const uint32_t off[6] = {and_or(ua, 0xfff8u, base), and_or(ua >> 16, 0xfff8u, base),
                                         and_or(ub, 0xfff8u, base), and_or(ub >> 16, 0xfff8u, base),
                                         and_or(uc, 0xfff8u, base), and_or(uc >> 13, 0xfff8u, base)};
#pragma unroll
                for (int t = 0; t < 6; ++t) vec[g][t] = *reinterpret_cast<lds_u32x2_ptr>(off[t]);
            }
            if (j0 + GB == 4) {  // every field of the slot has been read: refill it
                asm volatile("" ::: "memory");
#pragma unroll
                for (int j = 0; j < 4; ++j) it.q[j] = __builtin_amdgcn_raw_buffer_load_b64(win, noff + (j * 64 + lane) * 8, 0, 2);
                it.c = __builtin_amdgcn_raw_buffer_load_b128(win, noff + 2048 + lane * 16, 0, 2);
            }
#pragma unroll
            for (int g = 0; g < GB; ++g) {
                const int j = j0 + g;
                const float sc = __uint_as_float(stv[j].x);
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    float a = 0.f;
                    const uint32_t xv = xs[m][ls][j];
                    a = dot2_bcast4<0, false>(a, xv, vec[g][0].x, vec[g][0].y, vec[g][1].x, vec[g][1].y);
                    a = dot2_bcast4<4, false>(a, xv, vec[g][2].x, vec[g][2].y, vec[g][3].x, vec[g][3].y);
                    a = dot2_bcast4<8, true>(a, xv, vec[g][4].x, vec[g][4].y, vec[g][5].x, vec[g][5].y);
                    acc[m] = fmaf(sc, a, acc[m]);
                }
            }
        }
    };
    // the waves' partial sums of row-block i: slot (i * nwaves + wave) * MB + m, 16 neurons each
    auto park = [&](int i, float (&acc)[MB]) {
        const float av = anc[i * 16 + r];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float v = reduce_kb4(acc[m]) * av * xinv[m];
            if (lane < 16) red[((i * nwaves + wave) * MB + m) * 16 + lane] = v;
            acc[m] = 0.f;
        }
    };
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.f;
    // The walk is straight-line code over up to eight row-blocks with one exit per row-block and nothing conditional in
    // between (a wave without steps, or past the block's last row-block, walks zeros): with a loop, or a branch around an
    // item, the compiler could not count the requests in flight and would wait for all of them -- the refill it has just
    // issued included -- before every item.
#define NVQ_RB(II)                                                                                                   \
    if (II >= rpb) break;                                                                                            \
    static_for<SPW>([&](auto LS) {                                                                                   \
        constexpr int ls = decltype(LS)::value;                                                                      \
        process(ring[(II % DEPTH) * SPW + ls], ls < n && II + DEPTH < nrb ? (II + DEPTH) * rbb + ls * sb : kNoStep, xh, LS, acc); \
    });                                                                                                              \
    park(II, acc);
    do {
        NVQ_RB(0) NVQ_RB(1) NVQ_RB(2) NVQ_RB(3) NVQ_RB(4) NVQ_RB(5) NVQ_RB(6) NVQ_RB(7)
    } while (0);
#undef NVQ_RB
    __syncthreads();
    for (int o = tid; o < nrb * MB * 16; o += blockDim.x) {
        const int rr = o & 15, m = (o >> 4) % MB, i = (o >> 4) / MB;
        float sum = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) sum += red[((i * nwaves + wv) * MB + m) * 16 + rr];
        const int row = (rb_first + i) * 16 + rr;
        if (m0 + m < M && row < k.out) y[static_cast<int64_t>(m0 + m) * ldy + row] = sum;
    }
}

// ---- prefill: block-tiled MFMA GEMM, weight fragments built from the codebooks in LDS ----------------------
// Block = 8 waves side by side on 8 * NB row-blocks, wave tile MT * 16 tokens x NB * 16 neurons.  Activations as in
// the NINT prefill kernel: fp16 rows scaled per token (x_prep), the 96 k-values of a sub-step (unit j of a step) staged
// in LDS, two buffers, XD tiles in flight in registers.  Weights: PF unit buffers per row-block (PF - 1 sub-steps in
// flight), each fragment built as in nvq_mfma_kernel -- two codebook vectors, sign bits XOR-ed in, one packed fp16
// multiply by the state's scale -- and shared by the MT token tiles of the wave.
// LDS map (dwords): [codebook pairs: banks*entries*2][sign xor table: 512][lut pairs: 16][bank offset: 16][x tiles]
template <int MT, int NB, int PF, int XD>
__global__ __launch_bounds__(512) void nvq_prefill_kernel(NvqK k, const uint8_t *__restrict__ w,
                                                          const uint16_t *__restrict__ x16, int Kp,
                                                          const float *__restrict__ xscale, int M,
                                                          float *__restrict__ y, int64_t ldy, int spz, int64_t ystride) {
    static_assert((PF == 2 || PF == 4) && (XD == 1 || XD == 2 || XD == 4), "the sub-step loop is unrolled four times");
    // split blockIdx.z over K: steps [s_begin, s_end), partial result at y + z * ystride
    const int s_begin = static_cast<int>(blockIdx.z) * spz, s_end = min(k.nsteps, s_begin + spz);
    y += static_cast<int64_t>(blockIdx.z) * ystride;
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr int GS = 24, NM = 3, NT = 512, BM = MT * 16, EL = 8;
    constexpr int ROW = 4 * GS + 8;  // LDS row stride in halves
    constexpr int CPG = GS / EL, CHUNKS = 4 * CPG;
    constexpr int PER_THREAD = (BM * CHUNKS + NT - 1) / NT;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kb = lane >> 4;
    const int ncb = k.banks * k.entries;
    uint32_t *cbp = lds;
    uint32_t *sgx = cbp + 2 * ncb;
    uint32_t *luth = sgx + 512;
    uint32_t *bankoff = luth + 16;
    uint16_t *xt = reinterpret_cast<uint16_t *>(bankoff + 16);
    {
        const float *lut = reinterpret_cast<const float *>(w + k.tables_off);
        const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
        const uint32_t *cb = bfs + 16;  // 4 int8 magnitudes per entry
        for (int i = tid; i < ncb; i += NT) {
            const uint32_t e = cb[i];
            uint32_t h[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) h[t] = f32_to_f16_rne(static_cast<float>((e >> (8 * t)) & 0xffu));
            cbp[2 * i] = h[0] | (h[1] << 16);
            cbp[2 * i + 1] = h[2] | (h[3] << 16);
        }
        for (int i = tid; i < 128; i += NT) {
            const uint32_t m8 = parity8(i);
#pragma unroll
            for (int p = 0; p < 4; ++p)
                sgx[4 * i + p] = (((m8 >> (2 * p)) & 1u) << 15) | (((m8 >> (2 * p + 1)) & 1u) << 31);
        }
        if (tid < 16) {
            const uint32_t h = f32_to_f16_rne(lut[tid]);
            luth[tid] = h | (h << 16);
            bankoff[tid] = bfs[tid] * k.entries * 2;
        }
    }
    const DenseRows rows{static_cast<int>(blockIdx.y) * BM, M};
    const int rb0 = (static_cast<int>(blockIdx.x) * 8 + wave) * NB;
    const int nrb = max(0, min(NB, k.n_rowblocks - rb0));
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(min(rb0, k.n_rowblocks - 1)) * k.rowblock_bytes, nrb * rbb);
    float4_t acc[MT][NB];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    const uint16_t *xsrc[PER_THREAD];
    int xk[PER_THREAD];
#pragma unroll
    for (int p = 0; p < PER_THREAD; ++p) {
        const int c = min(tid + NT * p, BM * CHUNKS - 1);
        const int row = c / CHUNKS;
        xsrc[p] = x16 + static_cast<int64_t>(rows.src(row)) * Kp;
        xk[p] = EL * (c - row * CHUNKS);
    }
    u32x4_t xr[XD][PER_THREAD];
    auto xload = [&](int it, u32x4_t (&xq)[PER_THREAD]) {
        const int k0 = it * 4 * GS;
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int kk = k0 + xk[p];
            u32x4_t v = *reinterpret_cast<const u32x4_t *>(xsrc[p] + min(kk, Kp - EL));
            if (kk >= Kp) v = u32x4_t{0u, 0u, 0u, 0u};
            xq[p] = v;
        }
    };
    auto xstore = [&](int buf, const u32x4_t (&xq)[PER_THREAD]) {
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int c = tid + NT * p;
            const int row = c / CHUNKS, ch = c - row * CHUNKS;
            if (c < BM * CHUNKS) *reinterpret_cast<u32x4_t *>(xt + buf * (BM * ROW) + row * ROW + EL * ch) = xq[p];
        }
    };
    u32x2_t qr[PF][NB];
    u32x4_t hh[NB], hhn[NB];
    auto wload = [&](int it, u32x2_t (&qq)[NB]) {
        const int s = it >> 2, j = it & 3;
#pragma unroll
        for (int b = 0; b < NB; ++b)
            qq[b] = __builtin_amdgcn_raw_buffer_load_b64(
                win, b < nrb && s < s_end ? b * rbb + s * sb + (j * 64 + lane) * 8 : kNoStep, 0, 0);
    };
    auto hload = [&](int s, u32x4_t (&h)[NB]) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
            h[b] = __builtin_amdgcn_raw_buffer_load_b128(win, b < nrb && s < s_end ? b * rbb + s * sb + 2048 + lane * 16 : kNoStep,
                                                         0, 0);
    };
    xload(4 * s_begin, xr[0]);
#pragma unroll
    for (int i = 0; i < PF - 1; ++i) wload(4 * s_begin + i, qr[i]);
    hload(s_begin, hh);
    xstore(0, xr[0]);
#pragma unroll
    for (int i = 1; i < XD; ++i) xload(4 * s_begin + i, xr[i]);
    __syncthreads();  // tables and the first tile

    for (int s = s_begin; s < s_end; ++s) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int it = 4 * s + j;
            xload(it + XD, xr[j % XD]);
            wload(it + PF - 1, qr[(j + PF - 1) % PF]);
            if (j == 0) hload(s + 1, hhn);
            const uint32_t *bank[NB];
            half2_t sc[NB];
            uint32_t mk[NB][3], ix[NB][6];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const NvqUnit un = nvq_decode(qr[j % PF][b].x, qr[j % PF][b].y, hh[b][j]);
                const uint32_t state = un.state;
                bank[b] = cbp + bankoff[state];
                sc[b] = __builtin_bit_cast(half2_t, luth[state]);
#pragma unroll
                for (int t = 0; t < 3; ++t) mk[b][t] = un.mask[t];
#pragma unroll
                for (int t = 0; t < 6; ++t) ix[b][t] = un.idx[t];
            }
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                u32x4_t af[MT];
#pragma unroll
                for (int a = 0; a < MT; ++a)
                    af[a] = *reinterpret_cast<const u32x4_t *>(xt + (j & 1) * (BM * ROW) + (a * 16 + r) * ROW + kb * GS + 8 * m);
                u32x4_t bf[NB];
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const u32x4_t sx = *reinterpret_cast<const u32x4_t *>(sgx + 4 * mk[b][m]);
                    const u32x2_t c0 = *reinterpret_cast<const u32x2_t *>(bank[b] + 2 * ix[b][2 * m]);
                    const u32x2_t c1 = *reinterpret_cast<const u32x2_t *>(bank[b] + 2 * ix[b][2 * m + 1]);
                    const uint32_t wv[4] = {c0.x ^ sx.x, c0.y ^ sx.y, c1.x ^ sx.z, c1.y ^ sx.w};
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        bf[b][t] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, wv[t]) * sc[b]);
                }
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int a = 0; a < MT; ++a) acc[a][b] = mfma16(af[a], bf[b], acc[a][b]);
            }
            xstore((j + 1) & 1, xr[(j + 1) % XD]);
            if (j == 3) {
#pragma unroll
                for (int b = 0; b < NB; ++b) hh[b] = hhn[b];
            }
            __syncthreads();
        }
    }
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    float an[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) an[b] = anchors[min(rb0 + b, k.n_rowblocks - 1) * 16 + r];
#pragma unroll
    for (int a = 0; a < MT; ++a) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int ti = a * 16 + 4 * kb + v;
            const int m = rows.dst(ti);
            if (m < 0) continue;
            const float xs = xscale[m];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int col = (rb0 + b) * 16 + r;
                if (rb0 + b < k.n_rowblocks && col < k.out) y[static_cast<int64_t>(m) * ldy + col] = xs * (an[b] * acc[a][b][v]);
            }
        }
    }
}

static size_t nvq_prefill_lds(const NvqK &k, int bm) {
    return (static_cast<size_t>(k.banks) * k.entries * 2 + 512 + 32) * 4 + static_cast<size_t>(2 * bm) * (4 * 24 + 8) * 2;
}

int prefill_sum_splits(const float *part, int64_t ystride, int splits, int M, int N, float *y, int64_t ldy, hipStream_t st);

// Splits over K: grids of 64-token tiles that leave CUs idle are cut along K (up to eight splits of at least two
// steps); the partial results go to the workspace and are added in split order.  1 = no split.
static int nvq_prefill_splits(const NvqK &k, int M) {
    const int64_t blocks = ceil_div(k.n_rowblocks, 16) * ceil_div(M, 64);
    if (blocks > 128 || k.out % 4) return 1;
    int splits = static_cast<int>(256 / blocks);
    if (splits > 8) splits = 8;
    if (splits > k.nsteps / 2) splits = k.nsteps / 2;
    if (splits <= 1) return 1;
    const int spz = static_cast<int>(ceil_div(k.nsteps, splits));
    return static_cast<int>(ceil_div(k.nsteps, spz));  // no empty split
}

// x16 [M, Kp] fp16 rows scaled by 1 / xscale[m], zero beyond K (x_prep); part: splits * M * out floats when split
static int nvq_prefill(const NvqK &k, const uint8_t *w, const uint16_t *x16, int Kp, const float *xscale, int M, float *y,
                       int64_t ldy, float *part, hipStream_t st) {
    const int splits = part ? nvq_prefill_splits(k, M) : 1;
    const int spz = static_cast<int>(ceil_div(k.nsteps, splits));
    const int64_t ystride = static_cast<int64_t>(M) * k.out;
    float *yk = splits > 1 ? part : y;
    const int64_t ldk = splits > 1 ? k.out : ldy;
#define MFQ_NVQ_PREFILL(MT, NB, XD)                                                                                   \
    {                                                                                                                  \
        const dim3 grid(static_cast<unsigned>(ceil_div(k.n_rowblocks, 8 * NB)), static_cast<unsigned>(ceil_div(M, MT * 16)), \
                        static_cast<unsigned>(splits));                                                                \
        const size_t lds = nvq_prefill_lds(k, MT * 16);                                                                \
        auto kern = nvq_prefill_kernel<MT, NB, 4, XD>;                                                                 \
        if (lds > 65536) {                                                                                             \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                   \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));     \
            MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nvq_prefill: %s", hipGetErrorString(e));                     \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, k, w, x16, Kp, xscale, M, yk, ldk, spz, ystride);           \
        if (splits > 1) return prefill_sum_splits(part, ystride, splits, M, k.out, y, ldy, st);                        \
        return check_launch("nvq_prefill");                                                                            \
    }
    // 64 x 256 tiles while they give at most one block per CU (four activation tiles in flight); beyond, the cheaper
    // of 128 x 256 and 64 x 384 by rounds of 256 blocks x tile area (see nint_prefill; here the second runs at 0.85 of
    // the first's rate per area: building a fragment costs more, so sharing it among eight token tiles counts for more)
    if (ceil_div(k.n_rowblocks, 16) * ceil_div(M, 64) <= 256) MFQ_NVQ_PREFILL(4, 2, 4)
    const double cost_a = static_cast<double>(ceil_div(ceil_div(k.n_rowblocks, 16) * ceil_div(M, 128), 256)) * (128 * 256);
    const double cost_b = static_cast<double>(ceil_div(ceil_div(k.n_rowblocks, 24) * ceil_div(M, 64), 256)) * (64 * 384) / 0.85;
    if (cost_b < cost_a) MFQ_NVQ_PREFILL(4, 3, 2)
    MFQ_NVQ_PREFILL(8, 2, 2)
#undef MFQ_NVQ_PREFILL
}

static bool nvq_stream_capable(const NvqK &k) {
    return k.neuron_len >= 8 && k.neuron_len % 8 == 0 && 4 * k.rowblock_bytes < (1ll << 31);
}

template <int XF16, int NB>
static int nvq_launch_mfma(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                           hipStream_t st) {
    const int64_t groups = ceil_div(k.n_rowblocks, NB);
    int spw = static_cast<int>(ceil_div(k.nsteps, 8));
    while (spw < k.nsteps && groups * ceil_div(k.nsteps, spw) > 8192) ++spw;
    const int nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const size_t lds = (static_cast<size_t>(k.banks) * k.entries * 2 + 512 + 32) * 4 + static_cast<size_t>(nwaves) * NB * 1024;
    MFQ_REQUIRE(lds <= 65536, MFQ_ERR_UNSUPPORTED, "nvq_mfma: %zu bytes of LDS", lds);
    hipLaunchKernelGGL((nvq_mfma_kernel<XF16, NB>), dim3(static_cast<unsigned>(groups), static_cast<unsigned>(ceil_div(M, 16))),
                       dim3(64 * nwaves), lds, st, k, w, x, ldx, M, y, ldy, spw, PairSel{});
    return check_launch("nvq_mfma");
}

// the same kernel, a tile of one row per block row, over the pairs of a MoE decode step (see PairSel): eight times the
// generic kernel's rate on an expert of 2048 x 4096
template <int XF16, int NB>
static int nvq_launch_mfma_pairs(const NvqK &k, const uint16_t *x, int64_t ldx, int n_pairs, float *y, int64_t ldy, const PairSel &sel,
                                 hipStream_t st) {
    const int64_t groups = ceil_div(k.n_rowblocks, NB);
    int spw = static_cast<int>(ceil_div(k.nsteps, 8));
    while (spw < k.nsteps && groups * ceil_div(k.nsteps, spw) > 8192) ++spw;
    const int nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const size_t lds = (static_cast<size_t>(k.banks) * k.entries * 2 + 512 + 32) * 4 + static_cast<size_t>(nwaves) * NB * 1024;
    MFQ_REQUIRE(lds <= 65536, MFQ_ERR_UNSUPPORTED, "nvq_mfma_pairs: %zu bytes of LDS", lds);
    hipLaunchKernelGGL((nvq_mfma_kernel<XF16, NB, true>), dim3(static_cast<unsigned>(groups), static_cast<unsigned>(n_pairs)),
                       dim3(64 * nwaves), lds, st, k, static_cast<const uint8_t *>(nullptr), x, ldx, n_pairs, y, ldy, spw, sel);
    return check_launch("nvq_mfma_pairs");
}

// 16-row tiles through nvq_signed_kernel: at most one block per CU and tile, each with up to six row-blocks
static int nvq_signed_rpb(const NvqK &k, int more_rowblocks = 0) {
    return static_cast<int>(ceil_div(k.n_rowblocks + more_rowblocks, gemv_cu_count()));
}
static bool nvq_signed_capable(const NvqK &k, int M, int more_rowblocks = 0) {
    static const int off = tune_env("MFQ_NVQ_SIGNED_OFF", 0);
    const int rpb = nvq_signed_rpb(k, more_rowblocks);
    // two 16-row tiles still beat the older streaming kernel and the prefill kernel on the config 3 tensors
    // (17408 x 5120 at M = 32: 42 us against 54 and 46); MFQ_NVQ_SIGNED_MAX_M for tuning
    static const int max_m = tune_env("MFQ_NVQ_SIGNED_MAX_M", 32);
    return !off && M <= max_m && static_cast<int64_t>(k.banks) * k.entries * 128 <= 131072 && rpb <= 6 && k.nsteps >= 4 &&
           rpb * k.rowblock_bytes < (1ll << 31);
}
template <int XF16, int RPB, int RING, bool ONE>
static int nvq_launch_signed_as(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y,
                                int64_t ldy, hipStream_t st, const NvqSecond *second) {
    const int spw = static_cast<int>(ceil_div(k.nsteps, 16));
    const int nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const int blocks0 = static_cast<int>(ceil_div(k.n_rowblocks, RPB));
    NvqSecond s2{k, w, blocks0, 0};
    int blocks = blocks0;
    size_t ncb = static_cast<size_t>(k.banks) * k.entries;
    if (second) {
        s2 = *second;
        s2.blocks0 = blocks0;
        blocks += static_cast<int>(ceil_div(s2.k.n_rowblocks, RPB));
        if (static_cast<size_t>(s2.k.banks) * s2.k.entries > ncb) ncb = static_cast<size_t>(s2.k.banks) * s2.k.entries;
    }
    const size_t lds = ncb * 136 + 128 + static_cast<size_t>(nwaves) * 1024;
    auto kern = nvq_signed_kernel<XF16, RPB, RING, ONE>;
    if (lds > 65536) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(lds));
        MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nvq_signed: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks), static_cast<unsigned>(ceil_div(M, 16))), dim3(64 * nwaves), lds,
                       st, k, w, x, ldx, M, y, ldy, spw, s2);
    return check_launch("nvq_signed");
}
template <int XF16>
static int nvq_launch_signed(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                             hipStream_t st, const NvqSecond *s2 = nullptr) {
    // ring depths: what fits in 128 registers beside the activation fragments (48) and the accumulators
    const int rpb = nvq_signed_rpb(k, s2 ? s2->k.n_rowblocks : 0);
    if (k.nsteps <= 16) {  // one step per wave
        switch (rpb) {
        case 1: return nvq_launch_signed_as<XF16, 1, 1, true>(k, w, x, ldx, M, y, ldy, st, s2);
        case 2: return nvq_launch_signed_as<XF16, 2, 2, true>(k, w, x, ldx, M, y, ldy, st, s2);
        case 3: return nvq_launch_signed_as<XF16, 3, 3, true>(k, w, x, ldx, M, y, ldy, st, s2);
        case 4: return nvq_launch_signed_as<XF16, 4, 3, true>(k, w, x, ldx, M, y, ldy, st, s2);
        case 5: {
            // ring depths 1 .. 4 run within 7 % of each other on 17408 x 5120 (two is the fastest): MFQ_NVQ_RING for tuning
            static const int ring = tune_env("MFQ_NVQ_RING", 2);
            if (ring == 1) return nvq_launch_signed_as<XF16, 5, 1, true>(k, w, x, ldx, M, y, ldy, st, s2);
            if (ring == 3) return nvq_launch_signed_as<XF16, 5, 3, true>(k, w, x, ldx, M, y, ldy, st, s2);
            if (ring == 4) return nvq_launch_signed_as<XF16, 5, 4, true>(k, w, x, ldx, M, y, ldy, st, s2);
            return nvq_launch_signed_as<XF16, 5, 2, true>(k, w, x, ldx, M, y, ldy, st, s2);
        }
        default: return nvq_launch_signed_as<XF16, 6, 3, true>(k, w, x, ldx, M, y, ldy, st, s2);
        }
    }
    switch (rpb) {
    case 1: return nvq_launch_signed_as<XF16, 1, 1, false>(k, w, x, ldx, M, y, ldy, st, s2);
    case 2: return nvq_launch_signed_as<XF16, 2, 2, false>(k, w, x, ldx, M, y, ldy, st, s2);
    case 3: return nvq_launch_signed_as<XF16, 3, 3, false>(k, w, x, ldx, M, y, ldy, st, s2);
    case 4: return nvq_launch_signed_as<XF16, 4, 2, false>(k, w, x, ldx, M, y, ldy, st, s2);
    case 5: return nvq_launch_signed_as<XF16, 5, 1, false>(k, w, x, ldx, M, y, ldy, st, s2);
    default: return nvq_launch_signed_as<XF16, 6, 1, false>(k, w, x, ldx, M, y, ldy, st, s2);
    }
}

// One or two rows on nvq_bcast_kernel: the signed table fits the LDS, the rows can be fetched pair by pair (4-byte
// aligned, even K), at most three steps per wave (four would spill), and at least four waves (the table build spreads
// over them).
// Blocks of a launch over one tensor (nrb1 = 0) or two: every block gets the same number of consecutive row-blocks of
// one tensor, the fewest that leave one block per compute unit.  (Dealing the row-blocks out evenly over as many blocks
// as there are compute units measured slower on every shape tried, 17408 x 5120: 15.5 us against 15.0 -- the blocks
// that finish early do not shorten the launch, and each block more builds another table.)
static int nvq_bcast_split(int nrb0, int nrb1, int &b0, int &b1) {
    const int rpb = static_cast<int>(ceil_div(nrb0 + nrb1, gemv_cu_count()));
    b0 = static_cast<int>(ceil_div(nrb0, rpb));
    b1 = static_cast<int>(ceil_div(nrb1, rpb));
    return rpb;
}
static bool nvq_bcast_capable(const NvqK &k, const void *w, const void *x, int64_t ldx, int M, int more_rowblocks = 0) {
    static const int off = tune_env("MFQ_NVQ_BCAST_OFF", 0);
    int b0, b1;
    const int rpb = nvq_bcast_split(k.n_rowblocks, more_rowblocks, b0, b1);
    const int spw = static_cast<int>(ceil_div(k.nsteps, 16));
    return !off && M >= 1 && M <= 2 && static_cast<int64_t>(k.banks) * k.entries * 128 <= 131072 && rpb <= 8 && spw <= 3 &&
           ceil_div(k.nsteps, spw) >= 4 && k.neuron_len % 2 == 0 && (M == 1 || ldx % 2 == 0) &&
           (reinterpret_cast<uintptr_t>(x) & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 &&
           rpb * k.rowblock_bytes < (1ll << 31);
}
template <int XF16, int MB, int SPW>
static int nvq_launch_bcast_as(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                               hipStream_t st, const NvqSecond *second) {
    const int nwaves = static_cast<int>(ceil_div(k.nsteps, SPW));
    int blocks0, blocks1;
    const int rpb = nvq_bcast_split(k.n_rowblocks, second ? second->k.n_rowblocks : 0, blocks0, blocks1);
    NvqSecond s2{k, w, blocks0, 0};
    int blocks = blocks0;
    size_t ncb = static_cast<size_t>(k.banks) * k.entries;
    if (second) {
        s2 = *second;
        s2.blocks0 = blocks0;
        blocks += blocks1;
        if (static_cast<size_t>(s2.k.banks) * s2.k.entries > ncb) ncb = static_cast<size_t>(s2.k.banks) * s2.k.entries;
    }
    const size_t lds = ncb * 136 + 128 + static_cast<size_t>(rpb) * nwaves * MB * 64 + static_cast<size_t>(rpb) * 64;
    auto kern = nvq_bcast_kernel<XF16, MB, SPW>;
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds, "nvq_bcast")) return rc;
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(blocks), static_cast<unsigned>(ceil_div(M, MB))), dim3(64 * nwaves), lds,
                       st, k, w, x, ldx, M, y, ldy, rpb, s2);
    return check_launch("nvq_bcast");
}
template <int XF16>
static int nvq_launch_bcast(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                            hipStream_t st, const NvqSecond *s2 = nullptr) {
    const int spw = static_cast<int>(ceil_div(k.nsteps, 16));
#define MFQ_NVQ_BCAST(MB)                                                                                   \
    switch (spw) {                                                                                          \
    case 1: return nvq_launch_bcast_as<XF16, MB, 1>(k, w, x, ldx, M, y, ldy, st, s2);                       \
    case 2: return nvq_launch_bcast_as<XF16, MB, 2>(k, w, x, ldx, M, y, ldy, st, s2);                       \
    default: return nvq_launch_bcast_as<XF16, MB, 3>(k, w, x, ldx, M, y, ldy, st, s2);                      \
    }
    if (M == 1) { MFQ_NVQ_BCAST(1) }
    MFQ_NVQ_BCAST(2)
#undef MFQ_NVQ_BCAST
}

template <int XF16>
static int nvq_mfma_any(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                        hipStream_t st) {
    // two row-blocks per wave (they share the activation fragments) while that leaves about 1000 waves over all 16-row
    // tiles; four were slower on both config 3 shapes (1.2 vs 1.4 TB/s).  MFQ_NVQ_NB overrides for tuning.
    if (nvq_signed_capable(k, M)) return nvq_launch_signed<XF16>(k, w, x, ldx, M, y, ldy, st);
    const int64_t wpb = (k.nsteps < 8 ? k.nsteps : 8) * ceil_div(M, 16);  // waves of a block x 16-row tiles
    static const int env_nb = tune_env("MFQ_NVQ_NB", 0);
    if (env_nb == 4) return nvq_launch_mfma<XF16, 4>(k, w, x, ldx, M, y, ldy, st);
    if (env_nb == 1) return nvq_launch_mfma<XF16, 1>(k, w, x, ldx, M, y, ldy, st);
    if (env_nb == 2 || ceil_div(k.n_rowblocks, 2) * wpb >= 1024) return nvq_launch_mfma<XF16, 2>(k, w, x, ldx, M, y, ldy, st);
    return nvq_launch_mfma<XF16, 1>(k, w, x, ldx, M, y, ldy, st);
}

static void nvq_gemv_shape(const NvqK &k, int mb, int &spw, int &nwaves, size_t &lds_bytes) {
    int want = static_cast<int>(ceil_div(3 * gemv_target_waves(), k.n_rowblocks));
    if (want < 1) want = 1;
    if (want > 16) want = 16;
    if (want > k.nsteps) want = k.nsteps;
    spw = static_cast<int>(ceil_div(k.nsteps, want));
    nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    lds_bytes = (static_cast<size_t>(k.banks) * k.entries * 2 + 512 + 32) * 4 + gemv_lds_bytes(mb, spw, 24, nwaves);
}

template <int XF16, int MB>
static int nvq_launch(const NvqK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                      hipStream_t st) {
    int spw, nwaves;
    size_t lds;
    nvq_gemv_shape(k, MB, spw, nwaves, lds);
    MFQ_REQUIRE(lds <= 65536, MFQ_ERR_UNSUPPORTED, "nvq_gemv: neuron_len %d needs %zu bytes of LDS", k.neuron_len, lds);
    hipLaunchKernelGGL((nvq_gemv_kernel<XF16, MB>), dim3(k.n_rowblocks, static_cast<unsigned>(ceil_div(M, MB))),
                       dim3(64 * nwaves), lds, st, k, w, x, ldx, M, y, ldy, spw, PairSel{});
    return check_launch("nvq_gemv");
}

// the same kernel, one row per block, over the pairs of a MoE decode step (see PairSel)
template <int XF16>
static int nvq_launch_pairs(const NvqK &k, const uint16_t *x, int64_t ldx, int n_pairs, float *y, int64_t ldy, const PairSel &sel,
                            hipStream_t st) {
    int spw, nwaves;
    size_t lds;
    nvq_gemv_shape(k, 1, spw, nwaves, lds);
    MFQ_REQUIRE(lds <= 65536, MFQ_ERR_UNSUPPORTED, "nvq_gemv_pairs: neuron_len %d needs %zu bytes of LDS", k.neuron_len, lds);
    hipLaunchKernelGGL((nvq_gemv_kernel<XF16, 1>), dim3(k.n_rowblocks, static_cast<unsigned>(n_pairs)), dim3(64 * nwaves), lds, st, k,
                       static_cast<const uint8_t *>(nullptr), x, ldx, n_pairs, y, ldy, spw, sel);
    return check_launch("nvq_gemv_pairs");
}

static int nvq_gemv_any(const mfq_nvq_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                        float *y, int64_t ldy, hipStream_t st) {
    const NvqK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    if (nvq_bcast_capable(k, w, x, ldx, M))
        return x_dtype == MFQ_X_F16 ? nvq_launch_bcast<1>(k, w, xp, ldx, M, y, ldy, st)
                                    : nvq_launch_bcast<0>(k, w, xp, ldx, M, y, ldy, st);
    if (nvq_stream_capable(k) && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0)
        return x_dtype == MFQ_X_F16 ? nvq_mfma_any<1>(k, w, xp, ldx, M, y, ldy, st) : nvq_mfma_any<0>(k, w, xp, ldx, M, y, ldy, st);
    int mb = M >= 4 ? 4 : (M >= 2 ? 2 : 1);
    for (;;) {
        int spw, nwaves;
        size_t lds;
        nvq_gemv_shape(k, mb, spw, nwaves, lds);
        if (lds <= 65536 || mb == 1) break;
        mb >>= 1;
    }
    if (x_dtype == MFQ_X_F16) {
        if (mb == 4) return nvq_launch<1, 4>(k, w, xp, ldx, M, y, ldy, st);
        if (mb == 2) return nvq_launch<1, 2>(k, w, xp, ldx, M, y, ldy, st);
        return nvq_launch<1, 1>(k, w, xp, ldx, M, y, ldy, st);
    }
    if (mb == 4) return nvq_launch<0, 4>(k, w, xp, ldx, M, y, ldy, st);
    if (mb == 2) return nvq_launch<0, 2>(k, w, xp, ldx, M, y, ldy, st);
    return nvq_launch<0, 1>(k, w, xp, ldx, M, y, ldy, st);
}

int gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, const float *sa,
                const float *sb, float *y, int64_t ldy, hipStream_t st, float *part = nullptr);
float *dequant_gemm_part(float *wscale, int N, int K, int M);
int x_prep(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, hipStream_t st);
size_t dequant_gemm_workspace(int N, int K, int M);
void dequant_gemm_carve(void *ws, int N, int K, int M, uint16_t *&x16, float *&xscale, uint16_t *&w16, float *&wscale,
                        int &Kp);

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_nvq_plan(int index_bits, int banks, int out, int neuron_len, mfq_nvq_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvq_plan: null descriptor");
    MFQ_REQUIRE(index_bits == 8 || index_bits == 9, MFQ_ERR_UNSUPPORTED,
                "nvq_plan: only the D4 256/512-entry codebooks are on the accelerated path (index_bits=%d)", index_bits);
    MFQ_REQUIRE(banks == 1 || banks == 2 || banks == 4, MFQ_ERR_INVALID, "nvq_plan: banks=%d", banks);
    MFQ_REQUIRE(out > 0 && neuron_len > 0, MFQ_ERR_INVALID, "nvq_plan: empty tensor");
    d->index_bits = index_bits; d->entries = 1 << index_bits; d->banks = banks; d->out = out; d->neuron_len = neuron_len;
    d->ng = static_cast<int32_t>(ceil_div(neuron_len, 24));
    d->nvec = static_cast<int32_t>(ceil_div(neuron_len, 4));
    d->nsign = static_cast<int32_t>(ceil_div(neuron_len, 8));
    d->ngp = static_cast<int32_t>(ceil_div(d->ng, 16) * 16);
    d->nsteps = d->ngp / 16;
    d->n_rowblocks = static_cast<int32_t>(ceil_div(out, 16));
    d->step_bytes = 2048 + 1024;
    d->rowblock_bytes = d->step_bytes * d->nsteps;
    d->tables_off = d->rowblock_bytes * d->n_rowblocks;
    d->anchors_off = d->tables_off + 128 + static_cast<int64_t>(banks) * d->entries * 4;
    d->total_bytes = d->anchors_off + 16ll * d->n_rowblocks * 4;
    const int64_t o = out;
    d->payload_bytes = 2 * o + (o * d->ng * 4 + 7) / 8 + (o * d->nvec * index_bits + 7) / 8 + (o * d->nsign * 7 + 7) / 8 +
                       64 + static_cast<int64_t>(banks) * d->entries * 4;
    return MFQ_OK;
}

static int64_t nvq_stream_bytes(const mfq_nvq_desc *d) {
    const int64_t o = d->out;
    return 2 * o + (o * d->ng * 4 + 7) / 8 + (o * d->nvec * d->index_bits + 7) / 8 + (o * d->nsign * 7 + 7) / 8;
}

extern "C" int mfq_hip_nvq_repack(const mfq_nvq_desc *d, const void *payload, int64_t payload_bytes, void *weight,
                                  mfq_stream_t stream) {
    MFQ_REQUIRE(d && payload && weight, MFQ_ERR_INVALID, "nvq_repack: null argument");
    const int64_t cbb = static_cast<int64_t>(d->banks) * d->entries * 4;
    const int64_t expect = 64 + cbb + nvq_stream_bytes(d);
    MFQ_REQUIRE(payload_bytes == expect, MFQ_ERR_INVALID, "invalid NVQ-JSC blob tail: size=%lld, expected=%lld",
                static_cast<long long>(payload_bytes), static_cast<long long>(expect));
    const NvqK k = to_k(d);
    const uint8_t *p = static_cast<const uint8_t *>(payload);
    hipLaunchKernelGGL(nvq_repack_kernel, dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k, p + 64 + cbb,
                       nvq_stream_bytes(d), reinterpret_cast<const uint16_t *>(p + 4), p + 36,
                       reinterpret_cast<const int8_t *>(p + 64), static_cast<uint8_t *>(weight));
    return check_launch("nvq_repack");
}

extern "C" int mfq_hip_nvq_repack_plain(const mfq_nvq_desc *d, const void *payload, int64_t payload_bytes,
                                        const void *grid, void *weight, mfq_stream_t stream) {
    MFQ_REQUIRE(d && payload && weight && grid, MFQ_ERR_INVALID, "nvq_repack_plain: null argument");
    MFQ_REQUIRE(d->banks == 1, MFQ_ERR_INVALID, "nvq_repack_plain: plain NVQ has one codebook bank");
    MFQ_REQUIRE(payload_bytes == nvq_stream_bytes(d), MFQ_ERR_INVALID, "invalid NVQ blob tail: size=%lld, expected=%lld",
                static_cast<long long>(payload_bytes), static_cast<long long>(nvq_stream_bytes(d)));
    const NvqK k = to_k(d);
    hipLaunchKernelGGL(nvq_repack_kernel, dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(payload), payload_bytes, static_cast<const uint16_t *>(nullptr),
                       static_cast<const uint8_t *>(nullptr), static_cast<const int8_t *>(grid),
                       static_cast<uint8_t *>(weight));
    return check_launch("nvq_repack_plain");
}

extern "C" int mfq_hip_nvq_gemv_pairs(const mfq_nvq_desc *d, const void *const *expert_weights, const int32_t *expert_slot, int E,
                                      const void *x, int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                                      float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && expert_weights && expert_slot && x && ids && y, MFQ_ERR_INVALID, "nvq_gemv_pairs: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvq_gemv_pairs: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(T >= 0 && R >= 1 && E >= 1, MFQ_ERR_INVALID, "nvq_gemv_pairs: T=%d R=%d E=%d", T, R, E);
    MFQ_REQUIRE(static_cast<int64_t>(T) * R <= 65535, MFQ_ERR_UNSUPPORTED, "nvq_gemv_pairs: %lld pairs (at most 65535 per launch)",
                static_cast<long long>(T) * R);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nvq_gemv_pairs: ldx/ldy smaller than the tensor");
    if (T == 0) return MFQ_OK;
    const PairSel sel{ids, expert_slot, reinterpret_cast<const uint8_t *const *>(expert_weights), E, R, routed_input ? 1 : 0};
    const NvqK k = to_k(d);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    // the matrix-core kernel where the activation rows allow 16-byte reads; else the generic kernel
    static const int pairs_mfma = tune_env("MFQ_NVQ_PAIRS_MFMA", 1);
    if (pairs_mfma && nvq_stream_capable(k) && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        const bool two = ceil_div(k.n_rowblocks, 2) * (k.nsteps < 8 ? k.nsteps : 8) * T * R >= 1024;
        if (x_dtype == MFQ_X_F16)
            return two ? nvq_launch_mfma_pairs<1, 2>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream))
                       : nvq_launch_mfma_pairs<1, 1>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream));
        return two ? nvq_launch_mfma_pairs<0, 2>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream))
                   : nvq_launch_mfma_pairs<0, 1>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream));
    }
    return x_dtype == MFQ_X_F16 ? nvq_launch_pairs<1>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream))
                                : nvq_launch_pairs<0>(k, xp, ldx, T * R, y, ldy, sel, as_stream(stream));
}

extern "C" int mfq_hip_nvq_embedding(const mfq_nvq_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                                     int out_dtype, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight, MFQ_ERR_INVALID, "nvq_embedding: null argument");
    MFQ_REQUIRE(n_ids >= 0, MFQ_ERR_INVALID, "nvq_embedding: n_ids=%d", n_ids);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16 || out_dtype == MFQ_X_F32, MFQ_ERR_INVALID,
                "nvq_embedding: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(ldo >= d->neuron_len, MFQ_ERR_INVALID, "nvq_embedding: ldo %lld < neuron_len %d", static_cast<long long>(ldo),
                d->neuron_len);
    if (n_ids == 0) return MFQ_OK;
    MFQ_REQUIRE(ids && out, MFQ_ERR_INVALID, "nvq_embedding: null ids or output");
    const NvqK k = to_k(d);
    const size_t esize = out_dtype == MFQ_X_F32 ? 4 : 2;
    for (int n0 = 0; n0 < n_ids; n0 += 65535) {  // the grid's second dimension holds 65535 rows
        const int rows = n_ids - n0 < 65535 ? n_ids - n0 : 65535;
        hipLaunchKernelGGL(nvq_embedding_kernel, dim3(static_cast<unsigned>(ceil_div(k.nsteps, 4)), static_cast<unsigned>(rows)),
                           dim3(64), 0, as_stream(stream), k, static_cast<const uint8_t *>(weight), ids + n0,
                           static_cast<void *>(static_cast<uint8_t *>(out) + static_cast<size_t>(n0) * ldo * esize), out_dtype, ldo);
    }
    return check_launch("nvq_embedding");
}

extern "C" int mfq_hip_nvq_dequant_f32(const mfq_nvq_desc *d, const void *weight, float *w_out, int64_t ld,
                                       mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && w_out, MFQ_ERR_INVALID, "nvq_dequant_f32: null argument");
    MFQ_REQUIRE(ld >= d->neuron_len, MFQ_ERR_INVALID, "nvq_dequant_f32: ld smaller than neuron_len");
    const NvqK k = to_k(d);
    hipLaunchKernelGGL((nvq_dequant_kernel<float>), dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(weight), w_out, ld, static_cast<float *>(nullptr), 0);
    return check_launch("nvq_dequant_f32");
}

extern "C" int mfq_hip_nvq_gemv(const mfq_nvq_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                                float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nvq_gemv: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nvq_gemv: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvq_gemv: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nvq_gemv: ldx/ldy smaller than the tensor");
    return nvq_gemv_any(d, weight, x, x_dtype, ldx, M, y, ldy, as_stream(stream));
}

extern "C" int mfq_hip_nvq_gemv_multi2(const mfq_nvq_desc *d0, const void *weight0, const mfq_nvq_desc *d1, const void *weight1,
                                       const void *x, int x_dtype, int64_t ldx, int M, float *y, int64_t ldy,
                                       mfq_stream_t stream) {
    MFQ_REQUIRE(d0 && d1 && weight0 && weight1 && x && y, MFQ_ERR_INVALID, "nvq_gemv_multi2: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nvq_gemv_multi2: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvq_gemv_multi2: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(d0->neuron_len == d1->neuron_len, MFQ_ERR_INVALID,
                "NVQ multi-projection requires compatible formats and input layouts");
    MFQ_REQUIRE(ldx >= d0->neuron_len && ldy >= static_cast<int64_t>(d0->out) + d1->out, MFQ_ERR_INVALID,
                "nvq_gemv_multi2: ldx/ldy smaller than the tensors");
    const NvqK k0 = to_k(d0), k1 = to_k(d1);
    hipStream_t st = as_stream(stream);
    if (nvq_bcast_capable(k0, weight0, x, ldx, M, k1.n_rowblocks) && nvq_bcast_capable(k1, weight1, x, ldx, M, k0.n_rowblocks) &&
        nvq_bcast_capable(k0, weight0, x, ldx, M) && nvq_bcast_capable(k1, weight1, x, ldx, M)) {  // what each tensor's own call would run
        const NvqSecond s2{k1, static_cast<const uint8_t *>(weight1), 0, d0->out};
        const uint8_t *w0 = static_cast<const uint8_t *>(weight0);
        const uint16_t *xp = static_cast<const uint16_t *>(x);
        return x_dtype == MFQ_X_F16 ? nvq_launch_bcast<1>(k0, w0, xp, ldx, M, y, ldy, st, &s2)
                                    : nvq_launch_bcast<0>(k0, w0, xp, ldx, M, y, ldy, st, &s2);
    }
    const bool aligned = ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    if (aligned && nvq_stream_capable(k0) && nvq_stream_capable(k1) && nvq_signed_capable(k0, M, k1.n_rowblocks) &&
        nvq_signed_capable(k1, M, k0.n_rowblocks)) {
        const NvqSecond s2{k1, static_cast<const uint8_t *>(weight1), 0, d0->out};
        const uint8_t *w0 = static_cast<const uint8_t *>(weight0);
        const uint16_t *xp = static_cast<const uint16_t *>(x);
        return x_dtype == MFQ_X_F16 ? nvq_launch_signed<1>(k0, w0, xp, ldx, M, y, ldy, st, &s2)
                                    : nvq_launch_signed<0>(k0, w0, xp, ldx, M, y, ldy, st, &s2);
    }
    const int rc = nvq_gemv_any(d0, weight0, x, x_dtype, ldx, M, y, ldy, st);
    if (rc) return rc;
    return nvq_gemv_any(d1, weight1, x, x_dtype, ldx, M, y + d0->out, ldy, st);
}

// The reference keeps the D4 family on its GEMV up to M = 13; tensors the matrix-core streaming kernel
// takes stay on it up to kNvqStreamMaxM rows.
static constexpr int kNvqGemvMaxM = 13, kNvqStreamMaxM = 256;
static bool nvq_prefill_capable(const NvqK &k) {
    return nvq_stream_capable(k) && (static_cast<size_t>(k.banks) * k.entries * 2 + 544) * 4 <= 16384 &&
           (static_cast<size_t>(k.banks) * k.entries) % 2 == 0 && 2 * k.rowblock_bytes < (1ll << 31);
}
// Rows up to which re-streaming the weights (16 rows per pass) beats the prefill kernel, from a two-term model fitted
// to measurements (17408x5120 and 5120x17408): 64 rows of streaming cost about 6 us + 1.7 us per MB of payload, the
// prefill kernel a flat 38 us + 1 us per 1024 of K up to about a hundred rows (small grids are split over K).
static int nvq_stream_max(const mfq_nvq_desc *d, const NvqK &k) {
    static const int env = tune_env("MFQ_NVQ_STREAM_MAX_M", 0);
    if (env > 0) return env;
    if (!nvq_prefill_capable(k)) return kNvqStreamMaxM;
    const double t64 = 6.0 + 1.7e-6 * static_cast<double>(d->payload_bytes);
    const double tp = 38.0 + 1.0 * k.neuron_len / 1024.0;
    const int m = static_cast<int>(64.0 * tp / t64) / 16 * 16;
    return m < 32 ? 32 : (m > 512 ? 512 : m);
}
static bool nvq_streams(const mfq_nvq_desc *d, int M) {
    const NvqK k = to_k(d);
    return M <= kNvqGemvMaxM || (M <= nvq_stream_max(d, k) && nvq_stream_capable(k));
}
static size_t nvq_align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }
static int nvq_kp(int K) { return static_cast<int>(ceil_div(K, 32)) * 32; }

extern "C" size_t mfq_hip_nvq_gemm_workspace_bytes(const mfq_nvq_desc *d, int M) {
    if (!d || nvq_streams(d, M)) return 0;
    if (nvq_prefill_capable(to_k(d))) {  // x16 [M, Kp] | xscale [M] | partial results of a split over K
        const int splits = nvq_prefill_splits(to_k(d), M);
        return nvq_align256(static_cast<size_t>(M) * nvq_kp(d->neuron_len) * 2) + nvq_align256(static_cast<size_t>(M) * 4) +
               (splits > 1 ? static_cast<size_t>(splits) * M * d->out * 4 : 0);
    }
    return dequant_gemm_workspace(d->out, d->neuron_len, M);
}

extern "C" int mfq_hip_nvq_gemm(const mfq_nvq_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                                float *y, int64_t ldy, void *workspace, size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nvq_gemm: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nvq_gemm: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvq_gemm: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nvq_gemm: ldx/ldy smaller than the tensor");
    hipStream_t st = as_stream(stream);
    if (nvq_streams(d, M)) return nvq_gemv_any(d, weight, x, x_dtype, ldx, M, y, ldy, st);
    if (nvq_prefill_capable(to_k(d))) {
        const NvqK k = to_k(d);
        const int Kp = nvq_kp(k.neuron_len);
        const size_t need = mfq_hip_nvq_gemm_workspace_bytes(d, M);
        MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nvq_gemm: workspace %zu < %zu bytes",
                    workspace_bytes, need);
        uint16_t *x16 = static_cast<uint16_t *>(workspace);
        uint8_t *p = static_cast<uint8_t *>(workspace) + nvq_align256(static_cast<size_t>(M) * Kp * 2);
        float *xscale = reinterpret_cast<float *>(p);
        p += nvq_align256(static_cast<size_t>(M) * 4);
        float *part = nvq_prefill_splits(k, M) > 1 ? reinterpret_cast<float *>(p) : nullptr;
        const int rc = x_prep(x, x_dtype, ldx, M, k.neuron_len, Kp, x16, xscale, st);
        if (rc) return rc;
        return nvq_prefill(k, static_cast<const uint8_t *>(weight), x16, Kp, xscale, M, y, ldy, part, st);
    }
    const size_t need = dequant_gemm_workspace(d->out, d->neuron_len, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nvq_gemm: workspace %zu < %zu bytes",
                workspace_bytes, need);
    uint16_t *x16, *w16;
    float *xscale, *wscale;
    int Kp;
    dequant_gemm_carve(workspace, d->out, d->neuron_len, M, x16, xscale, w16, wscale, Kp);
    int rc = x_prep(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, st);
    if (rc) return rc;
    const NvqK k = to_k(d);
    hipLaunchKernelGGL((nvq_dequant_kernel<uint16_t>), dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, st, k,
                       static_cast<const uint8_t *>(weight), w16, static_cast<int64_t>(Kp), wscale, Kp);
    rc = check_launch("nvq_dequant_f16");
    if (rc) return rc;
    return gemm_f16_nt(x16, Kp, w16, Kp, M, d->out, Kp, xscale, wscale, y, ldy, st, dequant_gemm_part(wscale, d->out, d->neuron_len, M));
}
