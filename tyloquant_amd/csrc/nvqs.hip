// NVQ payloads read in place from their tensor-wide bit streams: the E8 family (8-dimensional vectors, 256 / 1024 /
// 4096 entries, plain or JSC, parity or index-parity signs) and the 1024-entry D4 codebook, which the 16-bit fields
// of the lane-major D4 layout (nvq.hip) cannot hold.  The device weight is the payload itself with its tables
// widened: no re-layout, every field is fetched by bit offset.  A wave owns a neuron, its lanes the 8-weight sign
// blocks of the row, so the three streams of a neuron are read as consecutive bytes.
// The 1-bit families ride on the same machinery: NVQ1-L / NVQ1-S (kind 1: ternary 8-dimensional codebooks, an integer
// relative scale and a delta sign per group, the sign also choosing NVQ1-S's bank) and NPQ0-L / NPQ0-S (kind 2: two
// 4-dimensional int8 sub-codebooks and a relative scale chosen by the group's state).
#include <type_traits>

#include "common.hpp"
#include "gemv_common.hpp"
#include "tune.hpp"

namespace mfq {

struct NvqsK {
    int vs, ib, entries, banks, index_parity;
    int out, neuron_len, ng, nvec, nsign;
    int64_t tables_off, anchors_off, state_off, index_off, sign_off;
    int64_t state_bytes, index_bytes, sign_bytes;
    int kind, sbits, cb_bytes;  // kind 0: sign-stream NVQ; 1: ternary + delta (sign_off = the delta-sign stream); 2: product;
                                // 3: product with a table pool (sign_off = one bank id byte per neuron and 96 weights)
    float delta, magmax;        // magmax: bound of |magnitude| for the fp16 row scaling
    int nbank, nsuper, bank_bytes;  // kind 3: tables of the pool, bank ids per neuron, codebook bytes of one table
    int row0, nrows;            // the neurons a launch works on (an expert of an expert-shaped tensor)
};

static NvqsK to_k(const mfq_nvqs_desc *d) {
    NvqsK k;
    k.vs = d->vector_size; k.ib = d->index_bits; k.entries = d->entries; k.banks = d->banks; k.index_parity = d->index_parity;
    k.out = d->out; k.neuron_len = d->neuron_len; k.ng = d->ng; k.nvec = d->nvec; k.nsign = d->nsign;
    k.tables_off = d->tables_off; k.anchors_off = d->anchors_off; k.state_off = d->state_off; k.index_off = d->index_off;
    k.sign_off = d->sign_off;
    k.kind = d->kind; k.sbits = d->state_bits; k.cb_bytes = d->cb_bytes; k.delta = d->delta;
    k.magmax = d->kind == 1 ? 2.f : 127.f;
    k.state_bytes = (static_cast<int64_t>(d->out) * d->ng * d->state_bits + 7) / 8;
    k.index_bytes = (static_cast<int64_t>(d->out) * d->nvec * d->index_bits + 7) / 8;
    k.sign_bytes = d->kind == 0 ? (static_cast<int64_t>(d->out) * d->nsign * 7 + 7) / 8
                 : d->kind == 1 ? (static_cast<int64_t>(d->out) * d->ng + 7) / 8
                 : d->kind == 3 ? static_cast<int64_t>(d->out) * d->nsuper : 0;
    k.nbank = d->nbank; k.nsuper = d->nsuper; k.bank_bytes = d->nbank > 0 ? (d->cb_bytes - 32 * d->nbank) / d->nbank : 0;
    k.row0 = 0; k.nrows = d->out;
    return k;
}

// tables: float lut[16] | uint32 bank_for_state[16] | int8 codebooks[banks * entries * vs]
__device__ __forceinline__ const float *nvqs_lut(const NvqsK &k, const uint8_t *w) {
    return reinterpret_cast<const float *>(w + k.tables_off);
}

// Field of `bits` (<= 12) bits at bit position `bit` of a stream that is followed by at least three readable bytes.
__device__ __forceinline__ uint32_t stream_bits(const uint8_t *s, int64_t bit, int bits) {
    const int64_t b = bit >> 3;
    const uint32_t v = s[b] | (static_cast<uint32_t>(s[b + 1]) << 8) | (static_cast<uint32_t>(s[b + 2]) << 16);
    return (v >> (bit & 7)) & ((1u << bits) - 1u);
}

// The eight weights of sign block sb of neuron n, as signed integer magnitudes, and the scale of their group:
// w[i] = f32(mag[i]) * fl(anchor * lut[state])  (mfq/quantize/nvq_jsc.py:1053-1079; the plain formats are the case
// lut[s] = s, one bank: mfq/quantize/nvq_quant.py:608-626).  Sign bit 7 of a block is the parity of its seven stored
// bits, flipped by bit 7 of the vector's index in the index-parity mode (E8 only).
struct NvqsBlock {
    float mag[8];
    float scale;
};
template <class CB>
__device__ __forceinline__ NvqsBlock nvqs_block(const NvqsK &k, const uint8_t *w, const float *lut, const uint32_t *bfs,
                                                CB cb, float anchor, int n, int sb) {
    const uint8_t *st_s = w + k.state_off, *ix_s = w + k.index_off, *sg_s = w + k.sign_off;
    const int g = sb / 3;  // groups of 24 weights = three 8-weight blocks
    const uint32_t state = stream_bits(st_s, (static_cast<int64_t>(n) * k.ng + g) * k.sbits, k.sbits);
    NvqsBlock b;
    b.scale = __fmul_rn(anchor, lut[state]);
    if (k.kind == 1) {
        // w = fl(anchor * sub_scale) * (code + delta): delta = -d / +d by the group's sign bit, which with two banks also
        // names the bank (mfq/quantize/nvq1_l_quant.py:384-414, nvq1_s_quant.py:142-174); code + delta is exact
        const uint32_t neg = stream_bits(sg_s, static_cast<int64_t>(n) * k.ng + g, 1);
        const uint32_t idx = sb < k.nvec ? stream_bits(ix_s, (static_cast<int64_t>(n) * k.nvec + sb) * k.ib, k.ib) : 0u;
        const int64_t e = (static_cast<int64_t>(k.banks == 2 ? neg : 0u) * k.entries + idx) * 8;
        const float dl = neg ? -k.delta : k.delta;
#pragma unroll
        for (int i = 0; i < 8; ++i) b.mag[i] = static_cast<float>(cb(e + i)) + dl;
        return b;
    }
    if (k.kind == 2) {
        // a vector = first[state][index & 7] | second[state][index >> 3], four int8 weights each
        // (mfq/quantize/npq0_l.py:766-790, npq0_s.py:812-836); banks = states, entries = second sub-codebook entries
        const uint32_t idx = sb < k.nvec ? stream_bits(ix_s, (static_cast<int64_t>(n) * k.nvec + sb) * k.ib, k.ib) : 0u;
        const int64_t e1 = (static_cast<int64_t>(state) * 8 + (idx & 7u)) * 4;
        const int64_t e2 = static_cast<int64_t>(k.banks) * 32 + (static_cast<int64_t>(state) * k.entries + (idx >> 3)) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            b.mag[i] = static_cast<float>(cb(e1 + i));
            b.mag[4 + i] = static_cast<float>(cb(e2 + i));
        }
        return b;
    }
    if (k.kind == 3) {
        // the product form with a pool of tables: the neuron's bank id for these 96 weights picks scale LUT and
        // sub-codebooks (dequantize_nepq, mfq/formats/nepq.py:492-521); tables: per bank first | second, then the LUTs
        const uint32_t pb = sg_s[static_cast<int64_t>(n) * k.nsuper + g / 4];
        const float *lut3 = reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(lut) + 128 +
                                                            static_cast<int64_t>(k.nbank) * k.bank_bytes);
        b.scale = __fmul_rn(anchor, lut3[pb * 8 + state]);
        const uint32_t idx = sb < k.nvec ? stream_bits(ix_s, (static_cast<int64_t>(n) * k.nvec + sb) * k.ib, k.ib) : 0u;
        const int64_t base = static_cast<int64_t>(pb) * k.bank_bytes;
        const int64_t e1 = base + (static_cast<int64_t>(state) * 8 + (idx & 7u)) * 4;
        const int64_t e2 = base + static_cast<int64_t>(k.banks) * 32 + (static_cast<int64_t>(state) * k.entries + (idx >> 3)) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            b.mag[i] = static_cast<float>(cb(e1 + i));
            b.mag[4 + i] = static_cast<float>(cb(e2 + i));
        }
        return b;
    }
    const uint32_t mask = stream_bits(sg_s, (static_cast<int64_t>(n) * k.nsign + sb) * 7, 7);
    const uint32_t bank = bfs[state];
    uint32_t last = __popc(mask) & 1u;
    if (k.vs == 8) {
        const uint32_t idx = stream_bits(ix_s, (static_cast<int64_t>(n) * k.nvec + sb) * k.ib, k.ib);
        if (k.index_parity) last ^= (idx >> 7) & 1u;
        const int64_t e = (static_cast<int64_t>(bank) * k.entries + idx) * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) b.mag[i] = static_cast<float>(cb(e + i));
    } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int v = 2 * sb + h;
            const uint32_t idx = v < k.nvec ? stream_bits(ix_s, (static_cast<int64_t>(n) * k.nvec + v) * k.ib, k.ib) : 0u;
            const int64_t e = (static_cast<int64_t>(bank) * k.entries + idx) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) b.mag[4 * h + i] = static_cast<float>(cb(e + i));
        }
    }
    const uint32_t neg = mask | (last << 7);
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if ((neg >> i) & 1u) b.mag[i] = -b.mag[i];
    return b;
}

// ---- load: widen the tables, copy the streams ------------------------------------------------------------------
// body: JSC = 64-byte header (fp16 lut at +4, u8 bank map at +36), int8 banks, then the plain layout; plain =
// fp16 anchors, 4-bit state / sub-scale stream, index stream, 7-bit sign stream.
__global__ __launch_bounds__(256) void nvqs_repack_kernel(NvqsK k, const uint8_t *__restrict__ body, int jsc,
                                                          const int8_t *__restrict__ grid, uint8_t *__restrict__ dst) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, nthreads = static_cast<int64_t>(gridDim.x) * 256;
    float *lut = reinterpret_cast<float *>(dst + k.tables_off);
    uint32_t *bfs = reinterpret_cast<uint32_t *>(lut + 16);
    int8_t *cb = reinterpret_cast<int8_t *>(bfs + 16);
    const int64_t ncb = static_cast<int64_t>(k.banks) * k.entries * k.vs;
    const uint8_t *streams = body + (jsc ? 64 + ncb : 0);
    if (tid < 16) {
        if (jsc) {
            lut[tid] = f16_to_f32(static_cast<uint16_t>(body[4 + 2 * tid] | (body[5 + 2 * tid] << 8)));
            bfs[tid] = body[36 + tid];
        } else {
            lut[tid] = static_cast<float>(tid);  // the state is the integer relative scale
            bfs[tid] = 0u;
        }
    }
    for (int64_t i = tid; i < ncb; i += nthreads) cb[i] = jsc ? static_cast<int8_t>(body[64 + i]) : grid[i];
    float *anchors = reinterpret_cast<float *>(dst + k.anchors_off);
    for (int64_t i = tid; i < k.out; i += nthreads)
        anchors[i] = f16_to_f32(static_cast<uint16_t>(streams[2 * i] | (streams[2 * i + 1] << 8)));
    const uint8_t *st = streams + 2 * static_cast<int64_t>(k.out), *ix = st + k.state_bytes, *sg = ix + k.index_bytes;
    for (int64_t i = tid; i < k.state_bytes + 4; i += nthreads) dst[k.state_off + i] = i < k.state_bytes ? st[i] : 0;
    for (int64_t i = tid; i < k.index_bytes + 4; i += nthreads) dst[k.index_off + i] = i < k.index_bytes ? ix[i] : 0;
    for (int64_t i = tid; i < k.sign_bytes + 4; i += nthreads) dst[k.sign_off + i] = i < k.sign_bytes ? sg[i] : 0;
}

// The 1-bit families.  body: [tables] | fp16 anchors | state stream | index stream | [delta-sign stream].  Tables:
// kind 1 -- packed ternary entries (2 bits per digit, digit = code + 1, a uint16 per entry) from the body when
// table_in_body, else from `grid` (the built-in 2048-entry grid); kind 2 -- a 64-byte header with the fp16 scale LUT at
// byte 8, then the int8 sub-codebooks, copied as they are.
__global__ __launch_bounds__(256) void nvqs_repack_lowbit_kernel(NvqsK k, const uint8_t *__restrict__ body, int table_in_body,
                                                                 const uint16_t *__restrict__ grid, uint8_t *__restrict__ dst) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, nthreads = static_cast<int64_t>(gridDim.x) * 256;
    float *lut = reinterpret_cast<float *>(dst + k.tables_off);
    uint32_t *bfs = reinterpret_cast<uint32_t *>(lut + 16);
    int8_t *cb = reinterpret_cast<int8_t *>(bfs + 16);
    int64_t table_bytes = 0;
    if (k.kind == 1) {
        const int64_t nent = static_cast<int64_t>(k.banks) * k.entries;
        table_bytes = table_in_body ? 2 * nent : 0;
        if (tid < 16) { lut[tid] = static_cast<float>(tid); bfs[tid] = 0u; }
        for (int64_t i = tid; i < nent * 8; i += nthreads) {
            const int64_t e = i >> 3;
            const uint32_t enc = table_in_body ? (body[2 * e] | (static_cast<uint32_t>(body[2 * e + 1]) << 8)) : grid[e];
            cb[i] = static_cast<int8_t>(static_cast<int>((enc >> (2 * (i & 7))) & 3u) - 1);
        }
    } else if (k.kind == 2) {
        table_bytes = 64 + k.cb_bytes;
        if (tid < 16) {
            lut[tid] = tid < k.banks ? f16_to_f32(static_cast<uint16_t>(body[8 + 2 * tid] | (body[9 + 2 * tid] << 8))) : 0.f;
            bfs[tid] = 0u;
        }
        for (int64_t i = tid; i < k.cb_bytes; i += nthreads) cb[i] = static_cast<int8_t>(body[64 + i]);
    } else {
        // a pool of nbank tables of 64 + bank_bytes bytes each: the sub-codebooks of all banks, then eight LUT floats per
        // bank; the 16-entry LUT in front holds the largest scale of any bank per state (the fp16 path's row bound)
        const int64_t tb = 64 + k.bank_bytes;
        table_bytes = k.nbank * tb;
        float *lut3 = reinterpret_cast<float *>(cb + static_cast<int64_t>(k.nbank) * k.bank_bytes);
        if (tid < 16) {
            float m = 0.f;
            for (int pb = 0; pb < k.nbank && tid < k.banks; ++pb)
                m = fmaxf(m, f16_to_f32(static_cast<uint16_t>(body[pb * tb + 8 + 2 * tid] | (body[pb * tb + 9 + 2 * tid] << 8))));
            lut[tid] = m;
            bfs[tid] = 0u;
        }
        for (int64_t i = tid; i < static_cast<int64_t>(k.nbank) * 8; i += nthreads) {
            const int64_t pb = i >> 3, st_ = i & 7;
            lut3[i] = st_ < k.banks ? f16_to_f32(static_cast<uint16_t>(body[pb * tb + 8 + 2 * st_] | (body[pb * tb + 9 + 2 * st_] << 8))) : 0.f;
        }
        for (int64_t i = tid; i < static_cast<int64_t>(k.nbank) * k.bank_bytes; i += nthreads)
            cb[i] = static_cast<int8_t>(body[(i / k.bank_bytes) * tb + 64 + i % k.bank_bytes]);
    }
    const uint8_t *streams = body + table_bytes;
    float *anchors = reinterpret_cast<float *>(dst + k.anchors_off);
    for (int64_t i = tid; i < k.out; i += nthreads)
        anchors[i] = f16_to_f32(static_cast<uint16_t>(streams[2 * i] | (streams[2 * i + 1] << 8)));
    const uint8_t *st = streams + 2 * static_cast<int64_t>(k.out), *ix = st + k.state_bytes, *sg = ix + k.index_bytes;
    for (int64_t i = tid; i < k.state_bytes + 4; i += nthreads) dst[k.state_off + i] = i < k.state_bytes ? st[i] : 0;
    for (int64_t i = tid; i < k.index_bytes + 4; i += nthreads) dst[k.index_off + i] = i < k.index_bytes ? ix[i] : 0;
    for (int64_t i = tid; i < k.sign_bytes + 4; i += nthreads) dst[k.sign_off + i] = i < k.sign_bytes ? sg[i] : 0;
}

// ---- dequant -------------------------------------------------------------------------------------------------------
// One thread per (neuron, sign block).  OutT = float: the bit-exact dequantizer.  OutT = uint16_t: fp16 rows scaled by a
// power of two per neuron (rowscale receives its reciprocal), zero-padded to kpad columns, for the fp16 GEMM.
template <typename OutT>
__global__ __launch_bounds__(256) void nvqs_dequant_kernel(NvqsK k, const uint8_t *__restrict__ w, OutT *__restrict__ outp,
                                                           int64_t ld, float *__restrict__ rowscale, int kpad) {
    const int row = blockIdx.y, n = k.row0 + row;  // output row, neuron
    const float *lut = nvqs_lut(k, w);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cbp = reinterpret_cast<const int8_t *>(bfs + 16);
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[n];
    float inv = 1.f;
    if constexpr (sizeof(OutT) == 2) {
        float lmax = 0.f;
        for (int i = 0; i < 16; ++i) lmax = fmaxf(lmax, lut[i]);
        const float bound = anchor * lmax * k.magmax;
        int e = 0;
        if (bound > 0.f) frexpf(bound, &e);
        inv = ldexpf(1.f, 12 - e);
        if (blockIdx.x == 0 && threadIdx.x == 0) rowscale[row] = ldexpf(1.f, e - 12);
        for (int col = k.nsign * 8 + blockIdx.x * 256 + threadIdx.x; col < kpad; col += gridDim.x * 256) outp[row * ld + col] = 0;
    }
    const int sb = blockIdx.x * 256 + threadIdx.x;
    if (sb >= k.nsign) return;
    const NvqsBlock b = nvqs_block(k, w, lut, bfs, [&](int64_t i) { return cbp[i]; }, anchor, n, sb);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int col = sb * 8 + i;
        const float v = __fmul_rn(b.mag[i], b.scale);
        if constexpr (sizeof(OutT) == 2) {
            if (col < kpad) outp[row * ld + col] = col < k.neuron_len ? f32_to_f16_rne(v * inv) : uint16_t(0);
        } else {
            if (col < k.neuron_len) outp[row * ld + col] = v;
        }
    }
}

// Embedding rows: one thread per (id, sign block); row n of the output = neuron ids[n] of the bit-exact dequantizer,
// rounded once more to the output type; ids outside [0, out) give a row of zeros.
__global__ __launch_bounds__(256) void nvqs_embedding_kernel(NvqsK k, const uint8_t *__restrict__ w,
                                                             const int64_t *__restrict__ ids, void *__restrict__ outp,
                                                             int out_dtype, int64_t ldo) {
    const int sb = blockIdx.x * 256 + threadIdx.x;
    if (sb >= k.nsign) return;
    const int row = blockIdx.y;
    const int64_t tok = ids[row];
    const int64_t at = static_cast<int64_t>(row) * ldo + sb * 8;
    const int ncol = min(8, k.neuron_len - sb * 8);
    if (tok < 0 || tok >= k.out) {
        for (int i = 0; i < ncol; ++i) store_rounded(outp, at + i, 0.f, out_dtype);
        return;
    }
    const int n = static_cast<int>(tok);
    const float *lut = nvqs_lut(k, w);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cbp = reinterpret_cast<const int8_t *>(bfs + 16);
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[n];
    const NvqsBlock b = nvqs_block(k, w, lut, bfs, [&](int64_t i) { return cbp[i]; }, anchor, n, sb);
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (i < ncol) store_rounded(outp, at + i, __fmul_rn(b.mag[i], b.scale), out_dtype);
}

// ---- GEMV: a wave per neuron, MB rows per pass --------------------------------------------------------------------
// LDS (CB_LDS): the int8 codebooks.  The activation rows are read as 16-byte chunks straight from global memory (they
// stay in L2: every wave of the grid reads the same rows).
template <int XF16, int MB, bool CB_LDS>
__global__ __launch_bounds__(256) void nvqs_gemv_kernel(NvqsK k, const uint8_t *__restrict__ w_in,
                                                        const uint16_t *__restrict__ x_in, int64_t ldx, int M_in,
                                                        float *__restrict__ y_in, int64_t ldy, PairSel sel) {
    extern __shared__ __attribute__((aligned(16))) int8_t cbl[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint8_t *w = w_in;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = blockIdx.y * MB;
    if (sel.ids) {  // a pair of a MoE decode step: one row, the expert's own tensor
        const uint16_t *xr[1];
        float *yr[1];
        int local;
        if (!select_rows<1>(sel, w, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        if (!sel.weights) k.row0 = local * k.nrows;  // the experts are row ranges of one tensor
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    const float *lut = nvqs_lut(k, w);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cbp = reinterpret_cast<const int8_t *>(bfs + 16);
    if constexpr (CB_LDS) {
        const int ncb = k.cb_bytes;
        table_to_lds(reinterpret_cast<uint32_t *>(cbl), reinterpret_cast<const uint32_t *>(cbp), ncb / 4, threadIdx.x, blockDim.x);
        __syncthreads();
    }
    const int row = blockIdx.x * (blockDim.x >> 6) + wave;
    if (row >= k.nrows) return;
    const int n = k.row0 + row;
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[n];
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.f;
    const bool vec = ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    for (int sb = lane; sb < k.nsign; sb += 64) {
        NvqsBlock b;
        if constexpr (CB_LDS) b = nvqs_block(k, w, lut, bfs, [&](int64_t i) { return cbl[i]; }, anchor, n, sb);
        else b = nvqs_block(k, w, lut, bfs, [&](int64_t i) { return cbp[i]; }, anchor, n, sb);
        float wv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) wv[i] = sb * 8 + i < k.neuron_len ? __fmul_rn(b.mag[i], b.scale) : 0.f;
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            if (m0 + m >= M) break;
            const uint16_t *xr = x + static_cast<int64_t>(m0 + m) * ldx + sb * 8;
            uint16_t xv[8];
            if (vec && sb * 8 + 8 <= k.neuron_len) {
                const u32x4_t q = *reinterpret_cast<const u32x4_t *>(xr);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    xv[2 * t] = static_cast<uint16_t>(q[t] & 0xffffu);
                    xv[2 * t + 1] = static_cast<uint16_t>(q[t] >> 16);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[i] = sb * 8 + i < k.neuron_len ? xr[i] : uint16_t(0);
            }
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) s = fmaf(wv[i], x_to_f32<XF16>(xv[i]), s);
            acc[m] += s;
        }
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float s = acc[m];
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if (lane == 0 && m0 + m < M) y[static_cast<int64_t>(m0 + m) * ldy + row] = s;
    }
}

// ---- the sign-stream codebooks whose tables fit the LDS (E8: NVQ2, NVQ2J, NVQ2J-L, one bank of NVQ2J-XL; D4: NVQ3J-L): one
// ---- to eight rows per pass
// The generic kernel above asks for every field of every block by itself -- a few bytes per request, some fifty requests
// per kilobyte of payload, where a compute unit keeps about 64 in flight -- and decodes a weight at a time.  Here a wave
// copies the three stream ranges of its neurons (consecutive neurons: consecutive bits) into LDS in 16-byte pieces, one
// to three requests per range, and a lane takes a group of 24 weights at a time: its 4-bit state, 21 sign bits and
// three index bytes are funnel shifts over aligned LDS dwords; a block of eight weights is one 16-byte read of the
// entry out of a table of the activations' type (bf16 or fp16: the int8 magnitudes are exact in both), one 16-byte read
// of the eight sign bits' XOR pattern, four XORs and four packed dot products against the row's 16 bytes in LDS;
// the group's scale multiplies the sum of its 24 products in fp32.  bf16 activations are used as they are
// (v_dot2c_f32_bf16): no conversion and no range to mind.
// LDS: [entries: banks * entries * 16][sign patterns: 256 * 16][states: 16 x {anchor-free scale f32, entry base}]
//      [rows: MB * kp * 2][per wave: index | sign | state ranges]
template <int XF16>
__device__ __forceinline__ float e8_dot8(u32x4_t wv, u32x4_t xv, float acc) {
    // (the elements go through dot2's by-value parameters: a bit cast applied to a vector element directly reads element 0)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc = dot2<XF16>(wv[t], xv[t], acc);
    return acc;
}
// int8 pair -> pair of the activations' type (exact)
template <int XF16>
__device__ __forceinline__ uint32_t e8_pair(int a, int b) {
    if constexpr (XF16) {
        return static_cast<uint32_t>(f32_to_f16_rne(static_cast<float>(a))) | (static_cast<uint32_t>(f32_to_f16_rne(static_cast<float>(b))) << 16);
    } else {
        return (__float_as_uint(static_cast<float>(a)) >> 16) | (__float_as_uint(static_cast<float>(b)) & 0xffff0000u);
    }
}
constexpr int kE8Waves = 16;
// bytes staged for a bit range of `bits` bits that starts anywhere in its first 16 bytes, with room for a field's two dwords
__host__ __device__ inline uint32_t nvqs_e8_range_bytes(int64_t bits) { return static_cast<uint32_t>((16 + (bits + 7) / 8 + 8 + 15) / 16 * 16); }
struct E8Shape {
    int npw;            // consecutive neurons per wave
    int kp;             // staged elements of a row: whole groups of 24
    uint32_t cap[3];    // LDS bytes of a wave's index / sign / state range
    uint32_t wave_bytes, lds_bytes;
};
template <int XF16, int MB>
__global__ __launch_bounds__(64 * kE8Waves) void nvqs_e8_kernel(NvqsK k, const uint8_t *__restrict__ w_in,
                                                                const uint16_t *__restrict__ x_in, int64_t ldx, int M_in,
                                                                float *__restrict__ y_in, int64_t ldy, E8Shape sh, PairSel sel) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds32[];
    typedef __attribute__((address_space(3))) const u32x4_t *lds_u32x4_ptr;
    typedef __attribute__((address_space(3))) const u32x2_t *lds_u32x2_ptr;
    typedef __attribute__((address_space(3))) const uint32_t *lds_u32_ptr;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint8_t *w = w_in;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = static_cast<int>(blockIdx.y) * MB;
    if (sel.ids) {
        const uint16_t *xr[1];
        float *yr[1];
        int local;
        if (!select_rows<1>(sel, w, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        if (!sel.weights) k.row0 = local * k.nrows;
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    // table entries of vs int8 values (kinds 2 and 3: pairs of the 4-value entries of the sub-codebooks, of every table of the pool)
    const int ncb = k.kind == 2 ? k.cb_bytes / k.vs : (k.kind == 3 ? k.nbank * k.bank_bytes / k.vs : k.banks * k.entries);
    uint8_t *lds8 = reinterpret_cast<uint8_t *>(lds32);
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)lds8));
    const uint32_t esz = static_cast<uint32_t>(k.vs) * 2u;  // bytes of a table entry: 8 (E8) or 4 (D4) values of the activations' type
    // (kind 3 keeps the pool's scale tables, eight floats per table, behind the state table)
    const uint32_t sgn_off = static_cast<uint32_t>(ncb) * esz, stab_off = sgn_off + 4096u, lut3_off = stab_off + 128u,
                   x_off = lut3_off + (k.kind == 3 ? static_cast<uint32_t>(k.nbank) * 32u : 0u);
    const uint32_t row_bytes = static_cast<uint32_t>(sh.kp) * 2u;
    const uint32_t wave_off = x_off + MB * row_bytes + static_cast<uint32_t>(wave) * sh.wave_bytes;

    // ---- the wave's stream ranges: requested first, parked after the tables are written ----------------------------------
    const int row_first = (static_cast<int>(blockIdx.x) * kE8Waves + wave) * sh.npw;  // of the launch's rows
    const int nn = max(0, min(sh.npw, k.nrows - row_first));
    const int64_t n0 = k.row0 + row_first;
    // bit ranges [n0 * per, (n0 + nn) * per) of the three streams, read from 16-byte aligned addresses
    // bits per neuron of the three ranges: indices, the sign stream (kind 0: 7 per block; kind 1: a delta sign per group;
    // kind 2: none; kind 3: a table id byte per 96 weights) and the states
    const uint32_t per1 = k.kind == 0 ? static_cast<uint32_t>(k.nsign) * 7u
                        : (k.kind == 1 ? static_cast<uint32_t>(k.ng) : (k.kind == 3 ? static_cast<uint32_t>(k.nsuper) * 8u : 0u));
    const uint32_t per2 = static_cast<uint32_t>(k.ng) * static_cast<uint32_t>(k.sbits);
    const int64_t bit0[3] = {n0 * k.nvec * k.ib, n0 * static_cast<int64_t>(per1), n0 * static_cast<int64_t>(per2)};
    const int64_t region[3] = {k.index_off, k.sign_off, k.state_off};
    const int64_t region_bytes[3] = {k.index_bytes + 4, k.sign_bytes + 4, k.state_bytes + 4};
    uint32_t shift[3];   // bits between the staged range's first bit and the first bit of neuron n0
    u32x4_t piece[3][2];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const int64_t a0 = (bit0[r] >> 3) & ~static_cast<int64_t>(15);
        shift[r] = static_cast<uint32_t>(bit0[r] - a0 * 8);
        // bytes of the region from a0 on.  A wave past the launch's last neuron has none: its window must be empty, not a
        // negative length wrapped to 4 GiB, inside which the "no data" offset would be a real address
        const int64_t left = nn > 0 ? region_bytes[r] - a0 : 0;
        const __amdgpu_buffer_rsrc_t win = wave_window(w + region[r] + (nn > 0 ? a0 : 0),
                                                       static_cast<uint32_t>(left <= 0 ? 0 : (left < (1ll << 31) ? left : (1ll << 31))));
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t off = static_cast<uint32_t>(t * 64 + lane) * 16u;
            piece[r][t] = __builtin_amdgcn_raw_buffer_load_b128(win, nn > 0 && off < sh.cap[r] ? off : kNoStep, 0, 2);
        }
    }
    // ---- tables and rows (all waves): every request first, then the conversions and the LDS writes ----------------------
    const float *lut = nvqs_lut(k, w);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cbp = reinterpret_cast<const int8_t *>(bfs + 16);
    const int chunks = sh.kp / 8;
    const bool vec = ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    auto x_chunk = [&](int c) -> u32x4_t {  // chunk c = (row, 8 elements) of the staged rows, zeros past M and K
        const int m = c / chunks, j = c - m * chunks;
        u32x4_t v = {0u, 0u, 0u, 0u};
        if (c < MB * chunks && m0 + m < M) {
            const uint16_t *xr = x + static_cast<int64_t>(m0 + m) * ldx + j * 8;
            if (vec && j * 8 + 8 <= k.neuron_len) {
                v = *reinterpret_cast<const u32x4_t *>(xr);
            } else {
                uint32_t h[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = j * 8 + i < k.neuron_len ? xr[i] : 0u;
                v = u32x4_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
            }
        }
        return v;
    };
    auto x_park = [&](int c, u32x4_t v) {
        const int m = c / chunks, j = c - m * chunks;
        if (c < MB * chunks)
            *reinterpret_cast<u32x4_t *>(lds8 + x_off + static_cast<uint32_t>(m) * row_bytes + static_cast<uint32_t>(j) * 16u) = v;
    };
    // slot e of the table: eight int8 magnitudes -- one E8 entry, or two consecutive D4 entries
    auto entry_park = [&](int e, u32x2_t raw) {
        u32x4_t v;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t src = t < 2 ? raw.x : raw.y;
            const int a = static_cast<int8_t>((src >> (16 * (t & 1))) & 0xffu), b = static_cast<int8_t>((src >> (16 * (t & 1) + 8)) & 0xffu);
            v[t] = e8_pair<XF16>(a, b);
        }
        *reinterpret_cast<u32x4_t *>(lds8 + static_cast<uint32_t>(e) * 16u) = v;
    };
    const int nslot = ncb * k.vs / 8;
    // the first slot and the first two chunks of every thread, and the state tables, are requested together
    const u32x2_t raw0 = tid < nslot ? *reinterpret_cast<const u32x2_t *>(cbp + static_cast<int64_t>(tid) * 8) : u32x2_t{0u, 0u};
    const u32x4_t xc0 = x_chunk(tid), xc1 = x_chunk(tid + static_cast<int>(blockDim.x));
    const float lutv = tid < 16 ? lut[tid] : 0.f;
    const uint32_t bfsv = tid < 16 ? bfs[tid] : 0u;
    if (tid < nslot) entry_park(tid, raw0);
    for (int e = tid + blockDim.x; e < nslot; e += blockDim.x) entry_park(e, *reinterpret_cast<const u32x2_t *>(cbp + static_cast<int64_t>(e) * 8));
    for (int e = tid; e < 256; e += blockDim.x) {
        u32x4_t v;
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = (((e >> (2 * t)) & 1u) << 15) | (((e >> (2 * t + 1)) & 1u) << 31);
        *reinterpret_cast<u32x4_t *>(lds8 + sgn_off + static_cast<uint32_t>(e) * 16u) = v;
    }
    if (tid < 16) {
        float *st = reinterpret_cast<float *>(lds8 + stab_off);
        st[2 * tid] = lutv;
        reinterpret_cast<uint32_t *>(st)[2 * tid + 1] = lds_base + bfsv * static_cast<uint32_t>(k.entries) * esz;
    }
    if (k.kind == 3) {
        const float *lut3 = reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(lut) + 128 + static_cast<int64_t>(k.nbank) * k.bank_bytes);
        for (int i = tid; i < k.nbank * 8; i += blockDim.x) *reinterpret_cast<float *>(lds8 + lut3_off + static_cast<uint32_t>(i) * 4u) = lut3[i];
    }
    x_park(tid, xc0);
    x_park(tid + static_cast<int>(blockDim.x), xc1);
    for (int c = tid + 2 * static_cast<int>(blockDim.x); c < MB * chunks; c += blockDim.x) x_park(c, x_chunk(c));
    uint32_t roff[3];  // LDS byte offsets of the wave's three ranges
    roff[0] = wave_off;
    roff[1] = roff[0] + sh.cap[0];
    roff[2] = roff[1] + sh.cap[1];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t off = static_cast<uint32_t>(t * 64 + lane) * 16u;
            if (off < sh.cap[r]) *reinterpret_cast<u32x4_t *>(lds8 + roff[r] + off) = piece[r][t];
        }
    __syncthreads();
    // `nbits` (<= 25) bits at bit position `bit` of the range at LDS address `base`
    auto field = [&](uint32_t base, uint32_t bit, uint32_t nbits) -> uint32_t {
        const u32x2_t d = u32x2_t{*reinterpret_cast<lds_u32_ptr>(base + ((bit >> 5) << 2)), *reinterpret_cast<lds_u32_ptr>(base + ((bit >> 5) << 2) + 4u)};
        return __builtin_amdgcn_alignbit(d.y, d.x, bit & 31u) & ((1u << nbits) - 1u);
    };
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    for (int j = 0; j < nn; ++j) {
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.f;
        const uint32_t ib = shift[0] + static_cast<uint32_t>(j) * k.nvec * k.ib, sb0 = shift[1] + static_cast<uint32_t>(j) * per1,
                       tb = shift[2] + static_cast<uint32_t>(j) * per2;
        for (int g = lane; g < k.ng; g += 64) {
            const uint32_t state = field(lds_base + roff[2], tb + static_cast<uint32_t>(k.sbits) * g, k.sbits);
            if (k.kind != 0) {
                // The 1-bit families.  Kind 1 (NVQ1-L / -S): w = scale * (code + d), code a ternary 8-vector of the bank the
                // group's delta sign names, d = -delta / +delta by that sign -- the products with the codes plus d times
                // the sum of the group's activations.  Kind 2 (NPQ0-L / -S): a block is a 4-vector of the state's first
                // sub-codebook (index bits 0..2) beside one of its second (the bits above).  Kind 3 (NEPQ0-S / -L): the same
                // with a pool of tables.
                const u32x2_t se1 = *reinterpret_cast<lds_u32x2_ptr>(lds_base + stab_off + state * 8u);
                uint32_t neg = 0u, tbase = 0u;  // tbase: LDS byte offset of the group's table
                float sc1 = __uint_as_float(se1.x);
                if (k.kind == 1) neg = field(lds_base + roff[1], sb0 + g, 1);
                if (k.kind == 3) {
                    // NEPQ0: the neuron's table of the pool for these 96 weights gives sub-codebooks and scale
                    const uint32_t pb = min(field(lds_base + roff[1], sb0 + 8u * (static_cast<uint32_t>(g) >> 2), 8), static_cast<uint32_t>(k.nbank - 1));
                    tbase = pb * static_cast<uint32_t>(k.bank_bytes) * 2u;
                    sc1 = __uint_as_float(*reinterpret_cast<lds_u32_ptr>(lds_base + lut3_off + (pb * 8u + state) * 4u));
                }
                u32x4_t wv1[3];
#pragma unroll
                for (int b = 0; b < 3; ++b) {
                    // (a block past the neuron's last vector meets staged zeros; entry 0 keeps its lookups inside the tables)
                    const uint32_t idx = 3 * g + b < k.nvec ? field(lds_base + roff[0], ib + static_cast<uint32_t>(3 * g + b) * k.ib, k.ib) : 0u;
                    if (k.kind == 1) {
                        wv1[b] = *reinterpret_cast<lds_u32x4_ptr>(lds_base + ((k.banks == 2 ? neg : 0u) * static_cast<uint32_t>(k.entries) + idx) * 16u);
                    } else {
                        const u32x2_t e0 = *reinterpret_cast<lds_u32x2_ptr>(lds_base + tbase + (state * 8u + (idx & 7u)) * 8u);
                        const u32x2_t e1 = *reinterpret_cast<lds_u32x2_ptr>(lds_base + tbase + (static_cast<uint32_t>(k.banks) * 8u + state * static_cast<uint32_t>(k.entries) + (idx >> 3)) * 8u);
                        wv1[b] = u32x4_t{e0.x, e0.y, e1.x, e1.y};
                    }
                }
                const float dl = neg ? -k.delta : k.delta;
                const uint32_t ones = XF16 ? 0x3c003c00u : 0x3f803f80u;
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    float part1 = 0.f, xsum = 0.f;
#pragma unroll
                    for (int b = 0; b < 3; ++b) {
                        const u32x4_t xv = *reinterpret_cast<lds_u32x4_ptr>(lds_base + x_off + static_cast<uint32_t>(m) * row_bytes + static_cast<uint32_t>(3 * g + b) * 16u);
                        part1 = e8_dot8<XF16>(wv1[b], xv, part1);
                        if (k.kind == 1) xsum = e8_dot8<XF16>(u32x4_t{ones, ones, ones, ones}, xv, xsum);
                    }
                    acc[m] = fmaf(sc1, fmaf(dl, xsum, part1), acc[m]);
                }
                continue;
            }
            // the indices of the group's three blocks: one 24-bit field of index bytes, three fields of 10 or 12 bits, or
            // (4-dimensional vectors) two fields per block
            uint32_t ix[3], ix2[3] = {0u, 0u, 0u};
            if (k.vs == 4) {
#pragma unroll
                for (int b = 0; b < 3; ++b) {
                    ix[b] = field(lds_base + roff[0], ib + static_cast<uint32_t>(6 * g + 2 * b) * k.ib, k.ib);
                    ix2[b] = field(lds_base + roff[0], ib + static_cast<uint32_t>(6 * g + 2 * b + 1) * k.ib, k.ib);
                }
            } else if (k.ib == 8) {
                const uint32_t idx3 = field(lds_base + roff[0], ib + 24u * g, 24);
                ix[0] = idx3 & 255u; ix[1] = (idx3 >> 8) & 255u; ix[2] = idx3 >> 16;
            } else {
#pragma unroll
                for (int b = 0; b < 3; ++b) ix[b] = field(lds_base + roff[0], ib + static_cast<uint32_t>(3 * g + b) * k.ib, k.ib);
            }
            const uint32_t mask3 = field(lds_base + roff[1], sb0 + 21u * g, 21);
            const u32x2_t se = *reinterpret_cast<lds_u32x2_ptr>(lds_base + stab_off + state * 8u);
            float part[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m) part[m] = 0.f;
            // (no test for blocks past K in the last group: whatever entry and signs their bits name meets staged zeros)
            u32x4_t wv[3];
#pragma unroll
            for (int b = 0; b < 3; ++b) {
                const uint32_t idx = ix[b], mk = (mask3 >> (7 * b)) & 127u;
                uint32_t last = __popc(mk) & 1u;
                if (k.index_parity) last ^= idx >> 7;
                const uint32_t neg = mk | (last << 7);
                u32x4_t ev;
                if (k.vs == 4) {
                    const u32x2_t e0 = *reinterpret_cast<lds_u32x2_ptr>(se.y + idx * 8u), e1 = *reinterpret_cast<lds_u32x2_ptr>(se.y + ix2[b] * 8u);
                    ev = u32x4_t{e0.x, e0.y, e1.x, e1.y};
                } else {
                    ev = *reinterpret_cast<lds_u32x4_ptr>(se.y + idx * 16u);
                }
                const u32x4_t sv = *reinterpret_cast<lds_u32x4_ptr>(lds_base + sgn_off + neg * 16u);
                wv[b] = ev ^ sv;
            }
#pragma unroll
            for (int m = 0; m < MB; ++m)
#pragma unroll
                for (int b = 0; b < 3; ++b) {
                    const u32x4_t xv = *reinterpret_cast<lds_u32x4_ptr>(lds_base + x_off + static_cast<uint32_t>(m) * row_bytes + static_cast<uint32_t>(3 * g + b) * 16u);
                    part[m] = e8_dot8<XF16>(wv[b], xv, part[m]);
                }
            const float sc = __uint_as_float(se.x);
#pragma unroll
            for (int m = 0; m < MB; ++m) acc[m] = fmaf(sc, part[m], acc[m]);
        }
        const float anchor = anchors[n0 + j];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float v = acc[m];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0 && m0 + m < M) y[static_cast<int64_t>(m0 + m) * ldy + row_first + j] = v * anchor;
        }
    }
}


// ---- the same formats for 3 to 192 rows on the matrix cores -----------------------------------------------------------
// nvqs_e8_kernel reads a row's activations again for every block of weights, so its time grows with the rows.  Here a
// block owns 16 consecutive neurons: their three bit ranges (contiguous in the streams) are staged whole, the waves
// split the groups of 24 weights, and lane (n, kb) -- neuron n = lane % 16, block kb = lane / 16 of the group, the lanes
// of kb = 3 idle -- decodes one 8-weight block, which is its B fragment of a 16 x 16 x 32 product against the rows'
// 24 activations of the group (A fragment: row lane % 16, the same block; zeros for kb = 3).  The product's four
// results of a lane belong to its own neuron, whose group scale it has decoded, and are scaled and added in fp32.
// The waves' partial sums meet in LDS.  Above 16 rows a block takes two or four 16-row tiles (blockIdx.y counts such
// sets), which share every decoded fragment.  The 16 neurons of a wave read their fields at a stride of the neuron's bytes in
// the stream -- 512 bytes of index bytes for K = 4096, one LDS bank for all of them -- so the staged copy of a range
// skips a bank after every 2^pad bytes, with pad chosen per range so that the 16 strides spread over the banks.
// LDS map (bytes): [entries][256 sign patterns x 16][state table 128][pool scale tables][index | sign | state ranges]
// [partial sums: waves x 1024]
struct E8TileShape {
    int gpw;            // groups of 24 weights per wave
    uint32_t cap[3];    // LDS bytes of the block's index / sign / state range, padding included
    uint32_t pad[3];    // log2 of the bytes of a range after which its LDS copy skips a bank (31: no padding)
    int compact;        // the table stays bytes in LDS (decoder 8)
    uint32_t lds_bytes;
};
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
template <int XF16>
__device__ __forceinline__ float4_t e8_mfma(u32x4_t a, u32x4_t b, float4_t c) {
    if constexpr (XF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
// DEC: the block decoder -- 0: sign-stream formats with 8-dimensional vectors, 4: with 4-dimensional ones, 1: NVQ1,
// 2: NPQ0 / NEPQ0, 8: 8-dimensional vectors whose table fits the LDS only as bytes (NVQ2J-XL with several banks: 128 KB
// of int8).  The bytes are kept with bit 7 flipped (u = v + 128, unsigned) and widened where they are used: for fp16
// activations a byte permute builds 1024 + u and a packed subtraction of 1152 leaves v exactly; bf16 has no packed
// arithmetic here, so the block is multiplied as u and 128 times the product of the same activations with the block's
// signs alone is taken off (exact factors, fp32 sums).  The partial sums then reuse the ranges' LDS.
template <int XF16, int MT, int DEC>
__global__ __launch_bounds__(64 * kE8Waves, 8) void nvqs_e8_tile_kernel(NvqsK k, const uint8_t *__restrict__ w,
                                                                     const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                                     float *__restrict__ y, int64_t ldy, E8TileShape sh) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds32[];
    typedef __attribute__((address_space(3))) const u32x4_t *lds_u32x4_ptr;
    typedef __attribute__((address_space(3))) const u32x2_t *lds_u32x2_ptr;
    typedef __attribute__((address_space(3))) const uint32_t *lds_u32_ptr;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ncb = k.kind == 2 ? k.cb_bytes / k.vs : (k.kind == 3 ? k.nbank * k.bank_bytes / k.vs : k.banks * k.entries);
    uint8_t *lds8 = reinterpret_cast<uint8_t *>(lds32);
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)lds8));
    const uint32_t esz = DEC == 8 ? 8u : static_cast<uint32_t>(k.vs) * 2u;
    const uint32_t sgn_off = static_cast<uint32_t>(ncb) * esz, stab_off = sgn_off + 4096u, lut3_off = stab_off + 128u;
    uint32_t roff[3];
    roff[0] = lut3_off + (k.kind == 3 ? static_cast<uint32_t>(k.nbank) * 32u : 0u);
    roff[1] = roff[0] + sh.cap[0];
    roff[2] = roff[1] + sh.cap[1];
    const uint32_t red_off = DEC == 8 ? roff[0] : roff[2] + sh.cap[2];

    // ---- the block's stream ranges: 16-byte pieces, four requests of a thread in flight ----------------------------
    const int row_first = static_cast<int>(blockIdx.x) * 16;
    const int nn = min(16, k.nrows - row_first);  // >= 1: the grid has no block past the last neuron
    const int64_t n0 = k.row0 + row_first;
    const uint32_t per[3] = {static_cast<uint32_t>(k.nvec) * static_cast<uint32_t>(k.ib),
                             k.kind == 0 ? static_cast<uint32_t>(k.nsign) * 7u
                                         : (k.kind == 1 ? static_cast<uint32_t>(k.ng) : (k.kind == 3 ? static_cast<uint32_t>(k.nsuper) * 8u : 0u)),
                             static_cast<uint32_t>(k.ng) * static_cast<uint32_t>(k.sbits)};
    const int64_t region[3] = {k.index_off, k.sign_off, k.state_off};
    const int64_t region_bytes[3] = {k.index_bytes + 4, k.sign_bytes + 4, k.state_bytes + 4};
    uint32_t shift[3];  // bits between the staged range's first bit and the first bit of neuron n0
    // the tables' first requests go out with the stream ranges'
    const float *lut = nvqs_lut(k, w);
    const uint32_t *bfs = reinterpret_cast<const uint32_t *>(lut + 16);
    const int8_t *cbp = reinterpret_cast<const int8_t *>(bfs + 16);
    const int nslot = ncb * k.vs / 8;  // slot e: eight int8 values -> eight values of the activations' type
    const u32x2_t raw0 = tid < nslot ? *reinterpret_cast<const u32x2_t *>(cbp + static_cast<int64_t>(tid) * 8) : u32x2_t{0u, 0u};
    const float lutv = lut[tid & 15];
    const uint32_t bfsv = bfs[tid & 15];
    // the first pieces of a thread in each range (two: 32 KB of a range; one where four row tiles leave few registers) are
    // requested together, so that the three ranges cost one round trip, not three; what a longer range has left follows
    // in turns of four pieces
    constexpr int HEAD = MT == 4 ? 1 : 2;
    constexpr uint32_t kTurn = 64u * kE8Waves * 16u;  // bytes the block's threads cover with one piece each
    __amdgpu_buffer_rsrc_t win[3];
    uint32_t raw[3];  // stream bytes of the ranges
    u32x4_t head[3][HEAD];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        const int64_t bit0 = n0 * static_cast<int64_t>(per[r]);
        const int64_t a0 = (bit0 >> 3) & ~static_cast<int64_t>(15);
        shift[r] = static_cast<uint32_t>(bit0 - a0 * 8);
        const int64_t left = region_bytes[r] - a0;
        win[r] = wave_window(w + region[r] + a0, static_cast<uint32_t>(left <= 0 ? 0 : (left < (1ll << 31) ? left : (1ll << 31))));
        raw[r] = nvqs_e8_range_bytes(16ll * per[r]);
#pragma unroll
        for (int t = 0; t < HEAD; ++t) {
            const uint32_t off = static_cast<uint32_t>(tid) * 16u + static_cast<uint32_t>(t) * kTurn;
            head[r][t] = __builtin_amdgcn_raw_buffer_load_b128(win[r], off < raw[r] ? off : kNoStep, 0, 2);
        }
    }
    // a piece lies inside one padding period (they are 64 bytes and more); the skipped bank before a period holds a copy
    // of the period's first dword, so that a field's two dwords are adjacent in LDS wherever it starts
    auto park = [&](int r, uint32_t off, u32x4_t piece) {
        if (off < raw[r]) {
            uint32_t *dst = reinterpret_cast<uint32_t *>(lds8 + roff[r] + off + ((off >> sh.pad[r]) << 2));
            dst[0] = piece.x; dst[1] = piece.y; dst[2] = piece.z; dst[3] = piece.w;
            if (off > 0u && (off & ((1u << sh.pad[r]) - 1u)) == 0u) dst[-1] = piece.x;
        }
    };
#pragma unroll
    for (int r = 0; r < 3; ++r) {
#pragma unroll
        for (int t = 0; t < HEAD; ++t) park(r, static_cast<uint32_t>(tid) * 16u + static_cast<uint32_t>(t) * kTurn, head[r][t]);
        for (uint32_t p0 = static_cast<uint32_t>(tid) * 16u + HEAD * kTurn; p0 < raw[r]; p0 += 4u * kTurn) {
            u32x4_t piece[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t off = p0 + static_cast<uint32_t>(t) * kTurn;
                piece[t] = __builtin_amdgcn_raw_buffer_load_b128(win[r], off < raw[r] ? off : kNoStep, 0, 2);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) park(r, p0 + static_cast<uint32_t>(t) * kTurn, piece[t]);
        }
    }
    // ---- tables -------------------------------------------------------------------------------------------------------
    for (int e = tid; e < nslot; e += blockDim.x) {
        const u32x2_t raw = e == tid ? raw0 : *reinterpret_cast<const u32x2_t *>(cbp + static_cast<int64_t>(e) * 8);
        if constexpr (DEC == 8) {
            *reinterpret_cast<u32x2_t *>(lds8 + static_cast<uint32_t>(e) * 8u) = u32x2_t{raw.x ^ 0x80808080u, raw.y ^ 0x80808080u};
            continue;
        }
        u32x4_t v;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t src = t < 2 ? raw.x : raw.y;
            const int a = static_cast<int8_t>((src >> (16 * (t & 1))) & 0xffu), b = static_cast<int8_t>((src >> (16 * (t & 1) + 8)) & 0xffu);
            v[t] = e8_pair<XF16>(a, b);
        }
        *reinterpret_cast<u32x4_t *>(lds8 + static_cast<uint32_t>(e) * 16u) = v;
    }
    for (int e = tid; e < 256; e += blockDim.x) {
        u32x4_t v;
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = (((e >> (2 * t)) & 1u) << 15) | (((e >> (2 * t + 1)) & 1u) << 31);
        *reinterpret_cast<u32x4_t *>(lds8 + sgn_off + static_cast<uint32_t>(e) * 16u) = v;
    }
    if (tid < 16) {
        float *st = reinterpret_cast<float *>(lds8 + stab_off);
        st[2 * tid] = lutv;
        reinterpret_cast<uint32_t *>(st)[2 * tid + 1] = lds_base + bfsv * static_cast<uint32_t>(k.entries) * esz;
    }
    if (k.kind == 3) {
        const float *lut3 = reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(lut) + 128 + static_cast<int64_t>(k.nbank) * k.bank_bytes);
        for (int i = tid; i < k.nbank * 8; i += blockDim.x) *reinterpret_cast<float *>(lds8 + lut3_off + static_cast<uint32_t>(i) * 4u) = lut3[i];
    }
    __syncthreads();

    // `nbits` (<= 25) bits at bit position `bit` of staged range r
    auto field = [&](int r, uint32_t bit, uint32_t nbits) -> uint32_t {
        const uint32_t b0 = (bit >> 5) << 2, a = lds_base + roff[r] + b0 + ((b0 >> sh.pad[r]) << 2);
        const u32x2_t d = u32x2_t{*reinterpret_cast<lds_u32_ptr>(a), *reinterpret_cast<lds_u32_ptr>(a + 4u)};
        return __builtin_amdgcn_alignbit(d.y, d.x, bit & 31u) & ((1u << nbits) - 1u);
    };
    const int r16 = lane & 15, kb = lane >> 4;
    const uint32_t nloc = static_cast<uint32_t>(min(r16, nn - 1));  // lanes past the last neuron repeat it; their sums are not stored
    const uint32_t ixb = shift[0] + nloc * per[0], sgb = shift[1] + nloc * per[1], stb = shift[2] + nloc * per[2];
    const int m0 = static_cast<int>(blockIdx.y) * 16 * MT;  // the block's MT tiles of 16 rows share every decoded fragment
    const bool vec = ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    // the eight activations of block kb of group g of the lane's row in tile mt; zeros past M and K and for kb = 3
    // whole aligned vectors everywhere (the common case): one range-checked load per fragment, the "no data" offset for
    // the fragments that are zero
    const bool fast = vec && k.neuron_len % 8 == 0 && 32 * ldx * 2 < (1ll << 31);
    const __amdgpu_buffer_rsrc_t xwin =
        wave_window(reinterpret_cast<const uint8_t *>(x + static_cast<int64_t>(m0) * ldx),
                    fast ? static_cast<uint32_t>(((min(M - m0, 16 * MT) - 1) * ldx + k.neuron_len) * 2) : 0u);
    auto x_frag_fast = [&](int g, int mt) -> u32x4_t {
        const int c0 = (3 * g + kb) * 8, ml = 16 * mt + r16;
        const bool ok = m0 + ml < M && kb < 3 && c0 < k.neuron_len;  // (g past the wave's groups is passed as ng: c0 >= K)
        return __builtin_amdgcn_raw_buffer_load_b128(xwin, ok ? static_cast<uint32_t>(ml * ldx * 2 + c0 * 2) : kNoStep, 0, 0);
    };
    auto x_frag = [&](int g, int mt) -> u32x4_t {
        u32x4_t v = {0u, 0u, 0u, 0u};
        const int c0 = (3 * g + kb) * 8, m = m0 + 16 * mt + r16;
        const uint16_t *xr = x + static_cast<int64_t>(min(m, M - 1)) * ldx;
        if (m < M && kb < 3 && g < k.ng && c0 < k.neuron_len) {
            if (vec && c0 + 8 <= k.neuron_len) {
                v = *reinterpret_cast<const u32x4_t *>(xr + c0);
            } else {
                uint32_t h[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = c0 + i < k.neuron_len ? xr[c0 + i] : 0u;
                v = u32x4_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
            }
        }
        return v;
    };
    const uint32_t ones = XF16 ? 0x3c003c00u : 0x3f803f80u;
    constexpr int GT = MT == 1 ? 4 : (MT == 2 ? 2 : 1);  // groups whose activations are requested together
    float4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int g0 = wave * sh.gpw, g1 = min(k.ng, g0 + sh.gpw);
    // bit positions of the lane's fields in the wave's first group; they advance by a constant per group (a product per
    // field and group would be a quarter-rate 64-bit multiply-add each)
    const uint32_t kb2 = static_cast<uint32_t>(min(kb, 2));  // the lanes of kb = 3 meet zero activations
    const uint32_t ix_inc = (DEC == 4 ? 6u : 3u) * static_cast<uint32_t>(k.ib), sg_inc = DEC == 1 ? 1u : 21u, st_inc = static_cast<uint32_t>(k.sbits);
    uint32_t ix_bit = ixb + (DEC == 4 ? 2u : 1u) * (3u * static_cast<uint32_t>(g0) + kb2) * static_cast<uint32_t>(k.ib);
    uint32_t sg_bit = sgb + (DEC == 1 ? static_cast<uint32_t>(g0) : 7u * (3u * static_cast<uint32_t>(g0) + kb2));
    uint32_t st_bit = stb + st_inc * static_cast<uint32_t>(g0);
    auto walk = [&](auto fast_c) {
    for (int gq = g0; gq < g1; gq += GT) {
        u32x4_t xf[GT][MT];
#pragma unroll
        for (int t = 0; t < GT; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int gx = gq + t < g1 ? gq + t : k.ng;
                if constexpr (decltype(fast_c)::value) xf[t][mt] = x_frag_fast(gx, mt);
                else xf[t][mt] = x_frag(gx, mt);
            }
#pragma unroll
        for (int t = 0; t < GT; ++t) {
            const int g = min(gq + t, g1 - 1);  // past the wave's last group: that group again, against zero activations
            const uint32_t sb = static_cast<uint32_t>(3 * g) + kb2;
            const uint32_t state = field(2, st_bit, k.sbits);
            const u32x2_t se = *reinterpret_cast<lds_u32x2_ptr>(lds_base + stab_off + state * 8u);
            float sc = __uint_as_float(se.x);
            u32x4_t wv;
            float dl = 0.f;
            [[maybe_unused]] u32x4_t sgn_ones = {0u, 0u, 0u, 0u};  // DEC 8, bf16: the block's signs on ones
            if constexpr (DEC == 0 || DEC == 4 || DEC == 8) {
                const uint32_t mk = field(1, sg_bit, 7);
                uint32_t last = __popc(mk) & 1u;
                u32x4_t ev;
                if constexpr (DEC == 4) {
                    const uint32_t i0 = field(0, ix_bit, k.ib);
                    const uint32_t i1 = 2u * sb + 1u < static_cast<uint32_t>(k.nvec) ? field(0, ix_bit + static_cast<uint32_t>(k.ib), k.ib) : 0u;
                    const u32x2_t e0 = *reinterpret_cast<lds_u32x2_ptr>(se.y + i0 * 8u), e1 = *reinterpret_cast<lds_u32x2_ptr>(se.y + i1 * 8u);
                    ev = u32x4_t{e0.x, e0.y, e1.x, e1.y};
                } else {
                    const uint32_t idx = field(0, ix_bit, k.ib);
                    if (k.index_parity) last ^= (idx >> 7) & 1u;
                    if constexpr (DEC == 8) {
                        const u32x2_t q = *reinterpret_cast<lds_u32x2_ptr>(se.y + idx * 8u);
                        const uint32_t qq[2] = {q.x, q.y};
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            if constexpr (XF16) {
                                const half2_t bias = {static_cast<_Float16>(1152.f), static_cast<_Float16>(1152.f)};
                                ev[2 * h] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(qq[h], 0x64006400u, 0x03050104u)) - bias);
                                ev[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(qq[h], 0x64006400u, 0x03070106u)) - bias);
                            } else {
                                const float f0 = static_cast<float>(qq[h] & 0xffu), f1 = static_cast<float>((qq[h] >> 8) & 0xffu),
                                            f2 = static_cast<float>((qq[h] >> 16) & 0xffu), f3 = static_cast<float>(qq[h] >> 24);
                                ev[2 * h] = (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
                                ev[2 * h + 1] = (__float_as_uint(f2) >> 16) | (__float_as_uint(f3) & 0xffff0000u);
                            }
                        }
                    } else {
                        ev = *reinterpret_cast<lds_u32x4_ptr>(se.y + idx * 16u);
                    }
                }
                const u32x4_t sv = *reinterpret_cast<lds_u32x4_ptr>(lds_base + sgn_off + (mk | (last << 7)) * 16u);
                wv = ev ^ sv;
                if constexpr (DEC == 8 && !XF16) sgn_ones = u32x4_t{ones, ones, ones, ones} ^ sv;
            } else {
                const uint32_t idx = sb < static_cast<uint32_t>(k.nvec) ? field(0, ix_bit, k.ib) : 0u;
                if constexpr (DEC == 1) {
                    const uint32_t neg = field(1, sg_bit, 1);
                    wv = *reinterpret_cast<lds_u32x4_ptr>(lds_base + ((k.banks == 2 ? neg : 0u) * static_cast<uint32_t>(k.entries) + idx) * 16u);
                    // w = scale * (code + d): d times the sum of the group's activations, as a product with ones
                    dl = neg ? -k.delta : k.delta;
                } else {
                    uint32_t tbase = 0u;
                    if (k.kind == 3) {
                        const uint32_t pb = min(field(1, sgb + 8u * (static_cast<uint32_t>(g) >> 2), 8), static_cast<uint32_t>(k.nbank - 1));
                        tbase = pb * static_cast<uint32_t>(k.bank_bytes) * 2u;
                        sc = __uint_as_float(*reinterpret_cast<lds_u32_ptr>(lds_base + lut3_off + (pb * 8u + state) * 4u));
                    }
                    const u32x2_t e0 = *reinterpret_cast<lds_u32x2_ptr>(lds_base + tbase + (state * 8u + (idx & 7u)) * 8u);
                    const u32x2_t e1 = *reinterpret_cast<lds_u32x2_ptr>(lds_base + tbase + (static_cast<uint32_t>(k.banks) * 8u + state * static_cast<uint32_t>(k.entries) + (idx >> 3)) * 8u);
                    wv = u32x4_t{e0.x, e0.y, e1.x, e1.y};
                }
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                float4_t part = {0.f, 0.f, 0.f, 0.f};
                if constexpr (DEC == 1) {
                    const float4_t xs = e8_mfma<XF16>(xf[t][mt], u32x4_t{ones, ones, ones, ones}, float4_t{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                    for (int v = 0; v < 4; ++v) part[v] = dl * xs[v];
                }
                if constexpr (DEC == 8 && !XF16) {
                    const float4_t xs = e8_mfma<XF16>(xf[t][mt], sgn_ones, float4_t{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                    for (int v = 0; v < 4; ++v) part[v] = -128.f * xs[v];
                }
                part = e8_mfma<XF16>(xf[t][mt], wv, part);
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[mt][v] = fmaf(sc, part[v], acc[mt][v]);
            }
            if (gq + t + 1 < g1) {  // (wave-uniform; past the wave's last group the positions stay on it)
                ix_bit += ix_inc; sg_bit += sg_inc; st_bit += st_inc;
            }
        }
    }
    };
    if (fast) walk(std::true_type{});
    else walk(std::false_type{});
    // ---- the waves' partial sums: red[wave][row][neuron] ------------------------------------------------------------
    float *red = reinterpret_cast<float *>(lds8 + red_off);
    if constexpr (DEC == 8) __syncthreads();  // the sums take the place of the ranges: every wave is done with them
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {  // one tile at a time through the same 16 KB
        if (mt > 0) __syncthreads();
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave * 256 + (4 * kb + v) * 16 + r16] = acc[mt][v];
        __syncthreads();
        if (tid < 256) {
            const int m = m0 + 16 * mt + (tid >> 4), n = tid & 15;
            float sum = 0.f;
#pragma unroll
            for (int wv = 0; wv < kE8Waves; ++wv) sum += red[wv * 256 + tid];
            if (m < M && n < nn) y[static_cast<int64_t>(m) * ldy + row_first + n] = sum * reinterpret_cast<const float *>(w + k.anchors_off)[n0 + n];
        }
    }
}

int gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, const float *sa,
                const float *sb, float *y, int64_t ldy, hipStream_t st, float *part = nullptr);
float *dequant_gemm_part(float *wscale, int N, int K, int M);
int x_prep(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, hipStream_t st);
size_t dequant_gemm_workspace(int N, int K, int M);
void dequant_gemm_carve(void *ws, int N, int K, int M, uint16_t *&x16, float *&xscale, uint16_t *&w16, float *&wscale,
                        int &Kp);

constexpr int kNvqsGemvMaxM = 16;  // rows up to which the weights are re-read per pass of eight rows
constexpr int kNvqsTileMaxM = 192;  // rows up to which the formats of the matrix-core tile kernel stay on it

// The E8 kernel takes the sign-stream format with 8- or 4-dimensional vectors, 4-bit states and tables that fit the LDS
// in the activations' type (E8: 256 or 1024 entries in up to four banks, 4096 in one; D4: 1024 entries), tensors whose streams fit 32-bit offsets and
// neurons of at most about 16000 weights with index bytes, 10000 with 12-bit indices (a wave's index range is two 1 KB
// requests at most), and the 1-bit families NVQ1-L / NVQ1-S (ternary 8-vectors, a delta sign per group) and NPQ0-L /
// NPQ0-S (two 4-vectors per block; NEPQ0-S / NEPQ0-L: out of a pool of tables that fits the LDS) with their states of
// 2 to 4 bits.  MB = rows per pass that fit the LDS.
static bool nvqs_e8_format(const NvqsK &k) {
    static const int off = tune_env("MFQ_NVQS_E8_OFF", 0);
    if (off || k.index_bytes >= (1ll << 31) || k.sign_bytes >= (1ll << 31)) return false;
    if (k.kind == 0) {
        if ((k.vs != 8 && k.vs != 4) || k.ib < 8 || k.ib > 12 || k.entries != (1 << k.ib) || k.sbits != 4 || k.banks > 4) return false;
    } else if (k.kind == 1) {  // NVQ1-L / NVQ1-S: 2048 or two banks of 512 ternary 8-vectors
        if (k.vs != 8 || k.ib < 8 || k.ib > 12 || k.entries != (1 << k.ib) || k.sbits < 2 || k.sbits > 4 || k.banks > 2) return false;
    } else if (k.kind == 2 || k.kind == 3) {  // NPQ0-L / NPQ0-S: a few dozen 4-vectors per state; NEPQ0: a pool of such tables
        if (k.ib < 4 || k.ib > 8 || k.entries * 8 != (1 << k.ib) || k.sbits < 2 || k.sbits > 4 || k.cb_bytes % 8 != 0) return false;
        if (k.kind == 3 && (k.nbank < 1 || k.nbank > 256 || k.bank_bytes % 8 != 0 || k.bank_bytes != k.banks * 32 + k.banks * k.entries * 4)) return false;
    } else {
        return false;
    }
    return true;
}
static uint32_t nvqs_e8_table_bytes(const NvqsK &k) {  // the tables as int8
    return k.kind == 2 ? static_cast<uint32_t>(k.cb_bytes)
                       : (k.kind == 3 ? static_cast<uint32_t>(k.nbank) * static_cast<uint32_t>(k.bank_bytes)
                                      : static_cast<uint32_t>(k.banks) * static_cast<uint32_t>(k.entries) * static_cast<uint32_t>(k.vs));
}
static int64_t nvqs_e8_sign_bits(const NvqsK &k) {  // bits per neuron of the second staged range
    return k.kind == 0 ? static_cast<int64_t>(k.nsign) * 7 : (k.kind == 1 ? k.ng : (k.kind == 3 ? k.nsuper * 8 : 0));
}
static uint32_t nvqs_e8_cap(int64_t bits) { return nvqs_e8_range_bytes(bits); }
static bool nvqs_e8_shape(const NvqsK &k, int M, int &mb, E8Shape &sh) {
    if (!nvqs_e8_format(k)) return false;
    auto cap = nvqs_e8_cap;
    int npw = static_cast<int>(ceil_div(k.nrows, static_cast<int64_t>(gemv_cu_count()) * kE8Waves));
    if (npw > 4) npw = 4;
    while (npw > 1 && cap(static_cast<int64_t>(npw) * k.nvec * k.ib) > 2048) --npw;
    if (cap(static_cast<int64_t>(npw) * k.nvec * k.ib) > 2048) return false;
    sh.npw = npw;
    sh.kp = k.ng * 24;
    sh.cap[0] = cap(static_cast<int64_t>(npw) * k.nvec * k.ib);
    sh.cap[1] = cap(static_cast<int64_t>(npw) * nvqs_e8_sign_bits(k));
    sh.cap[2] = cap(static_cast<int64_t>(npw) * k.ng * k.sbits);
    sh.wave_bytes = sh.cap[0] + sh.cap[1] + sh.cap[2];
    for (mb = M >= 2 ? 2 : 1; mb >= 1; mb >>= 1) {  // (three rows and more go to the matrix-core form)
        const uint32_t table = nvqs_e8_table_bytes(k);
        if (table > kMaxDynamicLds / 2) return false;
        sh.lds_bytes = table * 2u + 4096u + 128u + (k.kind == 3 ? static_cast<uint32_t>(k.nbank) * 32u : 0u) + static_cast<uint32_t>(mb) * sh.kp * 2u + kE8Waves * sh.wave_bytes;
        if (sh.lds_bytes <= kMaxDynamicLds) return true;
    }
    return false;
}
// The matrix-core form: from MFQ_NVQS_TILE_MIN_M rows on (from one row for the tables kept as bytes), when the 16 neurons'
// ranges and the tables fit the LDS.
static bool nvqs_e8_tile_shape(const NvqsK &k, int M, E8TileShape &sh) {
    static const int min_m = tune_env("MFQ_NVQS_TILE_MIN_M", 3);
    static const int max_m = tune_env("MFQ_NVQS_TILE_MAX_M", kNvqsTileMaxM);
    if (M < 1 || M > max_m || !nvqs_e8_format(k)) return false;
    const int64_t bits[3] = {16ll * k.nvec * k.ib, 16ll * nvqs_e8_sign_bits(k), 16ll * k.ng * k.sbits};
    uint64_t ranges = 0;
    for (int r = 0; r < 3; ++r) {
        if (bits[r] > (1ll << 22)) return false;
        // the padding period under which the first dwords of the 16 neurons spread best over 32 banks
        const uint32_t raw = nvqs_e8_range_bytes(bits[r]);
        const int periods[6] = {31, 6, 7, 8, 9, 10};
        int best = 17;
        for (int pi = 0; pi < 6; ++pi) {
            int hits[32] = {0}, worst = 0;
            for (int n = 0; n < 16; ++n) {
                const uint32_t b = static_cast<uint32_t>(n * (bits[r] / 16) / 32) * 4u;
                const int bank = static_cast<int>(((b + ((b >> periods[pi]) << 2)) >> 2) & 31u);
                if (++hits[bank] > worst) worst = hits[bank];
            }
            if (worst < best) { best = worst; sh.pad[r] = static_cast<uint32_t>(periods[pi]); }
        }
        sh.cap[r] = (raw + ((raw >> sh.pad[r]) << 2) + 16u + 15u) / 16u * 16u;
        ranges += sh.cap[r];
    }
    const uint64_t tables = 4096u + 128u + (k.kind == 3 ? static_cast<uint32_t>(k.nbank) * 32u : 0u);
    uint64_t total = static_cast<uint64_t>(nvqs_e8_table_bytes(k)) * 2u + tables + ranges + kE8Waves * 1024u;
    // 8-dimensional sign-stream tables too large for the LDS in the activations' type stay bytes there and the sums
    // reuse the ranges' place; the vector kernel cannot take those tensors, so the tile kernel does from one row on
    sh.compact = total > kMaxDynamicLds && k.kind == 0 && k.vs == 8;
    if (sh.compact) total = nvqs_e8_table_bytes(k) + tables + (ranges > kE8Waves * 1024u ? ranges : kE8Waves * 1024u);
    if (!sh.compact && M < min_m) return false;
    if (total > kMaxDynamicLds) return false;
    sh.lds_bytes = static_cast<uint32_t>(total);
    sh.gpw = static_cast<int>(ceil_div(k.ng, kE8Waves));
    return true;
}
template <int XF16>
static int nvqs_launch_e8_tile(const NvqsK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                               const E8TileShape &sh, hipStream_t st) {
    // one, two or four 16-row tiles per block, which share every decoded fragment (with four, one group's activations
    // are requested at a time to stay within 64 registers: two blocks of 16 waves per compute unit)
#define MFQ_E8_TILE(MTV, DECV)                                                                                        \
    {                                                                                                                 \
        auto kern = nvqs_e8_tile_kernel<XF16, MTV, DECV>;                                                             \
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), sh.lds_bytes, "nvqs_e8_tile")) return rc; \
        hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(ceil_div(k.nrows, 16)), static_cast<unsigned>(ceil_div(M, 16 * MTV))), \
                           dim3(64 * kE8Waves), sh.lds_bytes, st, k, w, x, ldx, M, y, ldy, sh);                        \
        return check_launch("nvqs_e8_tile");                                                                          \
    }
#define MFQ_E8_TILE_MT(DECV) \
    if (M <= 16) MFQ_E8_TILE(1, DECV) else if (M <= 32) MFQ_E8_TILE(2, DECV) else MFQ_E8_TILE(4, DECV)
    if (sh.compact) MFQ_E8_TILE_MT(8)
    if (k.kind == 0 && k.vs == 8) MFQ_E8_TILE_MT(0)
    if (k.kind == 0) MFQ_E8_TILE_MT(4)
    if (k.kind == 1) MFQ_E8_TILE_MT(1)
    MFQ_E8_TILE_MT(2)
#undef MFQ_E8_TILE_MT
#undef MFQ_E8_TILE
}
template <int XF16>
static int nvqs_launch_e8(const NvqsK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy, int mb,
                          const E8Shape &sh, const PairSel &sel, int n_pairs, hipStream_t st) {
    const dim3 grid(static_cast<unsigned>(ceil_div(k.nrows, static_cast<int64_t>(kE8Waves) * sh.npw)),
                    static_cast<unsigned>(n_pairs ? n_pairs : ceil_div(M, mb)));
#define MFQ_E8(MBV)                                                                                                   \
    if (mb == MBV) {                                                                                                  \
        auto kern = nvqs_e8_kernel<XF16, MBV>;                                                                        \
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), sh.lds_bytes, "nvqs_e8")) return rc;     \
        hipLaunchKernelGGL(kern, grid, dim3(64 * kE8Waves), sh.lds_bytes, st, k, w, x, ldx, M, y, ldy, sh, sel);       \
        return check_launch("nvqs_e8");                                                                               \
    }
    MFQ_E8(1) MFQ_E8(2)
#undef MFQ_E8
    return fail(MFQ_ERR_UNSUPPORTED, "nvqs_e8: %d rows per pass", mb);
}

template <int XF16, int MB>
static int nvqs_launch_gemv(const NvqsK &k, const uint8_t *w, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy,
                            hipStream_t st) {
    const size_t ncb = static_cast<size_t>(k.cb_bytes);
    const dim3 grid(static_cast<unsigned>(ceil_div(k.nrows, 4)), static_cast<unsigned>(ceil_div(M, MB)));
    if (ncb <= 49152 && ncb % 4 == 0)
        hipLaunchKernelGGL((nvqs_gemv_kernel<XF16, MB, true>), grid, dim3(256), ncb, st, k, w, x, ldx, M, y, ldy, PairSel{});
    else
        hipLaunchKernelGGL((nvqs_gemv_kernel<XF16, MB, false>), grid, dim3(256), 0, st, k, w, x, ldx, M, y, ldy, PairSel{});
    return check_launch("nvqs_gemv");
}

// the same kernel, one row per block row, over the pairs of a MoE decode step (see PairSel)
template <int XF16>
static int nvqs_launch_pairs(const NvqsK &k, const uint8_t *none, const uint16_t *x, int64_t ldx, int n_pairs, float *y, int64_t ldy,
                             const PairSel &sel, hipStream_t st) {
    const size_t ncb = static_cast<size_t>(k.cb_bytes);
    const dim3 grid(static_cast<unsigned>(ceil_div(k.nrows, 4)), static_cast<unsigned>(n_pairs));
    if (ncb <= 49152 && ncb % 4 == 0)
        hipLaunchKernelGGL((nvqs_gemv_kernel<XF16, 1, true>), grid, dim3(256), ncb, st, k, none, x, ldx, n_pairs, y, ldy, sel);
    else
        hipLaunchKernelGGL((nvqs_gemv_kernel<XF16, 1, false>), grid, dim3(256), 0, st, k, none, x, ldx, n_pairs, y, ldy, sel);
    return check_launch("nvqs_gemv_pairs");
}

}  // namespace mfq

using namespace mfq;

static size_t nvqs_align(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

extern "C" int mfq_hip_nvqs_plan(int vector_size, int index_bits, int banks, int index_parity, int out, int neuron_len,
                                 mfq_nvqs_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvqs_plan: null descriptor");
    MFQ_REQUIRE(vector_size == 4 || vector_size == 8, MFQ_ERR_INVALID, "nvqs_plan: vector_size=%d", vector_size);
    MFQ_REQUIRE(index_bits >= 8 && index_bits <= 12, MFQ_ERR_UNSUPPORTED, "nvqs_plan: index_bits=%d", index_bits);
    MFQ_REQUIRE(banks == 1 || banks == 2 || banks == 4, MFQ_ERR_INVALID, "nvqs_plan: banks=%d", banks);
    MFQ_REQUIRE(!index_parity || (vector_size == 8 && index_bits == 8), MFQ_ERR_INVALID,
                "nvqs_plan: index-parity signs need the 256-entry 8-dimensional codebook");
    MFQ_REQUIRE(out > 0 && neuron_len > 0, MFQ_ERR_INVALID, "nvqs_plan: empty tensor");
    d->vector_size = vector_size; d->index_bits = index_bits; d->entries = 1 << index_bits; d->banks = banks;
    d->index_parity = index_parity ? 1 : 0; d->out = out; d->neuron_len = neuron_len;
    d->ng = static_cast<int32_t>(ceil_div(neuron_len, 24));
    d->nvec = static_cast<int32_t>(ceil_div(neuron_len, vector_size));
    d->nsign = static_cast<int32_t>(ceil_div(neuron_len, 8));
    const int64_t ncb = static_cast<int64_t>(banks) * d->entries * vector_size;
    const int64_t st = (static_cast<int64_t>(out) * d->ng * 4 + 7) / 8, ix = (static_cast<int64_t>(out) * d->nvec * index_bits + 7) / 8,
                  sg = (static_cast<int64_t>(out) * d->nsign * 7 + 7) / 8;
    d->tables_off = 0;
    d->anchors_off = static_cast<int64_t>(nvqs_align(128 + static_cast<size_t>(ncb)));
    d->state_off = d->anchors_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(out) * 4));
    d->index_off = d->state_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(st) + 4));
    d->sign_off = d->index_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(ix) + 4));
    d->total_bytes = d->sign_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(sg) + 4));
    d->payload_bytes = 2ll * out + st + ix + sg;
    d->kind = 0; d->state_bits = 4; d->cb_bytes = static_cast<int32_t>(ncb); d->delta = 0.f;
    d->nbank = 0; d->nsuper = 0;
    return MFQ_OK;
}

extern "C" int mfq_hip_nvqs_plan_lowbit(int format, int state_bits, int out, int neuron_len, mfq_nvqs_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvqs_plan_lowbit: null descriptor");
    MFQ_REQUIRE(out > 0 && neuron_len > 0, MFQ_ERR_INVALID, "nvqs_plan_lowbit: empty tensor");
    d->vector_size = 8; d->index_parity = 0; d->out = out; d->neuron_len = neuron_len;
    d->nbank = 0; d->nsuper = 0;
    d->ng = static_cast<int32_t>(ceil_div(neuron_len, 24));
    d->nsign = static_cast<int32_t>(ceil_div(neuron_len, 8));
    d->nvec = d->nsign;
    switch (format) {
    case MFQ_NVQS_NVQ1_L:
        MFQ_REQUIRE(state_bits == 3 || state_bits == 4, MFQ_ERR_UNSUPPORTED, "unsupported NVQ1-L profile: %d-bit scales", state_bits);
        d->kind = 1; d->index_bits = 11; d->entries = 2048; d->banks = 1; d->state_bits = state_bits; d->delta = 0.125f;
        d->cb_bytes = 2048 * 8;
        break;
    case MFQ_NVQS_NVQ1_S:
        MFQ_REQUIRE(neuron_len % 8 == 0, MFQ_ERR_INVALID, "NVQ1-S neuron length must be divisible by 8");
        d->kind = 1; d->index_bits = 9; d->entries = 512; d->banks = 2; d->state_bits = 4; d->delta = 0.15625f;
        d->cb_bytes = 2 * 512 * 8;
        break;
    case MFQ_NVQS_NPQ0_L:
        MFQ_REQUIRE(neuron_len % 8 == 0, MFQ_ERR_INVALID, "NPQ0-L neuron length must be divisible by 8");
        d->kind = 2; d->index_bits = 7; d->entries = 16; d->banks = 8; d->state_bits = 3; d->delta = 0.f;
        d->cb_bytes = 8 * 32 + 8 * 16 * 4;
        break;
    case MFQ_NVQS_NPQ0_S:
        MFQ_REQUIRE(neuron_len % 8 == 0, MFQ_ERR_INVALID, "NPQ0-S neuron length must be divisible by 8");
        d->kind = 2; d->index_bits = 6; d->entries = 8; d->banks = 4; d->state_bits = 2; d->delta = 0.f;
        d->cb_bytes = 4 * 32 + 4 * 8 * 4;
        break;
    default:
        return fail(MFQ_ERR_INVALID, "nvqs_plan_lowbit: format=%d", format);
    }
    const int64_t st = (static_cast<int64_t>(out) * d->ng * d->state_bits + 7) / 8;
    const int64_t ix = (static_cast<int64_t>(out) * d->nvec * d->index_bits + 7) / 8;
    const int64_t sg = d->kind == 1 ? (static_cast<int64_t>(out) * d->ng + 7) / 8 : 0;
    d->tables_off = 0;
    d->anchors_off = static_cast<int64_t>(nvqs_align(128 + static_cast<size_t>(d->cb_bytes)));
    d->state_off = d->anchors_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(out) * 4));
    d->index_off = d->state_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(st) + 4));
    d->sign_off = d->index_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(ix) + 4));
    d->total_bytes = d->sign_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(sg) + 4));
    d->payload_bytes = 2ll * out + st + ix + sg;
    return MFQ_OK;
}

extern "C" int mfq_hip_nvqs_repack_lowbit(const mfq_nvqs_desc *d, const void *body, int64_t body_bytes, const void *grid,
                                          void *weight, mfq_stream_t stream) {
    MFQ_REQUIRE(d && body && weight, MFQ_ERR_INVALID, "nvqs_repack_lowbit: null argument");
    MFQ_REQUIRE(d->kind == 1 || d->kind == 2, MFQ_ERR_INVALID, "nvqs_repack_lowbit: not a 1-bit family descriptor");
    const int64_t table = d->kind == 1 ? 2ll * d->banks * d->entries : 64ll + d->cb_bytes;
    const bool builtin = d->kind == 1 && d->banks == 1 && body_bytes == d->payload_bytes;  // NVQ1-L without a table
    MFQ_REQUIRE(builtin || body_bytes == d->payload_bytes + table, MFQ_ERR_INVALID,
                "nvqs_repack_lowbit: body is %lld bytes, the tensor needs %lld", static_cast<long long>(body_bytes),
                static_cast<long long>(d->payload_bytes + table));
    MFQ_REQUIRE(!builtin || grid, MFQ_ERR_INVALID, "nvqs_repack_lowbit: a blob without a table needs the built-in grid");
    const NvqsK k = to_k(d);
    hipLaunchKernelGGL(nvqs_repack_lowbit_kernel, dim3(1024), dim3(256), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(body), builtin ? 0 : 1, static_cast<const uint16_t *>(grid),
                       static_cast<uint8_t *>(weight));
    return check_launch("nvqs_repack_lowbit");
}

extern "C" int mfq_hip_nvqs_repack(const mfq_nvqs_desc *d, const void *payload, int64_t payload_bytes, int jsc,
                                   const void *grid, void *weight, mfq_stream_t stream) {
    MFQ_REQUIRE(d && payload && weight, MFQ_ERR_INVALID, "nvqs_repack: null argument");
    MFQ_REQUIRE(jsc || grid, MFQ_ERR_INVALID, "nvqs_repack: a plain payload needs its magnitude grid");
    MFQ_REQUIRE(jsc || d->banks == 1, MFQ_ERR_INVALID, "nvqs_repack: a plain payload has one bank");
    const int64_t ncb = static_cast<int64_t>(d->banks) * d->entries * d->vector_size;
    const int64_t expect = d->payload_bytes + (jsc ? 64 + ncb : 0);
    MFQ_REQUIRE(payload_bytes == expect, MFQ_ERR_INVALID, "nvqs_repack: payload is %lld bytes, the tensor needs %lld",
                static_cast<long long>(payload_bytes), static_cast<long long>(expect));
    const NvqsK k = to_k(d);
    hipLaunchKernelGGL(nvqs_repack_kernel, dim3(1024), dim3(256), 0, as_stream(stream), k, static_cast<const uint8_t *>(payload),
                       jsc, static_cast<const int8_t *>(grid), static_cast<uint8_t *>(weight));
    return check_launch("nvqs_repack");
}

extern "C" int mfq_hip_nvqs_plan_nepq0(int profile, int banks, int rows, int neuron_len, mfq_nvqs_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvqs_plan_nepq0: null descriptor");
    MFQ_REQUIRE(profile == 0 || profile == 1, MFQ_ERR_INVALID, "nvqs_plan_nepq0: profile=%d (0: NEPQ0-S, 1: NEPQ0-L)", profile);
    MFQ_REQUIRE(banks >= 1 && banks <= 256, MFQ_ERR_INVALID, "nvqs_plan_nepq0: %d tables (1..256)", banks);
    MFQ_REQUIRE(rows > 0 && neuron_len > 0 && neuron_len % 8 == 0, MFQ_ERR_INVALID,
                "NEPQ shape dimensions must be positive, K divisible by 8");
    int rc = mfq_hip_nvqs_plan_lowbit(profile ? MFQ_NVQS_NPQ0_L : MFQ_NVQS_NPQ0_S, 0, rows, neuron_len, d);
    if (rc) return rc;
    const int per_bank = d->cb_bytes;  // sub-codebooks of one table
    d->kind = 3; d->nbank = banks; d->nsuper = static_cast<int32_t>(ceil_div(d->ng, 4));
    d->cb_bytes = banks * (per_bank + 32);
    const int64_t st = (static_cast<int64_t>(rows) * d->ng * d->state_bits + 7) / 8;
    const int64_t ix = (static_cast<int64_t>(rows) * d->nvec * d->index_bits + 7) / 8;
    const int64_t sel = static_cast<int64_t>(rows) * d->nsuper;
    d->anchors_off = static_cast<int64_t>(nvqs_align(128 + static_cast<size_t>(d->cb_bytes)));
    d->state_off = d->anchors_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(rows) * 4));
    d->index_off = d->state_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(st) + 4));
    d->sign_off = d->index_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(ix) + 4));
    d->total_bytes = d->sign_off + static_cast<int64_t>(nvqs_align(static_cast<size_t>(sel) + 4));
    d->payload_bytes = 2ll * rows + st + ix + sel;
    return MFQ_OK;
}

extern "C" int mfq_hip_nvqs_repack_nepq0(const mfq_nvqs_desc *d, const void *body, int64_t body_bytes, void *weight,
                                         mfq_stream_t stream) {
    MFQ_REQUIRE(d && body && weight, MFQ_ERR_INVALID, "nvqs_repack_nepq0: null argument");
    MFQ_REQUIRE(d->kind == 3, MFQ_ERR_INVALID, "nvqs_repack_nepq0: not a NEPQ0 descriptor");
    const NvqsK k = to_k(d);
    const int64_t expect = static_cast<int64_t>(k.nbank) * (64 + k.bank_bytes) + d->payload_bytes;
    MFQ_REQUIRE(body_bytes == expect, MFQ_ERR_INVALID, "invalid NEPQ tail: remaining=%lld, expected=%lld",
                static_cast<long long>(body_bytes), static_cast<long long>(expect));
    hipLaunchKernelGGL(nvqs_repack_lowbit_kernel, dim3(1024), dim3(256), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(body), 1, static_cast<const uint16_t *>(nullptr),
                       static_cast<uint8_t *>(weight));
    return check_launch("nvqs_repack_nepq0");
}

static bool nvqs_rows_ok(const mfq_nvqs_desc *d, int row0, int nrows) {
    return row0 >= 0 && nrows > 0 && static_cast<int64_t>(row0) + nrows <= d->out;
}

extern "C" int mfq_hip_nvqs_dequant_rows_f32(const mfq_nvqs_desc *d, const void *weight, int row0, int nrows, float *w_out,
                                             int64_t ld, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && w_out, MFQ_ERR_INVALID, "nvqs_dequant_f32: null argument");
    MFQ_REQUIRE(ld >= d->neuron_len, MFQ_ERR_INVALID, "nvqs_dequant_f32: ld smaller than neuron_len");
    MFQ_REQUIRE(nvqs_rows_ok(d, row0, nrows), MFQ_ERR_INVALID, "nvqs_dequant_f32: rows [%d, %d) outside the tensor's %d", row0,
                row0 + nrows, d->out);
    NvqsK k = to_k(d);
    for (int done = 0; done < nrows; done += 65535) {  // the grid's second dimension holds 65535 rows
        k.row0 = row0 + done; k.nrows = nrows - done < 65535 ? nrows - done : 65535;
        hipLaunchKernelGGL((nvqs_dequant_kernel<float>), dim3(static_cast<unsigned>(ceil_div(k.nsign, 256)), k.nrows), dim3(256),
                           0, as_stream(stream), k, static_cast<const uint8_t *>(weight), w_out + static_cast<int64_t>(done) * ld,
                           ld, static_cast<float *>(nullptr), 0);
    }
    return check_launch("nvqs_dequant_f32");
}

extern "C" int mfq_hip_nvqs_gemv_pairs(const mfq_nvqs_desc *d, const void *const *expert_weights, const void *weight,
                                       int out_per_expert, const int32_t *expert_slot, int E, const void *x, int x_dtype,
                                       int64_t ldx, int routed_input, const int32_t *ids, int T, int R, float *y, int64_t ldy,
                                       mfq_stream_t stream) {
    MFQ_REQUIRE(d && (expert_weights || weight) && expert_slot && x && ids && y, MFQ_ERR_INVALID, "nvqs_gemv_pairs: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvqs_gemv_pairs: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(T >= 0 && R >= 1 && E >= 1, MFQ_ERR_INVALID, "nvqs_gemv_pairs: T=%d R=%d E=%d", T, R, E);
    MFQ_REQUIRE(static_cast<int64_t>(T) * R <= 65535, MFQ_ERR_UNSUPPORTED, "nvqs_gemv_pairs: %lld pairs (at most 65535 per launch)",
                static_cast<long long>(T) * R);
    MFQ_REQUIRE(out_per_expert > 0 && (expert_weights ? out_per_expert == d->out : d->out % out_per_expert == 0), MFQ_ERR_INVALID,
                "nvqs_gemv_pairs: %d rows per expert, the tensor has %d", out_per_expert, d->out);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= out_per_expert, MFQ_ERR_INVALID, "nvqs_gemv_pairs: ldx/ldy smaller than the tensor");
    if (T == 0) return MFQ_OK;
    const PairSel sel{ids, expert_slot, reinterpret_cast<const uint8_t *const *>(expert_weights), E, R, routed_input ? 1 : 0};
    NvqsK k = to_k(d);
    k.row0 = 0;
    k.nrows = out_per_expert;
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    {
        int mb;
        E8Shape sh;
        if (nvqs_e8_shape(k, 1, mb, sh))
            return x_dtype == MFQ_X_F16 ? nvqs_launch_e8<1>(k, w, xp, ldx, T * R, y, ldy, 1, sh, sel, T * R, as_stream(stream))
                                        : nvqs_launch_e8<0>(k, w, xp, ldx, T * R, y, ldy, 1, sh, sel, T * R, as_stream(stream));
    }
    return x_dtype == MFQ_X_F16 ? nvqs_launch_pairs<1>(k, w, xp, ldx, T * R, y, ldy, sel, as_stream(stream))
                                : nvqs_launch_pairs<0>(k, w, xp, ldx, T * R, y, ldy, sel, as_stream(stream));
}

extern "C" int mfq_hip_nvqs_embedding(const mfq_nvqs_desc *d, const void *weight, const int64_t *ids, int n_ids, void *out,
                                      int out_dtype, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight, MFQ_ERR_INVALID, "nvqs_embedding: null argument");
    MFQ_REQUIRE(n_ids >= 0, MFQ_ERR_INVALID, "nvqs_embedding: n_ids=%d", n_ids);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16 || out_dtype == MFQ_X_F32, MFQ_ERR_INVALID,
                "nvqs_embedding: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(ldo >= d->neuron_len, MFQ_ERR_INVALID, "nvqs_embedding: ldo %lld < neuron_len %d", static_cast<long long>(ldo),
                d->neuron_len);
    if (n_ids == 0) return MFQ_OK;
    MFQ_REQUIRE(ids && out, MFQ_ERR_INVALID, "nvqs_embedding: null ids or output");
    const NvqsK k = to_k(d);
    const size_t esize = out_dtype == MFQ_X_F32 ? 4 : 2;
    for (int n0 = 0; n0 < n_ids; n0 += 65535) {  // the grid's second dimension holds 65535 rows
        const int rows = n_ids - n0 < 65535 ? n_ids - n0 : 65535;
        hipLaunchKernelGGL(nvqs_embedding_kernel, dim3(static_cast<unsigned>(ceil_div(k.nsign, 256)), static_cast<unsigned>(rows)),
                           dim3(256), 0, as_stream(stream), k, static_cast<const uint8_t *>(weight), ids + n0,
                           static_cast<void *>(static_cast<uint8_t *>(out) + static_cast<size_t>(n0) * ldo * esize), out_dtype, ldo);
    }
    return check_launch("nvqs_embedding");
}

extern "C" int mfq_hip_nvqs_dequant_f32(const mfq_nvqs_desc *d, const void *weight, float *w_out, int64_t ld,
                                        mfq_stream_t stream) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvqs_dequant_f32: null argument");
    return mfq_hip_nvqs_dequant_rows_f32(d, weight, 0, d->out, w_out, ld, stream);
}

extern "C" int mfq_hip_nvqs_gemv_rows(const mfq_nvqs_desc *d, const void *weight, int row0, int nrows, const void *x,
                                      int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nvqs_gemv: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nvqs_gemv: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvqs_gemv: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(nvqs_rows_ok(d, row0, nrows), MFQ_ERR_INVALID, "nvqs_gemv: rows [%d, %d) outside the tensor's %d", row0,
                row0 + nrows, d->out);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= nrows, MFQ_ERR_INVALID, "nvqs_gemv: ldx/ldy smaller than the tensor");
    NvqsK k = to_k(d);
    k.row0 = row0; k.nrows = nrows;
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    hipStream_t st = as_stream(stream);
    {
        E8TileShape ts;
        if (nvqs_e8_tile_shape(k, M, ts))
            return x_dtype == MFQ_X_F16 ? nvqs_launch_e8_tile<1>(k, w, xp, ldx, M, y, ldy, ts, st)
                                        : nvqs_launch_e8_tile<0>(k, w, xp, ldx, M, y, ldy, ts, st);
        int mb;
        E8Shape sh;
        if (nvqs_e8_shape(k, M, mb, sh))
            return x_dtype == MFQ_X_F16 ? nvqs_launch_e8<1>(k, w, xp, ldx, M, y, ldy, mb, sh, PairSel{}, 0, st)
                                        : nvqs_launch_e8<0>(k, w, xp, ldx, M, y, ldy, mb, sh, PairSel{}, 0, st);
    }
    if (x_dtype == MFQ_X_F16) {
        if (M == 1) return nvqs_launch_gemv<1, 1>(k, w, xp, ldx, M, y, ldy, st);
        if (M <= 4) return nvqs_launch_gemv<1, 4>(k, w, xp, ldx, M, y, ldy, st);
        return nvqs_launch_gemv<1, 8>(k, w, xp, ldx, M, y, ldy, st);
    }
    if (M == 1) return nvqs_launch_gemv<0, 1>(k, w, xp, ldx, M, y, ldy, st);
    if (M <= 4) return nvqs_launch_gemv<0, 4>(k, w, xp, ldx, M, y, ldy, st);
    return nvqs_launch_gemv<0, 8>(k, w, xp, ldx, M, y, ldy, st);
}

extern "C" int mfq_hip_nvqs_gemv(const mfq_nvqs_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                                 float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvqs_gemv: null argument");
    return mfq_hip_nvqs_gemv_rows(d, weight, 0, d->out, x, x_dtype, ldx, M, y, ldy, stream);
}

// batches above the GEMV range that the matrix-core tile kernel takes (no workspace)
static bool nvqs_tile_takes(const mfq_nvqs_desc *d, int M) {
    E8TileShape ts;
    return nvqs_e8_tile_shape(to_k(d), M, ts);
}
extern "C" size_t mfq_hip_nvqs_gemm_rows_workspace_bytes(const mfq_nvqs_desc *d, int nrows, int M) {
    if (!d || M <= kNvqsGemvMaxM || nvqs_tile_takes(d, M)) return 0;
    return dequant_gemm_workspace(nrows, d->neuron_len, M);
}
extern "C" size_t mfq_hip_nvqs_gemm_workspace_bytes(const mfq_nvqs_desc *d, int M) {
    return d ? mfq_hip_nvqs_gemm_rows_workspace_bytes(d, d->out, M) : 0;
}

extern "C" int mfq_hip_nvqs_gemm_rows(const mfq_nvqs_desc *d, const void *weight, int row0, int nrows, const void *x,
                                      int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, void *workspace,
                                      size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nvqs_gemm: null argument");
    if (M <= kNvqsGemvMaxM || nvqs_tile_takes(d, M))
        return mfq_hip_nvqs_gemv_rows(d, weight, row0, nrows, x, x_dtype, ldx, M, y, ldy, stream);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nvqs_gemm: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(nvqs_rows_ok(d, row0, nrows), MFQ_ERR_INVALID, "nvqs_gemm: rows [%d, %d) outside the tensor's %d", row0,
                row0 + nrows, d->out);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= nrows, MFQ_ERR_INVALID, "nvqs_gemm: ldx/ldy smaller than the tensor");
    MFQ_REQUIRE(nrows <= 65535, MFQ_ERR_UNSUPPORTED, "nvqs_gemm: %d neurons in one call (max 65535)", nrows);
    const size_t need = dequant_gemm_workspace(nrows, d->neuron_len, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nvqs_gemm: workspace %zu < %zu bytes", workspace_bytes,
                need);
    hipStream_t st = as_stream(stream);
    uint16_t *x16, *w16;
    float *xscale, *wscale;
    int Kp;
    dequant_gemm_carve(workspace, nrows, d->neuron_len, M, x16, xscale, w16, wscale, Kp);
    int rc = x_prep(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, st);
    if (rc) return rc;
    NvqsK k = to_k(d);
    k.row0 = row0; k.nrows = nrows;
    hipLaunchKernelGGL((nvqs_dequant_kernel<uint16_t>), dim3(static_cast<unsigned>(ceil_div(Kp / 8 > k.nsign ? Kp / 8 : k.nsign, 256)), nrows),
                       dim3(256), 0, st, k, static_cast<const uint8_t *>(weight), w16, static_cast<int64_t>(Kp), wscale, Kp);
    rc = check_launch("nvqs_dequant_f16");
    if (rc) return rc;
    return gemm_f16_nt(x16, Kp, w16, Kp, M, nrows, Kp, xscale, wscale, y, ldy, st, dequant_gemm_part(wscale, nrows, d->neuron_len, M));
}

extern "C" int mfq_hip_nvqs_gemm(const mfq_nvqs_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M,
                                 float *y, int64_t ldy, void *workspace, size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nvqs_gemm: null argument");
    return mfq_hip_nvqs_gemm_rows(d, weight, 0, d->out, x, x_dtype, ldx, M, y, ldy, workspace, workspace_bytes, stream);
}
