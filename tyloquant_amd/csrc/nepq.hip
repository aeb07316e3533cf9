// NEPQ1-S / NEPQ1-L: 8-dim ternary code vectors from a cross-expert table pool, one bank id per
// 96 weights, per-group integer state (scale), one delta-sign bit per group.
//
// Device layout (rows = experts * out_per_expert neurons, same row-block / step / lane interleave):
//   NEPQ1-S unit = one dword   idx0 | idx1 << 9 | idx2 << 18 | state << 27 | aux << 31
//   NEPQ1-L unit = dword + byte  idx0 | idx1 << 11 | (idx2 & 1023) << 22 ;  (idx2 >> 10) | state << 1 | aux << 4
//   step = Q [j][lane] dwords, T [lane][4 bytes] (L only), B [16 neurons][4 bank ids (one per j)]
// tail: uint16 table[banks][entries] (S: aux * 512 + idx, L: idx; 8 two-bit digits = code + 1 each),
//       float anchor[].
// value = fl(anchor * state) * (code + bias), bias = +-5/32 (S) or +-1/8 (L), minus when aux is set.
#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_prefill.hpp"

namespace mfq {

struct NepqK {
    int profile, sb, ib, banks, rows, neuron_len, ng, nvec, nsuper, nsteps, n_rowblocks, entries, tail;
    int64_t step_bytes, rowblock_bytes, tables_off, anchors_off;
};

static NepqK to_k(const mfq_nepq_desc *d) {
    NepqK k;
    k.profile = d->profile; k.sb = d->state_bits; k.ib = d->index_bits; k.banks = d->banks; k.rows = d->rows;
    k.neuron_len = d->neuron_len; k.ng = d->ng; k.nvec = d->nvec; k.nsuper = d->nsuper; k.nsteps = d->nsteps;
    k.n_rowblocks = d->n_rowblocks; k.entries = d->table_entries; k.tail = d->profile == 3 ? 1 : 0;
    k.step_bytes = d->step_bytes; k.rowblock_bytes = d->rowblock_bytes; k.tables_off = d->tables_off;
    k.anchors_off = d->anchors_off;
    return k;
}

struct NepqUnit {
    uint32_t idx[3], state, aux;
};
__device__ __forceinline__ NepqUnit nepq_decode(int profile, uint32_t d, uint32_t t) {
    NepqUnit u;
    if (profile == 2) {
        u.idx[0] = d & 511u; u.idx[1] = (d >> 9) & 511u; u.idx[2] = (d >> 18) & 511u;
        u.state = (d >> 27) & 15u; u.aux = d >> 31;
        // the S table is indexed by aux * 512 + idx
        u.idx[0] += u.aux << 9; u.idx[1] += u.aux << 9; u.idx[2] += u.aux << 9;
    } else {
        u.idx[0] = d & 2047u; u.idx[1] = (d >> 11) & 2047u; u.idx[2] = (d >> 22) | ((t & 1u) << 10);
        u.state = (t >> 1) & 7u; u.aux = (t >> 4) & 1u;
    }
    return u;
}

__global__ void nepq_repack_kernel(NepqK k, const uint8_t *__restrict__ payload, uint8_t *__restrict__ dst) {
    const int lane = threadIdx.x;
    const int rb = blockIdx.x, s = blockIdx.y;
    const int r = lane & 15, kb = lane >> 4;
    const int row = rb * 16 + r;
    const int64_t rows = k.rows;
    const int64_t tb = static_cast<int64_t>(k.banks) * k.entries * 2;
    const int64_t st_bytes = (rows * k.ng * k.sb + 7) / 8, ix_bytes = (rows * k.nvec * k.ib + 7) / 8,
                  ax_bytes = (rows * k.ng + 7) / 8;
    const uint8_t *an_s = payload + tb;
    const uint8_t *st_s = an_s + 2 * rows;
    const uint8_t *ix_s = st_s + st_bytes;
    const uint8_t *ax_s = ix_s + ix_bytes;
    const uint8_t *bk_s = ax_s + ax_bytes;
    uint8_t *sp = dst + rb * k.rowblock_bytes + s * k.step_bytes;
    uint32_t *qreg = reinterpret_cast<uint32_t *>(sp);
    uint8_t *treg = sp + 1024;
    uint8_t *breg = treg + (k.tail ? 256 : 0);
    for (int j = 0; j < 4; ++j) {
        const int g = 16 * s + 4 * j + kb;
        uint32_t d = 0, t = 0;
        if (row < k.rows && g < k.ng) {
            uint32_t idx[3];
            for (int v = 0; v < 3; ++v) {
                const int vi = 3 * g + v;
                idx[v] = vi < k.nvec ? read_bits(ix_s, static_cast<int64_t>(row) * k.nvec + vi, k.ib, ix_bytes) : 0u;
            }
            const uint32_t state = read_bits(st_s, static_cast<int64_t>(row) * k.ng + g, k.sb, st_bytes);
            const uint32_t aux = read_bits(ax_s, static_cast<int64_t>(row) * k.ng + g, 1, ax_bytes);
            if (k.profile == 2) {
                d = idx[0] | (idx[1] << 9) | (idx[2] << 18) | (state << 27) | (aux << 31);
            } else {
                d = idx[0] | (idx[1] << 11) | ((idx[2] & 1023u) << 22);
                t = (idx[2] >> 10) | (state << 1) | (aux << 4);
            }
        }
        qreg[j * 64 + lane] = d;
        if (k.tail) treg[lane * 4 + j] = static_cast<uint8_t>(t);
        if (kb == 0) {
            const int sg = 4 * s + j;
            breg[r * 4 + j] = (row < k.rows && sg < k.nsuper) ? bk_s[static_cast<int64_t>(row) * k.nsuper + sg] : 0;
        }
    }
    if (s == 0 && kb == 0) {
        float *anchors = reinterpret_cast<float *>(dst + k.anchors_off);
        anchors[row] = row < k.rows ? f16_to_f32(reinterpret_cast<const uint16_t *>(an_s)[row]) : 0.f;
    }
    if (rb == 0 && s == 0) {
        uint16_t *tab = reinterpret_cast<uint16_t *>(dst + k.tables_off);
        const uint16_t *src = reinterpret_cast<const uint16_t *>(payload);
        for (int i = lane; i < k.banks * k.entries; i += 64) tab[i] = src[i];
    }
}

template <typename OutT>
__global__ void nepq_dequant_kernel(NepqK k, const uint8_t *__restrict__ w, int rb0, int row0, int nrows,
                                    OutT *__restrict__ outp, int64_t ld, float *__restrict__ rowscale, int kpad) {
    const int lane = threadIdx.x;
    const int rb = rb0 + blockIdx.x, s = blockIdx.y;
    const int r = lane & 15, kb = lane >> 4;
    const int row = rb * 16 + r;
    const int orow = row - row0;
    if (orow < 0 || orow >= nrows) return;
    const uint8_t *sp = w + rb * k.rowblock_bytes + s * k.step_bytes;
    const uint32_t *qreg = reinterpret_cast<const uint32_t *>(sp);
    const uint8_t *treg = sp + 1024;
    const uint8_t *breg = treg + (k.tail ? 256 : 0);
    const uint16_t *tab = reinterpret_cast<const uint16_t *>(w + k.tables_off);
    const float anchor = reinterpret_cast<const float *>(w + k.anchors_off)[row];
    const float delta = k.profile == 2 ? 0.15625f : 0.125f;
    float inv = 1.f;
    if constexpr (sizeof(OutT) == 2) {
        const float bound = anchor * static_cast<float>((1 << k.sb) - 1) * 1.25f;
        int e = 0;
        if (bound > 0.f) frexpf(bound, &e);
        inv = ldexpf(1.f, 12 - e);
        if (s == 0 && kb == 0) {
            rowscale[orow] = ldexpf(1.f, e - 12);
            for (int col = k.neuron_len; col < kpad; ++col) outp[orow * ld + col] = 0;
        }
    }
    for (int j = 0; j < 4; ++j) {
        const int g = 16 * s + 4 * j + kb;
        if (g >= k.ng) continue;
        const NepqUnit u = nepq_decode(k.profile, qreg[j * 64 + lane], k.tail ? treg[lane * 4 + j] : 0u);
        const uint16_t *bank = tab + static_cast<int64_t>(breg[r * 4 + j]) * k.entries;
        const float scale = __fmul_rn(anchor, static_cast<float>(u.state));
        const float bias = u.aux ? -delta : delta;
        for (int i = 0; i < 24; ++i) {
            const int col = g * 24 + i;
            if (col >= k.neuron_len) break;
            const uint32_t e = bank[u.idx[i >> 3]];
            const float code = static_cast<float>(static_cast<int>((e >> (2 * (i & 7))) & 3u) - 1);
            const float v = __fmul_rn(scale, __fadd_rn(code, bias));
            if constexpr (sizeof(OutT) == 2) outp[orow * ld + col] = f32_to_f16_rne(v * inv);
            else outp[orow * ld + col] = v;
        }
    }
}

// GEMV: sum_i (code_i + bias) x_i = sum_i digit_i x_i + (bias - 1) * xsum, digit = code + 1 in {0,1,2};
// a table entry e (8 two-bit digits) becomes four biased pairs from t = e | e << 14.
// A block owns RPB consecutive row-blocks: the lookup table and the activations are staged once for all of them, and a
// wave requests the units of all its row-blocks of a step before it decodes the first.
// PROF: the profile (2 = S, 3 = L) as a constant -- a decoder that branches on it at run time splits every unit into
// basic blocks the scheduler cannot mix, and the kernel spills.
template <int XF16, int MB, int TAB_LDS, int RPB, int PROF>
__global__ __launch_bounds__(1024) void nepq_gemv_kernel(NepqK k, const uint8_t *__restrict__ w_in, int rb0, int row0,
                                                         int nrows, const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                         float *__restrict__ y, int64_t ldy, int spw, PairSel sel) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr uint32_t MAGIC = 0x64006400u;  // fp16 (1024, 1024): digit d becomes 1024 + d
    constexpr float BIAS = 1024.f;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const uint16_t *xr[MB];
    float *yr[MB];
    const uint8_t *w = w_in;
    int local;
    if (!select_rows<MB>(sel, w, local, x, ldx, y, ldy, M, xr, yr)) return;
    if (sel.ids) {  // a pair of a MoE decode step: the expert's rows of the expert-shaped tensor (nrows = rows per expert)
        row0 = local * nrows;
        rb0 = row0 / 16;
    }
    const int rb = rb0 + blockIdx.x * RPB;
    const int rb_last = rb0 + (nrows + 15) / 16 - 1;  // row-blocks past it repeat it; their sums are dropped
    const uint16_t *gtab = reinterpret_cast<const uint16_t *>(w + k.tables_off);
    const int ntab = k.banks * k.entries;  // u16 entries
    uint16_t *ltab = reinterpret_cast<uint16_t *>(lds);
    uint32_t *xbase = lds;
    if constexpr (TAB_LDS) {
        table_to_lds(lds, reinterpret_cast<const uint32_t *>(gtab), ntab / 2, tid, blockDim.x);
        xbase = lds + ntab / 2;
    }
    const uint16_t *tab = TAB_LDS ? ltab : gtab;
    const int s0 = wave * spw;
    const int s1 = min(k.nsteps, s0 + spw);
    const int ngl = spw * 16, npairs = ngl * 12;
    uint32_t *xs = xbase + wave * (MB * (npairs + 2 * ngl));
    float *xsum = reinterpret_cast<float *>(xs + MB * npairs);
    float *red = reinterpret_cast<float *>(xbase + nwaves * (MB * (npairs + 2 * ngl)));
    XRegs<MB> xg;
    stage_x_issue<MB>(xr, k.neuron_len, s0 * 16 * 24, npairs, lane, xg);
    float xinv[MB];  // bf16 rows are staged times a per-wave power of two; the sums are scaled back below
    stage_x<XF16, MB, PlainBias, true>(xr, k.neuron_len, s0 * 16 * 24, npairs, 24, ngl, xs, xsum, lane, xg, xinv);
    if constexpr (TAB_LDS) __syncthreads();  // the LDS table copy was made by the whole block

    const int r = lane & 15, kb = lane >> 4;
    const float delta = PROF == 2 ? 0.15625f : 0.125f;
    // requested here, ahead of the weights: at the end of the kernel each would cost a round trip to memory
    float anchor[RPB];
#pragma unroll
    for (int i = 0; i < RPB; ++i) anchor[i] = reinterpret_cast<const float *>(w + k.anchors_off)[min(rb + i, rb_last) * 16 + r];
    float acc[RPB][MB];
#pragma unroll
    for (int i = 0; i < RPB; ++i)
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[i][m] = 0.f;
    for (int s = s0; s < s1; ++s) {
        uint32_t q[RPB][4], tails[RPB], banks4[RPB];
#pragma unroll
        for (int i = 0; i < RPB; ++i) {
            const uint8_t *sp = w + static_cast<int64_t>(min(rb + i, rb_last)) * k.rowblock_bytes + s * k.step_bytes;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                q[i][j] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sp) + j * 64 + lane);
            tails[i] = 0;
            if ((PROF == 3)) tails[i] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sp + 1024) + lane);
            banks4[i] = *(reinterpret_cast<const uint32_t *>(sp + 1024 + ((PROF == 3) ? 256 : 0)) + r);
        }
        // unit column by unit column: the twelve activation pairs of a column are read once for all row-blocks
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int i = 0; i < RPB; ++i) {
                const int lg = (s - s0) * 16 + 4 * j + kb;
                const NepqUnit u = nepq_decode(PROF, q[i][j], (tails[i] >> (8 * j)) & 0xffu);
                const uint16_t *bank = tab + ((banks4[i] >> (8 * j)) & 0xffu) * k.entries;
                const float st = static_cast<float>(u.state);
                const float off = (u.aux ? -delta : delta) - 1.f - BIAS;
                float raw[MB];
#pragma unroll
                for (int m = 0; m < MB; ++m) raw[m] = 0.f;
#pragma unroll
                for (int v = 0; v < 3; ++v) {
                    const uint32_t e = bank[u.idx[v]];
                    const uint32_t t = e | (e << 14);
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const uint32_t pr = ((t >> (4 * p)) & 0x00030003u) | MAGIC;
#pragma unroll
                        for (int m = 0; m < MB; ++m) raw[m] = dot2h(pr, xs[m * npairs + lg * 12 + 4 * v + p], raw[m]);
                    }
                }
#pragma unroll
                for (int m = 0; m < MB; ++m) acc[i][m] = fmaf(st, fmaf(off, xsum[(m * ngl + lg) * 2], raw[m]), acc[i][m]);
                // one unit at a time: left alone, the scheduler starts the table reads of all units at once and spills
                if constexpr (RPB > 1 || MB > 2) __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RPB; ++i) {
        float v[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) v[m] = anchor[i] * acc[i][m] * xinv[m];
        park_rows<MB>(v, red, i * nwaves + wave, lane);
    }
    // a row-block past the tensor's last has rows beyond nrows: flush_rows drops them
    flush_rows<MB>(red, nwaves, RPB, rb, row0, nrows, yr);
}

// ---- matrix-core path: up to 16 activation rows per streamed pass ----------------------------------
// Same scheme as the NINT kernel (nint_mfma.hpp).  Fragment m of a unit is one table entry: 8 two-bit digits
// (code + 1) that become four (1024 + digit) fp16 pairs and, with one packed FMA each, state * digit (exact).
// The remaining part of the value, state * (bias - 1) * X_g, is one more MFMA per step against the group sums
// X_g (two fp16 halves), exactly as the NINT minimum term.  Padding groups have state 0.
template <int XF16, int NB, int TAB_LDS, int PROF>
__global__ __launch_bounds__(512) void nepq_mfma_kernel(NepqK k, const uint8_t *__restrict__ w, int rb_first, int row0,
                                                        int nrows, const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                        float *__restrict__ y, int64_t ldy, int spw) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint16_t *gtab = reinterpret_cast<const uint16_t *>(w + k.tables_off);
    const int ntab = k.banks * k.entries;  // u16 entries
    float *red = reinterpret_cast<float *>(lds);
    if constexpr (TAB_LDS) {
        table_to_lds(lds, reinterpret_cast<const uint32_t *>(gtab), ntab / 2, tid, blockDim.x);
        red = reinterpret_cast<float *>(lds + ntab / 2);
    }
    const uint16_t *tab = TAB_LDS ? reinterpret_cast<const uint16_t *>(lds) : gtab;
    const int rbl0 = blockIdx.x * NB, m0 = blockIdx.y * 16;  // row-blocks relative to rb_first
    const int rb0 = rb_first + rbl0, rb_end = rb_first + (nrows + 15) / 16;
    const int tok = min(m0 + (lane & 15), M - 1);
    const uint16_t *xrow = x + static_cast<int64_t>(tok) * ldx;
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;
    const int nrb = min(NB, rb_end - rb0);
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    float anchor[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
        anchor[i] = reinterpret_cast<const float *>(w + k.anchors_off)[min(rb0 + i, k.n_rowblocks - 1) * 16 + r];
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb0) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);
    float4_t acc[NB], accB[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) acc[i] = accB[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    if constexpr (TAB_LDS) __syncthreads();

    const float delta = PROF == 2 ? 0.15625f : 0.125f;
    const uint32_t toff = 1024u, boff = 1024u + ((PROF == 3) ? 256u : 0u);
    // Software pipeline as in nint_mfma_body: the four unit dwords of a row-block are refilled unit by unit for the
    // next step, tails and bank bytes one step ahead, activation fragments two units ahead and before the refill.
    uint32_t q[NB][4], tails[NB], banks4[NB], tailsn[NB], banks4n[NB];
    auto unit_off = [&](int i, int s, int j) -> uint32_t {
        return i < nrb && s < n ? i * rbb + s * sb + (j * 64 + lane) * 4 : kNoStep;
    };
    auto side_load = [&](int s, uint32_t (&tt)[NB], uint32_t (&bb)[NB]) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const uint32_t off = i < nrb && s < n ? i * rbb + s * sb : kNoStep;
            tt[i] = (PROF == 3) ? __builtin_amdgcn_raw_buffer_load_b32(win, off + toff + lane * 4, 0, 2) : 0u;
            bb[i] = __builtin_amdgcn_raw_buffer_load_b32(win, off + boff + r * 4, 0, 2);
        }
    };
    auto xfrags = [&](int it, u32x4_t (&dst)[3]) {
        const int kpos = (s0 + (it >> 2)) * 16 * 24 + kb * 24 + 4 * (it & 3) * 24;
#pragma unroll
        for (int m = 0; m < 3; ++m) dst[m] = load_xfrag_raw<true>(xrow, kpos + 8 * m, k.neuron_len);
    };
    side_load(0, tails, banks4);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < NB; ++i) q[i][j] = __builtin_amdgcn_raw_buffer_load_b32(win, unit_off(i, 0, j), 0, 2);
    u32x4_t a1[3], a2[3];
    xfrags(0, a1);
    xfrags(1, a2);
    for (int s = 0; s < n; ++s) {
        side_load(s + 1, tailsn, banks4n);
        float xsum[4];
        uint32_t stw[NB][4];  // per unit: state * (bias - 1) as an fp16
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x4_t a[3];
#pragma unroll
            for (int m = 0; m < 3; ++m) {
                a[m] = xfrag_finish<XF16, true>(a1[m], (s0 + s) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len);
                a1[m] = a2[m];
            }
            xfrags(4 * s + j + 2, a2);
            float xs = 0.f;
#pragma unroll
            for (int m = 0; m < 3; ++m)
#pragma unroll
                for (int t = 0; t < 4; ++t) xs = dot2h(a[m][t], 0x3c003c00u, xs);
            xsum[j] = xs;
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const NepqUnit u = nepq_decode(PROF, q[i][j], (tails[i] >> (8 * j)) & 0xffu);
                q[i][j] = __builtin_amdgcn_raw_buffer_load_b32(win, unit_off(i, s + 1, j), 0, 2);
                const uint16_t *bank = tab + ((banks4[i] >> (8 * j)) & 0xffu) * k.entries;
                const float st = static_cast<float>(u.state);
                const half2_t S = pk_h2(st, st), C = pk_h2(-1024.f * st, -1024.f * st);
                stw[i][j] = f32_to_f16_rne(st * ((u.aux ? -delta : delta) - 1.f));
#pragma unroll
                for (int m = 0; m < 3; ++m) {
                    const uint32_t e = bank[u.idx[m]];
                    const uint32_t t2 = e | (e << 14);
                    u32x4_t b;
#pragma unroll
                    for (int p = 0; p < 4; ++p)
                        b[p] = __builtin_bit_cast(uint32_t, h2_fma(((t2 >> (4 * p)) & 0x00030003u) | kMagicH2, S, C));
                    acc[i] = mfma16(a[m], b, acc[i]);
                }
            }
            // Keeps the requests of this unit (activation fragments two units ahead, the refill of its registers) where
            // they are written: the scheduler otherwise sinks every refill to the end of the step, and the next step
            // begins with a wait for all of them.
            __builtin_amdgcn_sched_barrier(0);
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
            const uint32_t b01 = stw[i][0] | (stw[i][1] << 16), b23 = stw[i][2] | (stw[i][3] << 16);
            accB[i] = mfma16(ax, u32x4_t{b01, b23, b01, b23}, accB[i]);
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            tails[i] = tailsn[i];
            banks4[i] = banks4n[i];
        }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * NB + i) * 4 + v) * 64 + lane] = anchor[i] * (acc[i][v] + accB[i][v]);
    // rows are relative to row0 in y
    __syncthreads();
    const int nwaves = blockDim.x >> 6;
    for (int o = threadIdx.x; o < NB * 256; o += blockDim.x) {
        const int rr = o & 15, t = (o >> 4) & 15, nb = o >> 8;
        const int slot = (nb * 4 + (t & 3)) * 64 + rr + 16 * (t >> 2);
        float sacc = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) sacc += red[wv * NB * 256 + slot];
        const int row = (rb0 + nb) * 16 + rr - row0;
        if (m0 + t < M && row >= 0 && row < nrows) y[static_cast<int64_t>(m0 + t) * ldy + row] = sacc;
    }
}

// ---- 16-row tiles, one block per compute unit --------------------------------------------------------------
// The kernel above re-reads the 16 activation rows (and the lookup tables) once per block: 128 KB at K = 4096, which on a
// 1.5-bit format is eight times the block's own weights when a wave owns one row-block.  Here a block owns RPB consecutive
// row-blocks and its waves split the K steps: a wave requests the units of its first step for all its row-blocks and the
// step's activation fragments (48 registers, converted once and shared by the row-blocks) before the table copy, then
// walks the row-blocks unit by unit, refilling each unit's register for the next step as soon as it is decoded.  The
// bias term goes into the same accumulator as the digits.
// LDS: [table: banks * entries u16, when TAB_LDS][red: waves * RPB * 1 KB]
template <int XF16, int RPB, int TAB_LDS, int PROF>
__global__ __launch_bounds__(1024) void nepq_tile_kernel(NepqK k, const uint8_t *__restrict__ w, int rb_first, int row0,
                                                         int nrows, const uint16_t *__restrict__ x, int64_t ldx, int M,
                                                         float *__restrict__ y, int64_t ldy, int spw) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr bool TAIL = PROF == 3;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint16_t *gtab = reinterpret_cast<const uint16_t *>(w + k.tables_off);
    const int ntab = k.banks * k.entries;  // u16 entries
    float *red = reinterpret_cast<float *>(lds + (TAB_LDS ? ntab / 2 : 0));
    const uint16_t *tab = TAB_LDS ? reinterpret_cast<const uint16_t *>(lds) : gtab;
    const int rb0 = rb_first + static_cast<int>(blockIdx.x) * RPB, rb_end = rb_first + (nrows + 15) / 16;
    const int m0 = static_cast<int>(blockIdx.y) * 16;
    const int tok = min(m0 + (lane & 15), M - 1);
    const uint16_t *xrow = x + static_cast<int64_t>(tok) * ldx;
    const int r = lane & 15, kb = lane >> 4;
    const int s0 = wave * spw;
    const int n = min(k.nsteps, s0 + spw) - s0;  // may be <= 0: the wave only takes part in the barriers
    const int nrb = min(RPB, rb_end - rb0);
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(rb0) * k.rowblock_bytes + static_cast<int64_t>(s0) * sb,
                    n > 0 ? (nrb - 1) * rbb + n * sb : 0u);
    constexpr uint32_t toff = 1024u, boff = 1024u + (TAIL ? 256u : 0u);
    uint32_t q[RPB][4], tails[RPB], banks4[RPB];
    auto step_off = [&](int i, int ls) -> uint32_t { return i < nrb && ls < n ? i * rbb + ls * sb : kNoStep; };
    auto side_load = [&](int i, int ls, uint32_t &tt, uint32_t &bb) {
        const uint32_t off = step_off(i, ls);
        tt = TAIL ? __builtin_amdgcn_raw_buffer_load_b32(win, off + toff + lane * 4, 0, 2) : 0u;
        bb = __builtin_amdgcn_raw_buffer_load_b32(win, off + boff + r * 4, 0, 2);
    };
    u32x4_t xf[4][3];
    auto xload = [&](int ls) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int m = 0; m < 3; ++m)
                xf[j][m] = load_xfrag_raw<true>(xrow, (s0 + ls) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len);
    };
    // everything the first step needs, before the table copy: the weights come from HBM, the rest from L2; the anchors
    // too (at the end of the kernel they would cost a round trip to memory of their own)
    float anchor[RPB];
#pragma unroll
    for (int i = 0; i < RPB; ++i)
        anchor[i] = reinterpret_cast<const float *>(w + k.anchors_off)[min(rb0 + i, k.n_rowblocks - 1) * 16 + r];
#pragma unroll
    for (int i = 0; i < RPB; ++i) {
        side_load(i, 0, tails[i], banks4[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) q[i][j] = __builtin_amdgcn_raw_buffer_load_b32(win, step_off(i, 0) + (j * 64 + lane) * 4, 0, 2);
    }
    if (n > 0) xload(0);
    if constexpr (TAB_LDS) {
        table_to_lds(lds, reinterpret_cast<const uint32_t *>(gtab), ntab / 2, tid, blockDim.x);
        __syncthreads();
    }

    const float delta = PROF == 2 ? 0.15625f : 0.125f;
    float4_t acc[RPB];
#pragma unroll
    for (int i = 0; i < RPB; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int ls = 0; ls < n; ++ls) {
        // the step's activations as fp16 fragments and the group sums the bias term multiplies
        u32x4_t ax;
        {
            float xsum[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float xs = 0.f;
#pragma unroll
                for (int m = 0; m < 3; ++m) {
                    xf[j][m] = xfrag_finish<XF16, true>(xf[j][m], (s0 + ls) * 16 * 24 + kb * 24 + 4 * j * 24 + 8 * m, k.neuron_len);
#pragma unroll
                    for (int t = 0; t < 4; ++t) xs = dot2h(xf[j][m][t], 0x3c003c00u, xs);
                }
                xsum[j] = xs;
            }
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
        for (int i = 0; i < RPB; ++i) {
            uint32_t tailsn, banksn;
            side_load(i, ls + 1, tailsn, banksn);
            uint32_t stw[4];  // per unit: state * (bias - 1) as an fp16
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const NepqUnit u = nepq_decode(PROF, q[i][j], (tails[i] >> (8 * j)) & 0xffu);
                q[i][j] = __builtin_amdgcn_raw_buffer_load_b32(win, step_off(i, ls + 1) + (j * 64 + lane) * 4, 0, 2);
                const uint16_t *bank = tab + ((banks4[i] >> (8 * j)) & 0xffu) * k.entries;
                const float st = static_cast<float>(u.state);
                const half2_t S = pk_h2(st, st), C = pk_h2(-1024.f * st, -1024.f * st);
                stw[j] = f32_to_f16_rne(st * ((u.aux ? -delta : delta) - 1.f));
#pragma unroll
                for (int m = 0; m < 3; ++m) {
                    const uint32_t e = bank[u.idx[m]];
                    const uint32_t t2 = e | (e << 14);
                    u32x4_t b;
#pragma unroll
                    for (int p = 0; p < 4; ++p)
                        b[p] = __builtin_bit_cast(uint32_t, h2_fma(((t2 >> (4 * p)) & 0x00030003u) | kMagicH2, S, C));
                    acc[i] = mfma16(xf[j][m], b, acc[i]);
                }
                __builtin_amdgcn_sched_barrier(0);  // the refill stays with its unit (the scheduler would sink it)
            }
            const uint32_t b01 = stw[0] | (stw[1] << 16), b23 = stw[2] | (stw[3] << 16);
            acc[i] = mfma16(ax, u32x4_t{b01, b23, b01, b23}, acc[i]);
            tails[i] = tailsn;
            banks4[i] = banksn;
        }
        if (ls + 1 < n) xload(ls + 1);
    }
#pragma unroll
    for (int i = 0; i < RPB; ++i) {
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * RPB + i) * 4 + v) * 64 + lane] = anchor[i] * acc[i][v];
    }
    __syncthreads();
    const int nwaves = blockDim.x >> 6;
    for (int o = threadIdx.x; o < RPB * 256; o += blockDim.x) {
        const int rr = o & 15, t = (o >> 4) & 15, nb = o >> 8;
        const int slot = (nb * 4 + (t & 3)) * 64 + rr + 16 * (t >> 2);
        float sacc = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) sacc += red[wv * RPB * 256 + slot];
        const int row = (rb0 + nb) * 16 + rr - row0;  // rows are relative to row0 in y
        if (m0 + t < M && nb < nrb && row >= 0 && row < nrows) y[static_cast<int64_t>(m0 + t) * ldy + row] = sacc;
    }
}

// ---- prefill: block-tiled MFMA GEMM, weight fragments built from the ternary tables ------------------------
// Same frame as the NVQ prefill kernel: block = 8 waves x NB row-blocks, wave tile MT * 16 tokens, activations as
// scaled fp16 rows (x_prep) through two LDS buffers with XD tiles in flight, PF unit dwords per row-block in flight.
// A fragment is one table entry: (1024 + digit) pairs -> state * digit with one exact packed FMA, plus
// state * (bias - 1) with one packed add (exact for the 1/8 bias, one fp16 rounding for 5/32), so no separate bias
// term is needed.  Rows [row0, row0 + nrows) of the tensor (an expert's slice) go to columns 0 .. nrows - 1 of y.
// LDS: [table: banks * entries u16, when TAB_LDS][x tiles]
template <int MT, int NB, int PF, int XD, int TAB_LDS, int PROF>
__global__ __launch_bounds__(512) void nepq_prefill_kernel(NepqK k, const uint8_t *__restrict__ w, int rb_first, int row0,
                                                           int nrows, const uint16_t *__restrict__ x16, int Kp,
                                                           const float *__restrict__ xscale, int M,
                                                           float *__restrict__ y, int64_t ldy, int spz, int64_t ystride) {
    static_assert((PF == 2 || PF == 4) && (XD == 1 || XD == 2 || XD == 4), "the sub-step loop is unrolled four times");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr int GS = 24, NM = 3, NT = 512, BM = MT * 16, EL = 8;
    constexpr int ROW = 4 * GS + 8;
    constexpr int CPG = GS / EL, CHUNKS = 4 * CPG;
    constexpr int PER_THREAD = (BM * CHUNKS + NT - 1) / NT;
    const int s_begin = static_cast<int>(blockIdx.z) * spz, s_end = min(k.nsteps, s_begin + spz);
    y += static_cast<int64_t>(blockIdx.z) * ystride;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kb = lane >> 4;
    const uint16_t *gtab = reinterpret_cast<const uint16_t *>(w + k.tables_off);
    const int ntab = k.banks * k.entries;  // u16 entries, even
    uint16_t *xt = reinterpret_cast<uint16_t *>(lds);
    if constexpr (TAB_LDS) {
        table_to_lds(lds, reinterpret_cast<const uint32_t *>(gtab), ntab / 2, tid, NT);
        xt = reinterpret_cast<uint16_t *>(lds + (ntab / 2 + 3) / 4 * 4);
    }
    const uint16_t *tab = TAB_LDS ? reinterpret_cast<const uint16_t *>(lds) : gtab;
    const DenseRows rows{static_cast<int>(blockIdx.y) * BM, M};
    const int rb_end = rb_first + (nrows + 15) / 16;
    const int rb0 = rb_first + (static_cast<int>(blockIdx.x) * 8 + wave) * NB;
    const int nrb = max(0, min(NB, rb_end - rb0));
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
    const uint32_t toff = 1024u, boff = 1024u + ((PROF == 3) ? 256u : 0u);
    uint32_t qr[PF][NB], tails[NB], banks4[NB], tailsn[NB], banks4n[NB];
    auto wload = [&](int it, uint32_t (&qq)[NB]) {
        const int s = it >> 2, j = it & 3;
#pragma unroll
        for (int b = 0; b < NB; ++b)
            qq[b] = __builtin_amdgcn_raw_buffer_load_b32(win, b < nrb && s < s_end ? b * rbb + s * sb + (j * 64 + lane) * 4 : kNoStep,
                                                         0, 0);
    };
    auto side_load = [&](int s, uint32_t (&tt)[NB], uint32_t (&bb)[NB]) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t off = b < nrb && s < s_end ? b * rbb + s * sb : kNoStep;
            tt[b] = (PROF == 3) ? __builtin_amdgcn_raw_buffer_load_b32(win, off + toff + lane * 4, 0, 0) : 0u;
            bb[b] = __builtin_amdgcn_raw_buffer_load_b32(win, off + boff + r * 4, 0, 0);
        }
    };
    xload(4 * s_begin, xr[0]);
#pragma unroll
    for (int i = 0; i < PF - 1; ++i) wload(4 * s_begin + i, qr[i]);
    side_load(s_begin, tails, banks4);
    xstore(0, xr[0]);
#pragma unroll
    for (int i = 1; i < XD; ++i) xload(4 * s_begin + i, xr[i]);
    __syncthreads();  // table and the first tile

    const float delta = PROF == 2 ? 0.15625f : 0.125f;
    for (int s = s_begin; s < s_end; ++s) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int it = 4 * s + j;
            xload(it + XD, xr[j % XD]);
            wload(it + PF - 1, qr[(j + PF - 1) % PF]);
            if (j == 0) side_load(s + 1, tailsn, banks4n);
            const uint16_t *bank[NB];
            half2_t S[NB], C[NB], Bv[NB];
            uint32_t ix[NB][3];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const NepqUnit u = nepq_decode(PROF, qr[j % PF][b], (tails[b] >> (8 * j)) & 0xffu);
                bank[b] = tab + ((banks4[b] >> (8 * j)) & 0xffu) * k.entries;
                const float st = static_cast<float>(u.state);
                S[b] = pk_h2(st, st);
                C[b] = pk_h2(-1024.f * st, -1024.f * st);
                const float bs = st * ((u.aux ? -delta : delta) - 1.f);
                Bv[b] = pk_h2(bs, bs);
                ix[b][0] = u.idx[0]; ix[b][1] = u.idx[1]; ix[b][2] = u.idx[2];
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
                    const uint32_t e = bank[b][ix[b][m]];
                    const uint32_t t2 = e | (e << 14);
#pragma unroll
                    for (int p = 0; p < 4; ++p)
                        bf[b][p] = __builtin_bit_cast(uint32_t, h2_fma(((t2 >> (4 * p)) & 0x00030003u) | kMagicH2, S[b], C[b]) + Bv[b]);
                }
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int a = 0; a < MT; ++a) acc[a][b] = mfma16(af[a], bf[b], acc[a][b]);
            }
            xstore((j + 1) & 1, xr[(j + 1) % XD]);
            if (j == 3) {
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    tails[b] = tailsn[b];
                    banks4[b] = banks4n[b];
                }
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
                const int col = (rb0 + b) * 16 + r - row0;
                if (rb0 + b < rb_end && col >= 0 && col < nrows) y[static_cast<int64_t>(m) * ldy + col] = xs * (an[b] * acc[a][b][v]);
            }
        }
    }
}

int prefill_sum_splits(const float *part, int64_t ystride, int splits, int M, int N, float *y, int64_t ldy, hipStream_t st);

static bool nepq_prefill_capable(const NepqK &k) {
    return k.neuron_len >= 8 && (k.banks * k.entries) % 2 == 0 && 3 * k.rowblock_bytes < (1ll << 31);
}
static int nepq_prefill_splits(const NepqK &k, int nrows, int M) {
    const int64_t blocks = ceil_div(ceil_div(nrows, 16), 16) * ceil_div(M, 64);
    if (blocks > 128 || nrows % 4) return 1;
    int splits = static_cast<int>(256 / blocks);
    if (splits > 8) splits = 8;
    if (splits > k.nsteps / 2) splits = k.nsteps / 2;
    if (splits <= 1) return 1;
    const int spz = static_cast<int>(ceil_div(k.nsteps, splits));
    return static_cast<int>(ceil_div(k.nsteps, spz));
}

// x16 [M, Kp] fp16 rows scaled by 1 / xscale[m], zero beyond K (x_prep); part: splits * M * nrows floats when split
static int nepq_prefill(const NepqK &k, const uint8_t *w, int row0, int nrows, const uint16_t *x16, int Kp,
                        const float *xscale, int M, float *y, int64_t ldy, float *part, hipStream_t st) {
    const int splits = part ? nepq_prefill_splits(k, nrows, M) : 1;
    const int spz = static_cast<int>(ceil_div(k.nsteps, splits));
    const int64_t ystride = static_cast<int64_t>(M) * nrows;
    float *yk = splits > 1 ? part : y;
    const int64_t ldk = splits > 1 ? nrows : ldy;
    const int nrb = static_cast<int>(ceil_div(nrows, 16));
    const size_t tabb = (static_cast<size_t>(k.banks) * k.entries * 2 + 15) / 16 * 16;
    // the tables live in LDS while they leave room for the activation tiles of the tallest block (53 KB): a 16-bank pool
    // of the L profile (64 KB) does
    const bool tab_lds = tabb <= 96 * 1024;
#define MFQ_NEPQ_PREFILL(MT, NB, XD)                                                                                   \
    {                                                                                                                  \
        const dim3 grid(static_cast<unsigned>(ceil_div(nrb, 8 * NB)), static_cast<unsigned>(ceil_div(M, MT * 16)),     \
                        static_cast<unsigned>(splits));                                                                \
        const size_t lds = (tab_lds ? tabb : 0) + static_cast<size_t>(2 * MT * 16) * (4 * 24 + 8) * 2;                 \
        auto launch = [&](auto kern) -> int {                                                                          \
            if (lds > 65536) {                                                                                         \
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                               \
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
                MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nepq_prefill: %s", hipGetErrorString(e));                \
            }                                                                                                          \
            hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, k, w, row0 / 16, row0, nrows, x16, Kp, xscale, M, yk, ldk, spz, \
                               ystride);                                                                               \
            return MFQ_OK;                                                                                             \
        };                                                                                                             \
        const int rc = k.profile == 2 ? (tab_lds ? launch(nepq_prefill_kernel<MT, NB, 4, XD, 1, 2>) : launch(nepq_prefill_kernel<MT, NB, 4, XD, 0, 2>)) \
                                      : (tab_lds ? launch(nepq_prefill_kernel<MT, NB, 4, XD, 1, 3>) : launch(nepq_prefill_kernel<MT, NB, 4, XD, 0, 3>)); \
        if (rc) return rc;                                                                                             \
        if (splits > 1) return prefill_sum_splits(part, ystride, splits, M, nrows, y, ldy, st);                        \
        return check_launch("nepq_prefill");                                                                           \
    }
    // tiles as in nvq_prefill
    if (ceil_div(nrb, 16) * ceil_div(M, 64) <= 256) MFQ_NEPQ_PREFILL(4, 2, 4)
    const double cost_a = static_cast<double>(ceil_div(ceil_div(nrb, 16) * ceil_div(M, 128), 256)) * (128 * 256);
    const double cost_b = static_cast<double>(ceil_div(ceil_div(nrb, 24) * ceil_div(M, 64), 256)) * (64 * 384) / 0.85;
    if (cost_b < cost_a) MFQ_NEPQ_PREFILL(4, 3, 2)
    MFQ_NEPQ_PREFILL(8, 2, 2)
#undef MFQ_NEPQ_PREFILL
}

// LDS a block may take when that lets the lookup tables live there (a 16-bank pool
// of the L profile is 64 KB; up to 80 KB two blocks still fit a compute unit)
constexpr size_t kNepqTableLds = 96 * 1024;
template <class Kern>
static int nepq_allow_lds(Kern kern, size_t lds) {
    if (lds <= 65536) return MFQ_OK;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(lds));
    MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nepq: %s", hipGetErrorString(e));
    return MFQ_OK;
}

static bool nepq_stream_capable(const NepqK &k) {
    return k.neuron_len >= 8 && k.neuron_len % 8 == 0 && 4 * k.rowblock_bytes < (1ll << 31);
}

template <int XF16, int NB>
static int nepq_launch_mfma(const NepqK &k, const uint8_t *w, int row0, int nrows, const uint16_t *x, int64_t ldx, int M,
                            float *y, int64_t ldy, hipStream_t st) {
    const int nrb = static_cast<int>(ceil_div(nrows, 16));
    const int64_t groups = ceil_div(nrb, NB);
    int spw = static_cast<int>(ceil_div(k.nsteps, 8));
    while (spw < k.nsteps && groups * ceil_div(k.nsteps, spw) > 8192) ++spw;
    const int nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const size_t redb = static_cast<size_t>(nwaves) * NB * 1024, tabb = static_cast<size_t>(k.banks) * k.entries * 2;
    const bool tab_lds = redb + tabb <= kNepqTableLds;
    const size_t lds = redb + (tab_lds ? tabb : 0);
    const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(ceil_div(M, 16))), block(64 * nwaves);
#define MFQ_NEPQ_MFMA(T, P)                                                                                                      \
    do {                                                                                                                         \
        if (int rc = nepq_allow_lds(nepq_mfma_kernel<XF16, NB, T, P>, lds)) return rc;                                           \
        hipLaunchKernelGGL((nepq_mfma_kernel<XF16, NB, T, P>), grid, block, lds, st, k, w, row0 / 16, row0, nrows, x, ldx, M, y, \
                           ldy, spw);                                                                                            \
    } while (0)
    if (k.profile == 2) {
        if (tab_lds) MFQ_NEPQ_MFMA(1, 2); else MFQ_NEPQ_MFMA(0, 2);
    } else {
        if (tab_lds) MFQ_NEPQ_MFMA(1, 3); else MFQ_NEPQ_MFMA(0, 3);
    }
#undef MFQ_NEPQ_MFMA
    return check_launch("nepq_mfma");
}

// One block per compute unit and 16-row tile: up to three row-blocks per block, up to 16 waves over the K steps.
static bool nepq_tile_shape(const NepqK &k, int nrows, int &rpb, int &spw, int &nwaves, size_t &lds, bool &tab_lds) {
    static const int off = tune_env("MFQ_NEPQ_TILE_OFF", 0);
    const int nrb = static_cast<int>(ceil_div(nrows, 16));
    rpb = static_cast<int>(ceil_div(nrb, gemv_cu_count()));
    if (off || rpb > 3 || 3 * k.rowblock_bytes >= (1ll << 31)) return false;
    spw = static_cast<int>(ceil_div(k.nsteps, 16));
    nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const size_t redb = static_cast<size_t>(nwaves) * rpb * 1024, tabb = static_cast<size_t>(k.banks) * k.entries * 2;
    tab_lds = redb + tabb <= 128 * 1024;
    lds = redb + (tab_lds ? tabb : 0);
    // one row-block per block and two steps per wave (4096 x 12288): the streaming kernel's eight waves of four steps,
    // with their fragments two units ahead, are faster (14.7 against 16 us) than a wait for the second step's fragments
    if (rpb == 1 && spw > 1) return false;
    return lds <= 128 * 1024;
}
template <int XF16, int RPB>
static int nepq_launch_tile(const NepqK &k, const uint8_t *w, int row0, int nrows, const uint16_t *x, int64_t ldx, int M,
                            float *y, int64_t ldy, hipStream_t st, int spw, int nwaves, size_t lds, bool tab_lds) {
    const dim3 grid(static_cast<unsigned>(ceil_div(ceil_div(nrows, 16), RPB)), static_cast<unsigned>(ceil_div(M, 16)));
    const dim3 block(64 * nwaves);
#define MFQ_NEPQ_TILE(T, P)                                                                                                       \
    do {                                                                                                                          \
        if (int rc = nepq_allow_lds(nepq_tile_kernel<XF16, RPB, T, P>, lds)) return rc;                                           \
        hipLaunchKernelGGL((nepq_tile_kernel<XF16, RPB, T, P>), grid, block, lds, st, k, w, row0 / 16, row0, nrows, x, ldx, M, y, \
                           ldy, spw);                                                                                             \
    } while (0)
    if (k.profile == 2) {
        if (tab_lds) MFQ_NEPQ_TILE(1, 2); else MFQ_NEPQ_TILE(0, 2);
    } else {
        if (tab_lds) MFQ_NEPQ_TILE(1, 3); else MFQ_NEPQ_TILE(0, 3);
    }
#undef MFQ_NEPQ_TILE
    return check_launch("nepq_tile");
}

template <int XF16>
static int nepq_mfma_any(const NepqK &k, const uint8_t *w, int row0, int nrows, const uint16_t *x, int64_t ldx, int M,
                         float *y, int64_t ldy, hipStream_t st) {
    {
        int rpb, spw, nwaves;
        size_t lds;
        bool tab_lds;
        if (M <= 32 && nepq_tile_shape(k, nrows, rpb, spw, nwaves, lds, tab_lds)) {
            if (rpb == 3) return nepq_launch_tile<XF16, 3>(k, w, row0, nrows, x, ldx, M, y, ldy, st, spw, nwaves, lds, tab_lds);
            if (rpb == 2) return nepq_launch_tile<XF16, 2>(k, w, row0, nrows, x, ldx, M, y, ldy, st, spw, nwaves, lds, tab_lds);
            return nepq_launch_tile<XF16, 1>(k, w, row0, nrows, x, ldx, M, y, ldy, st, spw, nwaves, lds, tab_lds);
        }
    }
    const int64_t wpb = (k.nsteps < 8 ? k.nsteps : 8) * ceil_div(M, 16);  // waves of a block x 16-row tiles
    static const int env_nb = tune_env("MFQ_NEPQ_NB", 0);
    if (env_nb == 4) return nepq_launch_mfma<XF16, 4>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
    if (env_nb == 2) return nepq_launch_mfma<XF16, 2>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
    if (env_nb == 1) return nepq_launch_mfma<XF16, 1>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
    if (ceil_div(ceil_div(nrows, 16), 4) * wpb >= 1536) return nepq_launch_mfma<XF16, 4>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
    return nepq_launch_mfma<XF16, 1>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
}

static void nepq_gemv_shape(const NepqK &k, int nrb, int mb, int rpb, int &spw, int &nwaves, size_t &lds_bytes, bool &tab_lds) {
    int want = static_cast<int>(ceil_div(3 * gemv_target_waves(), ceil_div(nrb, rpb)));
    if (want < 1) want = 1;
    if (want > 16) want = 16;
    if (want > k.nsteps) want = k.nsteps;
    spw = static_cast<int>(ceil_div(k.nsteps, want));
    nwaves = static_cast<int>(ceil_div(k.nsteps, spw));
    const size_t xb = gemv_lds_bytes(mb, spw, 24, nwaves, rpb);
    const size_t tabb = static_cast<size_t>(k.banks) * k.entries * 2;
    tab_lds = tabb + xb <= kNepqTableLds;
    lds_bytes = xb + (tab_lds ? tabb : 0);
}

template <int XF16, int MB, int RPB>
static int nepq_launch_as(const NepqK &k, const uint8_t *w, int row0, int nrows, const uint16_t *x, int64_t ldx, int M,
                          float *y, int64_t ldy, hipStream_t st) {
    const int rb0 = row0 / 16, nrb = static_cast<int>(ceil_div(nrows, 16));
    int spw, nwaves;
    size_t lds;
    bool tab_lds;
    nepq_gemv_shape(k, nrb, MB, RPB, spw, nwaves, lds, tab_lds);
    MFQ_REQUIRE(lds <= kNepqTableLds, MFQ_ERR_UNSUPPORTED, "nepq_gemv: neuron_len %d needs %zu bytes of LDS", k.neuron_len, lds);
    const dim3 grid(static_cast<unsigned>(ceil_div(nrb, RPB)), static_cast<unsigned>(ceil_div(M, MB))), block(64 * nwaves);
#define MFQ_NEPQ_GEMV(T, P)                                                                                                     \
    do {                                                                                                                        \
        if (int rc = nepq_allow_lds(nepq_gemv_kernel<XF16, MB, T, RPB, P>, lds)) return rc;                                     \
        hipLaunchKernelGGL((nepq_gemv_kernel<XF16, MB, T, RPB, P>), grid, block, lds, st, k, w, rb0, row0, nrows, x, ldx, M, y, \
                           ldy, spw, PairSel{});                                                                                \
    } while (0)
    if (k.profile == 2) {
        if (tab_lds) MFQ_NEPQ_GEMV(1, 2); else MFQ_NEPQ_GEMV(0, 2);
    } else {
        if (tab_lds) MFQ_NEPQ_GEMV(1, 3); else MFQ_NEPQ_GEMV(0, 3);
    }
#undef MFQ_NEPQ_GEMV
    return check_launch("nepq_gemv");
}

// the same kernel, one row and one row-block per block, over the pairs of a MoE decode step (see PairSel): the experts are
// the row ranges of one expert-shaped tensor
template <int XF16>
static int nepq_launch_pairs(const NepqK &k, const uint8_t *w, int out_per_expert, const uint16_t *x, int64_t ldx, int n_pairs,
                             float *y, int64_t ldy, const PairSel &sel, hipStream_t st) {
    const int nrb = static_cast<int>(ceil_div(out_per_expert, 16));
    int spw, nwaves;
    size_t lds;
    bool tab_lds;
    nepq_gemv_shape(k, nrb * n_pairs, 1, 1, spw, nwaves, lds, tab_lds);
    MFQ_REQUIRE(lds <= kNepqTableLds, MFQ_ERR_UNSUPPORTED, "nepq_gemv_pairs: neuron_len %d needs %zu bytes of LDS", k.neuron_len, lds);
    const dim3 grid(static_cast<unsigned>(nrb), static_cast<unsigned>(n_pairs)), block(64 * nwaves);
#define MFQ_NEPQ_PAIRS(T, P)                                                                                              \
    do {                                                                                                                  \
        if (int rc = nepq_allow_lds(nepq_gemv_kernel<XF16, 1, T, 1, P>, lds)) return rc;                                   \
        hipLaunchKernelGGL((nepq_gemv_kernel<XF16, 1, T, 1, P>), grid, block, lds, st, k, w, 0, 0, out_per_expert, x, ldx,  \
                           n_pairs, y, ldy, spw, sel);                                                                    \
    } while (0)
    if (k.profile == 2) {
        if (tab_lds) MFQ_NEPQ_PAIRS(1, 2); else MFQ_NEPQ_PAIRS(0, 2);
    } else {
        if (tab_lds) MFQ_NEPQ_PAIRS(1, 3); else MFQ_NEPQ_PAIRS(0, 3);
    }
#undef MFQ_NEPQ_PAIRS
    return check_launch("nepq_gemv_pairs");
}
template <int XF16, int MB>
static int nepq_launch(const NepqK &k, const uint8_t *w, int row0, int nrows, const uint16_t *x, int64_t ldx, int M,
                       float *y, int64_t ldy, hipStream_t st) {
    if constexpr (MB == 1) {
        // One row: as many row-blocks per block as it takes to have one block per CU (up to four), so that the table is
        // staged once per CU and every wave has several row-blocks' units in flight.  MFQ_NEPQ_RPB overrides for tuning.
        static const int env = tune_env("MFQ_NEPQ_RPB", 0);
        const int nrb = static_cast<int>(ceil_div(nrows, 16));
        int rpb = env > 0 ? env : static_cast<int>(ceil_div(nrb, gemv_cu_count()));
        int spw, nwaves;
        size_t lds;
        bool tl;
        for (rpb = rpb > 4 ? 4 : rpb; rpb > 1; --rpb) {  // the reduction area grows with the row-blocks
            nepq_gemv_shape(k, nrb, 1, rpb, spw, nwaves, lds, tl);
            if (lds <= kNepqTableLds) break;
        }
        if (rpb >= 4) return nepq_launch_as<XF16, 1, 4>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
        if (rpb == 3) return nepq_launch_as<XF16, 1, 3>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
        if (rpb == 2) return nepq_launch_as<XF16, 1, 2>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
    }
    return nepq_launch_as<XF16, MB, 1>(k, w, row0, nrows, x, ldx, M, y, ldy, st);
}

static int nepq_gemv_any(const mfq_nepq_desc *d, const void *weight, int row0, int nrows, const void *x, int x_dtype,
                         int64_t ldx, int M, float *y, int64_t ldy, hipStream_t st) {
    const NepqK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    const int nrb = static_cast<int>(ceil_div(nrows, 16));
    // a single row is still cheaper on the vector-ALU kernel
    static const int valu_max_m = tune_env("MFQ_NEPQ_VALU_MAX_M", 1);
    if (M > valu_max_m && nepq_stream_capable(k) && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0)
        return x_dtype == MFQ_X_F16 ? nepq_mfma_any<1>(k, w, row0, nrows, xp, ldx, M, y, ldy, st)
                                    : nepq_mfma_any<0>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
    int mb = M >= 4 ? 4 : (M >= 2 ? 2 : 1);
    for (;;) {
        int spw, nwaves;
        size_t lds;
        bool tl;
        nepq_gemv_shape(k, nrb, mb, 1, spw, nwaves, lds, tl);
        if (lds <= kNepqTableLds || mb == 1) break;
        mb >>= 1;
    }
    if (x_dtype == MFQ_X_F16) {
        if (mb == 4) return nepq_launch<1, 4>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
        if (mb == 2) return nepq_launch<1, 2>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
        return nepq_launch<1, 1>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
    }
    if (mb == 4) return nepq_launch<0, 4>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
    if (mb == 2) return nepq_launch<0, 2>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
    return nepq_launch<0, 1>(k, w, row0, nrows, xp, ldx, M, y, ldy, st);
}

// ---- signed block-Hadamard input transform ------------------------------------------------
template <int XF16>
__global__ __launch_bounds__(256) void hadamard_kernel(const uint16_t *__restrict__ x, int64_t ldx, int K, int block,
                                                       const int8_t *__restrict__ signs, uint16_t *__restrict__ out,
                                                       int64_t ldo) {
    extern __shared__ float hbuf[];
    const int b = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
    const uint16_t *xr = x + row * ldx + static_cast<int64_t>(b) * block;
    for (int i = tid; i < block; i += 256) hbuf[i] = x_to_f32<XF16>(xr[i]) * static_cast<float>(signs[b * block + i]);
    __syncthreads();
    for (int h = 1; h < block; h <<= 1) {
        for (int i = tid; i < block / 2; i += 256) {
            const int lo = ((i / h) * 2 * h) + (i % h);
            const float a = hbuf[lo], c = hbuf[lo + h];
            hbuf[lo] = a + c;
            hbuf[lo + h] = a - c;
        }
        __syncthreads();
    }
    const float norm = rsqrtf(static_cast<float>(block));
    uint16_t *o = out + row * ldo + static_cast<int64_t>(b) * block;
    for (int i = tid; i < block; i += 256) {
        const float v = hbuf[i] * norm;
        o[i] = XF16 ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
    }
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

extern "C" int mfq_hip_nepq_plan(int profile, int banks, int rows, int neuron_len, mfq_nepq_desc *d) {
    MFQ_REQUIRE(d != nullptr, MFQ_ERR_INVALID, "nepq_plan: null descriptor");
    MFQ_REQUIRE(profile == 2 || profile == 3, MFQ_ERR_UNSUPPORTED,
                "nepq_plan: only NEPQ1-S (2) and NEPQ1-L (3) are on the accelerated path (profile=%d)", profile);
    MFQ_REQUIRE(banks >= 1 && banks <= 256, MFQ_ERR_INVALID, "NEPQ bank count must be in [1,256]");
    MFQ_REQUIRE(rows > 0 && neuron_len > 0 && neuron_len % 8 == 0, MFQ_ERR_INVALID, "NEPQ K must be divisible by 8");
    d->profile = profile;
    d->state_bits = profile == 2 ? 4 : 3;
    d->index_bits = profile == 2 ? 9 : 11;
    d->banks = banks; d->rows = rows; d->neuron_len = neuron_len;
    d->ng = static_cast<int32_t>(ceil_div(neuron_len, 24));
    d->nvec = neuron_len / 8;
    d->nsuper = static_cast<int32_t>(ceil_div(d->ng, 4));
    d->ngp = static_cast<int32_t>(ceil_div(d->ng, 16) * 16);
    d->nsteps = d->ngp / 16;
    d->n_rowblocks = static_cast<int32_t>(ceil_div(rows, 16));
    d->table_entries = profile == 2 ? 1024 : 2048;
    d->step_bytes = 1024 + (profile == 3 ? 256 : 0) + 64;
    d->rowblock_bytes = d->step_bytes * d->nsteps;
    d->tables_off = d->rowblock_bytes * d->n_rowblocks;
    d->anchors_off = d->tables_off + static_cast<int64_t>(banks) * d->table_entries * 2;
    d->total_bytes = d->anchors_off + 16ll * d->n_rowblocks * 4;
    const int64_t r = rows;
    d->payload_bytes = static_cast<int64_t>(banks) * d->table_entries * 2 + 2 * r + (r * d->ng * d->state_bits + 7) / 8 +
                       (r * d->nvec * d->index_bits + 7) / 8 + (r * d->ng + 7) / 8 + r * d->nsuper;
    return MFQ_OK;
}

extern "C" int mfq_hip_nepq_repack(const mfq_nepq_desc *d, const void *payload, int64_t payload_bytes, void *weight,
                                   mfq_stream_t stream) {
    MFQ_REQUIRE(d && payload && weight, MFQ_ERR_INVALID, "nepq_repack: null argument");
    MFQ_REQUIRE(payload_bytes == d->payload_bytes, MFQ_ERR_INVALID, "invalid NEPQ tail: size=%lld, expected=%lld",
                static_cast<long long>(payload_bytes), static_cast<long long>(d->payload_bytes));
    const NepqK k = to_k(d);
    hipLaunchKernelGGL(nepq_repack_kernel, dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(payload), static_cast<uint8_t *>(weight));
    return check_launch("nepq_repack");
}

extern "C" int mfq_hip_nepq_dequant_f32(const mfq_nepq_desc *d, const void *weight, float *w_out, int64_t ld,
                                        mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && w_out, MFQ_ERR_INVALID, "nepq_dequant_f32: null argument");
    MFQ_REQUIRE(ld >= d->neuron_len, MFQ_ERR_INVALID, "nepq_dequant_f32: ld smaller than neuron_len");
    const NepqK k = to_k(d);
    hipLaunchKernelGGL((nepq_dequant_kernel<float>), dim3(k.n_rowblocks, k.nsteps), dim3(64), 0, as_stream(stream), k,
                       static_cast<const uint8_t *>(weight), 0, 0, k.rows, w_out, ld, static_cast<float *>(nullptr), 0);
    return check_launch("nepq_dequant_f32");
}

static int nepq_check_rows(const mfq_nepq_desc *d, int row0, int nrows) {
    MFQ_REQUIRE(row0 >= 0 && nrows > 0 && row0 + nrows <= d->rows, MFQ_ERR_INVALID, "nepq: rows [%d, %d) outside [0, %d)",
                row0, row0 + nrows, d->rows);
    MFQ_REQUIRE(row0 % 16 == 0, MFQ_ERR_UNSUPPORTED, "nepq: expert row offset %d must be a multiple of 16", row0);
    return MFQ_OK;
}

extern "C" int mfq_hip_nepq_gemv(const mfq_nepq_desc *d, const void *weight, int row0, int nrows, const void *x,
                                 int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nepq_gemv: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nepq_gemv: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nepq_gemv: x_dtype=%d", x_dtype);
    if (int rc = nepq_check_rows(d, row0, nrows)) return rc;
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= nrows, MFQ_ERR_INVALID, "nepq_gemv: ldx/ldy smaller than the tensor");
    return nepq_gemv_any(d, weight, row0, nrows, x, x_dtype, ldx, M, y, ldy, as_stream(stream));
}

extern "C" int mfq_hip_nepq_gemv_pairs(const mfq_nepq_desc *d, const void *weight, int out_per_expert, const int32_t *expert_slot,
                                       int E, const void *x, int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T,
                                       int R, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && expert_slot && x && ids && y, MFQ_ERR_INVALID, "nepq_gemv_pairs: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nepq_gemv_pairs: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(T >= 0 && R >= 1 && E >= 1, MFQ_ERR_INVALID, "nepq_gemv_pairs: T=%d R=%d E=%d", T, R, E);
    MFQ_REQUIRE(out_per_expert > 0 && out_per_expert % 16 == 0 && d->rows % out_per_expert == 0, MFQ_ERR_UNSUPPORTED,
                "nepq_gemv_pairs: %d rows per expert (a multiple of 16 that divides the tensor's %d)", out_per_expert, d->rows);
    MFQ_REQUIRE(static_cast<int64_t>(T) * R <= 65535, MFQ_ERR_UNSUPPORTED, "nepq_gemv_pairs: %lld pairs (at most 65535 per launch)",
                static_cast<long long>(T) * R);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= out_per_expert, MFQ_ERR_INVALID, "nepq_gemv_pairs: ldx/ldy smaller than the tensor");
    if (T == 0) return MFQ_OK;
    const PairSel sel{ids, expert_slot, nullptr, E, R, routed_input ? 1 : 0};
    const NepqK k = to_k(d);
    const uint8_t *w = static_cast<const uint8_t *>(weight);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    return x_dtype == MFQ_X_F16 ? nepq_launch_pairs<1>(k, w, out_per_expert, xp, ldx, T * R, y, ldy, sel, as_stream(stream))
                                : nepq_launch_pairs<0>(k, w, out_per_expert, xp, ldx, T * R, y, ldy, sel, as_stream(stream));
}

// The reference's Python policy keeps M <= 16 on the GEMV.  Two 16-row passes of the matrix-core streaming kernel cost
// what the prefill kernel costs up to about a hundred rows (40 us on 12288x4096), so the prefill kernel takes over
// from kNepqPrefillMinM rows; tensors it cannot take stay on the streaming kernel up to kNepqStreamMaxM rows.
static constexpr int kNepqGemvMaxM = 16, kNepqStreamMaxM = 256, kNepqPrefillMinM = 33;
static bool nepq_prefills(const NepqK &k, int M) {
    static const int env = tune_env("MFQ_NEPQ_PREFILL_MIN_M", 0);
    return M >= (env > 0 ? env : kNepqPrefillMinM) && nepq_prefill_capable(k);
}
static bool nepq_streams(const mfq_nepq_desc *d, int M) {
    const NepqK k = to_k(d);
    if (M > kNepqGemvMaxM && nepq_prefills(k, M)) return false;
    return M <= kNepqGemvMaxM || (M <= kNepqStreamMaxM && nepq_stream_capable(k));
}
static size_t nepq_align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }
static int nepq_kp(int K) { return static_cast<int>(ceil_div(K, 32)) * 32; }

extern "C" size_t mfq_hip_nepq_gemm_workspace_bytes(const mfq_nepq_desc *d, int nrows, int M) {
    if (!d || nepq_streams(d, M)) return 0;
    const NepqK k = to_k(d);
    if (nepq_prefills(k, M)) {  // x16 [M, Kp] | xscale [M] | partial results of a split over K
        const int splits = nepq_prefill_splits(k, nrows, M);
        return nepq_align256(static_cast<size_t>(M) * nepq_kp(k.neuron_len) * 2) + nepq_align256(static_cast<size_t>(M) * 4) +
               (splits > 1 ? static_cast<size_t>(splits) * M * nrows * 4 : 0);
    }
    return dequant_gemm_workspace(nrows, d->neuron_len, M);
}

extern "C" int mfq_hip_nepq_gemm(const mfq_nepq_desc *d, const void *weight, int row0, int nrows, const void *x,
                                 int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, void *workspace,
                                 size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nepq_gemm: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nepq_gemm: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nepq_gemm: x_dtype=%d", x_dtype);
    if (int rc = nepq_check_rows(d, row0, nrows)) return rc;
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= nrows, MFQ_ERR_INVALID, "nepq_gemm: ldx/ldy smaller than the tensor");
    hipStream_t st = as_stream(stream);
    if (nepq_streams(d, M)) return nepq_gemv_any(d, weight, row0, nrows, x, x_dtype, ldx, M, y, ldy, st);
    if (nepq_prefills(to_k(d), M)) {
        const NepqK k = to_k(d);
        const int Kp = nepq_kp(k.neuron_len);
        const size_t need = mfq_hip_nepq_gemm_workspace_bytes(d, nrows, M);
        MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nepq_gemm: workspace %zu < %zu bytes",
                    workspace_bytes, need);
        uint16_t *x16 = static_cast<uint16_t *>(workspace);
        uint8_t *p = static_cast<uint8_t *>(workspace) + nepq_align256(static_cast<size_t>(M) * Kp * 2);
        float *xscale = reinterpret_cast<float *>(p);
        p += nepq_align256(static_cast<size_t>(M) * 4);
        float *part = nepq_prefill_splits(k, nrows, M) > 1 ? reinterpret_cast<float *>(p) : nullptr;
        const int rc = x_prep(x, x_dtype, ldx, M, k.neuron_len, Kp, x16, xscale, st);
        if (rc) return rc;
        return nepq_prefill(k, static_cast<const uint8_t *>(weight), row0, nrows, x16, Kp, xscale, M, y, ldy, part, st);
    }
    const size_t need = dequant_gemm_workspace(nrows, d->neuron_len, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nepq_gemm: workspace %zu < %zu bytes",
                workspace_bytes, need);
    uint16_t *x16, *w16;
    float *xscale, *wscale;
    int Kp;
    dequant_gemm_carve(workspace, nrows, d->neuron_len, M, x16, xscale, w16, wscale, Kp);
    int rc = x_prep(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, st);
    if (rc) return rc;
    const NepqK k = to_k(d);
    hipLaunchKernelGGL((nepq_dequant_kernel<uint16_t>), dim3(static_cast<unsigned>(ceil_div(nrows, 16)), k.nsteps), dim3(64),
                       0, st, k, static_cast<const uint8_t *>(weight), row0 / 16, row0, nrows, w16,
                       static_cast<int64_t>(Kp), wscale, Kp);
    rc = check_launch("nepq_dequant_f16");
    if (rc) return rc;
    return gemm_f16_nt(x16, Kp, w16, Kp, M, nrows, Kp, xscale, wscale, y, ldy, st, dequant_gemm_part(wscale, nrows, d->neuron_len, M));
}

extern "C" int mfq_hip_nepq_hadamard(const void *x, int x_dtype, int64_t ldx, int rows, int K, int block,
                                     const int8_t *signs, void *x_out, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(x && signs && x_out, MFQ_ERR_INVALID, "nepq_hadamard: null argument");
    MFQ_REQUIRE(block >= 2 && block <= 8192 && (block & (block - 1)) == 0 && K % block == 0, MFQ_ERR_INVALID,
                "NEPQ rotation block must be a power of two dividing K (block=%d, K=%d)", block, K);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nepq_hadamard: x_dtype=%d", x_dtype);
    const dim3 grid(K / block, rows);
    if (x_dtype == MFQ_X_F16)
        hipLaunchKernelGGL((hadamard_kernel<1>), grid, dim3(256), block * 4, as_stream(stream),
                           static_cast<const uint16_t *>(x), ldx, K, block, signs, static_cast<uint16_t *>(x_out), ldo);
    else
        hipLaunchKernelGGL((hadamard_kernel<0>), grid, dim3(256), block * 4, as_stream(stream),
                           static_cast<const uint16_t *>(x), ldx, K, block, signs, static_cast<uint16_t *>(x_out), ldo);
    return check_launch("nepq_hadamard");
}
