// NINT prefill matmul: a block-tiled MFMA GEMM whose B operand is dequantized in registers.
//
// Block = 4 waves as WM (tokens) x 4/WM (neurons); a wave owns MT*16 tokens x NB*16 neurons and, like the
// small-batch kernel (nint_mfma.hpp), reads its weight units straight from HBM in the R16 layout, turns
// each dword of codes into an fp16 fragment (sub_scale * code / 64) with one AND-OR and one packed FMA
// per pair, and feeds v_mfma_f32_16x16x32_f16.  The activation tile (already fp16, see x_prep) of one
// sub-step -- the 4 * GS k-values of units j of a step -- is staged in LDS once per block and shared by the waves
// (two buffers filled through registers, or a ring of four filled by direct-to-LDS copies three sub-steps ahead);
// weights never touch LDS.  After the K loop the minimum term sum_g sub_min_g X_g runs as a
// short second loop (one MFMA per step and tile against precomputed group sums), then
//     y = xscale[token] * (64 * neuron_scale * S1 - neuron_min * S2).
#pragma once
#include "nint_mfma.hpp"

namespace mfq {

constexpr int kMinSteps = 8;  // steps whose minimum-term operands a block stages at once

// LDS bytes of a block of BM tile rows: nbuf activation buffers of [BM][4 * GS' + 8] halves (GS' = groupsize padded to 8),
// reused for the group sums of kMinSteps steps ([BM][kMinSteps * 16 + 4] dwords).
constexpr size_t prefill_lds_bytes(int bm, int gs, int nbuf = 2) {
    // a buffer of the ring of four (direct-to-LDS copies) is a whole number of wave-wide copies of 16-byte chunks
    const size_t row = 4 * ((gs + 7) / 8 * 8) + 8;
    const size_t buf = nbuf == 4 ? (bm * (row / 8) + 63) / 64 * 64 * 16 : bm * row * 2;
    const size_t xt = nbuf * buf;
    const size_t mn = static_cast<size_t>(bm) * (kMinSteps * 16 + 4) * 4;
    return xt > mn ? xt : mn;
}

// Rows of a block tile: src(i) = row of x16 / xscale / xg that tile row i reads (always valid), dst(i) = row of y it
// writes or -1.
// win_row0() / win_rows(bm): rows of x16 that the direct-to-LDS copies of a tile of bm rows address through one
// buffer window (a window spans less than 4 GiB).
struct DenseRows {
    int tok0, M;
    __device__ __forceinline__ int src(int i) const { return min(tok0 + i, M - 1); }
    __device__ __forceinline__ int dst(int i) const { return tok0 + i < M ? tok0 + i : -1; }
    __device__ __forceinline__ int win_row0() const { return min(tok0, M - 1); }
    __device__ __forceinline__ int64_t win_rows(int bm) const { return bm; }
};
struct MappedRows {  // both tables live in LDS; any row of x16 may be a source: the window spans all n_src of them
    const int *srcv, *dstv;
    int n_src;
    __device__ __forceinline__ int src(int i) const { return srcv[i]; }
    __device__ __forceinline__ int dst(int i) const { return dstv[i]; }
    __device__ __forceinline__ int win_row0() const { return 0; }
    __device__ __forceinline__ int64_t win_rows(int) const { return n_src; }
};

// One block: tile rows `rows`, neurons of the row-blocks [rb_base, rb_base + (NW / WM) * NB) below rb_end; y column of a
// neuron = (row-block - rb_col0) * 16 + r, stored when below ncols.  xg: the group sums x_prep leaves,
// [row][step][kb] x 16 bytes (see gemm.hip).  xt: LDS, prefill_lds_bytes(BM, GS, XD == 0 ? 4 : 2) bytes.
// XD: activation tiles in flight in registers, or 0 for direct-to-LDS copies (rows of x16 then hold whole steps:
// Kp >= 64 * GS * steps).  PF: register buffers of weight units per row-block; the unit of sub-step it + PF - 1 is requested while sub-step it
// multiplies (2 = ping-pong; 4 keeps a whole step in flight for tiles with few rows, where the weight stream and
// not the matrix cores sets the pace).
// GLU: the wave's NB row-blocks are NB / 2 gate row-blocks from rb_base on and the NB / 2 row-blocks glu.rb_stride further
// (up); rb_end bounds the gate row-blocks; instead of the two fp32 results the block stores act(gate) * up in 16 bits
// (y is then uint16_t [rows, ldy], column = the gate neuron's).
struct GluOut {
    int rb_stride;  // row-blocks from a gate row-block to its up row-block
    int gelu;       // 0: SiLU, 1: tanh form of GELU
    int f16;        // output halves are fp16 (else bf16)
};
template <class U, int MT, int NB, int WM, int NW, class Rows, int PF = 2, int XD = (PF == 4 ? 4 : 1), bool GLU = false>
__device__ __forceinline__ void nint_prefill_body(const NintK &k, const uint8_t *__restrict__ w, int rb_base, int rb_end,
                                                  int rb_col0, int ncols, const uint16_t *__restrict__ x16, int Kp,
                                                  const float *__restrict__ xscale, const uint32_t *__restrict__ xg,
                                                  const Rows &rows, float *__restrict__ y, int64_t ldy, uint16_t *xt,
                                                  int s_begin = 0, int s_end = -1, GluOut glu = GluOut{0, 0, 0}) {
    if (s_end < 0) s_end = k.nsteps;  // steps [s_begin, s_end) of K: a block of a split over K leaves a partial sum
    constexpr int D = U::D, GS = U::GROUP, NM = U::NPAIR / 4, BITS = U::CBITS;
    constexpr int NCLS = BITS == 0 ? 1 : (BITS == 3 ? 3 : 2);
    constexpr int NT = 64 * NW;                // threads
    constexpr int BM = WM * MT * 16;           // tokens per block
    constexpr int EL = GS % 8 == 0 ? 8 : 4;    // halves per copy chunk (16 or 8 bytes)
    constexpr int GSP = (GS + 7) / 8 * 8;      // group width in LDS: fragments stay 16-byte aligned
    constexpr int ROW = 4 * GSP + 8;           // LDS row stride in halves (16 bytes of padding)
    constexpr int CPG = GS / EL;               // chunks per group
    constexpr int CHUNKS = 4 * CPG;            // chunks per tile row
    constexpr int PER_THREAD = (BM * CHUNKS + NT - 1) / NT;
    static_assert(GS % EL == 0, "groupsize must be a multiple of 4");
    typedef uint32_t chunk_t __attribute__((ext_vector_type(EL / 2)));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int r = lane & 15, kb = lane >> 4;
    static_assert(!GLU || NB % 2 == 0, "gate and up row-blocks come in pairs");
    constexpr int NBG = GLU ? NB / 2 : NB;  // row-blocks from rb0 on; with GLU the other half lies glu.rb_stride further
    const int rb0 = rb_base + wn * NBG;
    const int nrb = max(0, min(NBG, rb_end - rb0));
    auto rbo = [&](int b) { return GLU ? (b % NBG) + (b / NBG) * glu.rb_stride : b; };  // row-block of b, relative to rb0
    auto live = [&](int b) { return (b % NBG) < nrb; };
    const uint32_t sb = static_cast<uint32_t>(k.step_bytes), rbb = static_cast<uint32_t>(k.rowblock_bytes);
    const __amdgpu_buffer_rsrc_t win =
        wave_window(w + static_cast<int64_t>(min(rb0, k.n_rowblocks - 1)) * k.rowblock_bytes,
                    nrb > 0 ? (rbo(NB - NBG) + nrb) * rbb : 0u);

    float4_t acc[MT][NB];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // global -> register copy of the activation tile of sub-step `it` (chunk c of a row = 8 halves at k0 + 8 c)
    // XD = 0: the tiles go from global memory straight into a ring of four LDS buffers (no registers in between),
    // three sub-steps ahead.  Needs 16-byte chunks (GS % 8 == 0) and Kp >= 64 * GS * steps: every tile lies inside a row.
    constexpr bool DMA = XD == 0;
    static_assert(XD == 0 || XD == 1 || XD == 2 || XD == 4, "activation tiles in flight in registers");
    static_assert(!DMA || (EL == 8 && GSP == GS), "direct-to-LDS tiles are made of 16-byte chunks");
    // A tile whose chunks do not fill the last wave-wide copy is followed by slack for the rest of that copy (which
    // repeats the tile's last chunk): TILE_CH counts the slack, BUF is the distance between two buffers in halves.
    constexpr int CPR = ROW / 8, TILE_CH = DMA ? (BM * CPR + 63) / 64 * 64 : BM * CPR, DPER = DMA ? (TILE_CH + NT - 1) / NT : 1;
    constexpr int LASTW = (TILE_CH - NT * (DPER - 1)) / 64;
    constexpr int BUF = DMA ? TILE_CH * 8 : BM * ROW;
    constexpr int XR = DMA ? 1 : XD;
    chunk_t xr[XR][PER_THREAD];
    // the thread's chunks of a tile: source row (looked up once: a mapped tile keeps its row table in LDS) and k offset
    const uint16_t *xsrc[PER_THREAD];
    int xk[PER_THREAD];
#pragma unroll
    for (int p = 0; p < PER_THREAD; ++p) {
        const int c = min(tid + NT * p, BM * CHUNKS - 1);
        const int row = c / CHUNKS;
        xsrc[p] = x16 + static_cast<int64_t>(rows.src(row)) * Kp;
        xk[p] = EL * (c - row * CHUNKS);  // groups are contiguous in k: chunk ch of the row starts EL * ch further
    }
    auto xload = [&](int it, chunk_t (&xq)[PER_THREAD]) {
        const int k0 = it * 4 * GS;
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int kk = k0 + xk[p];
            const int kc = min(kk, Kp - EL);
            chunk_t v = *reinterpret_cast<const chunk_t *>(xsrc[p] + kc);
            if (kk >= Kp) v = chunk_t(0u);
            xq[p] = v;
        }
    };
    auto xstore = [&](int buf, const chunk_t (&xq)[PER_THREAD]) {
#pragma unroll
        for (int p = 0; p < PER_THREAD; ++p) {
            const int c = tid + NT * p;
            const int row = c / CHUNKS, ch = c - row * CHUNKS;
            const int g = ch / CPG, ci = ch - g * CPG;
            if (c < BM * CHUNKS)
                *reinterpret_cast<chunk_t *>(xt + buf * BUF + row * ROW + g * GSP + EL * ci) = xq[p];
        }
    };
    // direct-to-LDS copies: chunk c of a tile (16 bytes; row c / CPR, the last chunk of a row is padding and takes a
    // copy of the one before) lands at byte 16 c of its buffer -- lane l of a wave-wide copy writes 16 l bytes behind
    // the wave's base, so a thread's chunks are tid, tid + NT, ...  The last round has work for LASTW waves only; the
    // others repeat it (same bytes to the same place), so that every wave issues the same number of requests.
    uint32_t dsrc[DPER];  // byte offset of the thread's chunk p inside x16 at k = 0
    int dbase[DPER];      // first chunk of the wave's copy p
    // buffer-addressed copies (the flat-addressed form makes the compiler wait for all outstanding requests at every
    // use of a loaded register); the tile rows of a block lie inside 4 GiB from xwin's base
    __amdgpu_buffer_rsrc_t xwin;
    if constexpr (DMA) {
        const int row_lo = rows.win_row0();
        xwin = wave_window(reinterpret_cast<const uint8_t *>(x16 + static_cast<int64_t>(row_lo) * Kp),
                           static_cast<uint32_t>(min(rows.win_rows(BM) * Kp * 2, static_cast<int64_t>(0xffffffffu))));
#pragma unroll
        for (int p = 0; p < DPER; ++p) {
            dbase[p] = NT * p + (p == DPER - 1 ? wave % LASTW : wave) * 64;
            const int c = min(dbase[p] + lane, BM * CPR - 1);  // the slack behind the tile takes copies of its last chunk
            const int row = c / CPR, cc = min(c - row * CPR, CPR - 2);
            dsrc[p] = static_cast<uint32_t>((static_cast<int64_t>(rows.src(row) - row_lo) * Kp + 8 * cc) * 2);
        }
    }
    const int it_last = 4 * k.nsteps - 1;  // tiles past the end of K re-read the last one (nobody multiplies them)
    auto xdma = [&](int it, int buf) {
        if constexpr (DMA) {
            const int k0 = min(it, it_last) * 4 * GS;
#pragma unroll
            for (int p = 0; p < DPER; ++p) {
                typedef __attribute__((address_space(3))) void *lds_ptr;
                uint16_t *dst = xt + buf * BUF + dbase[p] * 8;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(xwin, (lds_ptr)dst, 16, dsrc[p], k0 * 2, 0, 0);
            }
        }
    };
    // Requests of a thread in sub-step j: how many younger requests may
    // be outstanding when the copies issued two sub-steps earlier must have landed.
    constexpr int DMIN = DPER;
    constexpr int WCNT = NB;                                   // weight units
    constexpr int SCNT = NB * (U::TAIL ? 2 : 1);               // scale (and tail) loads, once per step
    if constexpr (GSP != GS) {  // the padding halves of a group are multiplied by zero weights: keep them finite
        for (int i = tid; i < 2 * BM * ROW / 2; i += NT) reinterpret_cast<uint32_t *>(xt)[i] = 0u;
        __syncthreads();
    }

    static_assert(PF == 2 || PF == 4, "the sub-step loop is unrolled four times");
    uint32_t qr[PF][NB][D], tails[NB], tailsn[NB];
    u32x2_t sc[NB], scn[NB];
    auto wload = [&](int it, uint32_t (&qq)[NB][D]) {
        const int s = it >> 2, j = it & 3;
#pragma unroll
        for (int b = 0; b < NB; ++b)
            load_unit_win<D, 0>(win, live(b) && s < s_end ? rbo(b) * rbb + s * sb + (j * 64 + lane) * (D * 4) : kNoStep, qq[b]);
    };
    auto sload = [&](int s, uint32_t (&tt)[NB], u32x2_t (&ss)[NB]) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint32_t off = live(b) && s < s_end ? rbo(b) * rbb + s * sb + 1024 * D : kNoStep;
            tt[b] = 0;
            if constexpr (U::TAIL) tt[b] = __builtin_amdgcn_raw_buffer_load_b32(win, off + lane * 4, 0, 0);
            ss[b] = __builtin_amdgcn_raw_buffer_load_b64(win, off + (U::TAIL ? 256 : 0) + lane * 8, 0, 0);
        }
    };

    if constexpr (DMA) {
#pragma unroll
        for (int i = 0; i < 3; ++i) xdma(4 * s_begin + i, i);
    } else {
        xload(4 * s_begin, xr[0]);
    }
#pragma unroll
    for (int i = 0; i < PF - 1; ++i) wload(4 * s_begin + i, qr[i]);
    sload(s_begin, tails, sc);
    if constexpr (!DMA) {
        xstore(0, xr[0]);
#pragma unroll
        for (int i = 1; i < XD; ++i) xload(4 * s_begin + i, xr[i]);
    }
    // Every request of the prologue lands before the loop, through a wait the compiler sees (not inline assembly): the
    // waits it places inside the loop then count only the requests of earlier sub-steps.  Entering the loop with requests
    // in flight makes it keep, for all iterations, the short distances of the first one -- a wait for a weight unit
    // requested a few instructions earlier, once per step.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    for (int s = s_begin; s < s_end; ++s) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int it = 4 * s + j;
        if constexpr (DMA) xdma(it + 3, (j + 3) & 3);  // the buffer the previous sub-step read
        else xload(it + XD, xr[j % XR]);                // past the end: clamped addresses, zeros
        wload(it + PF - 1, qr[(j + PF - 1) % PF]);
        if (j == (PF == 4 ? 0 : 3)) sload(s + 1, tailsn, scn);

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
                af[a] = *reinterpret_cast<const u32x4_t *>(xt + (DMA ? (j & 3) : (j & 1)) * BUF + ((wm * MT + a) * 16 + r) * ROW + kb * GSP + 8 * m);
            // all weight fragments of this k-slice first, then the MFMAs back to back: while one wave's MFMAs run,
            // the other wave of the SIMD unpacks
            u32x4_t bf[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                uint32_t v[U::NPAIR];
                U::unpack(qr[j % PF][b], (tails[b] >> (8 * j)) & 0xffu, v);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    bf[b][t] = __builtin_bit_cast(uint32_t, h2_fma(v[4 * m + t], S[b][U::cls(4 * m + t)], C[b][U::cls(4 * m + t)]));
            }
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int a = 0; a < MT; ++a) acc[a][b] = mfma16(af[a], bf[b], acc[a][b]);
        }
        if constexpr (DMA) {
            // tile it + 1 was requested two sub-steps ago; what this and the previous sub-step requested may still be
            // in flight (the scale loads of a step belong to sub-step JS)
            constexpr int JS = PF == 4 ? 0 : 3;
            constexpr int N0 = 2 * (DMIN + WCNT), N1 = N0 + SCNT;
            static_assert(N1 < 64, "vmcnt holds six bits");
            if (j == JS || ((j + 3) & 3) == JS) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N1) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N0) : "memory");
        } else {
            xstore((j + 1) & 1, xr[(j + 1) % XR]);  // the other buffer: nobody reads it during this sub-step
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (j == 3) {
                tails[b] = tailsn[b];
                sc[b] = scn[b];
            }
        }
        if constexpr (DMA) {
            // A bare barrier: the fences of __syncthreads would make every outstanding request land first (copies into
            // LDS count as stores).  The wait above covers the tile the next sub-step reads; this sub-step's LDS reads
            // have returned (the MFMAs above consumed them); nothing else in LDS is written in this loop.
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            __syncthreads();
        }
      }
    }

    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // late copies must not land in reused LDS
    // minimum term and epilogue
    const float *anchors = reinterpret_cast<const float *>(w + k.anchors_off);
    float ns[NB], nm[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int rb = min(rb0 + rbo(b), k.n_rowblocks - 1);
        ns[b] = anchors[rb * 16 + r] * 64.f;
        nm[b] = anchors[16 * k.n_rowblocks + rb * 16 + r];
    }
    // sum_g sub_min_g X_g: one MFMA per step and tile.  The operands of kMinSteps steps are requested at once --
    // the tile rows' group sums through LDS (the activation buffers are free now), the sub_min bytes straight
    // into registers -- so a chunk costs one round trip to memory instead of one per step.
    float4_t accM[MT][NB];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) accM[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
    constexpr int SC = kMinSteps, XGROW = SC * 16 + 4;  // dwords per tile row in LDS, padded against bank conflicts
    constexpr int XG_PER_THREAD = (BM * SC * 4 + NT - 1) / NT;
    uint32_t *xgl = reinterpret_cast<uint32_t *>(xt);
    for (int c0 = s_begin; c0 < s_end; c0 += SC) {
        __syncthreads();  // the last reads of the activation tile / of the previous chunk are done
        u32x4_t gx[XG_PER_THREAD];
#pragma unroll
        for (int p = 0; p < XG_PER_THREAD; ++p) {
            const int i = min(tid + NT * p, BM * SC * 4 - 1);
            const int row = i / (SC * 4), rem = i - row * (SC * 4);
            const int sc_ = min(c0 + (rem >> 2), k.nsteps - 1);
            gx[p] = *reinterpret_cast<const u32x4_t *>(xg + (static_cast<int64_t>(rows.src(row)) * k.nsteps + sc_) * 16 + (rem & 3) * 4);
        }
        u32x2_t scs[SC][NB];
#pragma unroll
        for (int t = 0; t < SC; ++t)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int s = c0 + t;
                const uint32_t off = live(b) && s < s_end ? rbo(b) * rbb + s * sb + 1024 * D + (U::TAIL ? 256 : 0) : kNoStep;
                scs[t][b] = __builtin_amdgcn_raw_buffer_load_b64(win, off + lane * 8, 0, 0);
            }
#pragma unroll
        for (int p = 0; p < XG_PER_THREAD; ++p) {
            const int i = tid + NT * p;
            const int row = i / (SC * 4), rem = i - row * (SC * 4);
            if (i < BM * SC * 4) *reinterpret_cast<u32x4_t *>(xgl + row * XGROW + rem * 4) = gx[p];
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < SC; ++t) {
            if (c0 + t >= s_end) break;
            u32x4_t ax[MT];
#pragma unroll
            for (int a = 0; a < MT; ++a)
                ax[a] = *reinterpret_cast<const u32x4_t *>(xgl + ((wm * MT + a) * 16 + r) * XGROW + t * 16 + kb * 4);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const half2_t m01 = pk_h2(ubyte_f32(scs[t][b].x, 1), ubyte_f32(scs[t][b].x, 3));
                const half2_t m23 = pk_h2(ubyte_f32(scs[t][b].y, 1), ubyte_f32(scs[t][b].y, 3));
                const uint32_t b01 = __builtin_bit_cast(uint32_t, m01), b23 = __builtin_bit_cast(uint32_t, m23);
                const u32x4_t bfm = u32x4_t{b01, b23, b01, b23};
#pragma unroll
                for (int a = 0; a < MT; ++a) accM[a][b] = mfma16(ax[a], bfm, accM[a][b]);
            }
        }
    }
    // The rows' scales, all requested before the first store: a load issued between the stores would wait behind them
    // (the output may alias anything, as far as the compiler knows), one round trip to memory per row.
    float xsv[MT][4];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int v = 0; v < 4; ++v) xsv[a][v] = xscale[rows.src((wm * MT + a) * 16 + 4 * kb + v)];
#pragma unroll
    for (int a = 0; a < MT; ++a) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int ti = (wm * MT + a) * 16 + 4 * kb + v;
            const int m = rows.dst(ti);
            if (m < 0) continue;
            const float xs = xsv[a][v];
            if constexpr (GLU) {
                uint16_t *h = reinterpret_cast<uint16_t *>(y);
#pragma unroll
                for (int b = 0; b < NBG; ++b) {
                    const int col = (rb0 + b - rb_col0) * 16 + r;
                    const float g = xs * (ns[b] * acc[a][b][v] - nm[b] * accM[a][b][v]);
                    const float u = xs * (ns[b + NBG] * acc[a][b + NBG][v] - nm[b + NBG] * accM[a][b + NBG][v]);
                    const float hv = glu_value(g, u, glu.gelu != 0);
                    if (rb0 + b < rb_end && col < ncols)
                        h[static_cast<int64_t>(m) * ldy + col] = glu.f16 ? f32_to_f16_rne(hv) : f32_to_bf16_rne(hv);
                }
            } else {
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const int col = (rb0 + b - rb_col0) * 16 + r;
                    if (rb0 + b < rb_end && col < ncols)
                        y[static_cast<int64_t>(m) * ldy + col] = xs * (ns[b] * acc[a][b][v] - nm[b] * accM[a][b][v]);
                }
            }
        }
    }
}

// Dense wrapper: block (neuron tile, token tile, K split).  Split z handles the steps [z * spz, (z + 1) * spz) and
// writes its partial result to y + z * ystride (one split: y itself).
template <class U, int MT, int NB, int WM, int NW, int PF = 2, int XD = (PF == 4 ? 4 : 1)>
__global__ __launch_bounds__(64 * NW) void nint_prefill_kernel(NintK k, const uint8_t *__restrict__ w,
                                                               const uint16_t *__restrict__ x16, int Kp,
                                                               const float *__restrict__ xscale,
                                                               const uint32_t *__restrict__ xg, int M,
                                                               float *__restrict__ y, int64_t ldy, int spz,
                                                               int64_t ystride) {
    extern __shared__ __attribute__((aligned(16))) uint16_t xt[];
    const DenseRows rows{static_cast<int>(blockIdx.y) * WM * MT * 16, M};
    const int z = blockIdx.z;
    nint_prefill_body<U, MT, NB, WM, NW, DenseRows, PF, XD>(k, w, static_cast<int>(blockIdx.x) * (NW / WM) * NB, k.n_rowblocks, 0,
                                                            k.out, x16, Kp, xscale, xg, rows, y + z * ystride, ldy, xt,
                                                            z * spz, min(k.nsteps, (z + 1) * spz));
}

}  // namespace mfq
