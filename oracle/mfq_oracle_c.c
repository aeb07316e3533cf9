/*
 * C restatement of the reference's CPU paths (NINT, NVQ3J, NEPQ1-S linears; the MoE feed-forward loop)  --  TEST
 * INFRASTRUCTURE ONLY.
 *
 * The reference computes a quantized linear on the CPU as numpy fp32 `dequantize(W)` followed by
 * `x.astype(f32) @ W.T` (mfq/runtime/linear.py:37-42, mfq/quantize/nint_quant.py:896-908).  This
 * file restates exactly that in plain C (bit-stream unpack as mfq/formats/io.py:165-188, the four
 * separate fp32 roundings of the dequantizer, then a blocked fp32 GEMV/GEMM), so that bench.py can
 * time "the reference CPU path" on the GPU box's host cores and the tests can check it bit for bit
 * against oracle/mfq_oracle.py.  The NVQ3J and NEPQ1-S dequantizers and the MoE loop further down restate
 * mfq/quantize/nvq_jsc.py:1053-1079, mfq/formats/nepq.py:492-544 and cpp_runtime/mfq_decode.cpp:3394-3416 the same
 * way, from the unpacked fields (the bit streams are unpacked once at load time in the reference too), and are checked
 * bit for bit against the Python oracle in tests/.  Nothing in the shipped product links or loads it.
 *
 * Build: make -C oracle     (gcc -O2 -fopenmp -ffp-contract=off)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t read_bits(const uint8_t *s, int64_t idx, int bits, int64_t nbytes) {
    const int64_t bit = idx * bits, b = bit >> 3;
    uint32_t v = s[b];
    if (b + 1 < nbytes) v |= (uint32_t)s[b + 1] << 8;
    if (b + 2 < nbytes) v |= (uint32_t)s[b + 2] << 16;
    return (v >> (bit & 7)) & ((1u << bits) - 1u);
}

static inline float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 31u, man = h & 1023u, out;
    if (exp == 0) {
        if (man == 0) out = sign;
        else {
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 1024u));
            out = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 1023u) << 13);
        }
    } else if (exp == 31) out = sign | 0x7f800000u | (man << 13);
    else out = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &out, 4);
    return f;
}

int oracle_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* body = ns f16[out] | nm f16[out] | sub_scale bits | sub_min bits | q bits; W is [out, K] fp32. */
void oracle_nint_dequant_rows(const uint8_t *body, int bits, int sub_bits, int gs, int out, int K, int row0, int nrows,
                              float *W);
void oracle_nint_dequant(const uint8_t *body, int bits, int sub_bits, int gs, int out, int K, float *W) {
    oracle_nint_dequant_rows(body, bits, sub_bits, gs, out, K, 0, out, W);
}

/* rows [row0, row0 + nrows) of the same tensor into W [nrows, K]: one expert of a NINTM cohort's flat payload */
void oracle_nint_dequant_rows(const uint8_t *body, int bits, int sub_bits, int gs, int out, int K, int row0, int nrows,
                              float *W) {
    const int64_t ng = (K + gs - 1) / gs;
    const int64_t subs = (int64_t)out * ng, qn = subs * gs;
    const int64_t ss_bytes = (subs * sub_bits + 7) / 8, q_bytes = (qn * bits + 7) / 8;
    const uint16_t *ns16 = (const uint16_t *)body, *nm16 = ns16 + out;
    const uint8_t *ss_s = body + 4 * (int64_t)out, *sm_s = ss_s + ss_bytes, *q_s = sm_s + ss_bytes;
#pragma omp parallel for schedule(static)
    for (int r = row0; r < row0 + nrows; ++r) {
        const float ns = half_to_float(ns16[r]), nm = half_to_float(nm16[r]);
        for (int64_t g = 0; g < ng; ++g) {
            const int64_t u = (int64_t)r * ng + g;
            const volatile float d_eff = ns * (float)read_bits(ss_s, u, sub_bits, ss_bytes);
            const volatile float m_eff = nm * (float)read_bits(sm_s, u, sub_bits, ss_bytes);
            for (int i = 0; i < gs; ++i) {
                const int64_t col = g * gs + i;
                if (col >= K) break;
                const volatile float prod = d_eff * (float)read_bits(q_s, u * gs + i, bits, q_bytes);
                W[(int64_t)(r - row0) * K + col] = prod - m_eff;
            }
        }
    }
}

/* y[M, N] = x[M, K] . W[N, K]^T, fp32 accumulate (the numpy `x @ W.T`), row-parallel. */
void oracle_matmul_nt(const float *x, const float *W, int M, int N, int K, float *y) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const float *w = W + (int64_t)n * K;
        for (int m0 = 0; m0 < M; m0 += 8) {
            const int mb = M - m0 < 8 ? M - m0 : 8;
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int k = 0; k < K; ++k) {
                const float wv = w[k];
                for (int m = 0; m < mb; ++m) acc[m] += x[(int64_t)(m0 + m) * K + k] * wv;
            }
            for (int m = 0; m < mb; ++m) y[(int64_t)(m0 + m) * N + n] = acc[m];
        }
    }
}

/* NVQ-JSC (mfq/quantize/nvq_jsc.py:1053-1079): W[r, c] = (f32(mag) * sign) * fl(anchor[r] * lut[state[r, g]]),
 * g = c / 24; mag = codebooks[bank_for_state[state]][index of vector c / dim][c % dim]; sign bit c % 8 of mask
 * c / 8, the eighth sign being the parity of the seven stored ones.  indices has nvec columns per row (vectors past
 * it read entry 0), signs nsign mask bytes per row. */
void oracle_nvq_jsc_dequant(const float *anchor, const float *lut, const uint8_t *bank_for_state, const uint8_t *state,
                            const uint16_t *indices, int nvec, const uint8_t *signs, int nsign, const int8_t *codebooks,
                            int entries, int dim, int out, int K, float *W) {
    const int ng = (K + 23) / 24;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < out; ++r) {
        for (int c = 0; c < K; ++c) {
            const int g = c / 24, v = c / dim;
            const int st = state[(int64_t)r * ng + g];
            const int idx = v < nvec ? indices[(int64_t)r * nvec + v] : 0;
            const float mag = (float)codebooks[((int64_t)bank_for_state[st] * entries + idx) * dim + c % dim];
            const int m = c / 8 < nsign ? signs[(int64_t)r * nsign + c / 8] : 0, b = c % 8;
            const int neg = b < 7 ? (m >> b) & 1 : __builtin_popcount(m & 0x7f) & 1;
            const volatile float scale = anchor[r] * lut[st];
            W[(int64_t)r * K + c] = (neg ? -mag : mag) * scale;
        }
    }
}

/* NEPQ1-S (mfq/formats/nepq.py:492-544): W[r, c] = fl(anchor[r] * f32(state[r, g])) * (f32(code) + delta), g = c / 24,
 * code = tables[bank][aux[r, g]][index of vector c / 8][c % 8] with bank = bank_ids[r, g / 4], delta = -0.15625 when
 * aux is set, else +0.15625 (code + delta is exact).  tables is [banks][2][512][8] int8 (ternary digits - 1). */
void oracle_nepq1s_dequant(const float *anchor, const uint8_t *state, const uint16_t *indices, const uint8_t *aux,
                           const uint8_t *bank_ids, int nsuper, const int8_t *tables, int rows, int K, float *W) {
    const int ng = (K + 23) / 24, nvec = K / 8;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        for (int c = 0; c < K; ++c) {
            const int g = c / 24, v = c / 8;
            const int a = aux[(int64_t)r * ng + g] != 0;
            const int bank = bank_ids[(int64_t)r * nsuper + g / 4];
            const int idx = indices[(int64_t)r * nvec + v];
            const float code = (float)tables[(((int64_t)bank * 2 + a) * 512 + idx) * 8 + c % 8];
            const volatile float scale = anchor[r] * (float)state[(int64_t)r * ng + g];
            const float biased = code + (a ? -0.15625f : 0.15625f);
            W[(int64_t)r * K + c] = scale * biased;
        }
    }
}

/* silu(gate) * up evaluated in double and rounded once to fp32 (mfq/kernels/cuda/moe.cu:2980-2996 as the oracle
 * states it): hidden[i] = f32((g / (1 + exp(-g))) * u), g = gu[i], u = gu[W + i]. */
#include <math.h>
static void swiglu_row(const float *gu, int W, float *hidden) {
    for (int i = 0; i < W; ++i) {
        const double g = gu[i], u = gu[W + i];
        hidden[i] = (float)((g / (1.0 + exp(-g))) * u);
    }
}

/* The MoE feed-forward loop for T tokens with top-k routing already done (cpp_runtime/mfq_decode.cpp:3394-3416): for
 * every (token, route) pair gate_up = x[t] . GU[e]^T, hidden = swiglu, down = hidden . DN[e]^T, out[t] += w[t, r] *
 * down in route order, all fp32 products accumulated in fp32.  gu_dense / dn_dense are per-expert pointers to dense
 * fp32 [2W, H] and [H, W] matrices (NULL for experts no token selects); scratch holds T * k * (2W + W + H) floats. */
void oracle_moe_ffn(const float *x, const int32_t *ids, const float *w, int T, int k, int E, const float *const *gu_dense,
                    const float *const *dn_dense, int H, int W, float *scratch, float *out) {
    const int64_t per = 2 * (int64_t)W + W + H;
#pragma omp parallel for schedule(dynamic, 1)
    for (int p = 0; p < T * k; ++p) {
        const int t = p / k, e = ids[p];
        float *gu = scratch + p * per, *hid = gu + 2 * W, *dn = hid + W;
        if (e < 0 || e >= E || !gu_dense[e] || !dn_dense[e]) {
            memset(dn, 0, sizeof(float) * H);
            continue;
        }
        for (int n = 0; n < 2 * W; ++n) {
            const float *wr = gu_dense[e] + (int64_t)n * H;
            float acc = 0.f;
            for (int j = 0; j < H; ++j) acc += x[(int64_t)t * H + j] * wr[j];
            gu[n] = acc;
        }
        swiglu_row(gu, W, hid);
        for (int n = 0; n < H; ++n) {
            const float *wr = dn_dense[e] + (int64_t)n * W;
            float acc = 0.f;
            for (int j = 0; j < W; ++j) acc += hid[j] * wr[j];
            dn[n] = acc;
        }
    }
#pragma omp parallel for schedule(static)
    for (int t = 0; t < T; ++t)
        for (int n = 0; n < H; ++n) {
            float acc = 0.f;
            for (int r = 0; r < k; ++r) acc += w[t * k + r] * scratch[((int64_t)t * k + r) * per + 3 * (int64_t)W + n];
            out[(int64_t)t * H + n] = acc;
        }
}
