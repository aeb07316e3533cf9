/*
 * C restatement of the reference's CPU path for a NINT linear  --  TEST INFRASTRUCTURE ONLY.
 *
 * The reference computes a quantized linear on the CPU as numpy fp32 `dequantize(W)` followed by
 * `x.astype(f32) @ W.T` (mfq/runtime/linear.py:37-42, mfq/quantize/nint_quant.py:896-908).  This
 * file restates exactly that in plain C (bit-stream unpack as mfq/formats/io.py:165-188, the four
 * separate fp32 roundings of the dequantizer, then a blocked fp32 GEMV/GEMM), so that bench.py can
 * time "the reference CPU path" on the GPU box's host cores and the tests can check it bit for bit
 * against oracle/mfq_oracle.py.  Nothing in the shipped product links or loads it.
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
void oracle_nint_dequant(const uint8_t *body, int bits, int sub_bits, int gs, int out, int K, float *W) {
    const int64_t ng = (K + gs - 1) / gs;
    const int64_t subs = (int64_t)out * ng, qn = subs * gs;
    const int64_t ss_bytes = (subs * sub_bits + 7) / 8, q_bytes = (qn * bits + 7) / 8;
    const uint16_t *ns16 = (const uint16_t *)body, *nm16 = ns16 + out;
    const uint8_t *ss_s = body + 4 * (int64_t)out, *sm_s = ss_s + ss_bytes, *q_s = sm_s + ss_bytes;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < out; ++r) {
        const float ns = half_to_float(ns16[r]), nm = half_to_float(nm16[r]);
        for (int64_t g = 0; g < ng; ++g) {
            const int64_t u = (int64_t)r * ng + g;
            const volatile float d_eff = ns * (float)read_bits(ss_s, u, sub_bits, ss_bytes);
            const volatile float m_eff = nm * (float)read_bits(sm_s, u, sub_bits, ss_bytes);
            for (int i = 0; i < gs; ++i) {
                const int64_t col = g * gs + i;
                if (col >= K) break;
                const volatile float prod = d_eff * (float)read_bits(q_s, u * gs + i, bits, q_bytes);
                W[(int64_t)r * K + col] = prod - m_eff;
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
