// OCP MX weights of full-precision MFQ files: MXFP4 (E2M1 nibbles, low nibble = even column, one E8M0 scale per 32
// columns of a row) and MXFP8 (E4M3FN bytes, one E8M0 scale per 128 x 128 block).  The payload's two byte matrices are
// used as they lie in the file (mfq/formats/mx.py:65-117): values [rows, cols / 2] or [rows, cols], scales
// [rows, cols / 32] or [ceil(rows / 128), cols / 128].
//   element x scale, one fp32 multiply           cpp_runtime/mfq_decode.cpp:1920-1947, mfq/kernels/cuda/mx_matmul.cu:17-47
//   up to kMxTileMaxM rows: matrix-core tiles      mx_matmul.cu launch_mxfp8_small_m (rows 1..8 there)
//     (a wave per neuron where the activations are not 16-byte aligned rows)
//   more rows: fp16 copy + MFMA GEMM              mfq_decode.cpp:8760-8802 (dequantize, then the fp16 GEMM)
#include <type_traits>

#include "common.hpp"
#include "gemv_common.hpp"
#include "tune.hpp"

namespace mfq {

int gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, const float *sa,
                const float *sb, float *y, int64_t ldy, hipStream_t st, float *part = nullptr);
float *dequant_gemm_part(float *wscale, int N, int K, int M);
int x_prep(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, hipStream_t st);
size_t dequant_gemm_workspace(int N, int K, int M);
void dequant_gemm_carve(void *ws, int N, int K, int M, uint16_t *&x16, float *&xscale, uint16_t *&w16, float *&wscale,
                        int &Kp);

namespace {

constexpr int kMxGemvMaxM = 16;   // rows up to which the wave-per-neuron kernel serves calls the tile kernel cannot take
constexpr int kMxTileMaxM = 256;  // rows up to which the tile kernel runs (passes of 32 rows); above: fp16 copy + GEMM

struct MxK {
    int kind, rows, cols, row0, nrows;
    const uint8_t *values, *scales;
};

__device__ __forceinline__ float mx_nan() { return __uint_as_float(0x7fffffffu); }
// E8M0: 2^(raw - 127); raw 0 is the subnormal 2^-127, raw 255 a NaN (mx_matmul.cu:17-28)
__device__ __forceinline__ float e8m0_f32(uint32_t raw) {
    if (raw == 255u) return mx_nan();
    return raw == 0u ? __uint_as_float(0x00400000u) : __uint_as_float(raw << 23);
}
// E4M3FN (mx_matmul.cu:30-47): bias 7, no infinities, exponent 15 with mantissa 7 is NaN.  The seven magnitude bits,
// moved to bits 7..13 of an fp16, are the same number scaled by 2^-8 -- subnormals included.
__device__ __forceinline__ float e4m3fn_f32(uint32_t b) {
    const uint32_t mag = b & 0x7fu;
    float v = f16_to_f32(static_cast<uint16_t>(mag << 7)) * 256.f;
    if (mag == 0x7fu) v = mx_nan();
    return (b & 0x80u) ? -v : v;
}
// E2M1 (mfq_decode.cpp:1926-1946): 0, 0.5, 1, 1.5, 2, 3, 4, 6 with a sign bit; the three magnitude bits at bits 9..11
// of an fp16 are the number scaled by 2^-14.
__device__ __forceinline__ float e2m1_f32(uint32_t c) {
    const float v = f16_to_f32(static_cast<uint16_t>((c & 7u) << 9)) * 16384.f;
    return (c & 8u) ? -v : v;
}

// element (row, col) of the tensor
template <int KIND>
__device__ __forceinline__ float mx_elem(const MxK &k, int row, int col) {
    if constexpr (KIND == 4) {
        const uint32_t byte = k.values[static_cast<int64_t>(row) * (k.cols / 2) + col / 2];
        return e2m1_f32((byte >> (4 * (col & 1))) & 15u);
    } else {
        return e4m3fn_f32(k.values[static_cast<int64_t>(row) * k.cols + col]);
    }
}
template <int KIND>
__device__ __forceinline__ uint32_t mx_scale_raw(const MxK &k, int row, int col) {
    if constexpr (KIND == 4) return k.scales[static_cast<int64_t>(row) * (k.cols / 32) + col / 32];
    else return k.scales[static_cast<int64_t>(row / 128) * (k.cols / 128) + col / 128];
}

// ---- dequantizers -------------------------------------------------------------------------------------------
// fp32 / fp16 (one more rounding) copy of rows [row0, row0 + nrows): out[r - row0][c]
template <int KIND, typename OutT>
__global__ __launch_bounds__(256) void mx_dequant_kernel(MxK k, OutT *__restrict__ out, int64_t ld) {
    const int row = k.row0 + blockIdx.y;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < k.cols; c += gridDim.x * 256) {
        const float v = mx_elem<KIND>(k, row, c) * e8m0_f32(mx_scale_raw<KIND>(k, row, c));
        if constexpr (sizeof(OutT) == 4) out[static_cast<int64_t>(blockIdx.y) * ld + c] = v;
        else out[static_cast<int64_t>(blockIdx.y) * ld + c] = f32_to_f16_rne(v);
    }
}

// fp16 rows for the GEMM, each relative to the largest scale of its row (wscale[r] = that scale): the elements stay
// within fp16 whatever the scales are -- the reference rounds the products themselves to fp16 and saturates
// (mx_matmul.cu:222-240) -- and blocks more than 2^-24 below the row's largest vanish as they would against it.
// w16 [nrows, Kp], zero beyond cols.
template <int KIND>
__global__ __launch_bounds__(256) void mx_stage_f16_kernel(MxK k, uint16_t *__restrict__ w16, int Kp,
                                                           float *__restrict__ wscale) {
    __shared__ uint32_t smax[4];
    const int row = k.row0 + blockIdx.x, tid = threadIdx.x;
    constexpr int BLK = KIND == 4 ? 32 : 128;
    uint32_t emax = 0;
    for (int g = tid; g < k.cols / BLK; g += 256) {
        const uint32_t raw = mx_scale_raw<KIND>(k, row, g * BLK);
        if (raw != 255u && raw > emax) emax = raw;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) emax = max(emax, static_cast<uint32_t>(__shfl_xor(static_cast<int>(emax), o, 64)));
    if ((tid & 63) == 0) smax[tid >> 6] = emax;
    __syncthreads();
    emax = max(max(smax[0], smax[1]), max(smax[2], smax[3]));
    if (tid == 0) wscale[blockIdx.x] = e8m0_f32(emax);
    for (int c = tid; c < Kp; c += 256) {
        float v = 0.f;
        if (c < k.cols) {
            const uint32_t raw = mx_scale_raw<KIND>(k, row, c);
            // 2^(raw - emax) as an fp32: exact down to 2^-126, zero below (the product would be below fp16 anyway)
            const int e = static_cast<int>(raw) - static_cast<int>(emax) + 127;
            const float rel = raw == 255u ? mx_nan() : (e > 0 ? __uint_as_float(static_cast<uint32_t>(e) << 23) : 0.f);
            v = mx_elem<KIND>(k, row, c) * rel;
        }
        w16[static_cast<int64_t>(blockIdx.x) * Kp + c] = f32_to_f16_rne(v);
    }
}

// ---- GEMV: a wave per neuron, MB activation rows per pass ------------------------------------------------------
// A lane takes 16 bytes of the neuron at a time -- 32 MXFP4 or 16 MXFP8 weights under one scale -- and the matching
// activations of the MB rows; fp32 accumulation, one wave reduction at the end.
template <int KIND, int XF16, int MB>
__global__ __launch_bounds__(256) void mx_gemv_kernel(MxK k, const uint16_t *__restrict__ x_in, int64_t ldx, int M_in,
                                                      float *__restrict__ y_in, int64_t ldy, PairSel sel) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = blockIdx.x * 4 + wave;
    if (r >= k.nrows) return;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = blockIdx.y * MB;
    if (sel.ids) {  // a pair of a MoE decode step: one row, the expert's rows of the pool (nrows = rows per expert)
        const uint16_t *xr[1];
        float *yr[1];
        const uint8_t *unused = nullptr;
        int local;
        if (!select_rows<1>(sel, unused, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        k.row0 = local * k.nrows;
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    const int row = k.row0 + r;
    constexpr int PER = KIND == 4 ? 32 : 16;  // weights in 16 bytes
    const int64_t row_bytes = KIND == 4 ? k.cols / 2 : k.cols;
    const uint8_t *vrow = k.values + static_cast<int64_t>(row) * row_bytes;
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.f;
    for (int c = lane; c * PER < k.cols; c += 64) {
        const u32x4_t q = *reinterpret_cast<const u32x4_t *>(vrow + 16 * c);
        const float sc = e8m0_f32(mx_scale_raw<KIND>(k, row, c * PER));
        float part[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) part[m] = 0.f;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            float wv[PER / 4];
#pragma unroll
            for (int t = 0; t < PER / 4; ++t) {
                if constexpr (KIND == 4) wv[t] = e2m1_f32((q[d] >> (4 * t)) & 15u);
                else wv[t] = e4m3fn_f32((q[d] >> (8 * t)) & 255u);
            }
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                const uint16_t *xp = x + static_cast<int64_t>(min(m0 + m, M - 1)) * ldx + c * PER + d * (PER / 4);
#pragma unroll
                for (int t = 0; t < PER / 4; ++t) part[m] = fmaf(wv[t], x_to_f32<XF16>(xp[t]), part[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = fmaf(sc, part[m], acc[m]);
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float v = acc[m];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if (lane == 0 && m0 + m < M) y[static_cast<int64_t>(m0 + m) * ldy + r] = v;
    }
}

// ---- up to 32 rows per tile on the matrix cores -----------------------------------------------------------------------
// The values are read as they lie in the file and converted by the hardware: v_cvt_scalef32_pk_{bf16,f16}_{fp4,fp8}
// turns two E2M1 nibbles (low nibble first) or two E4M3FN bytes into a pair of the activations' type and multiplies by
// the power of two in the exponent field of its scale operand -- an E8M0 byte shifted into place, with E8M0's own
// meaning of 0 (2^-127) and 255 (NaN).  For bf16 activations the product element x scale is exact in bf16 (its exponent
// range is fp32's), so a block's weights enter v_mfma_f32_16x16x32_bf16 already scaled and the accumulator runs through
// the whole K slice; for fp16 activations the elements enter unscaled, a scale block's sum comes out of an accumulator
// that starts at zero and the scale multiplies it in fp32 (fp16 would overflow).  No conversion of the activations.
// A unit is 64 value bytes of a neuron: four MXFP4 scale blocks (128 columns) or 64 MXFP8 columns; lane (r, kb) loads
// its 16 bytes at kb.  MXFP4: a 4 x 4 transposition of dwords between the lane's four 16-lane rows (two lane swaps per
// register pair) leaves register m with codes 8 kb .. 8 kb + 7 of block m, so MFMA m covers one scale block.  MXFP8: the
// four dwords are two MFMAs' worth of k as they are (an MFMA does not care which k sits in which slot as long as both
// operands agree).  A block of the grid owns NB row-blocks of 16 neurons and MT tiles of 16 rows; its waves split the
// units of K; two units are in flight per wave.  LDS: waves * NB * MT * 1 KB for the sum over the waves.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

template <int XF16>
__device__ __forceinline__ float4_t mx_mfma(u32x4_t a, u32x4_t b, float4_t c) {
    if constexpr (XF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
// eight E2M1 codes of a dword -> eight values of the activations' type, times 2^(exponent field of scale - 127)
template <int XF16>
__device__ __forceinline__ u32x4_t mx_cvt_fp4(uint32_t q, float scale) {
    u32x4_t b;
    if constexpr (XF16) {
        b.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, scale, 0));
        b.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, scale, 1));
        b.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, scale, 2));
        b.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, scale, 3));
    } else {
        b.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 0));
        b.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 1));
        b.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 2));
        b.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, scale, 3));
    }
    return b;
}
// eight E4M3FN codes of two dwords
template <int XF16>
__device__ __forceinline__ u32x4_t mx_cvt_fp8(uint32_t q0, uint32_t q1, float scale) {
    u32x4_t b;
    if constexpr (XF16) {
        b.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(q0, scale, false));
        b.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(q0, scale, true));
        b.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(q1, scale, false));
        b.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(q1, scale, true));
    } else {
        b.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q0, scale, false));
        b.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q0, scale, true));
        b.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q1, scale, false));
        b.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(q1, scale, true));
    }
    return b;
}

// SAL: a row's scale bytes start on a 4-byte boundary (MXFP4: cols % 128 == 0), one dword per unit; else four byte reads
template <int KIND, int XF16, int NB, int MT, bool SAL>
__global__ __launch_bounds__(1024) void mx_tile_kernel(MxK k, const uint16_t *__restrict__ x_in, int64_t ldx, int M_in,
                                                       float *__restrict__ y_in, int64_t ldy, int upw, PairSel sel) {
    constexpr int FR = KIND == 4 ? 4 : 2;        // MFMAs, and activation fragments per token tile, of a unit
    constexpr int UCOLS = KIND == 4 ? 128 : 64;  // columns of a unit
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    float *red = reinterpret_cast<float *>(lds);
    const int tid = threadIdx.x, lane = tid & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kb = lane >> 4;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = static_cast<int>(blockIdx.y) * 16 * MT;
    if (sel.ids) {  // a pair of a MoE decode step: one row, the expert's rows of the pool (nrows = rows per expert)
        const uint16_t *xr[1];
        float *yr[1];
        const uint8_t *unused = nullptr;
        int local;
        if (!select_rows<1>(sel, unused, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        k.row0 = local * k.nrows;
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    const int mt = min(16 * MT, M - m0);  // rows of this block's tiles
    const int nunits = (k.cols + UCOLS - 1) / UCOLS;
    const int u0 = wave * upw, u1 = min(nunits, u0 + upw);
    const int rb0 = static_cast<int>(blockIdx.x) * NB;
    const int rows_here = min(NB * 16, k.nrows - rb0 * 16);
    const uint32_t row_bytes = static_cast<uint32_t>(KIND == 4 ? k.cols / 2 : k.cols);
    const int row_first = k.row0 + rb0 * 16;  // of the tensor
    const __amdgpu_buffer_rsrc_t win = wave_window(k.values + static_cast<int64_t>(row_first) * row_bytes,
                                                   static_cast<uint32_t>(rows_here) * row_bytes);
    const uint32_t nblk = static_cast<uint32_t>(k.cols / (KIND == 4 ? 32 : 128));  // scale bytes of a row (MXFP4) or block row
    const uint32_t scale_bytes = KIND == 4 ? static_cast<uint32_t>(k.rows) * nblk : static_cast<uint32_t>((k.rows + 127) / 128) * nblk;
    const __amdgpu_buffer_rsrc_t swin = wave_window(k.scales, scale_bytes);
    const __amdgpu_buffer_rsrc_t xwin = wave_window(reinterpret_cast<const uint8_t *>(x + static_cast<int64_t>(m0) * ldx),
                                                    static_cast<uint32_t>((static_cast<int64_t>(mt - 1) * ldx + k.cols) * 2));
    const uint32_t ldx2 = static_cast<uint32_t>(ldx) * 2u;

    auto wload = [&](int u, u32x4_t (&q)[NB], uint32_t (&s)[NB]) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int rr = i * 16 + r;
            const bool row_ok = u < u1 && rr < rows_here;
            const bool ok = row_ok && (KIND == 8 || static_cast<uint32_t>(4 * u + kb) < nblk);
            q[i] = __builtin_amdgcn_raw_buffer_load_b128(win, ok ? static_cast<uint32_t>(rr) * row_bytes + static_cast<uint32_t>(u * 64 + kb * 16) : kNoStep, 0, 2);
            if constexpr (KIND == 4) {
                const uint32_t so = static_cast<uint32_t>(row_first + rr) * nblk + 4u * u;
                if constexpr (SAL) {
                    s[i] = __builtin_amdgcn_raw_buffer_load_b32(swin, row_ok ? so : kNoStep, 0, 0);
                } else {
                    uint32_t b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        b[j] = __builtin_amdgcn_raw_buffer_load_b8(swin, row_ok && static_cast<uint32_t>(4 * u + j) < nblk ? so + j : kNoStep, 0, 0);
                    s[i] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                }
            } else {
                const uint32_t so = static_cast<uint32_t>((row_first + rr) >> 7) * nblk + static_cast<uint32_t>(u >> 1);
                s[i] = __builtin_amdgcn_raw_buffer_load_b8(swin, row_ok ? so : kNoStep, 0, 0);
            }
        }
    };
    // lane (token, kb) of tile t: the 8 activations the lane's k slots of MFMA f stand for
    auto xload = [&](int u, u32x4_t (&a)[MT][FR]) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int f = 0; f < FR; ++f) {
                const int tok = 16 * t + r;
                const int col = KIND == 4 ? (4 * u + f) * 32 + 8 * kb : 64 * u + 16 * kb + 8 * f;
                const bool ok = u < u1 && tok < mt && col < k.cols;
                a[t][f] = __builtin_amdgcn_raw_buffer_load_b128(xwin, ok ? static_cast<uint32_t>(tok) * ldx2 + static_cast<uint32_t>(col) * 2u : kNoStep, 0, 0);
            }
    };
    float4_t acc[NB][MT];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[i][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    auto compute = [&](const u32x4_t (&q)[NB], const uint32_t (&s)[NB], const u32x4_t (&a)[MT][FR]) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if constexpr (KIND == 4) {
                const auto p02 = __builtin_amdgcn_permlane32_swap(q[i].x, q[i].z, false, false);
                const auto p13 = __builtin_amdgcn_permlane32_swap(q[i].y, q[i].w, false, false);
                const auto t01 = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
                const auto t23 = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
                const uint32_t tq[4] = {t01[0], t01[1], t23[0], t23[1]};
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    const uint32_t raw = (s[i] >> (8 * f)) & 255u;
                    if constexpr (XF16) {
                        const u32x4_t b = mx_cvt_fp4<1>(tq[f], 1.f);
                        const float sc = e8m0_f32(raw);
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            const float4_t part = mx_mfma<1>(a[t][f], b, float4_t{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                            for (int v = 0; v < 4; ++v) acc[i][t][v] = fmaf(sc, part[v], acc[i][t][v]);
                        }
                    } else {
                        const u32x4_t b = mx_cvt_fp4<0>(tq[f], __uint_as_float(raw << 23));
#pragma unroll
                        for (int t = 0; t < MT; ++t) acc[i][t] = mx_mfma<0>(a[t][f], b, acc[i][t]);
                    }
                }
            } else {
                if constexpr (XF16) {
                    const u32x4_t b0 = mx_cvt_fp8<1>(q[i].x, q[i].y, 1.f), b1 = mx_cvt_fp8<1>(q[i].z, q[i].w, 1.f);
                    const float sc = e8m0_f32(s[i]);
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        float4_t part = mx_mfma<1>(a[t][0], b0, float4_t{0.f, 0.f, 0.f, 0.f});
                        part = mx_mfma<1>(a[t][1], b1, part);
#pragma unroll
                        for (int v = 0; v < 4; ++v) acc[i][t][v] = fmaf(sc, part[v], acc[i][t][v]);
                    }
                } else {
                    const float sc = __uint_as_float(s[i] << 23);
                    const u32x4_t b0 = mx_cvt_fp8<0>(q[i].x, q[i].y, sc), b1 = mx_cvt_fp8<0>(q[i].z, q[i].w, sc);
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        acc[i][t] = mx_mfma<0>(a[t][0], b0, acc[i][t]);
                        acc[i][t] = mx_mfma<0>(a[t][1], b1, acc[i][t]);
                    }
                }
            }
        }
    };
    u32x4_t qa[NB], qb[NB], xa[MT][FR], xb[MT][FR];
    uint32_t sa[NB], sb[NB];
    wload(u0, qa, sa);
    xload(u0, xa);
    for (int u = u0; u < u1; u += 2) {
        wload(u + 1, qb, sb);
        xload(u + 1, xb);
        compute(qa, sa, xa);
        wload(u + 2, qa, sa);
        xload(u + 2, xa);
        compute(qb, sb, xb);
    }
    // lane (r, kb), register v of acc[i][t] = y[token m0 + 16 t + 4 kb + v][neuron (rb0 + i) * 16 + r]
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[(((wave * NB + i) * MT + t) * 4 + v) * 64 + lane] = acc[i][t][v];
    __syncthreads();
    for (int o = tid; o < NB * MT * 256; o += blockDim.x) {
        const int rr = o & 15, tk = (o >> 4) & 15, it = o >> 8;
        const int slot = (it * 4 + (tk & 3)) * 64 + rr + 16 * (tk >> 2);
        float sum = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) sum += red[wv * NB * MT * 256 + slot];
        const int row = (rb0 + it / MT) * 16 + rr, tok = 16 * (it % MT) + tk;
        if (tok < mt && row < k.nrows) y[static_cast<int64_t>(m0 + tok) * ldy + row] = sum;
    }
}

int mx_check(const char *what, int kind, const void *values, const void *scales, int rows, int cols, int row0, int nrows) {
    MFQ_REQUIRE(kind == 4 || kind == 8, MFQ_ERR_INVALID, "%s: kind %d is neither MXFP4 (4) nor MXFP8 (8)", what, kind);
    MFQ_REQUIRE(values && scales, MFQ_ERR_INVALID, "%s: null argument", what);
    MFQ_REQUIRE(rows > 0 && cols > 0, MFQ_ERR_INVALID, "%s: invalid MX logical shape: (%d, %d)", what, rows, cols);
    if (kind == 4) MFQ_REQUIRE(cols % 32 == 0, MFQ_ERR_INVALID, "MXFP4 columns must be divisible by 32");
    else MFQ_REQUIRE(cols % 128 == 0, MFQ_ERR_INVALID, "MXFP8 columns must be divisible by 128");
    MFQ_REQUIRE(row0 >= 0 && nrows > 0 && row0 <= rows - nrows, MFQ_ERR_INVALID, "%s: rows [%d, %d) outside the tensor's %d",
                what, row0, row0 + nrows, rows);
    MFQ_REQUIRE(nrows <= 65535 * 4, MFQ_ERR_UNSUPPORTED, "%s: %d neurons in one call (max %d)", what, nrows, 65535 * 4);
    return MFQ_OK;
}

// ---- up to 16 rows with the wave's slice of the activations and scales staged in LDS ----------------------------------
// A compute unit keeps about 64 memory requests in flight whatever their size, so what counts is bytes per request:
// mx_tile_kernel asks, per unit and row-block, for 1 KB of values, a scale word and its share of four activation
// fragments -- three requests a kilobyte, 3 TB/s.  Here a wave fetches its K slice of the tile's rows in whole 1 KB
// requests (64 lanes x 16 bytes, row after row) and the slice's scale bytes of all its row-blocks in one request per
// four blocks (lane L = row L of the block's NB * 16), parks both in its own corner of the LDS and reads fragments and
// scales from there; inside the walk only values are requested.  bf16 activations need no transposition either: the
// conversion applies each lane's own block scale, so MFMA f simply takes dword f of every lane (four scale blocks side
// by side in its 32 k slots) against activations 8 f .. 8 f + 7 of the lane's block.
// LDS per wave: [x: mt rows of n_units * (256 | 128) + 16 bytes][scales: NB * 16 rows x 32 bytes]; the partial sums
// overlay it after a barrier.
constexpr int kMxStageReq = 8;   // 1 KB requests a wave's activation slice may take
constexpr int kMxStageUnits = 8; // units per wave: the slice's MXFP4 scale bytes of a row are a 32-byte LDS row

template <int KIND, int XF16, int NB, bool SAL, int XR>
__global__ __launch_bounds__(1024) void mx_tile_lds_kernel(MxK k, const uint16_t *__restrict__ x_in, int64_t ldx, int M_in,
                                                           float *__restrict__ y_in, int64_t ldy, int upw, int upw_rcp,
                                                           int xrows, PairSel sel) {
    constexpr int UB = KIND == 4 ? 256 : 128;  // activation bytes of a unit and row
    constexpr bool TRANSPOSED = KIND == 4 && XF16;  // fp16 against MXFP4: one scale block per MFMA, scaled afterwards
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    float *red = reinterpret_cast<float *>(lds);
    const int tid = threadIdx.x, lane = tid & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kb = lane >> 4;
    const uint16_t *x = x_in;
    float *y = y_in;
    int M = M_in, m0 = static_cast<int>(blockIdx.y) * 16;
    if (sel.ids) {
        const uint16_t *xr[1];
        float *yr[1];
        const uint8_t *unused = nullptr;
        int local;
        if (!select_rows<1>(sel, unused, local, x_in, ldx, y_in, ldy, M_in, xr, yr)) return;
        k.row0 = local * k.nrows;
        x = xr[0];
        y = yr[0];
        M = 1;
        m0 = 0;
    }
    const int mt = min(16, M - m0);
    const int nunits = (k.cols + (KIND == 4 ? 127 : 63)) / (KIND == 4 ? 128 : 64);
    const int u0 = wave * upw, u1 = min(nunits, u0 + upw);
    const int rb0 = static_cast<int>(blockIdx.x) * NB;
    const int rows_here = min(NB * 16, k.nrows - rb0 * 16);
    const uint32_t row_bytes = static_cast<uint32_t>(KIND == 4 ? k.cols / 2 : k.cols);
    const int row_first = k.row0 + rb0 * 16;
    const __amdgpu_buffer_rsrc_t win = wave_window(k.values + static_cast<int64_t>(row_first) * row_bytes,
                                                   static_cast<uint32_t>(rows_here) * row_bytes);
    const uint32_t nblk = static_cast<uint32_t>(k.cols / (KIND == 4 ? 32 : 128));
    const uint32_t scale_bytes = KIND == 4 ? static_cast<uint32_t>(k.rows) * nblk : static_cast<uint32_t>((k.rows + 127) / 128) * nblk;
    const __amdgpu_buffer_rsrc_t swin = wave_window(k.scales, scale_bytes);
    const __amdgpu_buffer_rsrc_t xwin = wave_window(reinterpret_cast<const uint8_t *>(x + static_cast<int64_t>(m0) * ldx),
                                                    static_cast<uint32_t>((static_cast<int64_t>(mt - 1) * ldx + k.cols) * 2));
    const uint32_t xrow = static_cast<uint32_t>(upw) * UB + 16u;       // LDS bytes of a staged row
    const uint32_t wave_bytes = static_cast<uint32_t>(xrows) * xrow + NB * 512u;  // of a wave's corner
    uint8_t *xs = reinterpret_cast<uint8_t *>(lds) + static_cast<size_t>(wave) * wave_bytes;
    uint8_t *ss = xs + static_cast<uint32_t>(xrows) * xrow;
    typedef __attribute__((address_space(3))) const u32x4_t *lds_u32x4_ptr;
    typedef __attribute__((address_space(3))) const uint32_t *lds_u32_ptr;
    typedef __attribute__((address_space(3))) const uint8_t *lds_u8_ptr;
    const uint32_t xs_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)xs));
    const uint32_t ss_lds = xs_lds + static_cast<uint32_t>(xrows) * xrow;

    // ---- requests, in order of use: activations, scales, the first two units of values -------------------------------
    // piece g = 64 * q + lane of the slice: 16 bytes, row g / ppr, at 16 * (g % ppr) of the row's slice; XR requests
    // (a template constant: a request that moves nothing still takes its turn in the compute unit's queue)
    const uint32_t ppr = static_cast<uint32_t>(upw) * (UB / 16);
    u32x4_t xraw[XR];
    uint32_t xdst[XR];
#pragma unroll
    for (int q = 0; q < XR; ++q) {
        const uint32_t g = static_cast<uint32_t>(q * 64 + lane);
        const uint32_t tok = ((g / (UB / 16)) * static_cast<uint32_t>(upw_rcp)) >> 16;  // g / ppr
        const uint32_t piece = g - tok * ppr;
        const uint32_t col = static_cast<uint32_t>(u0) * (UB / 2) + piece * 8u;
        const bool ok = tok < static_cast<uint32_t>(mt) && col < static_cast<uint32_t>(k.cols) && u0 < u1;
        xraw[q] = __builtin_amdgcn_raw_buffer_load_b128(xwin, ok ? tok * static_cast<uint32_t>(ldx) * 2u + col * 2u : kNoStep, 0, 0);
        xdst[q] = tok < static_cast<uint32_t>(mt) ? tok * xrow + piece * 16u : kNoStep;
    }
    // scales of row `lane` of the block's rows, for the blocks of the slice (MXFP4: 4 per unit, MXFP8: one per two units)
    // (one of three straight-line copies by the slice's length: a request that moves nothing still takes its turn)
    uint32_t sraw[kMxStageUnits + 1];
#pragma unroll
    for (int c = 0; c <= kMxStageUnits; ++c) sraw[c] = 0u;
    {
        const bool row_ok = lane < rows_here && u0 < u1;
        auto scale_loads = [&](auto CNT) {
            constexpr int N = decltype(CNT)::value;  // units covered
            if constexpr (KIND == 4) {
                const uint32_t a = static_cast<uint32_t>(row_first + lane) * nblk + 4u * u0;
#pragma unroll
                for (int c = 0; c < N + (SAL ? 0 : 1); ++c)
                    sraw[c] = __builtin_amdgcn_raw_buffer_load_b32(swin, row_ok && c < upw + (SAL ? 0 : 1) ? (a & ~3u) + 4u * c : kNoStep, 0, 0);
                if constexpr (!SAL) {
#pragma unroll
                    for (int c = 0; c < N; ++c) sraw[c] = __builtin_amdgcn_alignbyte(sraw[c + 1], sraw[c], a & 3u);
                }
            } else {
                const uint32_t a = static_cast<uint32_t>((row_first + lane) >> 7) * nblk + static_cast<uint32_t>(u0 >> 1);
                uint32_t b[5] = {0u, 0u, 0u, 0u, 0u};  // N units from u0 on touch at most N / 2 + 1 blocks of 128 columns
#pragma unroll
                for (int c = 0; c < N / 2 + 1; ++c)
                    b[c] = __builtin_amdgcn_raw_buffer_load_b8(swin, row_ok && (u0 >> 1) + c < static_cast<int>(nblk) ? a + c : kNoStep, 0, 0);
                sraw[0] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                sraw[1] = b[4];
            }
        };
        if (upw <= 2) scale_loads(std::integral_constant<int, 2>{});
        else if (upw <= 4) scale_loads(std::integral_constant<int, 4>{});
        else scale_loads(std::integral_constant<int, kMxStageUnits>{});
    }
    auto wload = [&](int u, u32x4_t (&q)[NB]) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int rr = i * 16 + r;
            const bool ok = u < u1 && rr < rows_here && (KIND == 8 || static_cast<uint32_t>(4 * u + kb) < nblk);
            q[i] = __builtin_amdgcn_raw_buffer_load_b128(win, ok ? static_cast<uint32_t>(rr) * row_bytes + static_cast<uint32_t>(u * 64 + kb * 16) : kNoStep, 0, 2);
        }
    };
    u32x4_t qa[NB], qb[NB];
    wload(u0, qa);
    wload(u0 + 1, qb);
    // ---- the slice into the wave's corner ---------------------------------------------------------------------------
#pragma unroll
    for (int q = 0; q < XR; ++q)
        if (xdst[q] != kNoStep) *reinterpret_cast<u32x4_t *>(xs + xdst[q]) = xraw[q];
    if (lane < NB * 16) {
        if constexpr (KIND == 4) {
            *reinterpret_cast<u32x4_t *>(ss + lane * 32) = u32x4_t{sraw[0], sraw[1], sraw[2], sraw[3]};
            *reinterpret_cast<u32x4_t *>(ss + lane * 32 + 16) = u32x4_t{sraw[4], sraw[5], sraw[6], sraw[7]};
        } else {
            *reinterpret_cast<u32x2_t *>(ss + lane * 32) = u32x2_t{sraw[0], sraw[1]};
        }
    }
    // rows of the tile that are not there read the wave's row 0 and are multiplied into rows nobody stores
    const uint32_t arow = xs_lds + static_cast<uint32_t>(min(r, mt - 1)) * xrow + (TRANSPOSED ? kb * 16u : kb * (UB / 4));
    float4_t acc[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    auto compute = [&](int u, const u32x4_t (&q)[NB]) {
        const uint32_t lu = static_cast<uint32_t>(u - u0);
        constexpr int FR = KIND == 4 ? 4 : 2;
        u32x4_t a[FR];
#pragma unroll
        for (int f = 0; f < FR; ++f) a[f] = *reinterpret_cast<lds_u32x4_ptr>(arow + lu * UB + (TRANSPOSED ? f * 64u : f * 16u));
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const uint32_t srow = ss_lds + static_cast<uint32_t>(i * 16 + r) * 32u;
            if constexpr (KIND == 4 && !XF16) {
                uint32_t raw = *reinterpret_cast<lds_u8_ptr>(srow + 4u * lu + kb);
                raw = static_cast<uint32_t>(4 * u + kb) < nblk ? raw : 0u;  // past K: the bytes belong to the next row
                const float sc = __uint_as_float(raw << 23);
                const uint32_t qd[4] = {q[i].x, q[i].y, q[i].z, q[i].w};
#pragma unroll
                for (int f = 0; f < 4; ++f) acc[i] = mx_mfma<0>(a[f], mx_cvt_fp4<0>(qd[f], sc), acc[i]);
            } else if constexpr (KIND == 4) {
                const uint32_t s4 = *reinterpret_cast<lds_u32_ptr>(srow + 4u * lu);
                const auto p02 = __builtin_amdgcn_permlane32_swap(q[i].x, q[i].z, false, false);
                const auto p13 = __builtin_amdgcn_permlane32_swap(q[i].y, q[i].w, false, false);
                const auto t01 = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
                const auto t23 = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
                const uint32_t tq[4] = {t01[0], t01[1], t23[0], t23[1]};
#pragma unroll
                for (int f = 0; f < 4; ++f) {
                    const uint32_t raw = static_cast<uint32_t>(4 * u + f) < nblk ? (s4 >> (8 * f)) & 255u : 0u;
                    const float4_t part = mx_mfma<1>(a[f], mx_cvt_fp4<1>(tq[f], 1.f), float4_t{0.f, 0.f, 0.f, 0.f});
                    const float sc = e8m0_f32(raw);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[i][v] = fmaf(sc, part[v], acc[i][v]);
                }
            } else {
                const uint32_t raw = *reinterpret_cast<lds_u8_ptr>(srow + static_cast<uint32_t>((u >> 1) - (u0 >> 1)));
                if constexpr (XF16) {
                    float4_t part = mx_mfma<1>(a[0], mx_cvt_fp8<1>(q[i].x, q[i].y, 1.f), float4_t{0.f, 0.f, 0.f, 0.f});
                    part = mx_mfma<1>(a[1], mx_cvt_fp8<1>(q[i].z, q[i].w, 1.f), part);
                    const float sc = e8m0_f32(raw);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[i][v] = fmaf(sc, part[v], acc[i][v]);
                } else {
                    const float sc = __uint_as_float(raw << 23);
                    acc[i] = mx_mfma<0>(a[0], mx_cvt_fp8<0>(q[i].x, q[i].y, sc), acc[i]);
                    acc[i] = mx_mfma<0>(a[1], mx_cvt_fp8<0>(q[i].z, q[i].w, sc), acc[i]);
                }
            }
        }
    };
    for (int u = u0; u < u1; u += 2) {
        compute(u, qa);
        wload(u + 2, qa);
        if (u + 1 < u1) compute(u + 1, qb);
        wload(u + 3, qb);
    }
    __syncthreads();  // every wave is done with its corner: the partial sums overlay them
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[((wave * NB + i) * 4 + v) * 64 + lane] = acc[i][v];
    __syncthreads();
    for (int o = tid; o < NB * 256; o += blockDim.x) {
        const int rr = o & 15, tk = (o >> 4) & 15, i = o >> 8;
        const int slot = (i * 4 + (tk & 3)) * 64 + rr + 16 * (tk >> 2);
        float sum = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) sum += red[wv * NB * 256 + slot];
        const int row = (rb0 + i) * 16 + rr;
        if (tk < mt && row < k.nrows) y[static_cast<int64_t>(m0 + tk) * ldy + row] = sum;
    }
}

static int mx_tile_max_m() {
    static const int v = tune_env("MFQ_MX_TILE_MAX_M", kMxTileMaxM);
    return v < kMxGemvMaxM ? kMxGemvMaxM : v;
}
// What the tile kernel needs of a call: 16-byte activation fragments (aligned rows), a tile's rows and the tensor's
// scale bytes inside 32-bit buffer windows.
static bool mx_tile_eligible(const MxK &k, const void *x, int64_t ldx) {
    static const int off = tune_env("MFQ_MX_TILE_OFF", 0);
    const int64_t row_bytes = k.kind == 4 ? k.cols / 2 : k.cols;
    return !off && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && ldx % 8 == 0 && (31 * ldx + k.cols) * 2 < (1ll << 31) &&
           (reinterpret_cast<uintptr_t>(k.values) & 15) == 0 && 64 * row_bytes < (1ll << 31) &&
           static_cast<int64_t>(k.rows) * (k.cols / 32) < (1ll << 31);
}
// Row-blocks per block: the count in 1 .. max_nb that needs the fewest rounds of one block per compute unit, weighted by
// the block's length; ties go to the larger count (its row-blocks share the activation fragments).
static int mx_tile_nb(int64_t n_rowblocks, int64_t tiles, int max_nb) {
    int best = 1;
    int64_t best_cost = 0;
    for (int nb = 1; nb <= max_nb; ++nb) {
        const int64_t cost = ceil_div(ceil_div(n_rowblocks, nb) * tiles, gemv_cu_count()) * nb;
        if (nb == 1 || cost <= best_cost) {
            best = nb;
            best_cost = cost;
        }
    }
    return best;
}
// n_pairs = 0: dense rows (tiles of 16 or 32); else one row per pair of `sel`
template <int KIND, int XF16>
int mx_launch_tile(const MxK &k, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy, const PairSel &sel, int n_pairs,
                   hipStream_t st) {
    // fp16 activations against MXFP4: a partial accumulator and a scale per block leave registers for one row-block and
    // one tile (more spill); the other combinations scale inside the conversion
    constexpr bool narrow = KIND == 4 && XF16;
    static const int env_nb = tune_env("MFQ_MX_NB", 0), env_waves = tune_env("MFQ_MX_WAVES", 0);
    static const int lds_off = tune_env("MFQ_MX_STAGE_OFF", 0);
    const int nunits = static_cast<int>(ceil_div(k.cols, KIND == 4 ? 128 : 64));
    const int64_t n_rowblocks = ceil_div(k.nrows, 16);
    const bool sal = KIND == 8 || ((k.cols / 32) % 4 == 0 && (reinterpret_cast<uintptr_t>(k.scales) & 3) == 0);
    auto split = [&](int want, int &upw, int &nwaves) {
        want = want < 1 ? 1 : (want > 16 ? 16 : want);
        upw = static_cast<int>(ceil_div(nunits, want));
        nwaves = static_cast<int>(ceil_div(nunits, upw));
    };
    // ---- the staged form: tiles of up to 16 rows, at most eight units and eight 1 KB activation requests per wave ----
    // Up to four rows: blocks of eight waves on one row-block each, several per compute unit, so that one block's
    // reduction runs while the others stream (12288 x 4096 MXFP4 at one row: 8.2 us against 10.4 with 16 waves and three
    // row-blocks).  More rows: 16 waves and the row-blocks per block that fill the compute units in the fewest rounds (they
    // share the staged rows: 13.1 against 19.5 us at 16 rows).
    static const int stage_max_m = tune_env("MFQ_MX_STAGE_MAX_M", 48);
    if (!lds_off && (n_pairs || M <= stage_max_m)) {
        const int xrows = n_pairs ? 1 : (M < 16 ? M : 16);
        const int64_t tiles = n_pairs ? n_pairs : ceil_div(M, 16);
        int upw, nwaves;
        split(env_waves ? env_waves : (xrows <= 4 && nunits <= 8 * kMxStageUnits ? 8 : 16), upw, nwaves);
        const int max_nb = narrow ? 1 : 3;
        const int nb = env_nb >= 1 && env_nb <= max_nb ? env_nb : (xrows <= 4 ? 1 : mx_tile_nb(n_rowblocks, tiles, max_nb));
        const int ub = KIND == 4 ? 256 : 128;
        const size_t corner = static_cast<size_t>(xrows) * (static_cast<size_t>(upw) * ub + 16) + static_cast<size_t>(nb) * 512;
        const size_t lds = static_cast<size_t>(nwaves) * (corner > static_cast<size_t>(nb) * 1024 ? corner : static_cast<size_t>(nb) * 1024);
        const int64_t sbytes = KIND == 4 ? static_cast<int64_t>(k.rows) * (k.cols / 32) : ceil_div(k.rows, 128) * (k.cols / 128);
        const bool scales_ok = sal || (sbytes % 4 == 0 && (reinterpret_cast<uintptr_t>(k.scales) & 3) == 0);
        const int pieces = xrows * upw * (ub / 16);
        if (upw <= kMxStageUnits && pieces <= kMxStageReq * 64 && lds <= kMaxDynamicLds && scales_ok && tiles <= 65535) {
            const int upw_rcp = (65536 + upw - 1) / upw;
            const int xr = pieces <= 64 ? 1 : (pieces <= 256 ? 4 : kMxStageReq);
            const dim3 grid(static_cast<unsigned>(ceil_div(n_rowblocks, nb)), static_cast<unsigned>(tiles));
#define MFQ_MX_STAGED(NBV, SALV) MFQ_MX_STAGED_XR(NBV, SALV, 1) MFQ_MX_STAGED_XR(NBV, SALV, 4) MFQ_MX_STAGED_XR(NBV, SALV, kMxStageReq)
#define MFQ_MX_STAGED_XR(NBV, SALV, XRV)                                                                              \
    if (nb == NBV && sal == SALV && xr == XRV) {                                                                      \
        auto kern = mx_tile_lds_kernel<KIND, XF16, NBV, SALV, XRV>;                                                   \
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds, "mx_tile_lds")) return rc;         \
        hipLaunchKernelGGL(kern, grid, dim3(64 * nwaves), lds, st, k, x, ldx, M, y, ldy, upw, upw_rcp, xrows, sel);   \
        return check_launch("mx_tile_lds");                                                                           \
    }
            MFQ_MX_STAGED(1, true)
            if constexpr (KIND == 4) MFQ_MX_STAGED(1, false)
            if constexpr (!narrow) {
                MFQ_MX_STAGED(2, true) MFQ_MX_STAGED(3, true)
                if constexpr (KIND == 4) {
                    MFQ_MX_STAGED(2, false) MFQ_MX_STAGED(3, false)
                }
            }
#undef MFQ_MX_STAGED
#undef MFQ_MX_STAGED_XR
        }
    }
    // ---- activations straight from memory: tiles of 16 or 32 rows, any K ------------------------------------------------
    const int mt = (!n_pairs && M > 16 && !narrow) ? 2 : 1;
    const int64_t tiles = n_pairs ? n_pairs : ceil_div(M, 16 * mt);
    MFQ_REQUIRE(tiles <= 65535, MFQ_ERR_UNSUPPORTED, "mx_tile: %lld row tiles in one call (max 65535)", static_cast<long long>(tiles));
    const int max_nb = narrow ? 1 : (mt == 2 ? 2 : 4);
    const int nb = env_nb >= 1 && env_nb <= max_nb ? env_nb : mx_tile_nb(n_rowblocks, tiles, max_nb);
    int upw, nwaves;
    split(env_waves ? env_waves : 16, upw, nwaves);
    const size_t lds = static_cast<size_t>(nwaves) * nb * mt * 1024;
    const dim3 grid(static_cast<unsigned>(ceil_div(n_rowblocks, nb)), static_cast<unsigned>(tiles));
#define MFQ_MX_TILE(NBV, MTV, SALV)                                                                                   \
    if (nb == NBV && mt == MTV && sal == SALV) {                                                                      \
        auto kern = mx_tile_kernel<KIND, XF16, NBV, MTV, SALV>;                                                       \
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds, "mx_tile")) return rc;             \
        hipLaunchKernelGGL(kern, grid, dim3(64 * nwaves), lds, st, k, x, ldx, M, y, ldy, upw, sel);                   \
        return check_launch("mx_tile");                                                                               \
    }
    MFQ_MX_TILE(1, 1, true)
    if constexpr (KIND == 4) MFQ_MX_TILE(1, 1, false)
    if constexpr (!narrow) {
        MFQ_MX_TILE(2, 1, true) MFQ_MX_TILE(3, 1, true) MFQ_MX_TILE(4, 1, true) MFQ_MX_TILE(1, 2, true) MFQ_MX_TILE(2, 2, true)
        if constexpr (KIND == 4) {
            MFQ_MX_TILE(2, 1, false) MFQ_MX_TILE(3, 1, false) MFQ_MX_TILE(4, 1, false) MFQ_MX_TILE(1, 2, false) MFQ_MX_TILE(2, 2, false)
        }
    }
#undef MFQ_MX_TILE
    return fail(MFQ_ERR_UNSUPPORTED, "mx_tile: no kernel for %d row-blocks x %d tiles", nb, mt);
}

template <int KIND, int XF16>
int mx_launch_gemv(const MxK &k, const uint16_t *x, int64_t ldx, int M, float *y, int64_t ldy, hipStream_t st) {
    const unsigned gx = static_cast<unsigned>(ceil_div(k.nrows, 4));
    if (M == 1) hipLaunchKernelGGL((mx_gemv_kernel<KIND, XF16, 1>), dim3(gx, 1), dim3(256), 0, st, k, x, ldx, M, y, ldy, PairSel{});
    else if (M == 2) hipLaunchKernelGGL((mx_gemv_kernel<KIND, XF16, 2>), dim3(gx, 1), dim3(256), 0, st, k, x, ldx, M, y, ldy, PairSel{});
    else hipLaunchKernelGGL((mx_gemv_kernel<KIND, XF16, 4>), dim3(gx, static_cast<unsigned>(ceil_div(M, 4))), dim3(256), 0, st, k, x, ldx, M, y, ldy, PairSel{});
    return check_launch("mx_gemv");
}

// the same kernel over the pairs of a MoE decode step (see PairSel); k.nrows = rows per expert of the pool
template <int KIND, int XF16>
int mx_launch_pairs(const MxK &k, const uint16_t *x, int64_t ldx, int n_pairs, float *y, int64_t ldy, const PairSel &sel,
                    hipStream_t st) {
    hipLaunchKernelGGL((mx_gemv_kernel<KIND, XF16, 1>), dim3(static_cast<unsigned>(ceil_div(k.nrows, 4)), static_cast<unsigned>(n_pairs)),
                       dim3(256), 0, st, k, x, ldx, n_pairs, y, ldy, sel);
    return check_launch("mx_gemv_pairs");
}

}  // namespace
}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_mx_gemv_pairs(int kind, const void *values, const void *scales, int rows, int cols, int out_per_expert,
                                     const int32_t *expert_slot, int E, const void *x, int x_dtype, int64_t ldx, int routed_input,
                                     const int32_t *ids, int T, int R, float *y, int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(out_per_expert > 0 && rows % out_per_expert == 0, MFQ_ERR_INVALID,
                "mx_gemv_pairs: %d rows per expert do not divide the pool's %d", out_per_expert, rows);
    if (int rc = mx_check("mx_gemv_pairs", kind, values, scales, rows, cols, 0, out_per_expert)) return rc;
    MFQ_REQUIRE(kind == 4 || out_per_expert % 128 == 0, MFQ_ERR_UNSUPPORTED,
                "mx_gemv_pairs: MXFP8 experts must be whole 128-row scale blocks, got %d rows", out_per_expert);
    MFQ_REQUIRE(expert_slot && x && ids && y, MFQ_ERR_INVALID, "mx_gemv_pairs: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "mx_gemv_pairs: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(T >= 0 && R >= 1 && E >= 1, MFQ_ERR_INVALID, "mx_gemv_pairs: T=%d R=%d E=%d", T, R, E);
    MFQ_REQUIRE(static_cast<int64_t>(T) * R <= 65535, MFQ_ERR_UNSUPPORTED, "mx_gemv_pairs: %lld pairs (at most 65535 per launch)",
                static_cast<long long>(T) * R);
    MFQ_REQUIRE(ldx >= cols && ldy >= out_per_expert, MFQ_ERR_INVALID, "mx_gemv_pairs: ldx/ldy smaller than the tensor");
    if (T == 0) return MFQ_OK;
    const PairSel sel{ids, expert_slot, nullptr, E, R, routed_input ? 1 : 0};
    const MxK k{kind, rows, cols, 0, out_per_expert, static_cast<const uint8_t *>(values), static_cast<const uint8_t *>(scales)};
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    hipStream_t st = as_stream(stream);
    if (mx_tile_eligible(k, x, ldx)) {
        if (kind == 4) return x_dtype == MFQ_X_F16 ? mx_launch_tile<4, 1>(k, xp, ldx, T * R, y, ldy, sel, T * R, st) : mx_launch_tile<4, 0>(k, xp, ldx, T * R, y, ldy, sel, T * R, st);
        return x_dtype == MFQ_X_F16 ? mx_launch_tile<8, 1>(k, xp, ldx, T * R, y, ldy, sel, T * R, st) : mx_launch_tile<8, 0>(k, xp, ldx, T * R, y, ldy, sel, T * R, st);
    }
    if (kind == 4) return x_dtype == MFQ_X_F16 ? mx_launch_pairs<4, 1>(k, xp, ldx, T * R, y, ldy, sel, st) : mx_launch_pairs<4, 0>(k, xp, ldx, T * R, y, ldy, sel, st);
    return x_dtype == MFQ_X_F16 ? mx_launch_pairs<8, 1>(k, xp, ldx, T * R, y, ldy, sel, st) : mx_launch_pairs<8, 0>(k, xp, ldx, T * R, y, ldy, sel, st);
}

extern "C" int mfq_hip_mx_dequant_rows(int kind, const void *values, const void *scales, int rows, int cols, int row0,
                                       int nrows, int out_dtype, void *w_out, int64_t ld, mfq_stream_t stream) {
    if (int rc = mx_check("mx_dequant", kind, values, scales, rows, cols, row0, nrows)) return rc;
    MFQ_REQUIRE(w_out && ld >= cols, MFQ_ERR_INVALID, "mx_dequant: null output or ld smaller than the columns");
    MFQ_REQUIRE(out_dtype == MFQ_X_F32 || out_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "mx_dequant: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(nrows <= 65535, MFQ_ERR_UNSUPPORTED, "mx_dequant: %d rows in one call (max 65535)", nrows);
    const MxK k{kind, rows, cols, row0, nrows, static_cast<const uint8_t *>(values), static_cast<const uint8_t *>(scales)};
    const dim3 grid(static_cast<unsigned>(ceil_div(cols, 1024)), static_cast<unsigned>(nrows));
    hipStream_t st = as_stream(stream);
    if (out_dtype == MFQ_X_F32) {
        if (kind == 4) hipLaunchKernelGGL((mx_dequant_kernel<4, float>), grid, dim3(256), 0, st, k, static_cast<float *>(w_out), ld);
        else hipLaunchKernelGGL((mx_dequant_kernel<8, float>), grid, dim3(256), 0, st, k, static_cast<float *>(w_out), ld);
    } else {
        if (kind == 4) hipLaunchKernelGGL((mx_dequant_kernel<4, uint16_t>), grid, dim3(256), 0, st, k, static_cast<uint16_t *>(w_out), ld);
        else hipLaunchKernelGGL((mx_dequant_kernel<8, uint16_t>), grid, dim3(256), 0, st, k, static_cast<uint16_t *>(w_out), ld);
    }
    return check_launch("mx_dequant");
}

extern "C" size_t mfq_hip_mx_gemm_rows_workspace_bytes(int cols, int nrows, int M) {
    return M <= mx_tile_max_m() ? 0 : dequant_gemm_workspace(nrows, cols, M);
}

extern "C" int mfq_hip_mx_gemm_rows(int kind, const void *values, const void *scales, int rows, int cols, int row0, int nrows,
                                    const void *x, int x_dtype, int64_t ldx, int M, float *y, int64_t ldy, void *workspace,
                                    size_t workspace_bytes, mfq_stream_t stream) {
    if (int rc = mx_check("mx_gemm", kind, values, scales, rows, cols, row0, nrows)) return rc;
    MFQ_REQUIRE(x && y, MFQ_ERR_INVALID, "mx_gemm: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "mx_gemm: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "mx_gemm: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= cols && ldy >= nrows, MFQ_ERR_INVALID, "mx_gemm: ldx/ldy smaller than the tensor");
    const MxK k{kind, rows, cols, row0, nrows, static_cast<const uint8_t *>(values), static_cast<const uint8_t *>(scales)};
    hipStream_t st = as_stream(stream);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    if (M <= mx_tile_max_m()) {
        // 16-byte reads of the value rows: true for whole tensors from the file (cols % 32 == 0) at 16-byte aligned bases
        MFQ_REQUIRE((reinterpret_cast<uintptr_t>(values) & 15) == 0, MFQ_ERR_INVALID, "mx_gemm: values must be 16-byte aligned");
        if (mx_tile_eligible(k, x, ldx)) {
            if (kind == 4) return x_dtype == MFQ_X_F16 ? mx_launch_tile<4, 1>(k, xp, ldx, M, y, ldy, PairSel{}, 0, st) : mx_launch_tile<4, 0>(k, xp, ldx, M, y, ldy, PairSel{}, 0, st);
            return x_dtype == MFQ_X_F16 ? mx_launch_tile<8, 1>(k, xp, ldx, M, y, ldy, PairSel{}, 0, st) : mx_launch_tile<8, 0>(k, xp, ldx, M, y, ldy, PairSel{}, 0, st);
        }
        // activations the tile kernel cannot read in 16-byte pieces: a wave per neuron, four rows per pass
        if (kind == 4) return x_dtype == MFQ_X_F16 ? mx_launch_gemv<4, 1>(k, xp, ldx, M, y, ldy, st) : mx_launch_gemv<4, 0>(k, xp, ldx, M, y, ldy, st);
        return x_dtype == MFQ_X_F16 ? mx_launch_gemv<8, 1>(k, xp, ldx, M, y, ldy, st) : mx_launch_gemv<8, 0>(k, xp, ldx, M, y, ldy, st);
    }
    MFQ_REQUIRE(nrows <= 65535, MFQ_ERR_UNSUPPORTED, "mx_gemm: %d neurons in one call (max 65535)", nrows);
    const size_t need = dequant_gemm_workspace(nrows, cols, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "mx_gemm: workspace %zu < %zu bytes", workspace_bytes, need);
    uint16_t *x16, *w16;
    float *xscale, *wscale;
    int Kp;
    dequant_gemm_carve(workspace, nrows, cols, M, x16, xscale, w16, wscale, Kp);
    int rc = x_prep(x, x_dtype, ldx, M, cols, Kp, x16, xscale, st);
    if (rc) return rc;
    if (kind == 4) hipLaunchKernelGGL((mx_stage_f16_kernel<4>), dim3(nrows), dim3(256), 0, st, k, w16, Kp, wscale);
    else hipLaunchKernelGGL((mx_stage_f16_kernel<8>), dim3(nrows), dim3(256), 0, st, k, w16, Kp, wscale);
    rc = check_launch("mx_stage_f16");
    if (rc) return rc;
    return gemm_f16_nt(x16, Kp, w16, Kp, M, nrows, Kp, xscale, wscale, y, ldy, st, dequant_gemm_part(wscale, nrows, cols, M));
}
