// OCP MX weights of full-precision MFQ files: MXFP4 (E2M1 nibbles, low nibble = even column, one E8M0 scale per 32
// columns of a row) and MXFP8 (E4M3FN bytes, one E8M0 scale per 128 x 128 block).  The payload's two byte matrices are
// used as they lie in the file (mfq/formats/mx.py:65-117): values [rows, cols / 2] or [rows, cols], scales
// [rows, cols / 32] or [ceil(rows / 128), cols / 128].
//   element x scale, one fp32 multiply           cpp_runtime/mfq_decode.cpp:1920-1947, mfq/kernels/cuda/mx_matmul.cu:17-47
//   up to kMxGemvMaxM rows: a wave per neuron     mx_matmul.cu launch_mxfp8_small_m (rows 1..8 there)
//   more rows: fp16 copy + MFMA GEMM              mfq_decode.cpp:8760-8802 (dequantize, then the fp16 GEMM)
#include "common.hpp"
#include "gemv_common.hpp"

namespace mfq {

int gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, const float *sa,
                const float *sb, float *y, int64_t ldy, hipStream_t st, float *part = nullptr);
float *dequant_gemm_part(float *wscale, int N, int K, int M);
int x_prep(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, hipStream_t st);
size_t dequant_gemm_workspace(int N, int K, int M);
void dequant_gemm_carve(void *ws, int N, int K, int M, uint16_t *&x16, float *&xscale, uint16_t *&w16, float *&wscale,
                        int &Kp);

namespace {

constexpr int kMxGemvMaxM = 16;

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
    return M <= kMxGemvMaxM ? 0 : dequant_gemm_workspace(nrows, cols, M);
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
    if (M <= kMxGemvMaxM) {
        // 16-byte reads of the value rows: true for whole tensors from the file (cols % 32 == 0) at 16-byte aligned bases
        MFQ_REQUIRE((reinterpret_cast<uintptr_t>(values) & 15) == 0, MFQ_ERR_INVALID, "mx_gemm: values must be 16-byte aligned");
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
