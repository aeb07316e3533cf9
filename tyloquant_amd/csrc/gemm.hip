// Prefill / large-M path: activations are rescaled per row by an exact power of two into fp16,
// weights are dequantized into fp16 (scaled per neuron by an exact power of two), and an
// fp16 x fp16 -> fp32 MFMA GEMM (v_mfma_f32_32x32x16_f16) produces y; the epilogue multiplies
// the two power-of-two scales back.  fp16 (11 significant bits) keeps the weight rounding error
// near 1e-4 relative, which bf16 tiles (8 bits) cannot.
#include <stdlib.h>

#include "common.hpp"
#include "tune.hpp"

namespace mfq {

// ---- core: thread-local error text ---------------------------------------------------
char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

// group-sum tables one activation prep launch leaves: one per distinct groupsize of the tensors that will read x16
struct XGroups {
    int n;
    int gs[4], nsteps[4];
    uint32_t *xg[4];
};

// ---- activation prep: x16[m, k] = fp16(x[m, k] * 2^-f_m), xscale[m] = 2^f_m ---------------
// With xg != null the block also leaves the row's group sums for the NINT prefill kernel:
// xg[((m * nsteps + s) * 4 + kb) * 4 + {0,1,2,3}] = fp16 pairs (Xhi_j0, Xhi_j1), (Xhi_j2, Xhi_j3), (Xlo_j0, Xlo_j1),
// (Xlo_j2, Xlo_j3), X_j = sum of x16[m] over group 16 s + 4 j + kb (gs values), split into two fp16 halves.
template <int XF16>
__global__ __launch_bounds__(256) void x_prep_kernel(const uint16_t *__restrict__ x, int64_t ldx, int K, int Kp,
                                                     uint16_t *__restrict__ x16, float *__restrict__ xscale,
                                                     XGroups grp) {
    __shared__ float red[4];
    __shared__ float gsum[256];
    const int m = blockIdx.x, tid = threadIdx.x;
    const uint16_t *xr = x + static_cast<int64_t>(m) * ldx;
    float amax = 0.f;
    for (int k = tid; k < K; k += 256) {
        const float v = fabsf(x_to_f32<XF16>(xr[k]));
        if (v == v && v <= 3.0e38f) amax = fmaxf(amax, v);
    }
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int e = 0;
    if (amax > 0.f) frexpf(amax, &e);  // amax = f * 2^e, f in [0.5, 1)
    const float inv = ldexpf(1.f, 9 - e);  // row maximum lands in [256, 512)
    if (tid == 0) xscale[m] = ldexpf(1.f, e - 9);
    uint16_t *o16 = x16 + static_cast<int64_t>(m) * Kp;
    for (int k = tid; k < Kp; k += 256) o16[k] = k < K ? f32_to_f16_rne(x_to_f32<XF16>(xr[k]) * inv) : uint16_t(0);
    // group sums of the fp16 values just written (recomputed from x: the same roundings), 256 groups at a time
    for (int gi = 0; gi < grp.n; ++gi) {
    const int gs = grp.gs[gi], nsteps = grp.nsteps[gi];
    uint32_t *xg = grp.xg[gi];
    for (int g0 = 0; g0 < nsteps * 16; g0 += 256) {
        const int g = g0 + tid;
        float acc = 0.f;
        if (g < nsteps * 16)
            for (int i = 0; i < gs; ++i) {
                const int k = g * gs + i;
                if (k < K) acc += f16_to_f32(f32_to_f16_rne(x_to_f32<XF16>(xr[k]) * inv));
            }
        __syncthreads();
        gsum[tid] = acc;
        __syncthreads();
        // thread (s_local, kb) of this chunk: groups 16 s + 4 j + kb
        if (tid < 64 && g0 / 16 + (tid >> 2) < nsteps) {
            const int sl = tid >> 2, kb = tid & 3;
            float X[4];
            for (int j = 0; j < 4; ++j) X[j] = gsum[sl * 16 + 4 * j + kb];
            uint32_t out[4];
            for (int p = 0; p < 2; ++p) {
                const _Float16 h0 = static_cast<_Float16>(X[2 * p]), h1 = static_cast<_Float16>(X[2 * p + 1]);
                const _Float16 l0 = static_cast<_Float16>(X[2 * p] - static_cast<float>(h0));
                const _Float16 l1 = static_cast<_Float16>(X[2 * p + 1] - static_cast<float>(h1));
                out[p] = __builtin_bit_cast(uint16_t, h0) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h1)) << 16);
                out[2 + p] = __builtin_bit_cast(uint16_t, l0) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, l1)) << 16);
            }
            uint32_t *o = xg + ((static_cast<int64_t>(m) * nsteps + g0 / 16 + sl) * 4 + kb) * 4;
            for (int t = 0; t < 4; ++t) o[t] = out[t];
        }
    }
    }
}

// The same for 16-byte aligned rows with K % 8 == 0 and Kp * 2 bytes of LDS: 8 values per load and store, the row
// read once (twice beyond 8192 values), the group sums taken from the fp16 row kept in LDS.  Bit-identical results.
template <int XF16>
__global__ __launch_bounds__(256) void x_prep_vec_kernel(const uint16_t *__restrict__ x, int64_t ldx, int K, int Kp,
                                                         uint16_t *__restrict__ x16, float *__restrict__ xscale,
                                                         XGroups grp) {
    extern __shared__ __attribute__((aligned(16))) uint16_t rowh[];  // [Kp] halves
    __shared__ float red[4];
    __shared__ float gsum[256];
    constexpr int KEEP = 4;  // chunks of 8 values a thread keeps in registers between the two passes
    const int m = blockIdx.x, tid = threadIdx.x;
    const u32x4_t *xr = reinterpret_cast<const u32x4_t *>(x + static_cast<int64_t>(m) * ldx);
    const int nchunks = K >> 3;
    u32x4_t keep[KEEP];
    float amax = 0.f;
    auto chunk_amax = [&](u32x4_t v) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float a = fabsf(x_to_f32<XF16>(static_cast<uint16_t>(v[t] & 0xffffu)));
            const float b = fabsf(x_to_f32<XF16>(static_cast<uint16_t>(v[t] >> 16)));
            if (a == a && a <= 3.0e38f) amax = fmaxf(amax, a);
            if (b == b && b <= 3.0e38f) amax = fmaxf(amax, b);
        }
    };
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
        const int c = tid + 256 * i;
        keep[i] = u32x4_t{0u, 0u, 0u, 0u};
        if (c < nchunks) {
            keep[i] = xr[c];
            chunk_amax(keep[i]);
        }
    }
    for (int c = tid + 256 * KEEP; c < nchunks; c += 256) chunk_amax(xr[c]);
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int e = 0;
    if (amax > 0.f) frexpf(amax, &e);
    const float inv = ldexpf(1.f, 9 - e);
    if (tid == 0) xscale[m] = ldexpf(1.f, e - 9);
    u32x4_t *o16 = reinterpret_cast<u32x4_t *>(x16 + static_cast<int64_t>(m) * Kp);
    u32x4_t *rowv = reinterpret_cast<u32x4_t *>(rowh);
    auto emit = [&](int c, u32x4_t v) {
        u32x4_t h;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t lo = f32_to_f16_rne(x_to_f32<XF16>(static_cast<uint16_t>(v[t] & 0xffffu)) * inv);
            const uint32_t hi = f32_to_f16_rne(x_to_f32<XF16>(static_cast<uint16_t>(v[t] >> 16)) * inv);
            h[t] = lo | (hi << 16);
        }
        o16[c] = h;
        rowv[c] = h;
    };
#pragma unroll
    for (int i = 0; i < KEEP; ++i)
        if (tid + 256 * i < nchunks) emit(tid + 256 * i, keep[i]);
    for (int c = tid + 256 * KEEP; c < nchunks; c += 256) emit(c, xr[c]);
    for (int c = nchunks + tid; c < (Kp >> 3); c += 256) {
        o16[c] = u32x4_t{0u, 0u, 0u, 0u};
        rowv[c] = u32x4_t{0u, 0u, 0u, 0u};
    }
    if (grp.n == 0) return;
    __syncthreads();
    for (int gi = 0; gi < grp.n; ++gi) {
    const int gs = grp.gs[gi], nsteps = grp.nsteps[gi];
    uint32_t *xg = grp.xg[gi];
    for (int g0 = 0; g0 < nsteps * 16; g0 += 256) {
        const int g = g0 + tid;
        float acc = 0.f;
        if (g < nsteps * 16) {
            if (gs % 4 == 0 && (g + 1) * gs <= Kp) {
                // four halves per LDS read, added in k order; the row is zero from K to Kp
                const uint2 *q = reinterpret_cast<const uint2 *>(rowh + g * gs);
                for (int i = 0; i < gs / 4; ++i) {
                    const uint2 v = q[i];
                    acc += f16_to_f32(static_cast<uint16_t>(v.x & 0xffffu));
                    acc += f16_to_f32(static_cast<uint16_t>(v.x >> 16));
                    acc += f16_to_f32(static_cast<uint16_t>(v.y & 0xffffu));
                    acc += f16_to_f32(static_cast<uint16_t>(v.y >> 16));
                }
            } else {
                for (int i = 0; i < gs; ++i) {
                    const int k = g * gs + i;
                    if (k < K) acc += f16_to_f32(rowh[k]);
                }
            }
        }
        __syncthreads();
        gsum[tid] = acc;
        __syncthreads();
        if (tid < 64 && g0 / 16 + (tid >> 2) < nsteps) {
            const int sl = tid >> 2, kb = tid & 3;
            float X[4];
            for (int j = 0; j < 4; ++j) X[j] = gsum[sl * 16 + 4 * j + kb];
            u32x4_t out;
            for (int p = 0; p < 2; ++p) {
                const _Float16 h0 = static_cast<_Float16>(X[2 * p]), h1 = static_cast<_Float16>(X[2 * p + 1]);
                const _Float16 l0 = static_cast<_Float16>(X[2 * p] - static_cast<float>(h0));
                const _Float16 l1 = static_cast<_Float16>(X[2 * p + 1] - static_cast<float>(h1));
                out[p] = __builtin_bit_cast(uint16_t, h0) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h1)) << 16);
                out[2 + p] = __builtin_bit_cast(uint16_t, l0) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, l1)) << 16);
            }
            *reinterpret_cast<u32x4_t *>(xg + ((static_cast<int64_t>(m) * nsteps + g0 / 16 + sl) * 4 + kb) * 4) = out;
        }
    }
    }
}

// ---- fp16 NT GEMM: y[m, n] = sa[m] * sb[n] * sum_k a[m, k] * b[n, k] ----------------------
// 128 x 128 x 32 block tile, 256 threads = 4 waves of 64 x 64 (2 x 2 MFMA 32x32x16 tiles).
constexpr int GBM = 128, GBN = 128, GBK = 32, GLD = GBK + 8;  // LDS row stride in halves (80 bytes)

__global__ __launch_bounds__(256) void gemm_f16_nt_kernel(const uint16_t *__restrict__ a, int64_t lda,
                                                          const uint16_t *__restrict__ b, int64_t ldb, int M, int N,
                                                          int K, const float *__restrict__ sa,
                                                          const float *__restrict__ sb, float *__restrict__ y,
                                                          int64_t ldy, int kps, int64_t ystride) {
    // split blockIdx.z multiplies the K steps [z * kps, (z + 1) * kps) and writes its (scaled) partial tile to
    // y + z * ystride; one split: the whole K, y itself
    __shared__ __attribute__((aligned(16))) uint16_t As[2][GBM * GLD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][GBN * GLD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bm = blockIdx.y * GBM, bn = blockIdx.x * GBN;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    // global -> LDS: each thread moves 16 halves of A and of B per K step (row = tid/2, half-row = tid&1)
    const int lr = tid >> 1, lc = (tid & 1) * 16;
    const bool a_ok = bm + lr < M, b_ok = bn + lr < N;
    const uint16_t *ap = a + static_cast<int64_t>(bm + lr) * lda + lc;
    const uint16_t *bp = b + static_cast<int64_t>(bn + lr) * ldb + lc;
    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int t = 0; t < 16; ++t) acc[i][j][t] = 0.f;

    const int k_begin = static_cast<int>(blockIdx.z) * kps, nk = min(K / GBK, k_begin + kps);  // K is a multiple of 32 (callers pad)
    y += static_cast<int64_t>(blockIdx.z) * ystride;
    u32x4_t ra[2], rbv[2];
    auto gload = [&](int kt) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ra[h] = a_ok ? *reinterpret_cast<const u32x4_t *>(ap + kt * GBK + 8 * h) : u32x4_t{0, 0, 0, 0};
            rbv[h] = b_ok ? *reinterpret_cast<const u32x4_t *>(bp + kt * GBK + 8 * h) : u32x4_t{0, 0, 0, 0};
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<u32x4_t *>(&As[buf][lr * GLD + lc + 8 * h]) = ra[h];
            *reinterpret_cast<u32x4_t *>(&Bs[buf][lr * GLD + lc + 8 * h]) = rbv[h];
        }
    };
    gload(k_begin);
    lstore(0);
    __syncthreads();
    const int fr = lane & 31, fk = (lane >> 5) * 8;
    for (int kt = k_begin; kt < nk; ++kt) {
        const int buf = (kt - k_begin) & 1;
        if (kt + 1 < nk) gload(kt + 1);
#pragma unroll
        for (int kk = 0; kk < GBK; kk += 16) {
            half8_t fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const half8_t *>(&As[buf][(wm + 32 * i + fr) * GLD + kk + fk]);
                fb[i] = *reinterpret_cast<const half8_t *>(&Bs[buf][(wn + 32 * i + fr) * GLD + kk + fk]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) lstore(buf ^ 1);
        __syncthreads();
    }
    // D[row = m, col = n]: lane holds col = lane & 31, rows 8 * (t / 4) + 4 * (lane / 32) + t % 4
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = bn + wn + 32 * j + (lane & 31);
            if (n >= N) continue;
            const float sn = sb ? sb[n] : 1.f;
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int m = bm + wm + 32 * i + 8 * (t >> 2) + 4 * (lane >> 5) + (t & 3);
                if (m < M) y[static_cast<int64_t>(m) * ldy + n] = acc[i][j][t] * sn * (sa ? sa[m] : 1.f);
            }
        }
    }
}

int prefill_sum_splits(const float *part, int64_t ystride, int splits, int M, int N, float *y, int64_t ldy, hipStream_t st);

// Splits over K of the dequantize + GEMM path: a grid of 128 x 128 tiles that leaves compute units idle (64 rows against
// 4096 neurons are 32 blocks) is cut along K, up to eight ways, while a split keeps at least four K steps of 32 and the
// neuron count allows 16-byte partial rows; the partial tiles go to the end of the workspace and are added in split
// order (deterministic).  1 = no split.
static int gemm_splits(int M, int N, int K) {
    const int64_t blocks = ceil_div(N, GBN) * ceil_div(M, GBM);
    if (blocks > 128 || N % 4) return 1;
    int64_t splits = 256 / blocks;
    if (splits > 8) splits = 8;
    if (splits > K / GBK / 4) splits = K / GBK / 4;
    if (splits <= 1) return 1;
    const int kps = static_cast<int>(ceil_div(K / GBK, splits));
    return static_cast<int>(ceil_div(K / GBK, kps));
}

// part: splits * M * N floats when gemm_splits(M, N, K) > 1 (dequant_gemm_carve hands it out), else unused
int gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, const float *sa,
                const float *sb, float *y, int64_t ldy, hipStream_t st, float *part = nullptr) {
    MFQ_REQUIRE(K % GBK == 0 && lda % 8 == 0 && ldb % 8 == 0, MFQ_ERR_INVALID,
                "gemm_f16_nt: K=%d, lda=%lld, ldb=%lld must be multiples of 32 / 8 / 8", K, (long long)lda, (long long)ldb);
    const int splits = part ? gemm_splits(M, N, K) : 1;
    const int kps = static_cast<int>(ceil_div(K / GBK, splits));
    const dim3 grid(static_cast<unsigned>(ceil_div(N, GBN)), static_cast<unsigned>(ceil_div(M, GBM)), static_cast<unsigned>(splits));
    if (splits == 1) {
        hipLaunchKernelGGL(gemm_f16_nt_kernel, grid, dim3(256), 0, st, static_cast<const uint16_t *>(a), lda,
                           static_cast<const uint16_t *>(b), ldb, M, N, K, sa, sb, y, ldy, kps, static_cast<int64_t>(0));
        return check_launch("gemm_f16_nt");
    }
    const int64_t ystride = static_cast<int64_t>(M) * N;
    hipLaunchKernelGGL(gemm_f16_nt_kernel, grid, dim3(256), 0, st, static_cast<const uint16_t *>(a), lda,
                       static_cast<const uint16_t *>(b), ldb, M, N, K, sa, sb, part, static_cast<int64_t>(N), kps, ystride);
    if (int rc = check_launch("gemm_f16_nt")) return rc;
    return prefill_sum_splits(part, ystride, splits, M, N, y, ldy, st);
}
// The split buffer of the call that dequant_gemm_carve(ws, N, K, M, ...) prepared: behind the row scales of the weights.
float *dequant_gemm_part(float *wscale, int N, int K, int M);

int x_prep_multi(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, int n_groups,
                 const int *gs, const int *nsteps, uint32_t *const *xg, hipStream_t st) {
    MFQ_REQUIRE(n_groups >= 0 && n_groups <= 4, MFQ_ERR_UNSUPPORTED, "x_prep: %d group-sum tables (max 4)", n_groups);
    XGroups grp;
    grp.n = n_groups;
    for (int i = 0; i < 4; ++i) {
        grp.gs[i] = i < n_groups ? gs[i] : 0;
        grp.nsteps[i] = i < n_groups ? nsteps[i] : 0;
        grp.xg[i] = i < n_groups ? xg[i] : nullptr;
    }
    const bool vec = K % 8 == 0 && ldx % 8 == 0 && Kp % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(x16) & 15) == 0 && Kp <= 28 * 1024;
    if (vec) {
        const size_t lds = static_cast<size_t>(Kp) * 2;
        if (x_dtype == MFQ_X_F16)
            hipLaunchKernelGGL((x_prep_vec_kernel<1>), dim3(M), dim3(256), lds, st, static_cast<const uint16_t *>(x), ldx, K,
                               Kp, static_cast<uint16_t *>(x16), xscale, grp);
        else
            hipLaunchKernelGGL((x_prep_vec_kernel<0>), dim3(M), dim3(256), lds, st, static_cast<const uint16_t *>(x), ldx, K,
                               Kp, static_cast<uint16_t *>(x16), xscale, grp);
        return check_launch("x_prep");
    }
    if (x_dtype == MFQ_X_F16)
        hipLaunchKernelGGL((x_prep_kernel<1>), dim3(M), dim3(256), 0, st, static_cast<const uint16_t *>(x), ldx, K, Kp,
                           static_cast<uint16_t *>(x16), xscale, grp);
    else
        hipLaunchKernelGGL((x_prep_kernel<0>), dim3(M), dim3(256), 0, st, static_cast<const uint16_t *>(x), ldx, K, Kp,
                           static_cast<uint16_t *>(x16), xscale, grp);
    return check_launch("x_prep");
}
int x_prep_groups(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, int gs,
                  int nsteps, uint32_t *xg, hipStream_t st) {
    return x_prep_multi(x, x_dtype, ldx, M, K, Kp, x16, xscale, xg ? 1 : 0, &gs, &nsteps, &xg, st);
}
int x_prep(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, hipStream_t st) {
    return x_prep_groups(x, x_dtype, ldx, M, K, Kp, x16, xscale, 0, 0, nullptr, st);
}

// Workspace carve-up of the dequant + GEMM path: x16 [M, Kp] | xscale [M] | w16 [N, Kp] | wscale [N]
static size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }
size_t dequant_gemm_workspace(int N, int K, int M) {
    const size_t Kp = static_cast<size_t>(ceil_div(K, GBK)) * GBK;
    const int splits = gemm_splits(M, N, static_cast<int>(Kp));
    return align256(static_cast<size_t>(M) * Kp * 2) + align256(static_cast<size_t>(M) * 4) +
           align256(static_cast<size_t>(N) * Kp * 2) + align256(static_cast<size_t>(N) * 4) +
           (splits > 1 ? align256(static_cast<size_t>(splits) * M * N * 4) : 0);   // partial tiles of a split over K
}
float *dequant_gemm_part(float *wscale, int N, int K, int M) {
    const int Kp = static_cast<int>(ceil_div(K, GBK)) * GBK;
    if (gemm_splits(M, N, Kp) <= 1) return nullptr;
    return reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(wscale) + align256(static_cast<size_t>(N) * 4));
}
void dequant_gemm_carve(void *ws, int N, int K, int M, uint16_t *&x16, float *&xscale, uint16_t *&w16, float *&wscale,
                        int &Kp) {
    Kp = static_cast<int>(ceil_div(K, GBK)) * GBK;
    uint8_t *p = static_cast<uint8_t *>(ws);
    x16 = reinterpret_cast<uint16_t *>(p); p += align256(static_cast<size_t>(M) * Kp * 2);
    xscale = reinterpret_cast<float *>(p); p += align256(static_cast<size_t>(M) * 4);
    w16 = reinterpret_cast<uint16_t *>(p); p += align256(static_cast<size_t>(N) * Kp * 2);
    wscale = reinterpret_cast<float *>(p);
}

int nint_gemv_any(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                  int64_t ldy, hipStream_t st);
int nint_dequant_f16(const mfq_nint_desc *d, const void *weight, void *w16, int64_t ld, float *rowscale, hipStream_t st);
bool nint_stream_capable(const mfq_nint_desc *d);
bool nint_prefill_capable(const mfq_nint_desc *d);
size_t nint_prefill_xg_bytes(const mfq_nint_desc *d, int M);
size_t nint_prefill_split_bytes(const mfq_nint_desc *d, int M);
int nint_prefill(const mfq_nint_desc *d, const void *weight, const uint16_t *x16, int Kp, const float *xscale, uint32_t *xg,
                 int M, float *y, int64_t ldy, float *part, hipStream_t st);
int nint_prefill_splits(const mfq_nint_desc *d, int M);
bool nint_prefill_glu_capable(const mfq_nint_desc *d);
int nint_prefill_glu(const mfq_nint_desc *d, const void *weight, const uint16_t *x16, int Kp, const float *xscale,
                     const uint32_t *xg, int M, void *hidden, int64_t ldh, int f16, int gelu, hipStream_t st);

}  // namespace mfq

using namespace mfq;

extern "C" const char *mfq_hip_last_error(void) { return error_buffer(); }
extern "C" int mfq_hip_version(void) { return 1; }

extern "C" int mfq_hip_gemm_f16_nt(const void *a, int64_t lda, const void *b, int64_t ldb, int M, int N, int K, float *y,
                                   int64_t ldy, mfq_stream_t stream) {
    MFQ_REQUIRE(a && b && y, MFQ_ERR_INVALID, "gemm_f16_nt: null argument");
    return gemm_f16_nt(a, lda, b, ldb, M, N, K, nullptr, nullptr, y, ldy, as_stream(stream));
}

// Up to kGemvMaxM activation rows the weight stream dominates and the GEMV kernels win; tensors with a
// matrix-core streaming kernel (16 rows per pass over the packed weights) stay on it up to kStreamMaxM rows,
// where re-streaming the weights is still cheaper than dequantizing them to fp16 once, or up to the crossover
// with the prefill kernel.  That crossover comes from a two-line model fitted to measurements on 4096..12288-wide
// tensors: 64 rows of streaming cost about 8 us + 0.85 us per MB of payload (twice that for the natural-order
// unit), the prefill kernel a flat 30 us + 1.9 us per 1024 of K up to a few hundred rows (small grids are split
// over K; a quarter more for the natural-order unit).
static constexpr int kGemvMaxM = 8, kStreamMaxM = 256;
static bool nint_streams(const mfq_nint_desc *d, int M) {
    static const int env_max = tune_env("MFQ_STREAM_MAX_M", 0);
    int stream_max = kStreamMaxM;
    if (nint_prefill_capable(d)) {
        const bool natural = d->kind != 1;
        const double t64 = (8.0 + 0.85e-6 * static_cast<double>(d->payload_bytes)) * (natural ? 2.0 : 1.0);
        const double tp = (30.0 + 1.9 * d->neuron_len / 1024.0) * (natural ? 1.25 : 1.0);
        const int m = static_cast<int>(64.0 * tp / t64) / 16 * 16;
        stream_max = m < 32 ? 32 : (m > 512 ? 512 : m);
    }
    // NINT8-48 streams one row-block per wave (twelve dwords a unit), 16 rows per pass: 12288 x 4096 takes 133 us at 64
    // rows where the fp16 copy + GEMM takes 335 us at any batch up to a few hundred
    else if (d->bits == 8) stream_max = 160;
    if (env_max > 0) stream_max = env_max;
    return M <= kGemvMaxM || (M <= stream_max && nint_stream_capable(d));
}

// Row length of the fp16 activations of the prefill kernel: whole 16-group steps (tiles copied straight into LDS never
// cross a row end), and a multiple of the GEMM's K block.
static int prefill_kp(const mfq_nint_desc *d) {
    const int64_t whole = static_cast<int64_t>(d->nsteps) * 16 * d->gs;
    const int64_t k = whole > d->neuron_len ? whole : d->neuron_len;
    return static_cast<int>(ceil_div(k, GBK) * GBK);
}

// prefill workspace: x16 [M, Kp] | xscale [M] | group sums
static size_t prefill_workspace(const mfq_nint_desc *d, int M) {
    const size_t Kp = static_cast<size_t>(prefill_kp(d));
    return align256(static_cast<size_t>(M) * Kp * 2) + align256(static_cast<size_t>(M) * 4) +
           align256(nint_prefill_xg_bytes(d, M)) + nint_prefill_split_bytes(d, M);
}

extern "C" size_t mfq_hip_nint_gemm_workspace_bytes(const mfq_nint_desc *d, int M) {
    if (!d || nint_streams(d, M)) return 0;
    if (nint_prefill_capable(d)) return prefill_workspace(d, M);
    return dequant_gemm_workspace(d->out, d->neuron_len, M);
}

extern "C" int mfq_hip_nint_gemm(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                 int M, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                                 mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && y, MFQ_ERR_INVALID, "nint_gemm: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nint_gemm: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemm: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= d->neuron_len && ldy >= d->out, MFQ_ERR_INVALID, "nint_gemm: ldx/ldy smaller than the tensor");
    hipStream_t st = as_stream(stream);
    if (nint_streams(d, M)) return nint_gemv_any(d, weight, x, x_dtype, ldx, M, y, ldy, st);
    if (nint_prefill_capable(d)) {
        const size_t need = prefill_workspace(d, M);
        MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nint_gemm: workspace %zu < %zu bytes",
                    workspace_bytes, need);
        const int Kp = prefill_kp(d);
        uint8_t *p = static_cast<uint8_t *>(workspace);
        uint16_t *x16 = reinterpret_cast<uint16_t *>(p);
        p += align256(static_cast<size_t>(M) * Kp * 2);
        float *xscale = reinterpret_cast<float *>(p);
        p += align256(static_cast<size_t>(M) * 4);
        uint32_t *xg = reinterpret_cast<uint32_t *>(p);
        p += align256(nint_prefill_xg_bytes(d, M));
        float *part = nint_prefill_split_bytes(d, M) ? reinterpret_cast<float *>(p) : nullptr;
        int rc = x_prep_groups(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, d->gs, d->nsteps, xg, st);
        if (rc) return rc;
        return nint_prefill(d, weight, x16, Kp, xscale, xg, M, y, ldy, part, st);
    }
    const size_t need = dequant_gemm_workspace(d->out, d->neuron_len, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nint_gemm: workspace %zu < %zu bytes",
                workspace_bytes, need);
    uint16_t *x16, *w16;
    float *xscale, *wscale;
    int Kp;
    dequant_gemm_carve(workspace, d->out, d->neuron_len, M, x16, xscale, w16, wscale, Kp);
    int rc = x_prep(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, st);
    if (rc) return rc;
    rc = nint_dequant_f16(d, weight, w16, Kp, wscale, st);
    if (rc) return rc;
    return gemm_f16_nt(x16, Kp, w16, Kp, M, d->out, Kp, xscale, wscale, y, ldy, st, dequant_gemm_part(wscale, d->out, d->neuron_len, M));
}

// The batch sizes at which mfq_hip_nint_gemm runs the block-tiled prefill kernel in one pass over K: only there does
// the fused epilogue have both halves of a pair in one block.
// Below a few hundred rows the two calls are as fast (measured on 24576 x 4096 and 34816 x 5120 NINT4-32: 142 against
// 143 us and 245 against 258 us at 512 rows, 441 against 481 us and 742 against 813 us at 2048).
static bool nint_gemm_glu_fuses(const mfq_nint_desc *d, int M) {
    static const int min_m = tune_env("MFQ_GLU_PREFILL_MIN_M", 512);
    return M >= min_m && !nint_streams(d, M) && nint_prefill_glu_capable(d) && nint_prefill_splits(d, M) == 1;
}

extern "C" int mfq_hip_nint_gemm_glu(const mfq_nint_desc *d, const void *weight, const void *x, int x_dtype, int64_t ldx,
                                     int M, int activation, void *hidden, int out_dtype, int64_t ldh, void *workspace,
                                     size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(d && weight && x && hidden, MFQ_ERR_INVALID, "nint_gemm_glu: null argument");
    MFQ_REQUIRE(M >= 1, MFQ_ERR_INVALID, "nint_gemm_glu: M=%d", M);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemm_glu: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_gemm_glu: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(activation == MFQ_GLU_SILU || activation == MFQ_GLU_GELU, MFQ_ERR_INVALID, "nint_gemm_glu: activation=%d",
                activation);
    MFQ_REQUIRE(d->out % 2 == 0 && ldx >= d->neuron_len && ldh >= d->out / 2, MFQ_ERR_INVALID,
                "nint_gemm_glu: ldx/ldh smaller than the tensor");
    if (!nint_gemm_glu_fuses(d, M))
        return fail(MFQ_ERR_UNSUPPORTED, "nint_gemm_glu: %d rows of this tensor do not take the one-pass prefill kernel", M);
    const size_t need = prefill_workspace(d, M);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nint_gemm_glu: workspace %zu < %zu bytes",
                workspace_bytes, need);
    hipStream_t st = as_stream(stream);
    const int Kp = prefill_kp(d);
    uint8_t *p = static_cast<uint8_t *>(workspace);
    uint16_t *x16 = reinterpret_cast<uint16_t *>(p);
    p += align256(static_cast<size_t>(M) * Kp * 2);
    float *xscale = reinterpret_cast<float *>(p);
    p += align256(static_cast<size_t>(M) * 4);
    uint32_t *xg = reinterpret_cast<uint32_t *>(p);
    int rc = x_prep_groups(x, x_dtype, ldx, M, d->neuron_len, Kp, x16, xscale, d->gs, d->nsteps, xg, st);
    if (rc) return rc;
    return nint_prefill_glu(d, weight, x16, Kp, xscale, xg, M, hidden, ldh, out_dtype == MFQ_X_F16,
                            activation == MFQ_GLU_GELU, st);
}
