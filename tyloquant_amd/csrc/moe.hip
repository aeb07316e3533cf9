// MoE: router top-k, device-side expert bucketing (parallel prefix sum), the expert-grouped
// mixed-bit matmul ("mul_mat_id"), SwiGLU and the weighted reduce.
#include <float.h>

#include "common.hpp"
#include "gemv_common.hpp"
#include "tune.hpp"
#include "nint_body.hpp"
#include "nint_mfma.hpp"
#include "nint_prefill.hpp"
#include "moe_prefill.hpp"

namespace mfq {

// ---- router top-k: one wave per token -----------------------------------------------------
__device__ __forceinline__ void wave_argmax(float &score, float &weight, int &id) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float os = __shfl_xor(score, o, 64);
        const float ow = __shfl_xor(weight, o, 64);
        const int oi = __shfl_xor(id, o, 64);
        if (os > score || (os == score && oi < id)) { score = os; weight = ow; id = oi; }
    }
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

__global__ __launch_bounds__(256) void moe_topk_kernel(const float *__restrict__ logits, const float *__restrict__ bias,
                                                       int T, int E, int k, int mode, int normalize, float norm_floor,
                                                       float scale, int32_t *__restrict__ ids,
                                                       float *__restrict__ weights) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const float *row = logits + static_cast<int64_t>(t) * E;
    auto raw_at = [&](int e) {
        const float v = row[e];
        return v != v ? -FLT_MAX : v;
    };
    float smax = 0.f, ssum = 1.f;
    if (mode == MFQ_TOPK_SOFTMAX) {
        smax = -INFINITY;
        for (int e = lane; e < E; e += 64) smax = fmaxf(smax, raw_at(e));
        smax = wave_max(smax);
        ssum = 0.f;
        for (int e = lane; e < E; e += 64) ssum += expf(raw_at(e) - smax);
        ssum = wave_sum(ssum);
    }
    auto weight_of = [&](float raw) {
        if (mode == MFQ_TOPK_DELAYED_SOFTMAX) return raw;
        if (mode == MFQ_TOPK_SIGMOID) return 1.f / (1.f + expf(-raw));
        if (mode == MFQ_TOPK_SQRT_SOFTPLUS) return sqrtf(raw > 20.f ? raw : log1pf(expf(raw)));
        return expf(raw - smax) / ssum;
    };
    float mine = 0.f;  // lane r keeps the weight of rank r
    constexpr int PER = 8;  // experts a lane keeps in registers: rows up to 512 experts are read once
    if (E <= 64 * PER) {
        float sc[PER], wv[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + 64 * i;
            sc[i] = -INFINITY;
            wv[i] = -INFINITY;
            if (e < E) {
                wv[i] = weight_of(raw_at(e));
                sc[i] = wv[i] + (bias ? bias[e] : 0.f);
            }
        }
        bool taken[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) taken[i] = lane + 64 * i >= E;
        for (int rank = 0; rank < k; ++rank) {
            float bs = -INFINITY, bw = -INFINITY;
            int bi = INT_MAX;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const int e = lane + 64 * i;
                if (!taken[i] && (sc[i] > bs || (sc[i] == bs && e < bi))) { bs = sc[i]; bw = wv[i]; bi = e; }
            }
            wave_argmax(bs, bw, bi);
#pragma unroll
            for (int i = 0; i < PER; ++i) taken[i] = taken[i] || (lane + 64 * i == bi);
            if (lane == rank) mine = bw;
            if (lane == 0) ids[static_cast<int64_t>(t) * k + rank] = bi;
        }
    } else {
        int selected[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) selected[i] = -1;
        for (int rank = 0; rank < k; ++rank) {
            float bs = -INFINITY, bw = -INFINITY;
            int bi = INT_MAX;
            for (int e = lane; e < E; e += 64) {
                bool taken = false;
#pragma unroll
                for (int p = 0; p < 16; ++p) taken |= (p < rank && selected[p] == e);
                if (taken) continue;
                const float wv = weight_of(raw_at(e));
                const float sc = wv + (bias ? bias[e] : 0.f);
                if (sc > bs || (sc == bs && e < bi)) { bs = sc; bw = wv; bi = e; }
            }
            wave_argmax(bs, bw, bi);
            selected[rank] = bi;
            if (lane == rank) mine = bw;
            if (lane == 0) ids[static_cast<int64_t>(t) * k + rank] = bi;
        }
    }
    float v = lane < k ? mine : 0.f;
    if (mode == MFQ_TOPK_DELAYED_SOFTMAX) {
        const float mx = wave_max(lane < k ? v : -INFINITY);
        v = lane < k ? expf(v - mx) : 0.f;
        const float den = wave_sum(v);
        v /= den;
    } else if (normalize) {
        const float den = fmaxf(wave_sum(v), norm_floor);
        v /= den;
    }
    if (lane < k) weights[static_cast<int64_t>(t) * k + lane] = v * scale;
}

// Rank-by-counting variant for up to 256 * PER experts: one block per token, thread e counts the experts that beat
// expert e (higher score, or the same score and a lower id); the k experts with rank < k are the selection, in
// rank order.  No serial chain of k wave-wide arg-max reductions: a decode step's single token takes about a
// microsecond.  Same results as moe_topk_kernel.
template <int PER>
__global__ __launch_bounds__(256) void moe_topk_rank_kernel(const float *__restrict__ logits, const float *__restrict__ bias,
                                                            int E, int k, int mode, int normalize, float norm_floor,
                                                            float scale, int32_t *__restrict__ ids,
                                                            float *__restrict__ weights) {
    __shared__ __attribute__((aligned(16))) int s_key[256 * PER];
    __shared__ float s_red[8];
    __shared__ float s_w[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.x;
    const float *row = logits + static_cast<int64_t>(t) * E;
    float raw[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + 256 * i;
        const float v = e < E ? row[e] : -INFINITY;
        raw[i] = v != v ? -FLT_MAX : v;
    }
    float smax = 0.f, ssum = 1.f;
    if (mode == MFQ_TOPK_SOFTMAX) {
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i) m = fmaxf(m, raw[i]);
        m = wave_max(m);
        if (lane == 0) s_red[wave] = m;
        __syncthreads();
        smax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
        float a = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (tid + 256 * i < E) a += expf(raw[i] - smax);
        a = wave_sum(a);
        if (lane == 0) s_red[4 + wave] = a;
        __syncthreads();
        ssum = (s_red[4] + s_red[5]) + (s_red[6] + s_red[7]);
    }
    float wv[PER];
    int key[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + 256 * i;
        float w = raw[i];
        if (mode == MFQ_TOPK_SIGMOID) w = 1.f / (1.f + expf(-raw[i]));
        else if (mode == MFQ_TOPK_SQRT_SOFTPLUS) w = sqrtf(raw[i] > 20.f ? raw[i] : log1pf(expf(raw[i])));
        else if (mode == MFQ_TOPK_SOFTMAX) w = expf(raw[i] - smax) / ssum;
        wv[i] = w;
        const float sc = e < E ? w + (bias ? bias[e] : 0.f) : -INFINITY;
        // order-preserving map of the float to a signed int (-0 and +0 compare equal, as they do as floats)
        const int b = __float_as_int(sc + 0.f);
        key[i] = b ^ ((b >> 31) & 0x7fffffff);
        if (key[i] == INT_MIN) key[i] = INT_MIN + 1;  // unreachable from a float; keeps key - 1 from wrapping
        s_key[e] = e < E ? key[i] : INT_MIN;
    }
    __syncthreads();
    int rank[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) rank[i] = 0;
    const int n4 = (E + 3) >> 2;
    for (int j4 = 0; j4 < n4; ++j4) {
        const int4 o = reinterpret_cast<const int4 *>(s_key)[j4];
        const int ov[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int j = 4 * j4 + c;
#pragma unroll
            for (int i = 0; i < PER; ++i) rank[i] += ov[c] > key[i] - (j < tid + 256 * i);  // >= for the lower ids
        }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = tid + 256 * i;
        if (e < E && rank[i] < k) {
            ids[static_cast<int64_t>(t) * k + rank[i]] = e;
            s_w[rank[i]] = wv[i];
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float v = lane < k ? s_w[lane] : 0.f;
    if (mode == MFQ_TOPK_DELAYED_SOFTMAX) {
        const float mx = wave_max(lane < k ? v : -INFINITY);
        v = lane < k ? expf(v - mx) : 0.f;
        const float den = wave_sum(v);
        v /= den;
    } else if (normalize) {
        const float den = fmaxf(wave_sum(v), norm_floor);
        v /= den;
    }
    if (lane < k) weights[static_cast<int64_t>(t) * k + lane] = v * scale;
}

// ---- expert map ------------------------------------------------------------------------------
// counts: one block per expert counts its pairs (no atomics, nothing to pre-clear).
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t *__restrict__ ids, int n_pairs,
                                                        int32_t *__restrict__ counts) {
    __shared__ int red[4];
    const int e = blockIdx.x, tid = threadIdx.x;
    int c = 0;
    const bool vec = (reinterpret_cast<uintptr_t>(ids) & 15) == 0;  // four ids per load
    const int n4 = vec ? n_pairs & ~3 : 0;
    for (int p = tid * 4; p < n4; p += 1024) {
        const int4 v = *reinterpret_cast<const int4 *>(ids + p);
        c += (v.x == e) + (v.y == e) + (v.z == e) + (v.w == e);
    }
    for (int p = n4 + tid; p < n_pairs; p += 256) c += (ids[p] == e);
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
    if ((tid & 63) == 0) red[tid >> 6] = c;
    __syncthreads();
    if (tid == 0) counts[e] = red[0] + red[1] + red[2] + red[3];
}

// exclusive prefix sums over the experts by one block (Hillis-Steele over 1024-wide chunks), then
// every expert fills its own tile slots.
__global__ __launch_bounds__(1024) void moe_scan_kernel(const int32_t *__restrict__ counts, int E, int tile_m,
                                                        int32_t *__restrict__ expert_bounds,
                                                        int32_t *__restrict__ tile_bounds,
                                                        int32_t *__restrict__ tile_experts, int max_tiles) {
    __shared__ int sa[1024], sb[1024];
    __shared__ int carry_a, carry_b;
    const int tid = threadIdx.x;
    if (tid == 0) { carry_a = 0; carry_b = 0; }
    __syncthreads();
    for (int base = 0; base < E; base += 1024) {
        const int e = base + tid;
        const int c = e < E ? counts[e] : 0;
        const int tl = (c + tile_m - 1) / tile_m;
        sa[tid] = c; sb[tid] = tl;
        __syncthreads();
        for (int o = 1; o < 1024; o <<= 1) {
            const int va = tid >= o ? sa[tid - o] : 0, vb = tid >= o ? sb[tid - o] : 0;
            __syncthreads();
            sa[tid] += va; sb[tid] += vb;
            __syncthreads();
        }
        const int ea = carry_a + sa[tid] - c, eb = carry_b + sb[tid] - tl;  // exclusive
        if (e < E) {
            expert_bounds[e] = ea;
            tile_bounds[e] = eb;
            for (int i = 0; i < tl; ++i)
                if (eb + i < max_tiles) tile_experts[eb + i] = e;
        }
        __syncthreads();
        if (tid == 1023) { carry_a += sa[1023]; carry_b += sb[1023]; }
        __syncthreads();
    }
    if (tid == 0) { expert_bounds[E] = carry_a; tile_bounds[E] = carry_b; }
}

// scatter: one block per expert walks the pairs in order, so the order inside an expert is the
// ascending pair index (deterministic).
__global__ __launch_bounds__(256) void moe_scatter_kernel(const int32_t *__restrict__ ids, int n_pairs,
                                                          const int32_t *__restrict__ expert_bounds,
                                                          int32_t *__restrict__ ids_dst) {
    __shared__ int wsum[4];
    __shared__ int base;
    const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) base = expert_bounds[e];
    __syncthreads();
    // windows of 1024 pairs, four consecutive ones per thread: the pairs of the expert keep their order
    const bool vec = (reinterpret_cast<uintptr_t>(ids) & 15) == 0;
    for (int p0 = 0; p0 < n_pairs; p0 += 1024) {
        const int p = p0 + tid * 4;
        int v[4];
        if (vec && p + 3 < n_pairs) {
            const int4 q = *reinterpret_cast<const int4 *>(ids + p);
            v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t) v[t] = p + t < n_pairs ? ids[p + t] : -1;
        }
        const int mine = (v[0] == e) + (v[1] == e) + (v[2] == e) + (v[3] == e);
        int inc = mine;
        for (int o = 1; o < 64; o <<= 1) {
            const int u = __shfl_up(inc, o, 64);
            if (lane >= o) inc += u;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        int off = base + inc - mine;
        for (int wv = 0; wv < wave; ++wv) off += wsum[wv];
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (v[t] == e) ids_dst[off++] = p + t;
        __syncthreads();
        if (tid == 0) base += wsum[0] + wsum[1] + wsum[2] + wsum[3];
        __syncthreads();
    }
}

// ---- expert-grouped matmul ---------------------------------------------------------------------
// One cohort dispatch of the vector-ALU path: MB pairs of one expert, one 16-neuron row-block.  RING = false
// when no wave has more than three steps.
template <int XF16, int MB, bool RING>
__device__ __forceinline__ void moe_valu_chunk(const NintK &k, const uint8_t *w, int rb, int row_base, int out_per_expert,
                                               const uint16_t *const (&xr)[MB], float *const (&yr)[MB], int spw,
                                               uint32_t *lds) {
#define MFQ_MOE_CASE(B, G)                                                                                    \
    if (k.bits == B && k.gs == G) {                                                                           \
        nint_paired_body<B, G, XF16, MB, RING>(k, w, rb, 1, row_base, out_per_expert, xr, yr, spw, lds);            \
        return;                                                                                               \
    }
    if (k.kind == 1) {
        MFQ_MOE_CASE(4, 24) MFQ_MOE_CASE(3, 24) MFQ_MOE_CASE(2, 16) MFQ_MOE_CASE(4, 32) MFQ_MOE_CASE(4, 16)
        MFQ_MOE_CASE(4, 48) MFQ_MOE_CASE(2, 32)
    }
#undef MFQ_MOE_CASE
    nint_generic_body<XF16, MB>(k, w, rb, row_base, out_per_expert, xr, yr, spw, lds);
}

// Vector-ALU path (any NINT profile, any K).  Without a route map every pair is its own tile (MB = 1,
// decode); with one, tile t holds pairs ids_dst[lo .. lo + kMoeTileM), taken MB at a time.
template <int XF16, int MB, bool RING>
__global__ __launch_bounds__(512) void moe_grouped_kernel(MoePools P, const int32_t *__restrict__ expert_pool,
                                                           const int32_t *__restrict__ expert_local, int E,
                                                           int out_per_expert, const uint16_t *__restrict__ x,
                                                           int64_t ldx, int routed_input, const int32_t *__restrict__ ids,
                                                           int n_pairs, int R, const int32_t *__restrict__ ids_dst,
                                                           const int32_t *__restrict__ expert_bounds,
                                                           const int32_t *__restrict__ tile_bounds,
                                                           const int32_t *__restrict__ tile_experts,
                                                           float *__restrict__ out, int64_t ldo) {
    extern __shared__ uint32_t lds[];
    const int tile = blockIdx.y;  // row-blocks run fastest, so that the blocks of one tile spread over the XCDs
    int e, lo = 0, hi = 0;
    if (ids_dst == nullptr) {
        e = ids[tile];
    } else {
        if (tile >= tile_bounds[E]) return;
        e = tile_experts[tile];
        lo = expert_bounds[e] + (tile - tile_bounds[e]) * kMoeTileM;
        hi = min(expert_bounds[e + 1], lo + kMoeTileM);
    }
    const int rbl = blockIdx.x;  // row-block inside the expert
    const bool valid = e >= 0 && e < E && expert_pool[e] >= 0;
    for (int c = 0; c == 0 || lo + c < hi; c += MB) {
        int pairs[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) pairs[m] = ids_dst ? (lo + c + m < hi ? ids_dst[lo + c + m] : -1) : (m == 0 ? tile : -1);
        const uint16_t *xr[MB];
        float *yr[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const int p = pairs[m];
            xr[m] = p >= 0 ? x + static_cast<int64_t>(routed_input ? p : p / R) * ldx : nullptr;
            yr[m] = p >= 0 ? out + static_cast<int64_t>(p) * ldo : nullptr;
        }
        if (!valid) {  // invalid expert id: defined as a zero row
            const int row = rbl * 16 + (threadIdx.x & 15);
            if (threadIdx.x < 16 && row < out_per_expert)
#pragma unroll
                for (int m = 0; m < MB; ++m)
                    if (yr[m]) yr[m][row] = 0.f;
            return;
        }
        const int pool = expert_pool[e];
        const int row_base = expert_local[e] * out_per_expert;
        moe_valu_chunk<XF16, MB, RING>(P.k[pool], P.w[pool], row_base / 16 + rbl, row_base, out_per_expert, xr, yr, P.spw[pool],
                                 lds);
        __syncthreads();  // the next chunk reuses the reduction area
    }
}

// Batch-1 path (no route map): block (group of rbw row-blocks, row), the body of the dense GEMV with the unit of
// the row's cohort.  Rows below n_pairs are (token, route) pairs; row n_pairs + t applies the shared tensor
// (cohort slot P.n) to token t.  P.spw: steps per wave of each cohort; RING = false when no wave has more than
// three (row-block, step) items.  SWIGLU: the block takes row-block blockIdx.x of the gate half and of the up half
// of the expert and stores act(gate) * up as 16-bit values: bit 0 of out_f16 selects fp16 over bf16, bit 1 GELU over SiLU.
// XR (only without a ring): cohorts whose groups fit a row of lanes keep the activations in registers
// (nint_unit_body_xreg); the launch sets it when the rows are 4-byte aligned and K is even.
template <int XF16, bool RING, bool SWIGLU, bool XR = false>
__global__ __launch_bounds__(1024) void moe_decode_kernel(MoePools P, int rbw, const int32_t *__restrict__ expert_pool,
                                                          const int32_t *__restrict__ expert_local, int E,
                                                          int out_per_expert, const uint16_t *__restrict__ x, int64_t ldx,
                                                          int routed_input, const int32_t *__restrict__ ids, int n_pairs,
                                                          int R, void *__restrict__ out, int out_f16, int64_t ldo) {
    extern __shared__ uint32_t lds[];
    const int row = blockIdx.y;
    const int half_rb = out_per_expert / 32;  // SWIGLU: row-blocks of the gate half
    const int rbl0 = SWIGLU ? blockIdx.x : blockIdx.x * rbw;
    int pool, row_base, xi;
    if (row < n_pairs) {
        const int e = ids[row];
        if (e < 0 || e >= E || expert_pool[e] < 0) {  // invalid expert id: defined as a zero row
            if constexpr (SWIGLU) {
                if (threadIdx.x < 16) static_cast<uint16_t *>(out)[row * ldo + rbl0 * 16 + threadIdx.x] = 0;
            } else {
                for (int c = threadIdx.x; c < rbw * 16; c += blockDim.x)
                    static_cast<float *>(out)[row * ldo + rbl0 * 16 + c] = 0.f;
            }
            return;
        }
        pool = expert_pool[e];
        row_base = expert_local[e] * out_per_expert;
        xi = routed_input ? row : row / R;
    } else {
        pool = P.n;
        row_base = 0;
        xi = routed_input ? row : row - n_pairs;
    }
    const NintK &k = P.k[pool];
    const uint8_t *w = P.w[pool];
    const int spw = P.spw[pool];
    const uint16_t *xr[1] = {x + static_cast<int64_t>(xi) * ldx};
    float *yr[1] = {SWIGLU ? nullptr : static_cast<float *>(out) + static_cast<int64_t>(row) * ldo};
    const int rb0 = row_base / 16 + rbl0, nrb = SWIGLU ? 2 : rbw, step = SWIGLU ? half_rb : 1;
    bool in_regs = false;  // this block's cohort ran the register body: its partial sums start at the head of the LDS
#define MFQ_MOE_CASE(UNIT, B, G)                                                                                        \
    if (k.bits == B && k.gs == G) {                                                                                    \
        if constexpr (XR && !RING && UNIT<B, G>::NPAIR <= 16) {                                                        \
            in_regs = true;                                                                                            \
            nint_unit_body_xreg<UNIT<B, G>, XF16, 1, !SWIGLU>(k, w, rb0, nrb, row_base, out_per_expert, xr, yr, spw, lds, step); \
        } else {                                                                                                       \
            nint_unit_body<UNIT<B, G>, XF16, 1, RING, !SWIGLU>(k, w, rb0, nrb, row_base, out_per_expert, xr, yr, spw, lds, step); \
        }                                                                                                              \
    }
    if (k.kind == 1) {
        MFQ_MOE_CASE(PairedUnit, 4, 24)
        else MFQ_MOE_CASE(PairedUnit, 3, 24)
        else MFQ_MOE_CASE(PairedUnit, 2, 16)
        else MFQ_MOE_CASE(PairedUnit, 4, 32)
        else MFQ_MOE_CASE(PairedUnit, 4, 16)
        else MFQ_MOE_CASE(PairedUnit, 4, 48)
        else MFQ_MOE_CASE(PairedUnit, 2, 32)
    } else {
        MFQ_MOE_CASE(GenericUnit, 5, 28)
    }
#undef MFQ_MOE_CASE
    if constexpr (SWIGLU) {
        __syncthreads();
        if (threadIdx.x < 16) {
            const int nwaves = blockDim.x >> 6;
            const float *red = reinterpret_cast<const float *>(lds + (in_regs ? 0 : gemv_red_offset(nwaves, 1, spw, k.gs)));
            float g = 0.f, u = 0.f;
            for (int wv = 0; wv < nwaves; ++wv) {
                g += red[wv * 16 + threadIdx.x];
                u += red[(nwaves + wv) * 16 + threadIdx.x];
            }
            const float v = glu_value(g, u, out_f16 & 2);
            static_cast<uint16_t *>(out)[row * ldo + rbl0 * 16 + threadIdx.x] = (out_f16 & 1) ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
        }
    }
}

// Matrix-core path: a tile of up to 16 pairs of one expert against NB row-blocks, weights streamed once
// per tile (nint_mfma_body).  Needs K % 8 == 0, 16-byte aligned activation rows and cohorts with an MFMA
// unit; P.spw holds the steps per wave of each cohort.
template <int XF16, int NB>
__global__ __launch_bounds__(512) void moe_mfma_kernel(MoePools P, const int32_t *__restrict__ expert_pool,
                                                       const int32_t *__restrict__ expert_local, int E,
                                                       int out_per_expert, const uint16_t *__restrict__ x, int64_t ldx,
                                                       int routed_input, const int32_t *__restrict__ ids, int n_pairs,
                                                       int R, const int32_t *__restrict__ ids_dst,
                                                       const int32_t *__restrict__ expert_bounds,
                                                       const int32_t *__restrict__ tile_bounds,
                                                       const int32_t *__restrict__ tile_experts,
                                                       float *__restrict__ out, int64_t ldo) {
    extern __shared__ uint32_t lds[];
    float *red = reinterpret_cast<float *>(lds);
    const int tile = blockIdx.y;  // row-blocks run fastest, so that the blocks of one tile spread over the XCDs
    int e, lo = 0, hi = 0;
    if (ids_dst == nullptr) {
        e = ids[tile];
    } else {
        if (tile >= tile_bounds[E]) return;
        e = tile_experts[tile];
        lo = expert_bounds[e] + (tile - tile_bounds[e]) * kMoeTileM;
        hi = min(expert_bounds[e + 1], lo + kMoeTileM);
    }
    const int rbe = out_per_expert / 16, rbl0 = blockIdx.x * NB;
    auto pair_of = [&](int slot) -> int {  // -1 = empty slot
        if (ids_dst == nullptr) return slot == 0 ? tile : -1;
        return lo + slot < hi ? ids_dst[lo + slot] : -1;
    };
    if (e < 0 || e >= E || expert_pool[e] < 0) {  // invalid expert id: defined as a zero row (unmapped tiles only)
        const int p = pair_of(0);
        for (int c = threadIdx.x; c < min(NB, rbe - rbl0) * 16; c += blockDim.x)
            if (p >= 0) out[static_cast<int64_t>(p) * ldo + rbl0 * 16 + c] = 0.f;
        return;
    }
    const int pool = expert_pool[e];
    const int rb_first = expert_local[e] * rbe;
    const int p = pair_of(threadIdx.x & 15);   // -1: an empty slot of the tile, whose lanes request no activations
    const NintK &k = P.k[pool];
    if (P.prefill[pool]) return;
    // all activation rows through one window (the launcher checks that they span less than 4 GiB)
    const int n_rows = routed_input ? n_pairs : (n_pairs + R - 1) / R;
    const __amdgpu_buffer_rsrc_t xwin = wave_window(reinterpret_cast<const uint8_t *>(x),
                                                    static_cast<uint32_t>((static_cast<int64_t>(n_rows - 1) * ldx + k.neuron_len) * 2));
    const uint32_t xoff = p < 0 ? kNoStep : static_cast<uint32_t>(static_cast<int64_t>(routed_input ? p : p / R) * ldx * 2);
    const uint8_t *w = P.w[pool];
    const int spw = P.spw[pool];
#define MFQ_MOE_MFMA(UNIT, B, G) \
    if (k.bits == B && k.gs == G) nint_mfma_body<UNIT<B, G>, XF16, NB, mfma_x_ahead<UNIT<B, G>, NB, 8>()>(k, w, rb_first + rbl0, rb_first + rbe, xwin, xoff, spw, red);
    if (k.kind == 1) {
        MFQ_MOE_MFMA(PairedUnit, 4, 24)
        else MFQ_MOE_MFMA(PairedUnit, 3, 24)
        else MFQ_MOE_MFMA(PairedUnit, 2, 16)
        else MFQ_MOE_MFMA(PairedUnit, 4, 32)
        else MFQ_MOE_MFMA(PairedUnit, 4, 16)
        else MFQ_MOE_MFMA(PairedUnit, 4, 48)
        else MFQ_MOE_MFMA(PairedUnit, 2, 32)
    } else {
        MFQ_MOE_MFMA(GenericUnit, 5, 28)
    }
#undef MFQ_MOE_MFMA
    __syncthreads();
    const int nwaves = blockDim.x >> 6;
    for (int o = threadIdx.x; o < NB * 256; o += blockDim.x) {
        const int rr = o & 15, t = (o >> 4) & 15, nb = o >> 8;
        const int pt = pair_of(t);
        if (pt < 0 || rbl0 + nb >= rbe) continue;
        const int slot = (nb * 4 + (t & 3)) * 64 + rr + 16 * (t >> 2);
        float s = 0.f;
        for (int wv = 0; wv < nwaves; ++wv) s += red[wv * NB * 256 + slot];
        out[static_cast<int64_t>(pt) * ldo + (rbl0 + nb) * 16 + rr] = s;
    }
}

// rows of pairs whose expert id is out of range are not in any tile of the map: clear them
__global__ void moe_zero_invalid_kernel(const int32_t *__restrict__ ids, int n_pairs, int E,
                                        const int32_t *__restrict__ expert_pool, int width, float *__restrict__ out,
                                        int64_t ldo) {
    const int p = blockIdx.x;
    const int e = ids[p];
    if (e >= 0 && e < E && expert_pool[e] >= 0) return;
    for (int c = threadIdx.x; c < width; c += blockDim.x) out[static_cast<int64_t>(p) * ldo + c] = 0.f;
}

template <int F16OUT>
__global__ __launch_bounds__(256) void moe_swiglu_kernel(const float *__restrict__ gu, int64_t ld, int rows, int W,
                                                         uint16_t *__restrict__ hidden, int64_t ldh, int gelu) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(rows) * W) return;
    const int row = static_cast<int>(idx / W), col = static_cast<int>(idx - static_cast<int64_t>(row) * W);
    const float g = gu[row * ld + col], u = gu[row * ld + W + col];
    const float v = glu_value(g, u, gelu != 0);
    hidden[row * ldh + col] = F16OUT ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
}

__global__ __launch_bounds__(256) void moe_reduce_kernel(const float *__restrict__ pair, const float *__restrict__ wts,
                                                         int T, int R, int H, const float *__restrict__ shared,
                                                         const float *__restrict__ gate_logits,
                                                         float *__restrict__ out) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(T) * H) return;
    const int t = static_cast<int>(idx / H), c = static_cast<int>(idx - static_cast<int64_t>(t) * H);
    float v = 0.f;
    for (int r = 0; r < R; ++r) {
        const int64_t p = static_cast<int64_t>(t) * R + r;
        v = fmaf(wts[p], pair[p * H + c], v);
    }
    if (shared) {
        const float g = gate_logits ? 1.f / (1.f + expf(-gate_logits[t])) : 1.f;
        v = fmaf(g, shared[idx], v);
    }
    out[idx] = v;
}

// Expert residency: copies `n` byte ranges out of one staging buffer (already on the device) to their destinations --
// the body and anchors of every expert that has just been brought in, and the table words that now point at its
// slot.  blockIdx.x = transfer, blockIdx.y = slice of it: a multi-megabyte expert body is spread over many blocks so
// that one launch moves the whole batch at HBM speed.
__global__ __launch_bounds__(256) void cache_scatter_kernel(const uint8_t *__restrict__ staging, int64_t descriptor_offset) {
    const mfq_scatter_desc d = reinterpret_cast<const mfq_scatter_desc *>(staging + descriptor_offset)[blockIdx.x];
    uint8_t *dst = reinterpret_cast<uint8_t *>(static_cast<uintptr_t>(d.destination));
    const uint8_t *src = staging + d.source_offset;
    const uint64_t n = d.nbytes;
    if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | n) & 15u) == 0) {
        const uint64_t n16 = n >> 4, per = (n16 + gridDim.y - 1) / gridDim.y;
        const uint64_t lo = per * blockIdx.y, hi = lo + per < n16 ? lo + per : n16;
        const u32x4_t *in = reinterpret_cast<const u32x4_t *>(src);
        u32x4_t *out = reinterpret_cast<u32x4_t *>(dst);
        for (uint64_t i = lo + threadIdx.x; i < hi; i += 256) out[i] = __builtin_nontemporal_load(in + i);
        return;
    }
    const uint64_t per = (n + gridDim.y - 1) / gridDim.y;
    const uint64_t lo = per * blockIdx.y, hi = lo + per < n ? lo + per : n;
    for (uint64_t i = lo + threadIdx.x; i < hi; i += 256) dst[i] = src[i];
}

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_cache_scatter(const void *staging, int64_t descriptor_offset, int n_transfers, int64_t max_bytes,
                                     mfq_stream_t stream) {
    MFQ_REQUIRE(staging && descriptor_offset >= 0 && (descriptor_offset & 7) == 0, MFQ_ERR_INVALID,
                "cache_scatter: null staging buffer or misaligned descriptor table");
    MFQ_REQUIRE(n_transfers >= 0 && n_transfers <= 65535 * 32, MFQ_ERR_INVALID, "cache_scatter: %d transfers", n_transfers);
    if (n_transfers == 0) return MFQ_OK;
    // slices of about 64 KB of the largest transfer, at most 64 per transfer
    int64_t slices = max_bytes > 0 ? ceil_div(max_bytes, 65536) : 1;
    slices = slices < 1 ? 1 : (slices > 64 ? 64 : slices);
    hipLaunchKernelGGL(cache_scatter_kernel, dim3(static_cast<unsigned>(n_transfers), static_cast<unsigned>(slices)), dim3(256), 0,
                       as_stream(stream), static_cast<const uint8_t *>(staging), descriptor_offset);
    return check_launch("cache_scatter");
}

extern "C" int mfq_hip_moe_topk(const float *logits, const float *bias, int T, int E, int k, int mode, int normalize,
                                float norm_floor, float scale, int32_t *ids, float *weights, mfq_stream_t stream) {
    MFQ_REQUIRE(logits && ids && weights, MFQ_ERR_INVALID, "moe_topk: null argument");
    MFQ_REQUIRE(T > 0 && E > 0, MFQ_ERR_INVALID, "logits dimensions must be nonzero");
    MFQ_REQUIRE(k >= 1 && k <= 16 && k <= E, MFQ_ERR_INVALID, "top_k must be in [1, min(16, experts)]");
    MFQ_REQUIRE(mode >= 0 && mode <= 3, MFQ_ERR_INVALID, "moe_topk: unknown mode %d", mode);
    MFQ_REQUIRE(!(normalize && mode == MFQ_TOPK_DELAYED_SOFTMAX), MFQ_ERR_INVALID,
                "selected-weight normalization and delayed softmax are mutually exclusive");
#define MFQ_TOPK_RANK(PER)                                                                                        \
    hipLaunchKernelGGL(moe_topk_rank_kernel<PER>, dim3(static_cast<unsigned>(T)), dim3(256), 0, as_stream(stream), \
                       logits, bias, E, k, mode, normalize, norm_floor, scale, ids, weights)
    if (E <= 256) MFQ_TOPK_RANK(1);
    else if (E <= 512) MFQ_TOPK_RANK(2);
    else if (E <= 1024) MFQ_TOPK_RANK(4);
#undef MFQ_TOPK_RANK
    else
        hipLaunchKernelGGL(moe_topk_kernel, dim3(static_cast<unsigned>(ceil_div(T, 4))), dim3(256), 0, as_stream(stream),
                           logits, bias, T, E, k, mode, normalize, norm_floor, scale, ids, weights);
    return check_launch("moe_topk");
}

extern "C" int mfq_hip_moe_route_map(const int32_t *ids, int n_pairs, int E, int tile_m, int32_t *counts,
                                     int32_t *expert_bounds, int32_t *tile_bounds, int32_t *tile_experts, int max_tiles,
                                     int32_t *ids_dst, mfq_stream_t stream) {
    MFQ_REQUIRE(ids && counts && expert_bounds && tile_bounds && tile_experts && ids_dst, MFQ_ERR_INVALID,
                "moe_route_map: null argument");
    MFQ_REQUIRE(n_pairs > 0 && E > 0 && tile_m > 0, MFQ_ERR_INVALID, "moe_route_map: empty problem");
    MFQ_REQUIRE(max_tiles >= ceil_div(n_pairs, tile_m) + E, MFQ_ERR_INVALID, "moe_route_map: max_tiles %d < %lld", max_tiles,
                static_cast<long long>(ceil_div(n_pairs, tile_m) + E));
    hipStream_t st = as_stream(stream);
    hipLaunchKernelGGL(moe_count_kernel, dim3(E), dim3(256), 0, st, ids, n_pairs, counts);
    hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(1024), 0, st, counts, E, tile_m, expert_bounds, tile_bounds,
                       tile_experts, max_tiles);
    hipLaunchKernelGGL(moe_scatter_kernel, dim3(E), dim3(256), 0, st, ids, n_pairs, expert_bounds, ids_dst);
    return check_launch("moe_route_map");
}

// the grouped kernel batches this many routes of one expert per block

extern "C" int mfq_hip_moe_tile_m(void) { return kMoeTileM; }

extern "C" size_t mfq_hip_moe_grouped_workspace_bytes(const mfq_moe_pool *pools, int n_pools, int K, int x_rows) {
    return moe_prefill_workspace(pools, n_pools, K, x_rows);
}

// Block shape of the batch-1 launch: false when the shape does not fit the kernel.
struct MoeDecodeShape {
    int nwaves, rbw;
    size_t lds;
    bool ring;
};
static bool moe_decode_shape(MoePools &P, int n_slots, int max_steps, int out_per_expert, int n_rows, int swiglu,
                             MoeDecodeShape &sh) {
    static const int env_off = tune_env("MFQ_MOE_SPLIT", 1) == 0;
    static const int env_w = tune_env("MFQ_MOE_DEC_WAVES", 3);
    static const int env_rbw = tune_env("MFQ_MOE_DEC_RBW", 0);
    if (env_off || n_rows > 65535) return false;
    const int rbe = out_per_expert / 16;
    // Three waves split the K steps: a launch has one block per (row-block group, row), thousands of them, and small
    // blocks let five or six sit on a compute unit at the kernel's 128 registers, so that the grid runs in fewer
    // rounds (config-4 layer at T = 1 / 2 / 4: 50 / 72 / 118 us against 57 / 87 / 149 us with eight waves and
    // 64 / 101 / 178 us with five).  A wave takes more (row-block, step) items while the grid keeps
    // about gemv_target_waves() waves.  With the fused SwiGLU a block always takes two row-blocks:
    // gate and up.
    const int nwaves = max_steps < env_w ? max_steps : env_w;
    const int spw_max = static_cast<int>(ceil_div(max_steps, nwaves));
    int64_t items = 0;
    for (int i = 0; i < n_slots; ++i) items += P.k[i].nsteps;
    items = items / n_slots * rbe * n_rows;
    int per_wave = static_cast<int>(items / gemv_target_waves());
    per_wave = per_wave < 1 ? 1 : (per_wave > 3 ? 3 : per_wave);
    int rbw = per_wave / spw_max < 1 ? 1 : per_wave / spw_max;
    if (env_rbw) rbw = env_rbw;
    if (rbw > kMaxRbw) rbw = kMaxRbw;
    while (rbe % rbw) --rbw;
    if (swiglu) {
        if (out_per_expert % 32) return false;
        rbw = 2;
    }
    size_t lds = 0;
    bool ring = false;
    for (int i = 0; i < n_slots; ++i) {
        P.spw[i] = static_cast<int>(ceil_div(P.k[i].nsteps, nwaves));
        const size_t need = gemv_lds_bytes(1, P.spw[i], P.k[i].gs, nwaves, rbw);
        if (need > lds) lds = need;
        if (P.spw[i] * rbw > 3) ring = true;
        if (swiglu && static_cast<int64_t>(rbe / 2) * P.k[i].rowblock_bytes >= (1ll << 31)) return false;
    }
    if (lds > kMaxDynamicLds) return false;
    sh.nwaves = nwaves; sh.rbw = rbw; sh.lds = lds; sh.ring = ring;
    return true;
}

// Batch-1 launch (moe_decode_kernel) over n_rows rows: the n_pairs routed pairs, then one row per token for the
// shared tensor in cohort slot P.n, if any.  Every cohort slot has a GEMV unit.  Returns -1 when the shape does
// not fit the kernel (the caller takes another path), else a status.
static int moe_decode_launch(MoePools &P, int n_slots, int max_steps, const int32_t *expert_pool,
                             const int32_t *expert_local, int E, int out_per_expert, const uint16_t *xp, int x_dtype,
                             int64_t ldx, int routed_input, const int32_t *ids, int n_pairs, int n_rows, int R, int swiglu,
                             void *out, int out_f16, int64_t ldo, hipStream_t st) {
    MoeDecodeShape sh;
    if (!moe_decode_shape(P, n_slots, max_steps, out_per_expert, n_rows, swiglu, sh)) return -1;
    const int rbe = out_per_expert / 16, rbw = sh.rbw, nwaves = sh.nwaves;
    const size_t lds = sh.lds;
    const bool ring = sh.ring;
    const dim3 grid(static_cast<unsigned>(swiglu ? rbe / 2 : rbe / rbw), static_cast<unsigned>(n_rows)), block(64 * nwaves);
    static const int env_xreg = tune_env("MFQ_GEMV_XREG", 1);
    const bool xreg = !ring && ldx % 2 == 0 && (reinterpret_cast<uintptr_t>(xp) & 3) == 0 && P.k[0].neuron_len % 2 == 0 &&
                      env_xreg != 0;
#define MFQ_MOE_DECODE(XF, RG, SW)                                                                                   \
    do {                                                                                                             \
        auto kern = (!RG && xreg) ? moe_decode_kernel<XF, RG, SW, !RG> : moe_decode_kernel<XF, RG, SW, false>;       \
        if (int rc_ = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds, "moe_decode")) return rc_;        \
        hipLaunchKernelGGL(kern, grid, block, lds, st, P, rbw, expert_pool, expert_local, E, out_per_expert, xp, ldx, \
                           routed_input, ids, n_pairs, R, out, out_f16, ldo);                                        \
    } while (0)
#define MFQ_MOE_DECODE_X(XF)                        \
    if (swiglu) {                                   \
        if (ring) MFQ_MOE_DECODE(XF, true, true);   \
        else MFQ_MOE_DECODE(XF, false, true);       \
    } else {                                        \
        if (ring) MFQ_MOE_DECODE(XF, true, false);  \
        else MFQ_MOE_DECODE(XF, false, false);      \
    }
    if (x_dtype == MFQ_X_F16) MFQ_MOE_DECODE_X(1) else MFQ_MOE_DECODE_X(0)
#undef MFQ_MOE_DECODE_X
#undef MFQ_MOE_DECODE
    return check_launch("moe_decode");
}

extern "C" int mfq_hip_moe_grouped_matmul(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                                          const int32_t *expert_local, int E, int out_per_expert, int K, const void *x,
                                          int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                                          const int32_t *ids_dst, const int32_t *expert_bounds,
                                          const int32_t *tile_bounds, const int32_t *tile_experts, float *out,
                                          int64_t ldo, mfq_stream_t stream) {
    return mfq_hip_moe_grouped_matmul_ws(pools, n_pools, expert_pool, expert_local, E, out_per_expert, K, x, x_dtype, ldx,
                                         routed_input, ids, T, R, ids_dst, expert_bounds, tile_bounds, tile_experts, out, ldo,
                                         nullptr, 0, stream);
}

extern "C" int mfq_hip_moe_grouped_matmul_ws(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                                             const int32_t *expert_local, int E, int out_per_expert, int K, const void *x,
                                             int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                                             const int32_t *ids_dst, const int32_t *expert_bounds,
                                             const int32_t *tile_bounds, const int32_t *tile_experts, float *out,
                                             int64_t ldo, void *workspace, size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(pools && expert_pool && expert_local && x && ids && out, MFQ_ERR_INVALID, "moe_grouped_matmul: null argument");
    MFQ_REQUIRE(n_pools >= 1 && n_pools <= kMaxPools, MFQ_ERR_UNSUPPORTED, "moe_grouped_matmul: %d cohorts (max %d)", n_pools,
                kMaxPools);
    MFQ_REQUIRE(T > 0 && R > 0 && E > 0, MFQ_ERR_INVALID, "MoE ids must be int32 [tokens, routes]");
    MFQ_REQUIRE(out_per_expert % 16 == 0, MFQ_ERR_UNSUPPORTED, "moe_grouped_matmul: out_per_expert %d must be a multiple of 16",
                out_per_expert);
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "moe_grouped_matmul: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(ldx >= K && ldo >= out_per_expert, MFQ_ERR_INVALID, "moe_grouped_matmul: ldx/ldo smaller than the tensor");
    const int n_pairs = T * R;
    const bool mapped = ids_dst != nullptr;
    if (mapped)
        MFQ_REQUIRE(expert_bounds && tile_bounds && tile_experts, MFQ_ERR_INVALID,
                    "moe_grouped_matmul: route map without its bounds / tile tables");
    MoePools P;
    P.n = n_pools;
    int max_steps = 1;
    bool units = true;  // every cohort has a unit with GEMV, streaming and prefill bodies
    // (the matrix-core kernel addresses all activation rows through one buffer window: they span less than 4 GiB)
    bool mfma = K >= 8 && K % 8 == 0 && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                (static_cast<int64_t>(n_pairs) * ldx + K) * 2 < (1ll << 32);
    for (int i = 0; i < n_pools; ++i) {
        const mfq_nint_desc &d = pools[i].desc;
        MFQ_REQUIRE(d.neuron_len == K && pools[i].weight, MFQ_ERR_INVALID,
                    "moe_grouped_matmul: cohort %d has neuron_len %d, expected %d", i, d.neuron_len, K);
        if (d.nsteps > max_steps) max_steps = d.nsteps;
        moe_fill_k(P.k[i], d);
        P.w[i] = static_cast<const uint8_t *>(pools[i].weight);
        P.xg[i] = nullptr;
        P.prefill[i] = 0;
        units = units && moe_prefill_unit(d) && 4 * d.rowblock_bytes < (1ll << 31);
        mfma = mfma && units;
    }
    const int rbe = out_per_expert / 16;
    const int64_t tiles = mapped ? ceil_div(n_pairs, kMoeTileM) + E : n_pairs;
    MFQ_REQUIRE(tiles <= 65535, MFQ_ERR_UNSUPPORTED, "moe_grouped_matmul: %lld tiles in one call (max 65535)",
                static_cast<long long>(tiles));
    hipStream_t st = as_stream(stream);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    if (mapped)
        hipLaunchKernelGGL(moe_zero_invalid_kernel, dim3(n_pairs), dim3(256), 0, st, ids, n_pairs, E, expert_pool,
                           out_per_expert, out, ldo);
#define MFQ_MOE_LAUNCH(KERNEL, GRID, BLOCK, LDS)                                                                      \
    hipLaunchKernelGGL(KERNEL, GRID, BLOCK, LDS, st, P, expert_pool, expert_local, E, out_per_expert, xp, ldx,      \
                       routed_input, ids, n_pairs, R, ids_dst, expert_bounds, tile_bounds, tile_experts, out, ldo)
    // mapped calls with a workspace go through the prefill kernels (faster than the streaming kernel from about one pair
    // per expert on; MFQ_MOE_PREFILL_PAIRS raises the threshold for tuning)
    static const int min_pairs = tune_env("MFQ_MOE_PREFILL_PAIRS", 0);
    if (mfma && mapped && n_pairs >= static_cast<int64_t>(min_pairs) * E &&
        moe_prefill_eligible(pools, n_pools, E, K, routed_input, n_pairs, T, workspace, workspace_bytes))
        return moe_prefill_launch<false>(P, pools, n_pools, expert_pool, expert_local, E, out_per_expert, K, x, x_dtype, ldx,
                                         routed_input, n_pairs, T, R, ids_dst, expert_bounds, out, ldo, GluOut{0, 0, 0},
                                         workspace, st);
    // vector-ALU path: one block shape for every cohort, waves = min(16, fewest steps that keeps every wave busy)
    auto launch_valu = [&]() -> int {
        const int mb = mapped ? 4 : 1;
        int want = static_cast<int>(ceil_div(8192, static_cast<int64_t>(rbe) * (mapped ? ceil_div(n_pairs, mb) : n_pairs)));
        if (want < 1) want = 1;
        if (want > 8) want = 8;
        if (want > max_steps) want = max_steps;
        // with at most three steps per wave every load is in flight before the first use and the body needs no ring
        if (!mapped && want * 3 < max_steps && max_steps <= 24) want = static_cast<int>(ceil_div(max_steps, 3));
        const int nwaves = want;
        const bool ring = mapped || ceil_div(max_steps, nwaves) > 3;
        size_t lds = 0;
        for (int i = 0; i < n_pools; ++i) {
            P.spw[i] = static_cast<int>(ceil_div(P.k[i].nsteps, nwaves));
            const size_t need = gemv_lds_bytes(mb, P.spw[i], P.k[i].gs, nwaves);
            if (need > lds) lds = need;
        }
        MFQ_REQUIRE(lds <= 65536, MFQ_ERR_UNSUPPORTED, "moe_grouped_matmul: K=%d needs %zu bytes of LDS", K, lds);
        const dim3 grid(rbe, static_cast<unsigned>(tiles)), block(64 * nwaves);
        if (mapped) {
            if (x_dtype == MFQ_X_F16) MFQ_MOE_LAUNCH((moe_grouped_kernel<1, 4, true>), grid, block, lds);
            else MFQ_MOE_LAUNCH((moe_grouped_kernel<0, 4, true>), grid, block, lds);
        } else if (ring) {
            if (x_dtype == MFQ_X_F16) MFQ_MOE_LAUNCH((moe_grouped_kernel<1, 1, true>), grid, block, lds);
            else MFQ_MOE_LAUNCH((moe_grouped_kernel<0, 1, true>), grid, block, lds);
        } else {
            if (x_dtype == MFQ_X_F16) MFQ_MOE_LAUNCH((moe_grouped_kernel<1, 1, false>), grid, block, lds);
            else MFQ_MOE_LAUNCH((moe_grouped_kernel<0, 1, false>), grid, block, lds);
        }
        return check_launch("moe_grouped_matmul");
    };
    if (!mapped && units) {
        const int rc = moe_decode_launch(P, n_pools, max_steps, expert_pool, expert_local, E, out_per_expert, xp, x_dtype, ldx,
                                         routed_input, ids, n_pairs, n_pairs, R, 0, out, 0, ldo, st);
        if (rc >= 0) return rc;
    }
    if (mfma) {
        // row-blocks per wave: 4 while the grid still has a few thousand waves, else 1
        const int64_t live_tiles = mapped ? ceil_div(n_pairs, kMoeTileM) : n_pairs;
        static const int env_nb = tune_env("MFQ_MOE_NB", 0);
        const bool nb4 = env_nb ? env_nb == 4 : (live_tiles * rbe * max_steps >= 4 * 2048 && rbe >= 4);
        const int nb = nb4 ? 4 : 1;
        int nwaves = max_steps < 8 ? max_steps : 8;
        for (int i = 0; i < n_pools; ++i)
            if (!P.prefill[i]) P.spw[i] = static_cast<int>(ceil_div(P.k[i].nsteps, nwaves));
        const size_t lds = static_cast<size_t>(nwaves) * nb * 1024;
        const dim3 grid(static_cast<unsigned>(ceil_div(rbe, nb)), static_cast<unsigned>(tiles)), block(64 * nwaves);
        if (x_dtype == MFQ_X_F16) {
            if (nb4) MFQ_MOE_LAUNCH((moe_mfma_kernel<1, 4>), grid, block, lds);
            else MFQ_MOE_LAUNCH((moe_mfma_kernel<1, 1>), grid, block, lds);
        } else {
            if (nb4) MFQ_MOE_LAUNCH((moe_mfma_kernel<0, 4>), grid, block, lds);
            else MFQ_MOE_LAUNCH((moe_mfma_kernel<0, 1>), grid, block, lds);
        }
        return check_launch("moe_grouped_matmul");
    }
    return launch_valu();
#undef MFQ_MOE_LAUNCH
}

extern "C" int mfq_hip_moe_decode_matmul(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                                         const int32_t *expert_local, int E, int out_per_expert, int K, const void *x,
                                         int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                                         const mfq_nint_desc *shared_desc, const void *shared_weight, int swiglu,
                                         void *out, int out_dtype, int64_t ldo, mfq_stream_t stream) {
    MFQ_REQUIRE(pools && expert_pool && expert_local && x && ids && out, MFQ_ERR_INVALID, "moe_decode_matmul: null argument");
    MFQ_REQUIRE(T > 0 && R > 0 && E > 0, MFQ_ERR_INVALID, "MoE ids must be int32 [tokens, routes]");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "moe_decode_matmul: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(swiglu >= 0 && swiglu <= 2, MFQ_ERR_INVALID, "moe_decode_matmul: swiglu=%d (0 none, 1 SwiGLU, 2 GEGLU)", swiglu);
    MFQ_REQUIRE(!swiglu || out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16, MFQ_ERR_INVALID,
                "moe_decode_matmul: the fused SwiGLU stores bf16 or fp16, out_dtype=%d", out_dtype);
    MFQ_REQUIRE((shared_desc == nullptr) == (shared_weight == nullptr), MFQ_ERR_INVALID,
                "moe_decode_matmul: shared tensor without its descriptor (or the reverse)");
    const int n_slots = n_pools + (shared_desc ? 1 : 0);
    MFQ_REQUIRE(n_pools >= 1 && n_slots <= kMaxPools, MFQ_ERR_UNSUPPORTED, "moe_decode_matmul: %d cohorts (max %d)", n_slots,
                kMaxPools);
    MFQ_REQUIRE(out_per_expert % 16 == 0, MFQ_ERR_UNSUPPORTED, "moe_decode_matmul: out_per_expert %d must be a multiple of 16",
                out_per_expert);
    MFQ_REQUIRE(ldx >= K && ldo >= (swiglu ? out_per_expert / 2 : out_per_expert), MFQ_ERR_INVALID,
                "moe_decode_matmul: ldx/ldo smaller than the tensor");
    MoePools P;
    P.n = n_pools;
    int max_steps = 1;
    for (int i = 0; i < n_slots; ++i) {
        const mfq_nint_desc &d = i < n_pools ? pools[i].desc : *shared_desc;
        const void *wt = i < n_pools ? pools[i].weight : shared_weight;
        MFQ_REQUIRE(d.neuron_len == K && wt, MFQ_ERR_INVALID, "moe_decode_matmul: cohort %d has neuron_len %d, expected %d", i,
                    d.neuron_len, K);
        MFQ_REQUIRE(moe_prefill_unit(d) && 4 * d.rowblock_bytes < (1ll << 31), MFQ_ERR_UNSUPPORTED,
                    "moe_decode_matmul: no batch-1 kernel for NINT%d-%d", d.bits, d.gs);
        if (d.nsteps > max_steps) max_steps = d.nsteps;
        moe_fill_k(P.k[i], d);
        P.w[i] = static_cast<const uint8_t *>(wt);
        P.xg[i] = nullptr;
        P.prefill[i] = 0;
    }
    MFQ_REQUIRE(!shared_desc || shared_desc->out == out_per_expert, MFQ_ERR_UNSUPPORTED,
                "moe_decode_matmul: shared tensor has %d rows, the experts %d", shared_desc ? shared_desc->out : 0,
                out_per_expert);
    const int n_pairs = T * R, n_rows = n_pairs + (shared_desc ? T : 0);
    const int rc = moe_decode_launch(P, n_slots, max_steps, expert_pool, expert_local, E, out_per_expert,
                                     static_cast<const uint16_t *>(x), x_dtype, ldx, routed_input, ids, n_pairs, n_rows, R,
                                     swiglu, out, (out_dtype == MFQ_X_F16 ? 1 : 0) | (swiglu == 2 ? 2 : 0), ldo, as_stream(stream));
    if (rc < 0) return fail(MFQ_ERR_UNSUPPORTED, "moe_decode_matmul: shape outside the batch-1 kernel (rows %d, K %d)", n_rows, K);
    return rc;
}

extern "C" int mfq_hip_moe_decode_capable(const mfq_moe_pool *pools, int n_pools, int out_per_expert, int K,
                                          const mfq_nint_desc *shared_desc, int T, int R, int swiglu) {
    if (!pools || n_pools < 1 || T <= 0 || R <= 0 || out_per_expert % 16) return 0;
    const int n_slots = n_pools + (shared_desc ? 1 : 0);
    if (n_slots > kMaxPools) return 0;
    if (shared_desc && shared_desc->out != out_per_expert) return 0;
    MoePools P;
    P.n = n_pools;
    int max_steps = 1;
    for (int i = 0; i < n_slots; ++i) {
        const mfq_nint_desc &d = i < n_pools ? pools[i].desc : *shared_desc;
        if (d.neuron_len != K || !moe_prefill_unit(d) || 4 * d.rowblock_bytes >= (1ll << 31)) return 0;
        if (d.nsteps > max_steps) max_steps = d.nsteps;
        moe_fill_k(P.k[i], d);
    }
    MoeDecodeShape sh;
    return moe_decode_shape(P, n_slots, max_steps, out_per_expert, T * R + (shared_desc ? T : 0), swiglu, sh) ? 1 : 0;
}

extern "C" int mfq_hip_moe_glu(const float *gate_up, int64_t ld, int rows, int W, void *hidden, int out_dtype, int64_t ldh,
                               int activation, mfq_stream_t stream) {
    MFQ_REQUIRE(gate_up && hidden, MFQ_ERR_INVALID, "moe_glu: null argument");
    MFQ_REQUIRE(rows > 0 && W > 0 && ld >= 2 * W && ldh >= W, MFQ_ERR_INVALID, "moe_glu: bad shape");
    MFQ_REQUIRE(activation == MFQ_GLU_SILU || activation == MFQ_GLU_GELU, MFQ_ERR_INVALID, "moe_glu: activation=%d", activation);
    const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<int64_t>(rows) * W, 256));
    if (out_dtype == MFQ_X_F16)
        hipLaunchKernelGGL((moe_swiglu_kernel<1>), dim3(blocks), dim3(256), 0, as_stream(stream), gate_up, ld, rows, W,
                           static_cast<uint16_t *>(hidden), ldh, activation);
    else
        hipLaunchKernelGGL((moe_swiglu_kernel<0>), dim3(blocks), dim3(256), 0, as_stream(stream), gate_up, ld, rows, W,
                           static_cast<uint16_t *>(hidden), ldh, activation);
    return check_launch("moe_glu");
}

namespace mfq {
// dst row i = src row index[i] (gather), or dst row index[i] = src row i (scatter): rows of row_bytes bytes, a multiple
// of 4, as 32-bit words
__global__ __launch_bounds__(256) void moe_move_rows_kernel(const uint8_t *__restrict__ src, int64_t src_stride,
                                                            const int32_t *__restrict__ index, int row_bytes, int scatter,
                                                            uint8_t *__restrict__ dst, int64_t dst_stride) {
    const int i = blockIdx.x, j = index[i];
    const uint32_t *s = reinterpret_cast<const uint32_t *>(src + static_cast<int64_t>(scatter ? i : j) * src_stride);
    uint32_t *d = reinterpret_cast<uint32_t *>(dst + static_cast<int64_t>(scatter ? j : i) * dst_stride);
    for (int c = threadIdx.x; c < row_bytes / 4; c += blockDim.x) d[c] = s[c];
}
}  // namespace mfq

extern "C" int mfq_hip_moe_move_rows(const void *src, int64_t src_stride, const int32_t *index, int n, int row_bytes,
                                     int scatter, void *dst, int64_t dst_stride, mfq_stream_t stream) {
    MFQ_REQUIRE(src && index && dst, MFQ_ERR_INVALID, "moe_move_rows: null argument");
    MFQ_REQUIRE(n > 0 && row_bytes > 0 && row_bytes % 4 == 0 && src_stride % 4 == 0 && dst_stride % 4 == 0 &&
                    (reinterpret_cast<uintptr_t>(src) & 3) == 0 && (reinterpret_cast<uintptr_t>(dst) & 3) == 0,
                MFQ_ERR_INVALID, "moe_move_rows: rows must be made of whole aligned 32-bit words");
    hipLaunchKernelGGL(moe_move_rows_kernel, dim3(static_cast<unsigned>(n)), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t *>(src), src_stride, index, row_bytes, scatter ? 1 : 0,
                       static_cast<uint8_t *>(dst), dst_stride);
    return check_launch("moe_move_rows");
}

extern "C" int mfq_hip_moe_swiglu(const float *gate_up, int64_t ld, int rows, int W, void *hidden, int out_dtype,
                                  int64_t ldh, mfq_stream_t stream) {
    return mfq_hip_moe_glu(gate_up, ld, rows, W, hidden, out_dtype, ldh, MFQ_GLU_SILU, stream);
}

namespace mfq {
// The same sums, four neighbouring columns per thread (H % 4 == 0, 16-byte aligned rows): same order of the fused
// multiply-adds per element, a quarter of the load instructions.
__global__ __launch_bounds__(256) void moe_reduce4_kernel(const float *__restrict__ pair, const float *__restrict__ wts,
                                                          int T, int R, int H, const float *__restrict__ shared,
                                                          const float *__restrict__ gate_logits, float *__restrict__ out) {
    const int h4 = H >> 2;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(T) * h4) return;
    const int t = static_cast<int>(idx / h4), c = static_cast<int>(idx - static_cast<int64_t>(t) * h4) * 4;
    float4_t v = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int r = 0; r < R; ++r) {
        const int64_t p = static_cast<int64_t>(t) * R + r;
        const float w = wts[p];
        const float4_t q = *reinterpret_cast<const float4_t *>(pair + p * H + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = fmaf(w, q[i], v[i]);
    }
    if (shared) {
        const float g = gate_logits ? 1.f / (1.f + expf(-gate_logits[t])) : 1.f;
        const float4_t q = *reinterpret_cast<const float4_t *>(shared + static_cast<int64_t>(t) * H + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = fmaf(g, q[i], v[i]);
    }
    *reinterpret_cast<float4_t *>(out + static_cast<int64_t>(t) * H + c) = v;
}
}  // namespace mfq

extern "C" int mfq_hip_moe_weighted_reduce(const float *pair, const float *weights, int T, int R, int H,
                                           const float *shared, const float *gate_logits, float *out,
                                           mfq_stream_t stream) {
    MFQ_REQUIRE(pair && weights && out, MFQ_ERR_INVALID, "moe_weighted_reduce: null argument");
    MFQ_REQUIRE(T > 0 && R > 0 && H > 0, MFQ_ERR_INVALID, "moe_weighted_reduce: bad shape");
    const bool vec = H % 4 == 0 && ((reinterpret_cast<uintptr_t>(pair) | reinterpret_cast<uintptr_t>(out) |
                                     reinterpret_cast<uintptr_t>(shared)) & 15) == 0;
    if (vec) {
        const unsigned blocks4 = static_cast<unsigned>(ceil_div(static_cast<int64_t>(T) * (H / 4), 256));
        hipLaunchKernelGGL(moe_reduce4_kernel, dim3(blocks4), dim3(256), 0, as_stream(stream), pair, weights, T, R, H, shared,
                           gate_logits, out);
        return check_launch("moe_weighted_reduce");
    }
    const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<int64_t>(T) * H, 256));
    hipLaunchKernelGGL(moe_reduce_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), pair, weights, T, R, H, shared,
                       gate_logits, out);
    return check_launch("moe_weighted_reduce");
}
