// MoE: router top-k, device-side expert bucketing (parallel prefix sum), the expert-grouped
// mixed-bit matmul ("mul_mat_id"), SwiGLU and the weighted reduce.
#include <float.h>

#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_body.hpp"

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
    int selected[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) selected[i] = -1;
    float mine = 0.f;  // lane r keeps the weight of rank r
    for (int rank = 0; rank < k; ++rank) {
        float bs = -INFINITY, bw = -INFINITY;
        int bi = INT_MAX;
        for (int e = lane; e < E; e += 64) {
            bool taken = false;
#pragma unroll
            for (int p = 0; p < 16; ++p) taken |= (p < rank && selected[p] == e);
            if (taken) continue;
            const float raw = raw_at(e);
            float wv;
            if (mode == MFQ_TOPK_DELAYED_SOFTMAX) wv = raw;
            else if (mode == MFQ_TOPK_SIGMOID) wv = 1.f / (1.f + expf(-raw));
            else if (mode == MFQ_TOPK_SQRT_SOFTPLUS) wv = sqrtf(raw > 20.f ? raw : log1pf(expf(raw)));
            else wv = expf(raw - smax) / ssum;
            const float sc = wv + (bias ? bias[e] : 0.f);
            if (sc > bs || (sc == bs && e < bi)) { bs = sc; bw = wv; bi = e; }
        }
        wave_argmax(bs, bw, bi);
        selected[rank] = bi;
        if (lane == rank) mine = bw;
        if (lane == 0) ids[static_cast<int64_t>(t) * k + rank] = bi;
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

// ---- expert map ------------------------------------------------------------------------------
// counts: one block per expert counts its pairs (no atomics, nothing to pre-clear).
__global__ __launch_bounds__(256) void moe_count_kernel(const int32_t *__restrict__ ids, int n_pairs,
                                                        int32_t *__restrict__ counts) {
    __shared__ int red[4];
    const int e = blockIdx.x, tid = threadIdx.x;
    int c = 0;
    for (int p = tid; p < n_pairs; p += 256) c += (ids[p] == e);
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
    for (int p0 = 0; p0 < n_pairs; p0 += 256) {
        const int p = p0 + tid;
        const bool hit = p < n_pairs && ids[p] == e;
        const unsigned long long ball = __ballot(hit);
        const int before = __popcll(ball & ((1ull << lane) - 1ull));
        if (lane == 0) wsum[wave] = __popcll(ball);
        __syncthreads();
        int off = 0;
        for (int wv = 0; wv < wave; ++wv) off += wsum[wv];
        if (hit) ids_dst[base + off + before] = p;
        __syncthreads();
        if (tid == 0) base += wsum[0] + wsum[1] + wsum[2] + wsum[3];
        __syncthreads();
    }
}

// ---- expert-grouped matmul ---------------------------------------------------------------------
constexpr int kMaxPools = 8;
struct MoePools {
    NintK k[kMaxPools];
    const uint8_t *w[kMaxPools];
    int spw[kMaxPools];
    int n;
};

// A tile is up to MB (token, route) pairs of one expert.  Without a route map every pair is its
// own tile (MB = 1, decode); with one, tile t of the map holds pairs ids_dst[lo .. lo+MB).
template <int XF16, int MB>
__global__ __launch_bounds__(1024) void moe_grouped_kernel(MoePools P, const int32_t *__restrict__ expert_pool,
                                                           const int32_t *__restrict__ expert_local, int E,
                                                           int out_per_expert, const uint16_t *__restrict__ x,
                                                           int64_t ldx, int routed_input, const int32_t *__restrict__ ids,
                                                           int n_pairs, int R, const int32_t *__restrict__ ids_dst,
                                                           const int32_t *__restrict__ expert_bounds,
                                                           const int32_t *__restrict__ tile_bounds,
                                                           const int32_t *__restrict__ tile_experts,
                                                           float *__restrict__ out, int64_t ldo) {
    extern __shared__ uint32_t lds[];
    const int tile = blockIdx.x;
    int e;
    int pairs[MB];
    if (ids_dst == nullptr) {
        e = ids[tile];
        pairs[0] = tile;
#pragma unroll
        for (int m = 1; m < MB; ++m) pairs[m] = -1;
    } else {
        if (tile >= tile_bounds[E]) return;
        e = tile_experts[tile];
        const int lo = expert_bounds[e] + (tile - tile_bounds[e]) * MB, hi = expert_bounds[e + 1];
#pragma unroll
        for (int m = 0; m < MB; ++m) pairs[m] = lo + m < hi ? ids_dst[lo + m] : -1;
    }
    const uint16_t *xr[MB];
    float *yr[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const int p = pairs[m];
        xr[m] = p >= 0 ? x + static_cast<int64_t>(routed_input ? p : p / R) * ldx : nullptr;
        yr[m] = p >= 0 ? out + static_cast<int64_t>(p) * ldo : nullptr;
    }
    const int rbl = blockIdx.y;  // row-block inside the expert
    if (e < 0 || e >= E || expert_pool[e] < 0) {  // invalid expert id: defined as a zero row
        const int row = rbl * 16 + (threadIdx.x & 15);
        if (threadIdx.x < 16 && row < out_per_expert)
#pragma unroll
            for (int m = 0; m < MB; ++m)
                if (yr[m]) yr[m][row] = 0.f;
        return;
    }
    const int pool = expert_pool[e];
    const int row_base = expert_local[e] * out_per_expert;
    const int rb = row_base / 16 + rbl;
    const NintK &k = P.k[pool];
    const uint8_t *w = P.w[pool];
    const int spw = P.spw[pool];
#define MFQ_MOE_CASE(B, G)                                                                                    \
    if (k.bits == B && k.gs == G) {                                                                           \
        nint_paired_body<B, G, XF16, MB>(k, w, rb, 1, row_base, out_per_expert, xr, yr, spw, lds);            \
        return;                                                                                               \
    }
    if (k.kind == 1) {
        MFQ_MOE_CASE(4, 24) MFQ_MOE_CASE(3, 24) MFQ_MOE_CASE(2, 16) MFQ_MOE_CASE(4, 32) MFQ_MOE_CASE(4, 16)
        MFQ_MOE_CASE(4, 48) MFQ_MOE_CASE(2, 32)
    }
#undef MFQ_MOE_CASE
    nint_generic_body<XF16, MB>(k, w, rb, row_base, out_per_expert, xr, yr, spw, lds);
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
                                                         uint16_t *__restrict__ hidden, int64_t ldh) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<int64_t>(rows) * W) return;
    const int row = static_cast<int>(idx / W), col = static_cast<int>(idx - static_cast<int64_t>(row) * W);
    const float g = gu[row * ld + col], u = gu[row * ld + W + col];
    const float v = g / (1.f + expf(-g)) * u;
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

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_moe_topk(const float *logits, const float *bias, int T, int E, int k, int mode, int normalize,
                                float norm_floor, float scale, int32_t *ids, float *weights, mfq_stream_t stream) {
    MFQ_REQUIRE(logits && ids && weights, MFQ_ERR_INVALID, "moe_topk: null argument");
    MFQ_REQUIRE(T > 0 && E > 0, MFQ_ERR_INVALID, "logits dimensions must be nonzero");
    MFQ_REQUIRE(k >= 1 && k <= 16 && k <= E, MFQ_ERR_INVALID, "top_k must be in [1, min(16, experts)]");
    MFQ_REQUIRE(mode >= 0 && mode <= 3, MFQ_ERR_INVALID, "moe_topk: unknown mode %d", mode);
    MFQ_REQUIRE(!(normalize && mode == MFQ_TOPK_DELAYED_SOFTMAX), MFQ_ERR_INVALID,
                "selected-weight normalization and delayed softmax are mutually exclusive");
    hipLaunchKernelGGL(moe_topk_kernel, dim3(static_cast<unsigned>(ceil_div(T, 4))), dim3(256), 0, as_stream(stream), logits,
                       bias, T, E, k, mode, normalize, norm_floor, scale, ids, weights);
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
static constexpr int kMoeTileM = 4;

extern "C" int mfq_hip_moe_tile_m(void) { return kMoeTileM; }

extern "C" int mfq_hip_moe_grouped_matmul(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                                          const int32_t *expert_local, int E, int out_per_expert, int K, const void *x,
                                          int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                                          const int32_t *ids_dst, const int32_t *expert_bounds,
                                          const int32_t *tile_bounds, const int32_t *tile_experts, float *out,
                                          int64_t ldo, mfq_stream_t stream) {
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
    const int mb = mapped ? kMoeTileM : 1;
    MoePools P;
    P.n = n_pools;
    // one block shape for every cohort: waves = min(16, fewest steps that keeps every wave busy)
    int max_steps = 1;
    for (int i = 0; i < n_pools; ++i) {
        MFQ_REQUIRE(pools[i].desc.neuron_len == K && pools[i].weight, MFQ_ERR_INVALID,
                    "moe_grouped_matmul: cohort %d has neuron_len %d, expected %d", i, pools[i].desc.neuron_len, K);
        if (pools[i].desc.nsteps > max_steps) max_steps = pools[i].desc.nsteps;
    }
    const int rbe = out_per_expert / 16;
    const int64_t tiles = mapped ? ceil_div(n_pairs, mb) + E : n_pairs;
    int want = static_cast<int>(ceil_div(8192, static_cast<int64_t>(rbe) * (mapped ? ceil_div(n_pairs, mb) : n_pairs)));
    if (want < 1) want = 1;
    if (want > 16) want = 16;
    if (want > max_steps) want = max_steps;
    const int nwaves = want;
    size_t lds = 0;
    for (int i = 0; i < n_pools; ++i) {
        const mfq_nint_desc &d = pools[i].desc;
        NintK &k = P.k[i];
        k.bits = d.bits; k.sub_bits = d.sub_bits; k.gs = d.gs; k.out = d.out; k.neuron_len = d.neuron_len; k.ng = d.ng;
        k.kind = d.kind; k.dwords = d.dwords; k.tail = d.tail_bytes; k.nsteps = d.nsteps; k.n_rowblocks = d.n_rowblocks;
        k.step_bytes = d.step_bytes; k.rowblock_bytes = d.rowblock_bytes; k.anchors_off = d.anchors_off;
        P.w[i] = static_cast<const uint8_t *>(pools[i].weight);
        P.spw[i] = static_cast<int>(ceil_div(d.nsteps, nwaves));
        const size_t need = gemv_lds_bytes(mb, P.spw[i], d.gs, nwaves);
        if (need > lds) lds = need;
    }
    MFQ_REQUIRE(lds <= 65536, MFQ_ERR_UNSUPPORTED, "moe_grouped_matmul: K=%d needs %zu bytes of LDS", K, lds);
    hipStream_t st = as_stream(stream);
    const dim3 grid(static_cast<unsigned>(tiles), rbe), block(64 * nwaves);
    const uint16_t *xp = static_cast<const uint16_t *>(x);
    if (mapped) {
        MFQ_REQUIRE(expert_bounds && tile_bounds && tile_experts, MFQ_ERR_INVALID,
                    "moe_grouped_matmul: route map without its bounds / tile tables");
        hipLaunchKernelGGL(moe_zero_invalid_kernel, dim3(n_pairs), dim3(256), 0, st, ids, n_pairs, E, expert_pool,
                           out_per_expert, out, ldo);
        if (x_dtype == MFQ_X_F16)
            hipLaunchKernelGGL((moe_grouped_kernel<1, kMoeTileM>), grid, block, lds, st, P, expert_pool, expert_local, E,
                               out_per_expert, xp, ldx, routed_input, ids, n_pairs, R, ids_dst, expert_bounds, tile_bounds,
                               tile_experts, out, ldo);
        else
            hipLaunchKernelGGL((moe_grouped_kernel<0, kMoeTileM>), grid, block, lds, st, P, expert_pool, expert_local, E,
                               out_per_expert, xp, ldx, routed_input, ids, n_pairs, R, ids_dst, expert_bounds, tile_bounds,
                               tile_experts, out, ldo);
    } else {
        const int32_t *np = nullptr;
        if (x_dtype == MFQ_X_F16)
            hipLaunchKernelGGL((moe_grouped_kernel<1, 1>), grid, block, lds, st, P, expert_pool, expert_local, E,
                               out_per_expert, xp, ldx, routed_input, ids, n_pairs, R, np, np, np, np, out, ldo);
        else
            hipLaunchKernelGGL((moe_grouped_kernel<0, 1>), grid, block, lds, st, P, expert_pool, expert_local, E,
                               out_per_expert, xp, ldx, routed_input, ids, n_pairs, R, np, np, np, np, out, ldo);
    }
    return check_launch("moe_grouped_matmul");
}

extern "C" int mfq_hip_moe_swiglu(const float *gate_up, int64_t ld, int rows, int W, void *hidden, int out_dtype,
                                  int64_t ldh, mfq_stream_t stream) {
    MFQ_REQUIRE(gate_up && hidden, MFQ_ERR_INVALID, "moe_swiglu: null argument");
    MFQ_REQUIRE(rows > 0 && W > 0 && ld >= 2 * W && ldh >= W, MFQ_ERR_INVALID, "moe_swiglu: bad shape");
    const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<int64_t>(rows) * W, 256));
    if (out_dtype == MFQ_X_F16)
        hipLaunchKernelGGL((moe_swiglu_kernel<1>), dim3(blocks), dim3(256), 0, as_stream(stream), gate_up, ld, rows, W,
                           static_cast<uint16_t *>(hidden), ldh);
    else
        hipLaunchKernelGGL((moe_swiglu_kernel<0>), dim3(blocks), dim3(256), 0, as_stream(stream), gate_up, ld, rows, W,
                           static_cast<uint16_t *>(hidden), ldh);
    return check_launch("moe_swiglu");
}

extern "C" int mfq_hip_moe_weighted_reduce(const float *pair, const float *weights, int T, int R, int H,
                                           const float *shared, const float *gate_logits, float *out,
                                           mfq_stream_t stream) {
    MFQ_REQUIRE(pair && weights && out, MFQ_ERR_INVALID, "moe_weighted_reduce: null argument");
    MFQ_REQUIRE(T > 0 && R > 0 && H > 0, MFQ_ERR_INVALID, "moe_weighted_reduce: bad shape");
    const unsigned blocks = static_cast<unsigned>(ceil_div(static_cast<int64_t>(T) * H, 256));
    hipLaunchKernelGGL(moe_reduce_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), pair, weights, T, R, H, shared,
                       gate_logits, out);
    return check_launch("moe_weighted_reduce");
}
