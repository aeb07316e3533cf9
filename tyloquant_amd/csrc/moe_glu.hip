// MoE gate/up projection of a mapped call with the GLU fused into the matmul's epilogue: the prefill kernels of
// moe_prefill.hpp with their act(gate) * up output.
#include "moe_prefill.hpp"

using namespace mfq;

namespace mfq {
// rows of pairs whose expert id is out of range are not in any chunk: clear them
__global__ void moe_zero_invalid16_kernel(const int32_t *__restrict__ ids, int n_pairs, int E,
                                          const int32_t *__restrict__ expert_pool, int width, uint16_t *__restrict__ out,
                                          int64_t ldo) {
    const int p = blockIdx.x;
    const int e = ids[p];
    if (e >= 0 && e < E && expert_pool[e] >= 0) return;
    for (int c = threadIdx.x; c < width; c += blockDim.x) out[static_cast<int64_t>(p) * ldo + c] = 0;
}
}  // namespace mfq

extern "C" int mfq_hip_moe_grouped_glu_ws(const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                                          const int32_t *expert_local, int E, int out_per_expert, int K, const void *x,
                                          int x_dtype, int64_t ldx, int routed_input, const int32_t *ids, int T, int R,
                                          const int32_t *ids_dst, const int32_t *expert_bounds, int activation,
                                          void *hidden, int out_dtype, int64_t ldh, void *workspace,
                                          size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(pools && expert_pool && expert_local && x && ids && hidden, MFQ_ERR_INVALID, "moe_grouped_glu: null argument");
    MFQ_REQUIRE(n_pools >= 1 && n_pools <= kMaxPools, MFQ_ERR_UNSUPPORTED, "moe_grouped_glu: %d cohorts (max %d)", n_pools,
                kMaxPools);
    MFQ_REQUIRE(T > 0 && R > 0 && E > 0, MFQ_ERR_INVALID, "MoE ids must be int32 [tokens, routes]");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "moe_grouped_glu: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(out_dtype == MFQ_X_BF16 || out_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "moe_grouped_glu: out_dtype=%d", out_dtype);
    MFQ_REQUIRE(activation == MFQ_GLU_SILU || activation == MFQ_GLU_GELU, MFQ_ERR_INVALID, "moe_grouped_glu: activation=%d",
                activation);
    const int W = out_per_expert / 2;
    MFQ_REQUIRE(out_per_expert > 0 && out_per_expert % 32 == 0, MFQ_ERR_UNSUPPORTED,
                "moe_grouped_glu: out_per_expert %d must be two halves of whole 16-neuron row-blocks", out_per_expert);
    MFQ_REQUIRE(ldx >= K && ldh >= W, MFQ_ERR_INVALID, "moe_grouped_glu: ldx/ldh smaller than the tensor");
    MFQ_REQUIRE(ids_dst && expert_bounds, MFQ_ERR_UNSUPPORTED, "moe_grouped_glu: needs the route map of a mapped call");
    const int n_pairs = T * R;
    MoePools P;
    P.n = n_pools;
    bool ok = K >= 8 && K % 8 == 0 && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    for (int i = 0; i < n_pools; ++i) {
        const mfq_nint_desc &d = pools[i].desc;
        MFQ_REQUIRE(d.neuron_len == K && pools[i].weight, MFQ_ERR_INVALID,
                    "moe_grouped_glu: cohort %d has neuron_len %d, expected %d", i, d.neuron_len, K);
        moe_fill_k(P.k[i], d);
        P.w[i] = static_cast<const uint8_t *>(pools[i].weight);
        P.xg[i] = nullptr;
        P.spw[i] = 0;
        P.prefill[i] = 0;
        // a wave's buffer window spans from its gate row-blocks to its up row-blocks
        ok = ok && (static_cast<int64_t>(W / 16) + 4) * d.rowblock_bytes < (1ll << 31);
    }
    MFQ_REQUIRE(ok && moe_prefill_eligible(pools, n_pools, E, K, routed_input, n_pairs, T, workspace, workspace_bytes),
                MFQ_ERR_UNSUPPORTED, "moe_grouped_glu: these cohorts, activations or workspace keep the call off the prefill kernels");
    hipStream_t st = as_stream(stream);
    hipLaunchKernelGGL(moe_zero_invalid16_kernel, dim3(n_pairs), dim3(256), 0, st, ids, n_pairs, E, expert_pool, W,
                       static_cast<uint16_t *>(hidden), ldh);
    const GluOut glu{W / 16, activation == MFQ_GLU_GELU ? 1 : 0, out_dtype == MFQ_X_F16 ? 1 : 0};
    return moe_prefill_launch<true>(P, pools, n_pools, expert_pool, expert_local, E, out_per_expert, K, x, x_dtype, ldx,
                                    routed_input, n_pairs, T, R, ids_dst, expert_bounds, hidden, ldh, glu, workspace, st);
}
