// Mapped MoE calls through the prefill body: the chunk lists, the kernels of the three register groups and their launch,
// shared by the grouped matmul and by its form with the fused act(gate) * up output.
#pragma once
#include "common.hpp"
#include "gemv_common.hpp"
#include "tune.hpp"
#include "nint_mfma.hpp"
#include "nint_prefill.hpp"

namespace mfq {

constexpr int kMaxPools = 8;
struct MoePools {
    NintK k[kMaxPools];
    const uint8_t *w[kMaxPools];
    const uint32_t *xg[kMaxPools];  // prefill path: group sums of the activations for this cohort's groupsize
    int spw[kMaxPools];
    int n;
    int prefill[kMaxPools];  // cohort is taken by another kernel of this call (the streaming kernel skips it)
};

constexpr int kMoeTileM = 16;  // (token, route) pairs of one expert per tile of the route map

// Prefill path for the mapped call.  The pairs of an expert are cut into chunks of up to 128; a block takes one chunk
// against a tile of the expert's neurons, so that the weights are unpacked once per chunk.  The number of 16-row tiles of
// a chunk is a compile-time constant of the body it runs (no tile without rows is read or multiplied); the bodies are
// grouped by their register need into three kernels: 1-2 and 3-4 tiles x 512 neurons (four row-blocks per wave), 5-8
// tiles x 256 neurons (two per wave).  moe_chunk_list_kernel leaves one list of chunks per group.
constexpr int kMoeChunkRows = 128, kMoeGroups = 3;
__host__ __device__ constexpr int moe_group_rows(int grp) { return grp == 0 ? 32 : grp == 1 ? 64 : 128; }
__host__ __device__ constexpr int moe_group_nb(int grp) { return grp == 2 ? 2 : 4; }
__host__ __device__ constexpr int moe_group_of(int rows) { return rows <= 32 ? 0 : rows <= 64 ? 1 : 2; }
// weight unit buffers per row-block and activation tiles of a body of mt row tiles: up to two tiles keep a whole step
// of weights and activations in flight in registers (the weight stream sets the pace); from three on the activations
// are copied straight into a ring of four LDS buffers where the groups are whole 16-byte chunks and the ring fits
__host__ __device__ constexpr int moe_body_pf(int mt) { return mt <= 2 || mt >= 5 ? 4 : 2; }
__host__ __device__ constexpr int moe_body_xd(int mt, int gs, int d) {
    if (mt <= 2) return mt == 1 ? 4 : 2;
    if (gs % 8 == 0 && prefill_lds_bytes(mt * 16, gs, 4) + 1024 <= kMaxDynamicLds) return 0;
    return mt <= 4 ? 2 : (d >= 5 ? 1 : 2);
}
__host__ __device__ constexpr size_t moe_body_lds(int mt, int gs) {
    return prefill_lds_bytes(mt * 16, gs, moe_body_xd(mt, gs, 1) == 0 ? 4 : 2);
}

// lists: [0..2] chunks per group, [8 + 2 * (grp * cap + i)] = {expert, first pair} of chunk i of group grp.  One wave per
// group walks the experts in order (deterministic lists).
static __global__ __launch_bounds__(256) void moe_chunk_list_kernel(const int32_t *__restrict__ expert_bounds,
                                                             const int32_t *__restrict__ expert_pool, int E,
                                                             int32_t *__restrict__ lists, int cap) {
    const int grp = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (grp >= kMoeGroups) return;
    int32_t *items = lists + 8 + 2 * grp * cap;
    int total = 0;
    for (int base = 0; base < E; base += 64) {
        const int e = base + lane;
        int n = 0, lo = 0;
        if (e < E && expert_pool[e] >= 0) {
            lo = expert_bounds[e];
            n = expert_bounds[e + 1] - lo;
        }
        const int full = n / kMoeChunkRows, rem = n - full * kMoeChunkRows;
        const bool rem_mine = rem > 0 && moe_group_of(rem) == grp;
        const int mine = (grp == 2 ? full : 0) + (rem_mine ? 1 : 0);
        int inc = mine;
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(inc, o, 64);
            if (lane >= o) inc += v;
        }
        int pos = total + inc - mine;
        if (grp == 2)
            for (int c = 0; c < full; ++c, ++pos)
                if (pos < cap) { items[2 * pos] = e; items[2 * pos + 1] = lo + kMoeChunkRows * c; }
        if (rem_mine && pos < cap) { items[2 * pos] = e; items[2 * pos + 1] = lo + kMoeChunkRows * full; }
        total += __shfl(inc, 63, 64);
    }
    if (lane == 0) lists[grp] = min(total, cap);
}

// Block b of group GRP: XCD b % 8 (blocks go to the XCDs in turn) takes chunk (b / 8 / ncol) * 8 + b % 8, neuron
// tile (b / 8) % ncol -- the blocks that share a chunk's activation rows run next to each other on one XCD and find
// them in its L2.  x16 / xscale / P.xg are indexed by the source row of a pair (n_src rows).
// GLU: out_per_expert = 2 W neurons, gate rows first; the block takes NB / 2 gate row-blocks per wave with their up
// row-blocks and stores act(gate) * up as 16-bit values [pairs, W] (out is then uint16_t, ldo in halves).
template <int GRP, bool GLU>
__global__ __launch_bounds__(512) void moe_prefill_kernel(MoePools P, const int32_t *__restrict__ expert_pool,
                                                          const int32_t *__restrict__ expert_local, int out_per_expert,
                                                          const uint16_t *__restrict__ x16, int Kp, int n_src,
                                                          const float *__restrict__ xscale, int routed_input, int R,
                                                          const int32_t *__restrict__ ids_dst,
                                                          const int32_t *__restrict__ expert_bounds,
                                                          const int32_t *__restrict__ lists, int cap, int ncol,
                                                          float *__restrict__ out, int64_t ldo, GluOut glu) {
    constexpr int BMR = moe_group_rows(GRP), NB = moe_group_nb(GRP), NBG = GLU ? NB / 2 : NB;
    extern __shared__ __attribute__((aligned(16))) uint32_t plds[];
    const int b = blockIdx.x, j = b >> 3;
    const int item = (j / ncol) * 8 + (b & 7), col = j % ncol;
    if (item >= lists[GRP]) return;
    const int e = lists[8 + 2 * (GRP * cap + item)], lo = lists[8 + 2 * (GRP * cap + item) + 1];
    const int hi = min(expert_bounds[e + 1], lo + BMR);
    const int pool = expert_pool[e];
    int *srcv = reinterpret_cast<int *>(plds), *dstv = srcv + BMR;
    uint16_t *xt = reinterpret_cast<uint16_t *>(plds + 2 * BMR);
    if (threadIdx.x < BMR) {
        const int p = lo + static_cast<int>(threadIdx.x) < hi ? ids_dst[lo + threadIdx.x] : -1;
        const int pp = p >= 0 ? p : ids_dst[lo];
        dstv[threadIdx.x] = p;
        srcv[threadIdx.x] = routed_input ? pp : pp / R;
    }
    __syncthreads();
    const int rbe = out_per_expert / 16, rb_first = expert_local[e] * rbe;
    const int rb_base = rb_first + col * 8 * NBG;
    const int rb_end = rb_first + (GLU ? rbe / 2 : rbe), ncols = GLU ? out_per_expert / 2 : out_per_expert;
    const NintK &k = P.k[pool];
    const MappedRows rows{srcv, dstv, n_src};
    const int mt = (hi - lo + 15) / 16;  // block-uniform
#define MFQ_MOE_BODY(UNIT, B, G, MTV)                                                                                 \
    nint_prefill_body<UNIT<B, G>, MTV, NB, 1, 8, MappedRows, moe_body_pf(MTV), moe_body_xd(MTV, G, UNIT<B, G>::D), GLU>( \
        k, P.w[pool], rb_base, rb_end, rb_first, ncols, x16, Kp, xscale, P.xg[pool], rows, out, ldo, xt, 0, -1, glu)
#define MFQ_MOE_PREFILL(UNIT, B, G)                                                                                   \
    if (k.bits == B && k.gs == G) {                                                                                   \
        if constexpr (GRP == 0) {                                                                                     \
            if (mt <= 1) MFQ_MOE_BODY(UNIT, B, G, 1);                                                                 \
            else MFQ_MOE_BODY(UNIT, B, G, 2);                                                                         \
        } else if constexpr (GRP == 1) {                                                                              \
            if (mt <= 3) MFQ_MOE_BODY(UNIT, B, G, 3);                                                                 \
            else MFQ_MOE_BODY(UNIT, B, G, 4);                                                                         \
        } else {                                                                                                      \
            if (mt <= 5) MFQ_MOE_BODY(UNIT, B, G, 5);                                                                 \
            else if (mt <= 6) MFQ_MOE_BODY(UNIT, B, G, 6);                                                            \
            else MFQ_MOE_BODY(UNIT, B, G, 8);                                                                         \
        }                                                                                                             \
    }
    if (k.kind == 1) {
        MFQ_MOE_PREFILL(PairedUnit, 4, 24)
        else MFQ_MOE_PREFILL(PairedUnit, 3, 24)
        else MFQ_MOE_PREFILL(PairedUnit, 2, 16)
        else MFQ_MOE_PREFILL(PairedUnit, 4, 32)
        else MFQ_MOE_PREFILL(PairedUnit, 4, 16)
        else MFQ_MOE_PREFILL(PairedUnit, 4, 48)
        else MFQ_MOE_PREFILL(PairedUnit, 2, 32)
    } else {
        MFQ_MOE_PREFILL(GenericUnit, 5, 28)
    }
#undef MFQ_MOE_PREFILL
#undef MFQ_MOE_BODY
}

int x_prep_multi(const void *x, int x_dtype, int64_t ldx, int M, int K, int Kp, void *x16, float *xscale, int n_groups,
                 const int *gs, const int *nsteps, uint32_t *const *xg, hipStream_t st);

// prefill workspace: x16 [rows, Kp] | xscale [rows] | one group-sum table per distinct groupsize of the paired cohorts
static size_t moe_align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }
// Row length of the fp16 activations: whole 16-group steps of every cohort (a tile copied straight into LDS never crosses
// a row end), a multiple of 32.
static int moe_kp(const mfq_moe_pool *pools, int n_pools, int K) {
    int64_t k = K;
    for (int i = 0; i < n_pools; ++i) {
        const int64_t whole = static_cast<int64_t>(pools[i].desc.nsteps) * 16 * pools[i].desc.gs;
        if (whole > k) k = whole;
    }
    return static_cast<int>(ceil_div(k, 32) * 32);
}
constexpr int kMoeChunkCap = 16384;  // chunks per class a call can list
constexpr size_t kMoeListBytes = (8 + 2 * static_cast<size_t>(kMoeGroups) * kMoeChunkCap) * 4;
static bool moe_prefill_unit(const mfq_nint_desc &d) { return d.kind == 1 || (d.bits == 5 && d.gs == 28); }
static bool moe_prefill_pools(const mfq_moe_pool *pools, int n_pools) {  // every cohort has a prefill unit
    for (int i = 0; i < n_pools; ++i)
        if (!moe_prefill_unit(pools[i].desc) || 4 * pools[i].desc.rowblock_bytes >= (1ll << 31)) return false;
    return true;
}

static void moe_fill_k(NintK &k, const mfq_nint_desc &d) {
    k.bits = d.bits; k.sub_bits = d.sub_bits; k.gs = d.gs; k.out = d.out; k.neuron_len = d.neuron_len; k.ng = d.ng;
    k.kind = d.kind; k.dwords = d.dwords; k.tail = d.tail_bytes; k.nsteps = d.nsteps; k.n_rowblocks = d.n_rowblocks;
    k.step_bytes = d.step_bytes; k.rowblock_bytes = d.rowblock_bytes; k.anchors_off = d.anchors_off;
}


// prefill workspace of x_rows activation rows; 0 when a cohort has no prefill body
static size_t moe_prefill_workspace(const mfq_moe_pool *pools, int n_pools, int K, int x_rows) {
    if (!pools || n_pools < 1 || n_pools > kMaxPools || x_rows < 1 || !moe_prefill_pools(pools, n_pools)) return 0;
    size_t total = moe_align256(static_cast<size_t>(x_rows) * moe_kp(pools, n_pools, K) * 2) +
                   moe_align256(static_cast<size_t>(x_rows) * 4) + moe_align256(kMoeListBytes);
    for (int i = 0; i < n_pools; ++i) {
        bool seen = false;
        for (int j = 0; j < i; ++j) seen = seen || pools[j].desc.gs == pools[i].desc.gs;
        if (!seen) total += moe_align256(static_cast<size_t>(x_rows) * pools[i].desc.nsteps * 64);
    }
    return total;
}

// A mapped call can take the prefill kernels: every cohort has a body, the chunk lists and the fp16 activations (one
// buffer window) are within their limits, the workspace is large enough.
static bool moe_prefill_eligible(const mfq_moe_pool *pools, int n_pools, int E, int K, int routed_input, int n_pairs, int T,
                                 const void *workspace, size_t workspace_bytes) {
    const int x_rows = routed_input ? n_pairs : T;
    const int cap = E + n_pairs / kMoeChunkRows + 1;
    return workspace && moe_prefill_pools(pools, n_pools) && cap <= kMoeChunkCap &&
           static_cast<int64_t>(x_rows) * moe_kp(pools, n_pools, K) * 2 < (1ll << 32) &&
           workspace_bytes >= moe_prefill_workspace(pools, n_pools, K, x_rows);
}

// Chunk lists, activation prep (fp16 rows, scales, one group-sum table per distinct groupsize) and the three group
// launches.  P holds the cohorts (moe_fill_k, weights); out: float [pairs, ldo], or with GLU uint16_t [pairs, ldo].
template <bool GLU>
static int moe_prefill_launch(MoePools &P, const mfq_moe_pool *pools, int n_pools, const int32_t *expert_pool,
                              const int32_t *expert_local, int E, int out_per_expert, int K, const void *x, int x_dtype,
                              int64_t ldx, int routed_input, int n_pairs, int T, int R, const int32_t *ids_dst,
                              const int32_t *expert_bounds, void *out, int64_t ldo, GluOut glu, void *workspace,
                              hipStream_t st) {
    const int x_rows = routed_input ? n_pairs : T;
    const int Kp = moe_kp(pools, n_pools, K);
    const int cap = E + n_pairs / kMoeChunkRows + 1;  // chunks of a group: at most one partial chunk per expert
    const int rbe = out_per_expert / 16;
    uint8_t *p = static_cast<uint8_t *>(workspace);
    uint16_t *x16 = reinterpret_cast<uint16_t *>(p);
    p += moe_align256(static_cast<size_t>(x_rows) * Kp * 2);
    float *xscale = reinterpret_cast<float *>(p);
    p += moe_align256(static_cast<size_t>(x_rows) * 4);
    int32_t *lists = reinterpret_cast<int32_t *>(p);
    p += moe_align256(kMoeListBytes);
    hipLaunchKernelGGL(moe_chunk_list_kernel, dim3(1), dim3(256), 0, st, expert_bounds, expert_pool, E, lists, cap);
    // one activation prep launch leaves a group-sum table per distinct groupsize (at most four per launch)
    int ng = 0, g_gs[4], g_steps[4];
    size_t glds[kMoeGroups] = {0, 0, 0};  // activation buffers of a group: the largest need among its bodies and the cohorts
    uint32_t *g_xg[4];
    for (int i = 0; i < n_pools; ++i) {
        P.prefill[i] = 1;
        P.xg[i] = nullptr;
        for (int j = 0; j < i; ++j)
            if (P.k[j].gs == P.k[i].gs) P.xg[i] = P.xg[j];
        if (!P.xg[i]) {
            uint32_t *xg = reinterpret_cast<uint32_t *>(p);
            p += moe_align256(static_cast<size_t>(x_rows) * P.k[i].nsteps * 64);
            g_gs[ng] = P.k[i].gs; g_steps[ng] = P.k[i].nsteps; g_xg[ng] = xg;
            if (++ng == 4) {
                const int rc = x_prep_multi(x, x_dtype, ldx, x_rows, K, Kp, x16, xscale, ng, g_gs, g_steps, g_xg, st);
                if (rc) return rc;
                ng = 0;
            }
            P.xg[i] = xg;
        }
        for (int mt = 1; mt <= 8; ++mt) {
            const int g = moe_group_of(mt * 16);
            const size_t need = moe_body_lds(mt, P.k[i].gs);
            if (need > glds[g]) glds[g] = need;
        }
    }
    if (ng) {
        const int rc = x_prep_multi(x, x_dtype, ldx, x_rows, K, Kp, x16, xscale, ng, g_gs, g_steps, g_xg, st);
        if (rc) return rc;
    }
    static const int grp_mask = tune_env("MFQ_MOE_GROUPS", 7);
#define MFQ_MOE_GRP(GRP)                                                                                              \
    if (grp_mask >> GRP & 1) {                                                                                        \
        const int ncol = static_cast<int>(ceil_div(GLU ? rbe / 2 : rbe, 8 * (GLU ? moe_group_nb(GRP) / 2 : moe_group_nb(GRP)))); \
        const size_t lds = 8 * moe_group_rows(GRP) + glds[GRP];                                                       \
        const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(&moe_prefill_kernel<GRP, GLU>), lds, "moe_prefill"); \
        if (rc) return rc;                                                                                            \
        const unsigned grid = static_cast<unsigned>(ceil_div(cap, 8) * 8 * ncol);                                     \
        hipLaunchKernelGGL((moe_prefill_kernel<GRP, GLU>), dim3(grid), dim3(512), lds, st, P, expert_pool, expert_local, \
                           out_per_expert, x16, Kp, x_rows, xscale, routed_input, R, ids_dst, expert_bounds, lists, cap, \
                           ncol, static_cast<float *>(out), ldo, glu);                                                \
    }
    // the heaviest group first
    MFQ_MOE_GRP(2) MFQ_MOE_GRP(1) MFQ_MOE_GRP(0)
#undef MFQ_MOE_GRP
    return check_launch("moe_prefill");
}

}  // namespace mfq
