// Decode feed-forward block in one launch: hidden = act(gate x) * (up x), y = down hidden, for one activation row.
//
// One block of 16 waves per compute unit, all resident at once.  Phase A is the gate/up GEMV with the gated linear
// unit fused (the waves of a block form a gate team and an up team that split the K steps of the block's row-block
// pairs); phase B is the down GEMV (every wave a slice of K of the block's row-blocks).  Between the two the
// 16-bit hidden vector crosses the chip through the workspace behind a grid-wide barrier.  What the fusion buys over
// two launches is the second launch's gap and ramp: a wave requests its phase-B weights the moment its phase-A sums
// are done, so the down tensor streams while the hidden vector is written, the barrier is crossed and the hidden
// slices are fetched.
//
// Grid barrier: one flag word per block in the workspace.  All flags hold the same value between launches (zero at
// first); a block reads its own flag e at its start, stores e + 1 once its hidden values are out (32-bit stores that go
// past the XCD's L2), and its sync wave then polls the whole flag array with one wave-wide load per round until every
// flag has reached e + 1 -- no read-modify-write on a shared word (256 of those on one address take microseconds),
// nothing to reset.  The polling sleeps between rounds and stops after `spin_limit` rounds: every wave reaches the end
// of the kernel whatever happens; a block that gives up stores NaN outputs and raises the error word.  The sync wave
// of a block (its last one) requests its phase-B weights only after the barrier: loads return in order, so a wave
// that polls with weight loads outstanding would see the flags only after they land.
#include <atomic>

#include "common.hpp"
#include "gemv_common.hpp"
#include "nint_body.hpp"
#include "tune.hpp"

namespace mfq {

struct FfnK {
    NintK a, b;            // gate/up tensor [2 W, H] (gate rows first), down tensor [N, W]
    const uint8_t *wa, *wb;
    const uint16_t *x;     // [H] bf16 / fp16
    float *y;              // [N]
    uint16_t *hidden;      // [W] fp16 (workspace)
    int *sync;             // one flag per block, then the error word (workspace)
    int pairs;             // W / 16: gate row-block p pairs with up row-block pairs + p
    int ppb;               // pairs per block
    int wpt, spw_a, act_a; // waves per team, K steps per wave, waves of a team that own steps (phase A)
    int rbpb, spw_b, act_b;  // row-blocks per block, K steps per wave, waves that own steps (phase B)
    int stage_dwords;      // wave-private LDS area, sized for the larger phase
    int gelu;
    int spin_limit;
    long long *trace;      // tuning aid (MFQ_FFN_TRACE): four clock readings per block, or null
};

constexpr int kFfnWaves = 16;
constexpr int kFfnItems = 3;   // (row-block, step) items a wave holds in registers in phase A
constexpr int kFfnItemsB = 2;  // and in phase B (the kernel below is written for exactly two)

// item i of a wave that owns n steps of each of its row-blocks: row-block i / n, step i % n
__device__ __forceinline__ void ffn_item(int i, int n, int &irb, int &is) {
    irb = n == 1 ? i : (n == 2 ? (i >> 1) : (n == 3 ? (i == 3 ? 1 : 0) : 0));
    is = i - irb * n;
}

template <class UA, class UB, int XF16>
__global__ __launch_bounds__(1024) void nint_ffn_decode_kernel(FfnK p) {
    extern __shared__ uint32_t lds[];
    constexpr int DA = UA::D, DB = UB::D, GSA = UA::GROUP, GSB = UB::GROUP;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int r = lane & 15, kb = lane >> 4;
    const int G = gridDim.x;
    const bool sync_wave = wave == kFfnWaves - 1;
    if (p.trace && sync_wave && lane == 0) p.trace[blockIdx.x * 4] = wall_clock64();
    int epoch = 0;  // the sync wave's view of the barrier: every flag holds this value when the kernel starts
    if (sync_wave) epoch = __hip_atomic_load(p.sync + blockIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t *xs = lds + wave * p.stage_dwords;
    float *red = reinterpret_cast<float *>(lds + kFfnWaves * p.stage_dwords);  // 2 teams * 3 row-blocks * wpt * 16
    int *flag = reinterpret_cast<int *>(red + 2 * kFfnItems * kFfnWaves * 16);
    float *anc = reinterpret_cast<float *>(flag + 16) + wave * (2 * kFfnItems + 2 * kFfnItemsB) * 16;

    // ---- roles ----------------------------------------------------------------------------------------------
    const int team = wave / p.wpt, tw = wave - team * p.wpt;
    const int p0 = blockIdx.x * p.ppb;
    const int npair = max(0, min(p.ppb, p.pairs - p0));
    const int sa0 = tw * p.spw_a;
    const int na = (team < 2 && npair > 0) ? max(0, min(p.a.nsteps, sa0 + p.spw_a) - sa0) : 0;
    const int items_a = npair * na;
    const int rba0 = min(team, 1) * p.pairs + min(p0, p.pairs - 1);
    const uint32_t sba = static_cast<uint32_t>(p.a.step_bytes), rbba = static_cast<uint32_t>(p.a.rowblock_bytes);
    const int ngl_a = p.spw_a * 16, npairs_a = ngl_a * (GSA / 2);

    const int rbb0 = blockIdx.x * p.rbpb;
    const int nrb_b = max(0, min(p.rbpb, p.b.n_rowblocks - rbb0));
    const int sb0 = wave * p.spw_b;
    const int nb = nrb_b > 0 ? max(0, min(p.b.nsteps, sb0 + p.spw_b) - sb0) : 0;
    const int items_b = nrb_b * nb;
    const uint32_t sbb = static_cast<uint32_t>(p.b.step_bytes), rbbb = static_cast<uint32_t>(p.b.rowblock_bytes);
    const int ngl_b = p.spw_b * 16, npairs_b = ngl_b * (GSB / 2);

    // ---- requests, in order of use: activations, anchors, the phase-A items ----------------------------------------
    const uint16_t *xr[1] = {p.x};
    XRegs<1> xg;
    stage_x_issue<1>(xr, p.a.neuron_len, sa0 * 16 * GSA, npairs_a, lane, xg);
    const float *anc_a = reinterpret_cast<const float *>(p.wa + p.a.anchors_off);
    const float *anc_b = reinterpret_cast<const float *>(p.wb + p.b.anchors_off);
    // anchors: lanes 0..15 fetch them (one neuron each) for both phases right away; they wait in the wave's LDS area
    // until a row-block's sums are complete, so that they neither occupy registers nor queue behind the weights
    float anc_v[2 * kFfnItems + 2 * kFfnItemsB];
#pragma unroll
    for (int i = 0; i < kFfnItems; ++i) {
        const int ra = min(rba0 + i, p.a.n_rowblocks - 1);
        anc_v[2 * i] = anc_a[ra * 16 + r];
        anc_v[2 * i + 1] = anc_a[16 * p.a.n_rowblocks + ra * 16 + r];
    }
#pragma unroll
    for (int i = 0; i < kFfnItemsB; ++i) {
        const int rb = min(rbb0 + i, p.b.n_rowblocks - 1);
        anc_v[2 * kFfnItems + 2 * i] = anc_b[rb * 16 + r];
        anc_v[2 * kFfnItems + 2 * i + 1] = anc_b[16 * p.b.n_rowblocks + rb * 16 + r];
    }
    const __amdgpu_buffer_rsrc_t win_a =
        wave_window(p.wa + static_cast<int64_t>(rba0) * p.a.rowblock_bytes + static_cast<int64_t>(sa0) * sba,
                    items_a > 0 ? (npair - 1) * rbba + na * sba : 0u);
    const __amdgpu_buffer_rsrc_t win_b =
        wave_window(p.wb + static_cast<int64_t>(min(rbb0, p.b.n_rowblocks - 1)) * p.b.rowblock_bytes +
                        static_cast<int64_t>(sb0) * sbb,
                    items_b > 0 ? (nrb_b - 1) * rbbb + nb * sbb : 0u);
    const __amdgpu_buffer_rsrc_t win_h = wave_window(reinterpret_cast<const uint8_t *>(p.hidden),
                                                     static_cast<uint32_t>(p.b.neuron_len) * 2u);

    uint32_t qa[kFfnItems][4][DA], ta[kFfnItems], qb[kFfnItemsB][4][DB], tb[kFfnItemsB];
    u32x2_t ca[kFfnItems], cb[kFfnItemsB];
#pragma unroll
    for (int i = 0; i < kFfnItems; ++i) {
        int irb, is;
        ffn_item(i, na, irb, is);
        nint_load_step<DA, UA::TAIL>(win_a, i < items_a ? irb * rbba + is * sba : kNoStep, lane, qa[i], ta[i], ca[i]);
    }
    float *xsum_a = reinterpret_cast<float *>(xs + npairs_a);
    float xinv[1];
    stage_x<XF16, 1, typename UA::Bias, true>(xr, p.a.neuron_len, sa0 * 16 * GSA, npairs_a, GSA, ngl_a, xs, xsum_a, lane, xg, xinv);

    if (kb == 0) {
#pragma unroll
        for (int i = 0; i < 2 * kFfnItems + 2 * kFfnItemsB; ++i) anc[i * 16 + r] = anc_v[i];
    }
    wave_sync();

    // ---- phase A: compute item i, then hand its registers' successor request to phase B ------------------------------
    float accS[1] = {0.f}, accM[1] = {0.f};
#pragma unroll
    for (int i = 0; i < kFfnItems; ++i) {
        if (i < items_a) {
            int irb, is;
            ffn_item(i, na, irb, is);
            nint_compute_step<UA, 1>(qa[i], ta[i], ca[i], is * 16 + kb, xs, xsum_a, npairs_a, ngl_a, accS, accM);
            if (is == na - 1) {
                float v[1] = {(anc[(2 * irb) * 16 + r] * accS[0] - anc[(2 * irb + 1) * 16 + r] * accM[0]) * xinv[0]};
                park_rows<1>(v, red, (team * kFfnItems + irb) * p.wpt + tw, lane);
                accS[0] = accM[0] = 0.f;
            }
        }
    }
    // phase B's weights: requested now, so that they stream while the hidden vector crosses the chip
    if (!sync_wave) {
#pragma unroll
        for (int i = 0; i < kFfnItemsB; ++i) {
            int irb, is;
            ffn_item(i, nb, irb, is);
            nint_load_step<DB, UB::TAIL>(win_b, i < items_b ? irb * rbbb + is * sbb : kNoStep, lane, qb[i], tb[i], cb[i]);
        }
    }

    // ---- hidden values of the block's pairs, written back chip-wide by the sync wave, then the grid barrier --------
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();  // bare: the phase-B requests stay in flight
    asm volatile("" ::: "memory");
    if (sync_wave) {
        // one lane per pair of neighbouring neurons; the 32-bit stores go past this XCD's L2 (agent-scope atomics), so no
        // cache write-back is needed before the counter moves
        for (int o = lane; o < npair * 8; o += 64) {
            const int i = o >> 3, rr = (o & 7) * 2;
            float g0 = 0.f, u0 = 0.f, g1 = 0.f, u1 = 0.f;
            for (int t = 0; t < p.act_a; ++t) {
                const float *rg = red + ((0 * kFfnItems + i) * p.wpt + t) * 16 + rr;
                const float *ru = red + ((1 * kFfnItems + i) * p.wpt + t) * 16 + rr;
                g0 += rg[0]; g1 += rg[1]; u0 += ru[0]; u1 += ru[1];
            }
            const uint32_t h = static_cast<uint32_t>(f32_to_f16_rne(glu_value(g0, u0, p.gelu != 0))) |
                               (static_cast<uint32_t>(f32_to_f16_rne(glu_value(g1, u1, p.gelu != 0))) << 16);
            __hip_atomic_store(reinterpret_cast<uint32_t *>(p.hidden) + (p0 + i) * 8 + (rr >> 1), h, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores above are acknowledged (this wave has no loads in flight)
        if (lane == 0) {
            if (p.trace) p.trace[blockIdx.x * 4 + 1] = wall_clock64();
            __hip_atomic_store(p.sync + blockIdx.x, epoch + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // every lane watches four flags per round (G <= 256: one load instruction for the whole array)
        int ok = 0;
        for (int spins = 0; spins < p.spin_limit; ++spins) {
            bool all = true;
            for (int j0 = 0; j0 < G; j0 += 256) {
                const int j = j0 + lane * 4;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int f = j + t < G ? __hip_atomic_load(p.sync + j + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : epoch + 1;
                    all = all && (f - (epoch + 1)) >= 0;
                }
            }
            if (__all(all)) { ok = 1; break; }
            __builtin_amdgcn_s_sleep(1);
        }
        if (lane == 0) {
            if (!ok) __hip_atomic_store(p.sync + G, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (p.trace) p.trace[blockIdx.x * 4 + 2] = wall_clock64();
            flag[0] = ok;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const int ok = flag[0];
    if (sync_wave) {
#pragma unroll
        for (int i = 0; i < kFfnItemsB; ++i) {
            int irb, is;
            ffn_item(i, nb, irb, is);
            nint_load_step<DB, UB::TAIL>(win_b, i < items_b ? irb * rbbb + is * sbb : kNoStep, lane, qb[i], tb[i], cb[i]);
        }
    }

    // ---- phase B: the wave's slice of the hidden vector (read past every non-coherent cache), then its items ---------
    {
        const int k0 = sb0 * 16 * GSB;
#pragma unroll
        for (int c = 0; c < kXChunks; ++c) {
            const int i = lane * 4 + c * 256;
            const bool in = nb > 0 && i < npairs_b && k0 + 2 * i + 8 <= p.b.neuron_len;
            xg.v[0][c] = __builtin_amdgcn_raw_buffer_load_b128(win_h, in ? static_cast<uint32_t>(k0 + 2 * i) * 2u : kNoStep, 0, 17);
        }
        xg.on = true;
    }
    float *xsum_b = reinterpret_cast<float *>(xs + npairs_b);
    const uint16_t *hr[1] = {p.hidden};
    stage_x<1, 1, typename UB::Bias>(hr, p.b.neuron_len, sb0 * 16 * GSB, npairs_b, GSB, ngl_b, xs, xsum_b, lane, xg);
    accS[0] = accM[0] = 0.f;
#pragma unroll
    for (int i = 0; i < kFfnItemsB; ++i) {
        if (i < items_b) {
            int irb, is;
            ffn_item(i, nb, irb, is);
            nint_compute_step<UB, 1>(qb[i], tb[i], cb[i], is * 16 + kb, xs, xsum_b, npairs_b, ngl_b, accS, accM);
            if (is == nb - 1) {
                float v[1] = {anc[(2 * kFfnItems + 2 * irb) * 16 + r] * accS[0] -
                              anc[(2 * kFfnItems + 2 * irb + 1) * 16 + r] * accM[0]};
                park_rows<1>(v, red, irb * kFfnWaves + wave, lane);
                accS[0] = accM[0] = 0.f;
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    for (int o = threadIdx.x; o < nrb_b * 16; o += blockDim.x) {
        const int i = o >> 4, rr = o & 15;
        float s = 0.f;
        for (int t = 0; t < p.act_b; ++t) s += red[(i * kFfnWaves + t) * 16 + rr];
        const int row = (rbb0 + i) * 16 + rr;
        if (row < p.b.out) p.y[row] = ok ? s : __builtin_nanf("");
    }
    if (p.trace && sync_wave && lane == 0) p.trace[blockIdx.x * 4 + 3] = wall_clock64();
}

// workspace: the barrier's flag words (one per block, then the error word), then the fp16 hidden vector
constexpr size_t kFfnSyncBytes = 4096;

__global__ void ffn_sync_clear_kernel(int *sync) {
    for (int i = threadIdx.x; i < static_cast<int>(kFfnSyncBytes / 4); i += blockDim.x) sync[i] = 0;
}

// profiles whose two phases fit a wave's 128 registers together
static bool ffn_unit(const mfq_nint_desc *d) {
    return d->kind == 1 && ((d->bits == 4 && (d->gs == 32 || d->gs == 24)) || (d->bits == 3 && d->gs == 24) || (d->bits == 2 && d->gs == 16));
}

// Fills the launch shape; false when the pair of tensors is outside what the kernel holds in registers.
static bool ffn_shape(const mfq_nint_desc *gu, const mfq_nint_desc *dn, int G, FfnK &p, size_t &lds) {
    if (!ffn_unit(gu) || !ffn_unit(dn) || gu->bits != dn->bits || gu->gs != dn->gs) return false;
    if (G < 1 || static_cast<size_t>(G + 1) * 4 > kFfnSyncBytes) return false;
    if (gu->out % 32 || gu->out / 2 != dn->neuron_len || gu->neuron_len % 8 || dn->neuron_len % 8) return false;
    if (kFfnItems * gu->rowblock_bytes >= (1ll << 31) || kFfnItems * dn->rowblock_bytes >= (1ll << 31)) return false;
    p.pairs = gu->out / 32;
    p.ppb = static_cast<int>(ceil_div(p.pairs, G));
    p.wpt = kFfnWaves / 2;
    p.spw_a = static_cast<int>(ceil_div(gu->nsteps, p.wpt));
    p.act_a = static_cast<int>(ceil_div(gu->nsteps, p.spw_a));
    p.rbpb = static_cast<int>(ceil_div(dn->n_rowblocks, G));
    p.spw_b = static_cast<int>(ceil_div(dn->nsteps, kFfnWaves));
    p.act_b = static_cast<int>(ceil_div(dn->nsteps, p.spw_b));
    if (p.ppb * p.spw_a > kFfnItems || p.rbpb * p.spw_b > kFfnItemsB) return false;
    const int pa = p.spw_a * 16 * (gu->gs / 2), pb = p.spw_b * 16 * (dn->gs / 2);
    if (pa > 256 * kXChunks || pb > 256 * kXChunks) return false;  // what one wave stages from registers
    const int da = pa + 2 * p.spw_a * 16, db = pb + 2 * p.spw_b * 16;
    p.stage_dwords = da > db ? da : db;
    lds = (static_cast<size_t>(kFfnWaves) * p.stage_dwords + 2 * kFfnItems * kFfnWaves * 16 + 16 +
           kFfnWaves * (2 * kFfnItems + 2 * kFfnItemsB) * 16) * 4;
    return lds <= kMaxDynamicLds;
}

}  // namespace mfq

using namespace mfq;

extern "C" size_t mfq_hip_nint_ffn_decode_workspace_bytes(const mfq_nint_desc *gate_up, const mfq_nint_desc *down) {
    if (!gate_up || !down) return 0;
    FfnK p;
    size_t lds;
    if (!ffn_shape(gate_up, down, device_cu_count(), p, lds)) return 0;
    return kFfnSyncBytes + static_cast<size_t>(ceil_div(down->neuron_len, 8)) * 16;
}

extern "C" int mfq_hip_nint_ffn_decode_workspace_init(void *workspace, mfq_stream_t stream) {
    MFQ_REQUIRE(workspace && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0, MFQ_ERR_INVALID,
                "nint_ffn_decode: null or unaligned workspace");
    hipLaunchKernelGGL(ffn_sync_clear_kernel, dim3(1), dim3(256), 0, as_stream(stream), static_cast<int *>(workspace));
    return check_launch("nint_ffn_decode_workspace_init");
}

extern "C" int mfq_hip_nint_ffn_decode_status(void *workspace, mfq_stream_t stream) {
    MFQ_REQUIRE(workspace, MFQ_ERR_INVALID, "nint_ffn_decode_status: null workspace");
    const hipStream_t st = as_stream(stream);
    // the error word follows the flags of however many blocks the launches used: any of the words behind the first
    // device_cu_count() flags up to the end of the barrier area can only have been set by a timed-out barrier
    int words[kFfnSyncBytes / 4];
    hipError_t e = hipMemcpyAsync(words, workspace, kFfnSyncBytes, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    MFQ_REQUIRE(e == hipSuccess, MFQ_ERR_LAUNCH, "nint_ffn_decode_status: %s", hipGetErrorString(e));
    const int G = device_cu_count();
    if (words[G] == 0) return MFQ_OK;
    hipLaunchKernelGGL(ffn_sync_clear_kernel, dim3(1), dim3(256), 0, st, static_cast<int *>(workspace));
    if (int rc = check_launch("nint_ffn_decode_status")) return rc;
    return fail(MFQ_ERR_LAUNCH, "nint_ffn_decode: a grid barrier gave up (the blocks did not all run at once); the outputs of the "
                                "calls since the last check are NaN, the workspace has been reset");
}

extern "C" int mfq_hip_nint_ffn_decode(const mfq_nint_desc *gate_up, const void *gate_up_weight, const mfq_nint_desc *down,
                                       const void *down_weight, const void *x, int x_dtype, int activation, float *y,
                                       void *workspace, size_t workspace_bytes, mfq_stream_t stream) {
    MFQ_REQUIRE(gate_up && gate_up_weight && down && down_weight && x && y, MFQ_ERR_INVALID, "nint_ffn_decode: null argument");
    MFQ_REQUIRE(x_dtype == MFQ_X_BF16 || x_dtype == MFQ_X_F16, MFQ_ERR_INVALID, "nint_ffn_decode: x_dtype=%d", x_dtype);
    MFQ_REQUIRE(activation == MFQ_GLU_SILU || activation == MFQ_GLU_GELU, MFQ_ERR_INVALID, "nint_ffn_decode: activation=%d",
                activation);
    MFQ_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0, MFQ_ERR_UNSUPPORTED, "nint_ffn_decode: activations must be 16-byte aligned");
    FfnK p;
    size_t lds;
    const int G = device_cu_count();
    MFQ_REQUIRE(ffn_shape(gate_up, down, G, p, lds), MFQ_ERR_UNSUPPORTED,
                "nint_ffn_decode: NINT%d-%d [%d, %d] + NINT%d-%d [%d, %d] is outside the one-launch kernel (same profile with a "
                "batch-1 unit, down.neuron_len = gate_up.out / 2, at most three gate/up and two down items per wave on %d compute units)",
                gate_up->bits, gate_up->gs, gate_up->out, gate_up->neuron_len, down->bits, down->gs, down->out,
                down->neuron_len, G);
    const size_t need = mfq_hip_nint_ffn_decode_workspace_bytes(gate_up, down);
    MFQ_REQUIRE(workspace && workspace_bytes >= need, MFQ_ERR_WORKSPACE, "nint_ffn_decode: workspace %zu < %zu bytes",
                workspace_bytes, need);
    MFQ_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, MFQ_ERR_INVALID, "nint_ffn_decode: unaligned workspace");
    p.a = to_k(gate_up);
    p.b = to_k(down);
    p.wa = static_cast<const uint8_t *>(gate_up_weight);
    p.wb = static_cast<const uint8_t *>(down_weight);
    p.x = static_cast<const uint16_t *>(x);
    p.y = y;
    p.sync = static_cast<int *>(workspace);
    p.hidden = reinterpret_cast<uint16_t *>(static_cast<uint8_t *>(workspace) + kFfnSyncBytes);
    p.gelu = activation == MFQ_GLU_GELU ? 1 : 0;
    static const int spin_limit = tune_env("MFQ_FFN_SPIN_LIMIT", 1 << 18), want_trace = tune_env("MFQ_FFN_TRACE", 0);
    p.spin_limit = spin_limit;
    // MFQ_FFN_TRACE=1: a workspace with 32 more bytes per compute unit behind the hidden vector receives each block's
    // clock (100 MHz) at its start, at its arrival at the barrier, after the barrier and at its end
    p.trace = want_trace && workspace_bytes >= need + 32u * G
                  ? reinterpret_cast<long long *>(static_cast<uint8_t *>(workspace) + ((need + 31) & ~size_t(31)))
                  : nullptr;
    const hipStream_t st = as_stream(stream);
#define MFQ_FFN(UNIT, B, GS)                                                                                          \
    if (gate_up->bits == B && gate_up->gs == GS) {                                                                     \
        auto kern = x_dtype == MFQ_X_F16 ? nint_ffn_decode_kernel<UNIT<B, GS>, UNIT<B, GS>, 1>                         \
                                         : nint_ffn_decode_kernel<UNIT<B, GS>, UNIT<B, GS>, 0>;                        \
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds, "nint_ffn_decode")) return rc;       \
        /* all blocks must be resident at once: asked once per kernel and LDS size */                                  \
        static std::atomic<size_t> fits_lds{0};                                                                        \
        static std::atomic<int> resident_blocks{1};                                                                    \
        if (fits_lds.load(std::memory_order_relaxed) < lds) {                                                          \
            int resident = 0;                                                                                          \
            const hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, kern, 64 * kFfnWaves, lds);   \
            MFQ_REQUIRE(e == hipSuccess && resident >= 1, MFQ_ERR_UNSUPPORTED,                                         \
                        "nint_ffn_decode: a block of %d waves with %zu bytes of LDS does not fit a compute unit", kFfnWaves, lds); \
            fits_lds.store(lds, std::memory_order_relaxed);                                                            \
            resident_blocks.store(resident, std::memory_order_relaxed);                                                \
        }                                                                                                              \
        MFQ_REQUIRE(G <= device_real_cu_count() * resident_blocks.load(std::memory_order_relaxed), MFQ_ERR_UNSUPPORTED, \
                    "nint_ffn_decode: %d blocks cannot all run at once on %d compute units (%d block(s) each): the grid " \
                    "barrier would never be crossed", G, device_real_cu_count(), resident_blocks.load(std::memory_order_relaxed)); \
        hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(G)), dim3(64 * kFfnWaves), lds, st, p);                    \
        return check_launch("nint_ffn_decode");                                                                        \
    }
    if (gate_up->kind == 1) {
        MFQ_FFN(PairedUnit, 4, 32) MFQ_FFN(PairedUnit, 4, 24) MFQ_FFN(PairedUnit, 3, 24) MFQ_FFN(PairedUnit, 2, 16)
    }
#undef MFQ_FFN
    return fail(MFQ_ERR_UNSUPPORTED, "nint_ffn_decode: no one-launch kernel for NINT%d-%d", gate_up->bits, gate_up->gs);
}
