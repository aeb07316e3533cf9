// Tuning knobs (environment variables, read once), the device's CU count and the dynamic-LDS opt-in.
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "common.hpp"
#include "tune.hpp"

namespace mfq {

namespace {
struct Knob {
    const char *name;
    const char *what;
    int value;
    bool read;
};
// 0 = "automatic" wherever the default is 0
Knob g_knobs[] = {
    {"MFQ_GEMV_WAVES", "waves a decode GEMV grid aims for before a wave takes more than one item", 0, false},
    {"MFQ_GEMV_SPW", "K steps per wave of the NINT GEMV (0 = by shape)", 0, false},
    {"MFQ_GEMV_RBW", "row-blocks per block of the NINT GEMV (0 = by shape)", 0, false},
    {"MFQ_GEMV_XREG", "0 = the one- and two-row NINT GEMV stages its activations in LDS instead of registers", 0, false},
    {"MFQ_GEMV_VALU_MAX_M", "rows up to which the vector-ALU GEMV runs before the streaming MFMA kernel", 0, false},
    {"MFQ_MFMA_RESIDENT", "0 = small batches never take the kernel that keeps the activations in LDS", 0, false},
    {"MFQ_MFMA_WIDE", "0 = the NINT streaming MFMA kernel keeps eight waves per block on small grids", 0, false},
    {"MFQ_MFMA_NB", "row-blocks per wave of the NINT streaming MFMA kernel (0 = by shape)", 0, false},
    {"MFQ_STREAM_MAX_M", "rows up to which NINT streams instead of the prefill kernel (0 = cost model)", 0, false},
    {"MFQ_PREFILL_SPLITS", "splits over K of a NINT prefill launch (0 = by shape)", 0, false},
    {"MFQ_PREFILL_BIG", "experimental 128 x 384 prefill tiles (0 = off)", 0, false},
    {"MFQ_NVQ_NB", "row-blocks per wave of the NVQ streaming kernel (0 = by shape)", 0, false},
    {"MFQ_NVQ_STREAM_MAX_M", "rows up to which NVQ streams instead of the prefill kernel (0 = cost model)", 0, false},
    {"MFQ_NVQ_BCAST_OFF", "1 = one and two NVQ rows on the matrix-core signed-table kernel instead of the vector-ALU one", 0, false},
    {"MFQ_NVQ_SIGNED_OFF", "1 = NVQ small batches on the older streaming kernel", 0, false},
    {"MFQ_NVQ_SIGNED_MAX_M", "rows up to which the NVQ signed-table kernel runs", 0, false},
    {"MFQ_NVQ_RING", "weight ring depth of the five-row-block NVQ kernel", 0, false},
    {"MFQ_NEPQ_NB", "row-blocks per wave of the NEPQ streaming kernel (0 = by shape)", 0, false},
    {"MFQ_N8Z_TILE_MIN_M", "rows from which NINT8-0 small batches run on the matrix cores (default 2)", 0, false},
    {"MFQ_NEPQ_TILE_OFF", "1 = NEPQ small batches on the older streaming kernel", 0, false},
    {"MFQ_NEPQ_RPB", "row-blocks per block of the one-row NEPQ GEMV (0 = by shape)", 0, false},
    {"MFQ_NEPQ_VALU_MAX_M", "rows up to which NEPQ runs on the vector-ALU GEMV before the streaming MFMA kernel", 0, false},
    {"MFQ_NEPQ_PREFILL_MIN_M", "rows from which NEPQ takes the prefill kernel (0 = default)", 0, false},
    {"MFQ_MOE_SPLIT", "0 = no one-launch MoE decode form", 0, false},
    {"MFQ_MOE_DEC_WAVES", "waves per block of the MoE decode launch", 0, false},
    {"MFQ_MOE_DEC_RBW", "row-blocks per block of the MoE decode launch (0 = by shape)", 0, false},
    {"MFQ_MOE_PREFILL_PAIRS", "pairs per expert from which mapped MoE calls take the prefill kernel (0 = default)", 0, false},
    {"MFQ_FFN_SPIN_LIMIT", "polls after which the one-launch FFN's grid barrier gives up", 0, false},
    {"MFQ_FFN_TRACE", "1 = the one-launch FFN records per-block clocks behind its workspace", 0, false},
    {"MFQ_NVQS_E8_OFF", "1 = the E8 formats on the generic stream kernel", 0, false},
    {"MFQ_NVQS_TILE_MIN_M", "rows from which the stream formats whose ranges fit the LDS run on the matrix-core tile kernel (default 3)", 0, false},
    {"MFQ_NVQS_TILE_MAX_M", "rows up to which they stay on it before the fp16 copy + GEMM (default 192)", 0, false},
    {"MFQ_MX_TILE_OFF", "1 = MXFP4 / MXFP8 small batches on the wave-per-neuron kernel instead of the matrix-core tile kernel", 0, false},
    {"MFQ_MX_STAGE_OFF", "1 = the MX tile kernel never stages a wave's activation slice and scales in LDS", 0, false},
    {"MFQ_MX_STAGE_MAX_M", "rows up to which MX matmuls run as 16-row tiles with the activations staged in LDS (default 48)", 0, false},
    {"MFQ_MX_TILE_MAX_M", "rows up to which MX matmuls run on the tile kernel before the fp16 copy + GEMM (default 256)", 0, false},
    {"MFQ_MX_NB", "row-blocks per block of the MX tile kernel (0 = by shape)", 0, false},
    {"MFQ_MX_WAVES", "waves per block the MX tile kernels split K over (0 = by shape)", 0, false},
    {"MFQ_NVQ_PAIRS_MFMA", "0 = a MoE decode step on an NVQ cohort always takes the generic one-row kernel", 0, false},
    {"MFQ_MOE_NB", "row-blocks per wave of the MoE streaming kernel (0 = by shape)", 0, false},
    {"MFQ_MOE_GROUPS", "bit mask of the register groups the mapped MoE prefill path launches (7 = all)", 0, false},
    {"MFQ_GLU_PREFILL_MIN_M", "rows from which the dense gate/up prefill fuses the GLU into its epilogue", 0, false},
};
std::mutex g_mu;
std::atomic<int> g_cu_override{0};
std::atomic<int> g_cu_cached[64];
}  // namespace

int tune_env(const char *name, int dflt) {
    std::lock_guard<std::mutex> lock(g_mu);
    for (Knob &k : g_knobs) {
        if (strcmp(k.name, name) != 0) continue;
        if (!k.read) {
            const char *e = getenv(name);
            k.value = e ? atoi(e) : dflt;
            k.read = true;
        }
        return k.value;
    }
    const char *e = getenv(name);  // not in the table: still honoured, but not listed
    return e ? atoi(e) : dflt;
}

int device_cu_count() {
    const int forced = g_cu_override.load(std::memory_order_relaxed);
    if (forced > 0) return forced;
    return device_real_cu_count();
}

int device_real_cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = g_cu_cached[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    g_cu_cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

int allow_dynamic_lds(const void *kernel, size_t lds, const char *what) {
    if (lds <= 65536) return MFQ_OK;
    if (lds > kMaxDynamicLds) return fail(MFQ_ERR_UNSUPPORTED, "%s: %zu bytes of LDS exceed the %zu a block can have", what, lds, kMaxDynamicLds);
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return fail(MFQ_ERR_LAUNCH, "%s: %zu bytes of LDS: %s", what, lds, hipGetErrorString(e));
    return MFQ_OK;
}

// Read-only streaming probe: a wave owns 16 KB, requested up front.
__global__ __launch_bounds__(512) void read_probe_kernel(const u32x4_t *__restrict__ p, size_t n16, uint32_t *sink) {
    const size_t wave = static_cast<size_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const size_t base = wave * (16 * 64) + (threadIdx.x & 63);
    u32x4_t v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const size_t idx = base + static_cast<size_t>(i) * 64;
        v[i] = idx < n16 ? __builtin_nontemporal_load(p + idx) : u32x4_t{0u, 0u, 0u, 0u};
    }
    uint32_t a = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) a ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    if (a == 0x12345678u) sink[0] = a;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t *__restrict__ p, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256) p[i] = 0u;
}

}  // namespace mfq

using namespace mfq;

extern "C" int mfq_hip_fill_zero(void *data, size_t bytes, mfq_stream_t stream) {
    if (bytes == 0) return MFQ_OK;
    MFQ_REQUIRE(data && (reinterpret_cast<uintptr_t>(data) & 3) == 0 && bytes % 4 == 0, MFQ_ERR_INVALID,
                "fill_zero: null or unaligned buffer");
    const size_t n = bytes / 4;
    const size_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(static_cast<unsigned>(blocks < 4096 ? blocks : 4096)), dim3(256), 0, as_stream(stream),
                       static_cast<uint32_t *>(data), n);
    return check_launch("fill_zero");
}

extern "C" int mfq_hip_read_probe(const void *data, size_t bytes, void *sink, mfq_stream_t stream) {
    MFQ_REQUIRE(data && sink && (reinterpret_cast<uintptr_t>(data) & 15) == 0, MFQ_ERR_INVALID, "read_probe: null or unaligned buffer");
    const size_t n16 = bytes / 16, waves = ceil_div(static_cast<int64_t>(n16), 16 * 64);
    MFQ_REQUIRE(n16 > 0 && waves / 8 + 1 < (1ull << 31), MFQ_ERR_INVALID, "read_probe: %zu bytes", bytes);
    hipLaunchKernelGGL(read_probe_kernel, dim3(static_cast<unsigned>(ceil_div(static_cast<int64_t>(waves), 8))), dim3(512), 0,
                       as_stream(stream), static_cast<const u32x4_t *>(data), n16, static_cast<uint32_t *>(sink));
    return check_launch("read_probe");
}

extern "C" void mfq_hip_set_cu_count(int n) { g_cu_override.store(n > 0 ? n : 0, std::memory_order_relaxed); }

extern "C" const char *mfq_hip_config(void) {
    static thread_local char buf[2048];
    size_t off = 0;
    off += snprintf(buf + off, sizeof(buf) - off, "cu_count=%d", device_cu_count());
    std::lock_guard<std::mutex> lock(g_mu);
    for (const Knob &k : g_knobs)
        if (k.read && off < sizeof(buf)) off += snprintf(buf + off, sizeof(buf) - off, " %s=%d", k.name, k.value);
    return buf;
}
