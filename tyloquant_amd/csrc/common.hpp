// Shared host/device helpers for the MFQ gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/mfq_hip.h"

namespace mfq {

// ---- host-side error reporting -------------------------------------------------------
char *error_buffer();
int fail(int code, const char *fmt, ...);

#define MFQ_REQUIRE(cond, code, ...)                 \
    do {                                             \
        if (!(cond)) return ::mfq::fail((code), __VA_ARGS__); \
    } while (0)

inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MFQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MFQ_OK;
}

inline hipStream_t as_stream(mfq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device helpers --------------------------------------------------------------------
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// acc + a.lo*b.lo + a.hi*b.hi with both operands holding two bf16 (or fp16) values.
template <int XF16>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    if constexpr (XF16) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), acc, false);
    } else {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                               false);
    }
}

// Block-wide copy of n dwords (a lookup table) from global memory into LDS.  A thread requests four 16-byte pieces
// before it stores the first: a plain dword loop waits one round trip to memory per piece, which for a 32 KB table
// and a block of a thousand threads is eight round trips in a row at the head of the kernel.  dst: 16-byte aligned.
__device__ __forceinline__ void table_to_lds(uint32_t *dst, const uint32_t *src, int n, int tid, int nt) {
    if ((reinterpret_cast<uintptr_t>(src) & 15) == 0 && n % 4 == 0) {
        const u32x4_t *s4 = reinterpret_cast<const u32x4_t *>(src);
        u32x4_t *d4 = reinterpret_cast<u32x4_t *>(dst);
        const int n4 = n / 4;
        for (int i0 = tid; i0 < n4; i0 += 4 * nt) {
            u32x4_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = s4[min(i0 + u * nt, n4 - 1)];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (i0 + u * nt < n4) d4[i0 + u * nt] = v[u];
        }
    } else {
        for (int i = tid; i < n; i += nt) dst[i] = src[i];
    }
}

__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }
__device__ __forceinline__ float f16_to_f32(uint16_t v) {
    return static_cast<float>(__builtin_bit_cast(_Float16, v));
}
template <int XF16>
__device__ __forceinline__ float x_to_f32(uint16_t v) {
    if constexpr (XF16) return f16_to_f32(v);
    else return bf16_to_f32(v);
}
// Gated-linear-unit value act(gate) * up of the reference's mfq_glu (mfq/kernels/cuda/glu.cuh:5-16): SiLU, or the
// tanh form of GELU when `gelu` is set.  Kernels carry the choice in bit 1 of their 16-bit output mode
// (bit 0: fp16 rather than bf16).
// Both are gate * sigmoid(z) * up -- 0.5 (1 + tanh(u)) = sigmoid(2 u) -- with the sigmoid from the hardware's base-2
// exponential and reciprocal (one unit in the last place each; the 16-bit result keeps 8 or 11 bits): a dozen
// instructions per value where expf, tanhf and a division take several dozen, which the prefill epilogues notice.
__device__ __forceinline__ float sigmoid_fast(float z) {
    return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * z));
}
__device__ __forceinline__ float glu_value(float gate, float up, bool gelu) {
    const float z = gelu ? 1.59576912160573071176f * gate * (1.0f + 0.044715f * gate * gate) : gate;
    return gate * sigmoid_fast(z) * up;
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}
__device__ __forceinline__ uint16_t f32_to_f16_rne(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

// outp[at] = v rounded once to out_dtype (MFQ_X_F32: as is); outp is an array of that type.
__device__ __forceinline__ void store_rounded(void *outp, int64_t at, float v, int out_dtype) {
    if (out_dtype == MFQ_X_F32) static_cast<float *>(outp)[at] = v;
    else static_cast<uint16_t *>(outp)[at] = out_dtype == MFQ_X_F16 ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
}

// A 1.0/1.0 pair in the activation type, for group sums through dot2.
template <int XF16>
__device__ __forceinline__ constexpr uint32_t ones_pair() { return XF16 ? 0x3c003c00u : 0x3f803f80u; }

__device__ __forceinline__ float ubyte_f32(uint32_t v, int byte) {
    return static_cast<float>((v >> (8 * byte)) & 0xffu);
}

// Sum over the four lanes l, l^16, l^32, l^48 (the K-split inside a 16-neuron row-block).
__device__ __forceinline__ float reduce_kb4(float v) {
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// Little-endian bit-stream read of value `idx` of width `bits` (<= 16).
__device__ __forceinline__ uint32_t read_bits(const uint8_t *s, int64_t idx, int bits, int64_t nbytes) {
    const int64_t bit = idx * bits;
    const int64_t b = bit >> 3;
    uint32_t v = s[b];
    if (b + 1 < nbytes) v |= static_cast<uint32_t>(s[b + 1]) << 8;
    if (b + 2 < nbytes) v |= static_cast<uint32_t>(s[b + 2]) << 16;
    return (v >> (bit & 7)) & ((1u << bits) - 1u);
}

// Input gate of a projection: x * act(gate), act = SiLU (mode 0) or the logistic function (mode 1), formed in fp32
// and rounded once to the 16-bit type of x (F16: fp16, else bf16).
template <int F16>
__device__ __forceinline__ uint16_t input_gate_value(uint16_t xv, uint16_t gv, int mode) {
    const float g = F16 ? f16_to_f32(gv) : __uint_as_float(static_cast<uint32_t>(gv) << 16);
    const float x = F16 ? f16_to_f32(xv) : __uint_as_float(static_cast<uint32_t>(xv) << 16);
    const float s = 1.f / (1.f + expf(-g));
    const float v = x * (mode == 1 ? s : g * s);
    return F16 ? f32_to_f16_rne(v) : f32_to_bf16_rne(v);
}

}  // namespace mfq
