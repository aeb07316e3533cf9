// C++ host runtime over the C ABI of libmfq_hip.so (see mfq_runtime.h for the map to the reference).
#include "mfq_runtime.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <limits>
#include <stdexcept>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace mfq_rt {

namespace {

[[noreturn]] void fail(const std::string &msg) { throw std::runtime_error(msg); }

void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) fail(std::string(what) + ": " + hipGetErrorString(e));
}
void abi_check(int rc) {
    if (rc != MFQ_OK) fail(std::string("mfq_hip: ") + mfq_hip_last_error());
}
hipStream_t hs(mfq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

template <typename T>
T rd(const uint8_t *p, size_t off) {
    T v;
    std::memcpy(&v, p + off, sizeof(T));
    return v;
}
int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
float half_to_float(uint16_t h) {  // IEEE binary16 -> binary32, subnormals and specials included
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else {
            int e = -1;
            uint32_t m = man;
            do { ++e; m <<= 1; } while (!(m & 0x400u));
            u = sign | static_cast<uint32_t>(127 - 15 - e) << 23 | (m & 0x3ffu) << 13;
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | man << 13;
    } else {
        u = sign | (exp + 112u) << 23 | man << 13;
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

}  // namespace

// ---- DeviceBuffer ---------------------------------------------------------------------------------
DeviceBuffer::DeviceBuffer(size_t bytes) : bytes_(bytes) {
    if (bytes) hip_check(hipMalloc(&ptr_, bytes), "hipMalloc");
}
DeviceBuffer::~DeviceBuffer() {
    if (ptr_) (void)hipFree(ptr_);
}
DeviceBuffer::DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
DeviceBuffer &DeviceBuffer::operator=(DeviceBuffer &&o) noexcept {
    if (this != &o) {
        if (ptr_) (void)hipFree(ptr_);
        ptr_ = o.ptr_; bytes_ = o.bytes_;
        o.ptr_ = nullptr; o.bytes_ = 0;
    }
    return *this;
}
void DeviceBuffer::ensure(size_t bytes) {
    if (bytes <= bytes_) return;
    if (ptr_) hip_check(hipFree(ptr_), "hipFree");
    ptr_ = nullptr; bytes_ = 0;
    hip_check(hipMalloc(&ptr_, bytes), "hipMalloc");
    bytes_ = bytes;
}
DeviceBuffer DeviceBuffer::from_host(const void *src, size_t bytes) {
    DeviceBuffer b(bytes);
    if (bytes) hip_check(hipMemcpy(b.get(), src, bytes, hipMemcpyHostToDevice), "hipMemcpy");
    return b;
}

// ---- header parsers ---------------------------------------------------------------------------------
NintHeader parse_nint(const uint8_t *b, size_t n) {
    if (n < 18) fail("truncated NINT header");
    NintHeader h;
    h.bits = b[0]; h.sub_bits = b[1];
    h.gs = rd<int32_t>(b, 2); h.axis = rd<int32_t>(b, 6); h.neuron_len = rd<int32_t>(b, 10);
    const uint32_t ndim = rd<uint32_t>(b, 14);
    size_t off = 18;
    if (ndim > 8 || n < off + 8 * ndim + 8) fail("truncated NINT header");
    for (uint32_t i = 0; i < ndim; ++i) h.shape.push_back(rd<int64_t>(b, off + 8 * i));
    off += 8 * ndim;
    h.out = static_cast<int>(rd<uint32_t>(b, off)); h.ng = static_cast<int>(rd<uint32_t>(b, off + 4));
    off += 8;
    if (h.bits < 1 || h.bits > 8 || h.sub_bits < 1 || h.sub_bits > 8 || h.gs <= 0 || h.neuron_len <= 0 || h.out <= 0)
        fail("unsupported NINT spec");
    if (h.ng != cdiv(h.neuron_len, h.gs)) fail("NINT header group count does not match neuron_len");
    const int64_t subs = static_cast<int64_t>(h.out) * h.ng, qn = subs * h.gs;
    const int64_t packed = 4ll * h.out + 2 * ((subs * h.sub_bits + 7) / 8) + (qn * h.bits + 7) / 8;
    const int64_t old = 4ll * h.out + 2 * subs + qn;
    const int64_t remaining = static_cast<int64_t>(n) - static_cast<int64_t>(off);
    if (remaining == packed) h.legacy = false;
    else if (remaining == old) h.legacy = true;
    else fail("invalid NINT blob tail: remaining=" + std::to_string(remaining - 4ll * h.out) + ", packed=" +
              std::to_string(packed - 4ll * h.out) + ", old=" + std::to_string(old - 4ll * h.out));
    h.body_off = off; h.body_bytes = static_cast<size_t>(remaining);
    return h;
}

NvqHeader parse_nvq(const uint8_t *b, size_t n) {
    if (n < 20) fail("truncated NVQ header");
    if (std::memcmp(b, "NVQ1", 4) != 0 && std::memcmp(b, "NIQ1", 4) != 0) fail("invalid NVQ magic");
    NvqHeader h;
    const uint8_t enc = b[4];
    h.sub_bits = b[5]; h.gs = rd<uint16_t>(b, 6);
    h.neuron_len = rd<int32_t>(b, 12);
    const uint32_t ndim = rd<uint32_t>(b, 16);
    static const char *names[] = {"", "e8_256", "d4_256", "d4_512", "e8_1024", "e8_4096", "d4_1024"};
    static const int ibits[] = {0, 8, 8, 9, 10, 12, 10};
    const int cid = enc & 0x1f;
    if (cid < 1 || cid > 6) fail("unknown NVQ codebook id: " + std::to_string(cid));
    h.codebook = names[cid]; h.index_bits = ibits[cid];
    h.vector_size = h.codebook[0] == 'e' ? 8 : 4;
    h.jsc = enc & 0x20; h.index_parity = enc & 0x80;
    const bool custom = enc & 0x40;
    if (ndim > 8) fail("truncated NVQ header");
    size_t off = 20 + 8 * static_cast<size_t>(ndim);
    if (n < off + 4) fail("truncated NVQ header");
    h.out = static_cast<int>(rd<uint32_t>(b, off));
    off += 4;
    if (h.gs <= 0 || h.neuron_len <= 0 || h.out <= 0 || h.sub_bits < 1 || h.sub_bits > 8)
        fail("NVQ dimensions must be positive (groupsize, neuron_len, rows) and sub_bits in [1,8]");
    const int64_t o = h.out, ng = cdiv(h.neuron_len, h.gs), nvec = cdiv(h.neuron_len, h.vector_size),
                  nsign = cdiv(h.neuron_len, 8);
    const int64_t streams = 2 * o + (o * ng * h.sub_bits + 7) / 8 + (o * nvec * h.index_bits + 7) / 8 + (o * nsign * 7 + 7) / 8;
    int64_t expect = streams;
    h.banks = 0;
    if (h.jsc) {
        if (custom || h.index_parity || h.gs != 24 || h.sub_bits != 4) fail("invalid NVQ-JSC profile flags");
        if (n < off + 64) fail("truncated NVQ-JSC metadata header");
        const uint8_t *m = b + off;
        h.banks = m[1];
        bool reserved = false;
        for (int i = 52; i < 64; ++i) reserved |= m[i] != 0;
        if (m[0] != 1 || (h.banks != 1 && h.banks != 2 && h.banks != 4) || m[2] != 16 || m[3] > 1 || reserved)
            fail("invalid NVQ-JSC metadata");
        for (int i = 36; i < 52; ++i)
            if (m[i] >= h.banks) fail("invalid NVQ-JSC state-to-bank map");
        expect += 64 + static_cast<int64_t>(h.banks) * (1ll << h.index_bits) * h.vector_size;
        static const std::unordered_map<std::string, std::string> dt = {
            {"e8_256", "NVQ2J"}, {"e8_1024", "NVQ2J-L"}, {"e8_4096", "NVQ2J-XL"},
            {"d4_256", "NVQ3J"}, {"d4_512", "NVQ3J-512"}, {"d4_1024", "NVQ3J-L"}};
        h.dtype = dt.at(h.codebook);
    } else {
        if (custom) fail("custom-codebook NVQ blobs are outside this runtime's scope");
        h.dtype = h.codebook == "e8_256" ? "NVQ2" : h.codebook == "d4_256" ? "NVQ3" : "";
        if (h.dtype.empty()) fail(h.codebook + " requires an NVQ-JSC file profile");
    }
    if (static_cast<int64_t>(n) - static_cast<int64_t>(off) != expect)
        fail("invalid NVQ blob tail: consumed=" + std::to_string(off + expect) + ", size=" + std::to_string(n));
    h.body_off = off; h.body_bytes = static_cast<size_t>(expect);
    return h;
}

NepqHeader parse_nepq(const uint8_t *b, size_t n) {
    if (n < 36) fail("truncated NEPQ header");
    if (std::memcmp(b, "NEP1", 4) != 0 || b[4] != 1) fail("invalid or unsupported NEPQ header");
    NepqHeader h;
    h.profile = b[5];
    const int gps = b[6], flags = b[7];
    h.n_experts = static_cast<int>(rd<uint32_t>(b, 8)); h.out_per_expert = static_cast<int>(rd<uint32_t>(b, 12));
    h.neuron_len = static_cast<int>(rd<uint32_t>(b, 16)); h.banks = static_cast<int>(rd<uint32_t>(b, 20));
    h.rotation_block = static_cast<int>(rd<uint32_t>(b, 24)); h.rotation_seed = rd<uint64_t>(b, 28);
    static const char *labels[] = {"NEPQ0-S", "NEPQ0-L", "NEPQ1-S", "NEPQ1-L"};
    if (h.profile > 3 || gps != 4) fail("unsupported NEPQ super-group profile");
    h.label = labels[h.profile];
    if ((flags & ~1) || ((flags & 1) != 0) != (h.rotation_block != 0)) fail("inconsistent NEPQ rotation flag");
    if (h.n_experts <= 0 || h.out_per_expert <= 0 || h.neuron_len <= 0 || h.neuron_len % 8 || h.banks < 1 || h.banks > 256)
        fail("NEPQ shape dimensions must be positive, K divisible by 8, banks in [1,256]");
    static const int sbits[] = {2, 3, 4, 3}, ibits[] = {6, 7, 9, 11}, abits[] = {0, 0, 1, 1}, tbytes[] = {320, 832, 2048, 4096};
    const int sb = sbits[h.profile], ib = ibits[h.profile], ab = abits[h.profile], tb = tbytes[h.profile];
    const int64_t rows = static_cast<int64_t>(h.n_experts) * h.out_per_expert, ng = cdiv(h.neuron_len, 24),
                  nvec = h.neuron_len / 8, nsuper = cdiv(ng, 4);
    const int64_t expect = static_cast<int64_t>(h.banks) * tb + 2 * rows + (rows * ng * sb + 7) / 8 +
                           (rows * nvec * ib + 7) / 8 + (rows * ng * ab + 7) / 8 + rows * nsuper;
    if (static_cast<int64_t>(n) - 36 != expect)
        fail("invalid NEPQ tail: consumed=" + std::to_string(36 + expect) + ", size=" + std::to_string(n));
    if (h.profile < 2) {  // NEPQ0: every table of the pool is an NPQ0 table (mfq/formats/nepq.py:270-290)
        const int states = h.profile == 0 ? 4 : 8, version = h.profile == 0 ? 2 : 1;
        for (int bank = 0; bank < h.banks; ++bank) {
            const uint8_t *t = b + 36 + static_cast<size_t>(bank) * tb;
            if (t[0] != version || t[1] != states || t[2] != 3 || t[3] != ib - 3 || t[4] != 24 || t[5] != 8)
                fail("unsupported " + h.label + " table profile");
            bool reserved = t[6] || t[7];
            for (int i = 8 + 2 * states; i < 64; ++i) reserved = reserved || t[i];
            if (reserved) fail("invalid " + h.label + " reserved table bytes");
            float lmax = 0.f;
            for (int i = 0; i < states; ++i) {
                const float v = half_to_float(rd<uint16_t>(t, 8 + 2 * static_cast<size_t>(i)));
                if (!(v >= 0.f) || std::isinf(v)) fail(h.label + " scale LUT must be finite and non-negative");
                lmax = std::max(lmax, v);
            }
            if (lmax <= 0.f) fail(h.label + " scale LUT must be finite and non-negative");
        }
    }
    h.body_off = 36; h.body_bytes = static_cast<size_t>(expect);
    return h;
}

NintmHeader parse_nintm(const uint8_t *b, size_t n, bool allow_partial) {
    if (n < 20) fail("truncated NINTM header");
    const bool delta = std::memcmp(b, "NID2", 4) == 0;
    if (delta && !allow_partial) fail("NINTM delta cannot be loaded as a full tensor");
    if (!delta && std::memcmp(b, "NIM2", 4) != 0) fail("invalid NINTM magic");
    NintmHeader h;
    h.n_experts = static_cast<int>(rd<uint32_t>(b, 4)); h.out_per_expert = static_cast<int>(rd<uint32_t>(b, 8));
    h.neuron_len = static_cast<int>(rd<uint32_t>(b, 12));
    const uint32_t npools = rd<uint32_t>(b, 16);
    if (npools == 0 || static_cast<int>(npools) > h.n_experts) fail("invalid NINTM pool count");
    std::vector<int> owner(h.n_experts, -1);
    size_t off = 20;
    for (uint32_t pi = 0; pi < npools; ++pi) {
        if (off + 24 > n) fail("truncated NINTM v2 pool header");
        const uint32_t n_ids = rd<uint32_t>(b, off), dlen = rd<uint32_t>(b, off + 4);
        const uint64_t plen = rd<uint64_t>(b, off + 8), rlen = rd<uint64_t>(b, off + 16);
        off += 24;
        if (n_ids == 0 || dlen == 0 || dlen > 32) fail("invalid NINTM v2 pool metadata");
        // every length is compared with what is left, so that no sum of 64-bit header fields can wrap
        size_t left = n - off;
        if (4ull * n_ids > left) fail("truncated NINTM v2 pool payload");
        left -= 4ull * n_ids;
        if (dlen > left) fail("truncated NINTM v2 pool payload");
        left -= dlen;
        if (rlen > left) fail("truncated NINTM v2 pool payload");
        left -= rlen;
        if (plen > left) fail("truncated NINTM v2 pool payload");
        const size_t end = off + 4ull * n_ids + dlen + static_cast<size_t>(rlen) + static_cast<size_t>(plen);
        NintmPool p;
        for (uint32_t i = 0; i < n_ids; ++i) {
            const int32_t e = rd<int32_t>(b, off + 4ull * i);
            if (e < 0 || e >= h.n_experts) fail("NINTM pool " + std::to_string(pi) + " contains an invalid expert id");
            if (owner[e] == static_cast<int>(pi)) fail("NINTM pool " + std::to_string(pi) + " repeats an expert id");
            if (owner[e] >= 0) fail("an expert belongs to multiple NINTM pools");
            owner[e] = static_cast<int>(pi);
            p.expert_ids.push_back(e);
        }
        off += 4ull * n_ids;
        p.dtype.assign(reinterpret_cast<const char *>(b + off), dlen);
        off += dlen;
        p.runtime_off = off; p.runtime_bytes = rlen;
        p.payload_off = off + rlen; p.payload_bytes = plen;
        off = end;
        h.pools.push_back(std::move(p));
    }
    if (off != n) fail("invalid NINTM tail: " + std::to_string(n - off) + " extra bytes");
    for (int e = 0; e < h.n_experts && !allow_partial; ++e)
        if (owner[e] < 0) fail("NINTM pools do not cover expert " + std::to_string(e));
    return h;
}

// ---- weights -------------------------------------------------------------------------------------------
NintWeight NintWeight::from_blob(const uint8_t *blob, size_t n, mfq_stream_t stream) {
    const NintHeader h = parse_nint(blob, n);
    if (h.axis != 0) fail("NINT linear weights must be quantized along axis 0");
    NintWeight w;
    abi_check(mfq_hip_nint_plan(h.bits, h.sub_bits, h.gs, h.out, h.neuron_len, &w.desc));
    w.shape = h.shape;
    DeviceBuffer payload = DeviceBuffer::from_host(blob + h.body_off, h.body_bytes);
    w.data = DeviceBuffer(static_cast<size_t>(w.desc.total_bytes));
    abi_check(mfq_hip_nint_repack(&w.desc, payload.get(), static_cast<int64_t>(h.body_bytes), h.legacy ? 1 : 0,
                                  w.data.get(), stream));
    hip_check(hipStreamSynchronize(hs(stream)), "nint repack");  // the staged payload is freed on return
    return w;
}

// "<4siiI" ("NI80", axis, neuron_len, ndim) + shape i64[ndim] + out u32 + ng u32 + 34-byte blocks; the checks and
// messages of unpack_nint8_zero (cpp_runtime/mfq_decode.cpp:1601-1650)
Nint8ZeroWeight Nint8ZeroWeight::from_blob(const uint8_t *blob, size_t n, mfq_stream_t stream) {
    if (n < 24 || std::memcmp(blob, "NI80", 4) != 0) fail("invalid NINT8-0 header");
    const int axis = rd<int32_t>(blob, 4), neuron_len = rd<int32_t>(blob, 8);
    const uint32_t ndim = rd<uint32_t>(blob, 12);
    if (ndim == 0 || ndim > 8 || axis < 0 || axis >= static_cast<int>(ndim) || neuron_len <= 0 || neuron_len % 32 != 0)
        fail("invalid NINT8-0 dimensions");
    size_t off = 16;
    if (n < off + 8ull * ndim + 8) fail("invalid NINT8-0 header");
    Nint8ZeroWeight w;
    w.shape.resize(ndim);
    for (uint32_t i = 0; i < ndim; ++i, off += 8) w.shape[i] = rd<int64_t>(blob, off);
    const int64_t out = rd<uint32_t>(blob, off), ng = rd<uint32_t>(blob, off + 4);
    off += 8;
    if (out <= 0 || ng != neuron_len / 32 || w.shape[static_cast<size_t>(axis)] != out) fail("NINT8-0 shape/header mismatch");
    int64_t elements = 1;
    for (int64_t v : w.shape) {
        if (v <= 0 || elements > INT64_MAX / v) fail("invalid NINT8-0 logical shape");
        elements *= v;
    }
    if (elements != out * neuron_len) fail("NINT8-0 logical element count mismatch");
    if (n - off != static_cast<size_t>(out * ng) * 34) fail("invalid NINT8-0 block payload length");
    if (axis != 0) fail("NINT8-0 linear weights must be quantized along axis 0");
    abi_check(mfq_hip_nint8z_plan(static_cast<int>(out), neuron_len, &w.desc));
    DeviceBuffer payload = DeviceBuffer::from_host(blob + off, n - off);
    w.data = DeviceBuffer(static_cast<size_t>(w.desc.total_bytes));
    abi_check(mfq_hip_nint8z_repack(&w.desc, payload.get(), static_cast<int64_t>(n - off), w.data.get(), stream));
    hip_check(hipStreamSynchronize(hs(stream)), "nint8-0 repack");
    return w;
}

// parse_mx_layout / validate_mx_shapes (mfq/formats/mx.py:65-173; unpack_mxfp8 / unpack_mxfp4, cpp_runtime/mfq_decode.cpp:1832-1918)
MxWeight MxWeight::from_blob(const std::string &dtype, const uint8_t *blob, size_t n, int64_t out_per_expert, mfq_stream_t stream) {
    const int want_kind = dtype == "MXFP4" ? 4 : dtype == "MXFP8" ? 8 : 0;
    if (!want_kind) fail("unsupported MX dtype: " + dtype);
    if (n < 56) fail("truncated MFQ MX tensor header");
    const int version = blob[4], kind = blob[5];
    if (std::memcmp(blob, "MXT1", 4) != 0 || version != 1 || kind != want_kind || rd<uint16_t>(blob, 6) != 0)
        fail("invalid " + dtype + " payload header");
    uint64_t d[6];
    for (int i = 0; i < 6; ++i) d[i] = rd<uint64_t>(blob, 8 + 8 * static_cast<size_t>(i));
    const uint64_t rows = d[0], cols = d[1];
    if (rows == 0 || cols == 0 || rows > INT32_MAX || cols > INT32_MAX) fail("invalid MX logical shape");
    uint64_t sr, sc, qr, qc;
    if (kind == 4) {
        if (cols % 32) fail("MXFP4 columns must be divisible by 32");
        sr = rows; sc = cols / 2; qr = rows; qc = cols / 32;
    } else {
        if (cols % 128) fail("MXFP8 columns must be divisible by 128");
        sr = rows; sc = cols; qr = (rows + 127) / 128; qc = cols / 128;
    }
    if (d[2] != sr || d[3] != sc) fail(dtype + " storage shape does not match its logical shape");
    if (d[4] != qr || d[5] != qc) fail(dtype + " scale shape does not match its logical shape");
    const uint64_t nv = sr * sc, ns = qr * qc;
    if (n != 56 + nv + ns) fail(dtype + " payload size " + std::to_string(n) + " != " + std::to_string(56 + nv + ns));
    MxWeight w;
    w.kind = kind; w.rows = static_cast<int64_t>(rows); w.cols = static_cast<int64_t>(cols); w.dtype = dtype;
    w.out_per_expert = out_per_expert > 0 ? out_per_expert : w.rows;
    if (w.rows % w.out_per_expert) fail(dtype + ": the rows are not a whole number of experts");
    if (kind == 8 && w.out_per_expert != w.rows && w.out_per_expert % 128) fail("MXFP8 expert slices must preserve 128-row blocks");
    w.values = DeviceBuffer::from_host(blob + 56, nv);
    w.scales = DeviceBuffer::from_host(blob + 56 + nv, ns);
    hip_check(hipStreamSynchronize(hs(stream)), "mx upload");
    return w;
}
int64_t MxWeight::payload_bytes() const { return (kind == 4 ? rows * cols / 2 + rows * (cols / 32) : rows * cols + (rows + 127) / 128 * (cols / 128)); }

namespace {
// bits [bit0, bit0 + nbits) of the little-endian bit stream at s (which has `avail` readable bytes), as a stream of its own
std::vector<uint8_t> slice_bits(const uint8_t *s, size_t avail, int64_t bit0, int64_t nbits) {
    std::vector<uint8_t> out(static_cast<size_t>((nbits + 7) / 8), 0);
    const int sh = static_cast<int>(bit0 & 7);
    for (size_t i = 0; i < out.size(); ++i) {
        const size_t b = static_cast<size_t>(bit0 >> 3) + i;
        const uint32_t lo = b < avail ? s[b] : 0u, hi = b + 1 < avail ? s[b + 1] : 0u;
        out[i] = static_cast<uint8_t>(((lo | (hi << 8)) >> sh) & 0xffu);
    }
    if (nbits & 7) out.back() &= static_cast<uint8_t>((1u << (nbits & 7)) - 1u);
    return out;
}
}  // namespace

std::vector<std::vector<uint8_t>> split_rows(const std::string &dtype, const uint8_t *b, size_t n, int parts) {
    size_t body_off, tables;
    int64_t out, K;
    std::vector<int64_t> per_row;
    if (dtype == "NINT8-0") {  // [rows, K] along axis 0: a row is its ng blocks of 34 bytes, back to back
        if (n < 40 || std::memcmp(b, "NI80", 4) != 0) fail("invalid NINT8-0 header");
        const int axis = rd<int32_t>(b, 4), neuron_len = rd<int32_t>(b, 8);
        const uint32_t ndim = rd<uint32_t>(b, 12);
        if (axis != 0 || ndim != 2 || neuron_len <= 0 || neuron_len % 32) fail("NINT8-0 cohorts are [rows, K] tensors quantized along axis 0");
        const int64_t rows_all = rd<uint32_t>(b, 32), ng = rd<uint32_t>(b, 36);
        if (rows_all <= 0 || ng != neuron_len / 32 || n - 40 != static_cast<size_t>(rows_all * ng) * 34) fail("invalid NINT8-0 block payload length");
        if (parts <= 0 || rows_all % parts) fail(dtype + ": " + std::to_string(rows_all) + " neurons do not split into " + std::to_string(parts) + " equal parts");
        const int64_t rows = rows_all / parts;
        const size_t piece_bytes = static_cast<size_t>(rows * ng) * 34;
        std::vector<std::vector<uint8_t>> res;
        for (int i = 0; i < parts; ++i) {
            std::vector<uint8_t> v(b, b + 16);  // magic, axis, neuron_len, ndim
            auto put = [&](const void *p, size_t len) { const uint8_t *q = static_cast<const uint8_t *>(p); v.insert(v.end(), q, q + len); };
            const int64_t shape[2] = {rows, neuron_len};
            const uint32_t tail[2] = {static_cast<uint32_t>(rows), static_cast<uint32_t>(ng)};
            put(shape, 16); put(tail, 8);
            put(b + 40 + static_cast<size_t>(i) * piece_bytes, piece_bytes);
            res.push_back(std::move(v));
        }
        return res;
    }
    if (is_lowbit_linear_dtype(dtype)) {
        if (n < 20) fail("truncated " + dtype + " header");
        const int ver = b[4], sbits = b[5];
        K = rd<int32_t>(b, 12);
        const uint32_t ndim = rd<uint32_t>(b, 16);
        if (ndim == 0 || ndim > 8 || K <= 0 || n < 24 + 8 * static_cast<size_t>(ndim)) fail("invalid " + dtype + " dimensions");
        out = rd<uint32_t>(b, 20 + 8 * static_cast<size_t>(ndim));
        body_off = 24 + 8 * static_cast<size_t>(ndim);
        const bool nvq1l = dtype == "NVQ1-L", ternary = dtype[1] == 'V';
        tables = nvq1l ? (ver == 2 ? 4096 : 0) : dtype == "NVQ1-S" ? 2048 : dtype == "NPQ0-L" ? 832 : 320;
        const int ib = nvq1l ? 11 : dtype == "NVQ1-S" ? 9 : dtype == "NPQ0-L" ? 7 : 6;
        const int64_t ng = cdiv(K, 24), nvec = nvq1l ? cdiv(K, 8) : K / 8;
        per_row = {sbits * ng, ib * nvec};
        if (ternary) per_row.push_back(ng);
    } else {
        const NvqHeader h = parse_nvq(b, n);
        body_off = h.body_off; out = h.out; K = h.neuron_len;
        tables = h.jsc ? 64 + static_cast<size_t>(h.banks) * (1ull << h.index_bits) * h.vector_size : 0;
        per_row = {static_cast<int64_t>(h.sub_bits) * cdiv(K, h.gs), static_cast<int64_t>(h.index_bits) * cdiv(K, h.vector_size),
                   7 * cdiv(K, 8)};
    }
    if (parts <= 0 || out <= 0 || out % parts) fail(dtype + ": " + std::to_string(out) + " neurons do not split into " +
                                                     std::to_string(parts) + " equal parts");
    const int64_t rows = out / parts;
    const size_t anchors_off = body_off + tables;
    std::vector<size_t> stream_off;
    size_t off = anchors_off + 2 * static_cast<size_t>(out);
    for (int64_t bits : per_row) {
        stream_off.push_back(off);
        off += static_cast<size_t>((out * bits + 7) / 8);
    }
    if (off != n) fail("invalid " + dtype + " blob tail: consumed=" + std::to_string(off) + ", size=" + std::to_string(n));
    std::vector<std::vector<uint8_t>> res;
    for (int i = 0; i < parts; ++i) {
        std::vector<uint8_t> piece(b, b + 8);  // magic, flags / version, state bits, groupsize
        auto put = [&](const void *p, size_t bytes) {
            const uint8_t *q = static_cast<const uint8_t *>(p);
            piece.insert(piece.end(), q, q + bytes);
        };
        const int32_t axis = 0, k32 = static_cast<int32_t>(K);
        const uint32_t ndim = 2, o32 = static_cast<uint32_t>(rows);
        const int64_t shape[2] = {rows, K};
        put(&axis, 4); put(&k32, 4); put(&ndim, 4); put(shape, 16); put(&o32, 4);
        put(b + body_off, tables);
        put(b + anchors_off + 2 * static_cast<size_t>(i * rows), 2 * static_cast<size_t>(rows));
        for (size_t si = 0; si < per_row.size(); ++si) {
            const std::vector<uint8_t> bits = slice_bits(b + stream_off[si], n - stream_off[si], i * rows * per_row[si], rows * per_row[si]);
            put(bits.data(), bits.size());
        }
        res.push_back(std::move(piece));
    }
    return res;
}

// Header, shape and table checks of the reference's loaders for the 1-bit families, with their messages
// (mfq/formats/nvq1_l.py:287-345, nvq1_s.py:293-347, npq0_l.py:354-415, npq0_s.py:348-406; mfq_decode.cpp:3800-3910).
NvqWeight NvqWeight::from_lowbit_blob(const std::string &dtype, const uint8_t *b, size_t n, const uint16_t *iq1s_grid,
                                      mfq_stream_t stream) {
    struct Fmt { const char *magic; int version, state_bits, index_bits, format, table_version, states, second; };
    static const std::unordered_map<std::string, Fmt> fmts = {
        {"NVQ1-L", {"NQ1L", 0, 0, 11, MFQ_NVQS_NVQ1_L, 0, 0, 0}}, {"NVQ1-S", {"NQ1S", 1, 4, 9, MFQ_NVQS_NVQ1_S, 0, 0, 0}},
        {"NPQ0-L", {"NPQL", 1, 3, 7, MFQ_NVQS_NPQ0_L, 1, 8, 16}}, {"NPQ0-S", {"NPQS", 2, 2, 6, MFQ_NVQS_NPQ0_S, 2, 4, 8}}};
    const auto it = fmts.find(dtype);
    if (it == fmts.end()) fail("unsupported quantized linear dtype: " + dtype);
    const Fmt &f = it->second;
    if (n < 20) fail("truncated " + dtype + " header");
    if (std::memcmp(b, f.magic, 4) != 0) fail("invalid " + dtype + " magic");
    const int ver = b[4], sbits = b[5], gs = rd<uint16_t>(b, 6), neuron_len = rd<int32_t>(b, 12);
    const uint32_t ndim = rd<uint32_t>(b, 16);
    const bool nvq1l = dtype == "NVQ1-L", ternary = dtype[1] == 'V';
    if (nvq1l) {
        if (ver != 1 && ver != 2) fail("unsupported NVQ1-L profile: " + std::to_string(ver));
        if (gs != 24 || (sbits != 3 && sbits != 4)) fail("unsupported NVQ1-L profile");
    } else if (ver != f.version || sbits != f.state_bits || gs != 24) {
        fail("unsupported " + dtype + " stream profile");
    }
    if (ndim == 0 || ndim > 8 || neuron_len <= 0 || (!nvq1l && neuron_len % 8)) fail("invalid " + dtype + " dimensions");
    size_t off = 20 + 8 * static_cast<size_t>(ndim);
    if (n < off + 4) fail("truncated " + dtype + " shape");
    int64_t elements = 1;
    for (uint32_t i = 0; i < ndim; ++i) {
        const int64_t v = rd<int64_t>(b, 20 + 8 * static_cast<size_t>(i));
        if (v <= 0 || elements > INT64_MAX / v) fail(dtype + " shape does not match neuron dimensions");
        elements *= v;
    }
    const int64_t out = rd<uint32_t>(b, off);
    off += 4;
    if (out <= 0 || out > INT32_MAX || elements != out * neuron_len) fail(dtype + " shape does not match neuron dimensions");
    size_t table = 0;
    if (nvq1l) table = ver == 2 ? 4096 : 0;
    else if (ternary) table = 2048;
    else {
        table = 64 + static_cast<size_t>(f.states) * 32 + static_cast<size_t>(f.states) * f.second * 4;
        if (n < off + table) fail("truncated " + dtype + " product tables");
        const uint8_t *t = b + off;
        if (t[0] != f.table_version || t[1] != f.states || t[2] != 3 || t[3] != f.index_bits - 3 || t[4] != 24 || t[5] != 8)
            fail("unsupported " + dtype + " table profile");
        bool reserved = t[6] || t[7];
        for (int i = 8 + 2 * f.states; i < 64; ++i) reserved = reserved || t[i];
        if (reserved) fail("invalid " + dtype + " reserved table bytes");
        float lmax = 0.f;
        for (int i = 0; i < f.states; ++i) {
            const float v = half_to_float(rd<uint16_t>(t, 8 + 2 * static_cast<size_t>(i)));
            if (!(v >= 0.f) || std::isinf(v)) fail(dtype + " scale LUT must be finite and non-negative");
            lmax = std::max(lmax, v);
        }
        if (lmax <= 0.f) fail(dtype + " scale LUT must be finite and non-negative");
    }
    if (ternary && table) {
        if (n < off + table) fail("truncated " + dtype + " codebook");
        for (size_t i = 0; i < table / 2; ++i) {
            const uint16_t e = rd<uint16_t>(b, off + 2 * i);
            if (e & (e >> 1) & 0x5555u) fail("packed " + dtype + " codebook contains a non-ternary digit");
        }
    }
    const int64_t ng = cdiv(neuron_len, 24), nvec = nvq1l ? cdiv(neuron_len, 8) : neuron_len / 8;
    const int64_t streams = 2 * out + (out * ng * sbits + 7) / 8 + (out * nvec * f.index_bits + 7) / 8 +
                            (ternary ? (out * ng + 7) / 8 : 0);
    const int64_t expect = static_cast<int64_t>(table) + streams;
    if (static_cast<int64_t>(n) - static_cast<int64_t>(off) != expect)
        fail("invalid " + dtype + " blob tail: remaining=" + std::to_string(n - off) + ", expected=" + std::to_string(expect));
    NvqWeight w;
    w.dtype = dtype;
    w.streams = true;
    abi_check(mfq_hip_nvqs_plan_lowbit(f.format, sbits, static_cast<int>(out), neuron_len, &w.sdesc));
    DeviceBuffer body = DeviceBuffer::from_host(b + off, static_cast<size_t>(expect));
    DeviceBuffer grid;
    if (nvq1l && !table) {
        if (!iq1s_grid) fail("an NVQ1-L blob without a table needs the built-in 2048-entry ternary grid");
        grid = DeviceBuffer::from_host(iq1s_grid, 4096);
    }
    w.data = DeviceBuffer(static_cast<size_t>(w.sdesc.total_bytes));
    abi_check(mfq_hip_nvqs_repack_lowbit(&w.sdesc, body.get(), expect, grid.get(), w.data.get(), stream));
    hip_check(hipStreamSynchronize(hs(stream)), "1-bit family repack");
    return w;
}

NvqWeight NvqWeight::from_blob(const uint8_t *blob, size_t n, const int8_t *grid256, mfq_stream_t stream) {
    const NvqHeader h = parse_nvq(blob, n);
    NvqWeight w;
    w.dtype = h.dtype;
    if (h.vector_size != 4 || h.index_bits > 9) {  // E8 family, d4_1024: the streams are read in place
        if (h.gs != 24 || h.sub_bits != 4) fail(h.dtype + ": NVQ runs only with gs24 and 4-bit states");
        if (!h.jsc && !grid256) fail("plain NVQ2 needs the 256-entry E8 magnitude grid");
        w.streams = true;
        abi_check(mfq_hip_nvqs_plan(h.vector_size, h.index_bits, h.jsc ? h.banks : 1, h.index_parity ? 1 : 0, h.out,
                                    h.neuron_len, &w.sdesc));
        DeviceBuffer payload = DeviceBuffer::from_host(blob + h.body_off, h.body_bytes);
        DeviceBuffer grid;
        if (!h.jsc) grid = DeviceBuffer::from_host(grid256, 256ull * h.vector_size);
        w.data = DeviceBuffer(static_cast<size_t>(w.sdesc.total_bytes));
        abi_check(mfq_hip_nvqs_repack(&w.sdesc, payload.get(), static_cast<int64_t>(h.body_bytes), h.jsc ? 1 : 0, grid.get(),
                                      w.data.get(), stream));
        hip_check(hipStreamSynchronize(hs(stream)), "nvq repack");
        return w;
    }
    abi_check(mfq_hip_nvq_plan(h.index_bits, h.jsc ? h.banks : 1, h.out, h.neuron_len, &w.desc));
    DeviceBuffer payload = DeviceBuffer::from_host(blob + h.body_off, h.body_bytes);
    w.data = DeviceBuffer(static_cast<size_t>(w.desc.total_bytes));
    if (h.jsc) {
        abi_check(mfq_hip_nvq_repack(&w.desc, payload.get(), static_cast<int64_t>(h.body_bytes), w.data.get(), stream));
    } else {
        if (h.gs != 24 || h.sub_bits != 4 || h.index_parity)
            fail("plain NVQ3 runs only with gs24, 4-bit sub-scales and parity signs");
        if (!grid256) fail("plain NVQ3 needs the 256-entry D4 magnitude grid");
        DeviceBuffer grid = DeviceBuffer::from_host(grid256, 1024);
        abi_check(mfq_hip_nvq_repack_plain(&w.desc, payload.get(), static_cast<int64_t>(h.body_bytes), grid.get(),
                                           w.data.get(), stream));
        hip_check(hipStreamSynchronize(hs(stream)), "nvq repack");
    }
    hip_check(hipStreamSynchronize(hs(stream)), "nvq repack");
    return w;
}

NepqWeight NepqWeight::from_blob(const uint8_t *blob, size_t n, const int8_t *rotation_signs, mfq_stream_t stream) {
    const NepqHeader h = parse_nepq(blob, n);
    NepqWeight w;
    w.label = h.label; w.n_experts = h.n_experts; w.out_per_expert = h.out_per_expert; w.rotation_block = h.rotation_block;
    DeviceBuffer payload = DeviceBuffer::from_host(blob + h.body_off, h.body_bytes);
    if (h.profile < 2) {  // NEPQ0: read in place by the stream kernels
        w.streams = true;
        abi_check(mfq_hip_nvqs_plan_nepq0(h.profile, h.banks, h.n_experts * h.out_per_expert, h.neuron_len, &w.sdesc));
        w.data = DeviceBuffer(static_cast<size_t>(w.sdesc.total_bytes));
        abi_check(mfq_hip_nvqs_repack_nepq0(&w.sdesc, payload.get(), static_cast<int64_t>(h.body_bytes), w.data.get(), stream));
    } else {
        abi_check(mfq_hip_nepq_plan(h.profile, h.banks, h.n_experts * h.out_per_expert, h.neuron_len, &w.desc));
        w.data = DeviceBuffer(static_cast<size_t>(w.desc.total_bytes));
        abi_check(mfq_hip_nepq_repack(&w.desc, payload.get(), static_cast<int64_t>(h.body_bytes), w.data.get(), stream));
    }
    hip_check(hipStreamSynchronize(hs(stream)), "nepq repack");
    if (h.rotation_block) {
        if (!rotation_signs) fail("rotated NEPQ cohort lacks its runtime sign vector");
        for (int i = 0; i < h.neuron_len; ++i)
            if (rotation_signs[i] != 1 && rotation_signs[i] != -1) fail("NEPQ rotation sign vector is corrupt");
        w.signs = DeviceBuffer::from_host(rotation_signs, static_cast<size_t>(h.neuron_len));
    }
    return w;
}

void nint_matmul(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) {
    const size_t need = mfq_hip_nint_gemm_workspace_bytes(&w.desc, M);
    w.workspace.ensure(need);
    abi_check(mfq_hip_nint_gemm(&w.desc, w.data.get(), x, x_dtype, ldx, M, y, w.desc.out, w.workspace.get(), need, stream));
}
static void nint_matmul_glu(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, void *hidden, float *scratch,
                            int activation, const char *what, mfq_stream_t stream) {
    const int W = w.desc.out / 2;
    const bool unit = w.desc.kind == 1 || (w.desc.bits == 5 && w.desc.gs == 28);
    if (M <= 2 && w.desc.out % 32 == 0 && unit) {
        abi_check(mfq_hip_nint_gemv_glu(&w.desc, w.data.get(), x, x_dtype, ldx, M, hidden, MFQ_X_F16, W, activation, stream));
        return;
    }
    if (w.desc.out % 32 == 0 && unit) {  // prefill batches: the block-tiled kernel with the GLU in its epilogue, where it runs
        const size_t need = mfq_hip_nint_gemm_workspace_bytes(&w.desc, M);
        w.workspace.ensure(need);
        const int rc = mfq_hip_nint_gemm_glu(&w.desc, w.data.get(), x, x_dtype, ldx, M, activation, hidden, MFQ_X_F16, W,
                                             w.workspace.get(), need, stream);
        if (rc == MFQ_OK) return;
        if (rc != MFQ_ERR_UNSUPPORTED) abi_check(rc);
    }
    if (!scratch) fail(std::string(what) + ": this batch needs a [M, 2W] fp32 scratch buffer");
    nint_matmul(w, x, x_dtype, ldx, M, scratch, stream);
    abi_check(mfq_hip_moe_glu(scratch, 2 * W, M, W, hidden, MFQ_X_F16, W, activation, stream));
}
void nint_matmul_swiglu(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, void *hidden, float *scratch,
                        mfq_stream_t stream) {
    nint_matmul_glu(w, x, x_dtype, ldx, M, hidden, scratch, MFQ_GLU_SILU, "nint_matmul_swiglu", stream);
}
void nint_matmul_geglu(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, void *hidden, float *scratch,
                       mfq_stream_t stream) {
    nint_matmul_glu(w, x, x_dtype, ldx, M, hidden, scratch, MFQ_GLU_GELU, "nint_matmul_geglu", stream);
}
void nint_matmul_input_mul(const NintWeight &w, const void *x, const void *gate, int x_dtype, int64_t ldx, int64_t ldg, int M,
                           int mode, void *gated, float *y, mfq_stream_t stream) {
    const int K = w.desc.neuron_len;
    if (M <= 2) {  // the GEMV gates its own activation slices
        const int rc = mfq_hip_nint_gemv_gate(&w.desc, w.data.get(), x, gate, x_dtype, ldx, ldg, M, mode, y, w.desc.out, stream);
        if (rc == MFQ_OK) return;
        if (rc != MFQ_ERR_UNSUPPORTED) abi_check(rc);
    }
    if (!gated) fail("nint_matmul_input_mul: needs a [M, K] 16-bit buffer for the gated activations");
    abi_check(mfq_hip_input_gate(x, gate, x_dtype, ldx, ldg, M, K, mode, gated, K, stream));
    nint_matmul(w, gated, x_dtype, K, M, y, stream);
}
void nint_embedding(const NintWeight &w, const int64_t *ids, int n_ids, void *out, int out_dtype, mfq_stream_t stream) {
    abi_check(mfq_hip_nint_embedding(&w.desc, w.data.get(), ids, n_ids, out, out_dtype, w.desc.neuron_len, stream));
}
void nint8_zero_embedding(const Nint8ZeroWeight &w, const int64_t *ids, int n_ids, void *out, int out_dtype,
                          mfq_stream_t stream) {
    abi_check(mfq_hip_nint8z_embedding(&w.desc, w.data.get(), ids, n_ids, out, out_dtype, w.desc.neuron_len, stream));
}
void nvq_embedding(const NvqWeight &w, const int64_t *ids, int n_ids, void *out, int out_dtype, mfq_stream_t stream) {
    if (w.streams) abi_check(mfq_hip_nvqs_embedding(&w.sdesc, w.data.get(), ids, n_ids, out, out_dtype, w.sdesc.neuron_len, stream));
    else abi_check(mfq_hip_nvq_embedding(&w.desc, w.data.get(), ids, n_ids, out, out_dtype, w.desc.neuron_len, stream));
}
void nint_matmul_argmax(const NintWeight &w, const void *x, int x_dtype, int64_t ldx, int M, int64_t *token, float *logits,
                        mfq_stream_t stream) {
    const size_t need = mfq_hip_nint_gemv_argmax_workspace_bytes(&w.desc, M);
    w.workspace.ensure(need);
    abi_check(mfq_hip_nint_gemv_argmax(&w.desc, w.data.get(), x, x_dtype, ldx, M, logits, w.desc.out, token,
                                       w.workspace.get(), need, stream));
}
void nvq_matmul(const NvqWeight &w, const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) {
    if (w.streams) {
        const size_t need = mfq_hip_nvqs_gemm_workspace_bytes(&w.sdesc, M);
        w.workspace.ensure(need);
        abi_check(mfq_hip_nvqs_gemm(&w.sdesc, w.data.get(), x, x_dtype, ldx, M, y, w.sdesc.out, w.workspace.get(), need, stream));
        return;
    }
    const size_t need = mfq_hip_nvq_gemm_workspace_bytes(&w.desc, M);
    w.workspace.ensure(need);
    abi_check(mfq_hip_nvq_gemm(&w.desc, w.data.get(), x, x_dtype, ldx, M, y, w.desc.out, w.workspace.get(), need, stream));
}
void nvq_matmul_multi2(const NvqWeight &first, const NvqWeight &second, const void *x, int x_dtype, int64_t ldx, int M,
                       float *y, mfq_stream_t stream) {
    if (first.neuron_len() != second.neuron_len()) fail("NVQ multi-projection requires compatible formats and input layouts");
    const int64_t N = first.out() + second.out();
    if (first.streams || second.streams) {  // no joint launch for tensors read from their streams: each into its columns
        // a grow-only buffer of the first tensor holds one projection at a time; the stream orders its two uses
        DeviceBuffer &tmp = first.pair_tmp;
        tmp.ensure(static_cast<size_t>(M) * static_cast<size_t>(std::max(first.out(), second.out())) * 4);
        for (const NvqWeight *w : {&first, &second}) {
            nvq_matmul(*w, x, x_dtype, ldx, M, static_cast<float *>(tmp.get()), stream);
            hip_check(hipMemcpy2DAsync(y + (w == &second ? first.out() : 0), static_cast<size_t>(N) * 4, tmp.get(),
                                       static_cast<size_t>(w->out()) * 4, static_cast<size_t>(w->out()) * 4, M,
                                       hipMemcpyDeviceToDevice, hs(stream)), "nvq_matmul_multi2");
        }
        return;
    }
    if (M <= 32) {
        abi_check(mfq_hip_nvq_gemv_multi2(&first.desc, first.data.get(), &second.desc, second.data.get(), x, x_dtype, ldx, M, y, N,
                                          stream));
        return;
    }
    // larger batches: the two matmuls, each into its columns
    for (const NvqWeight *w : {&first, &second}) {
        const size_t need = mfq_hip_nvq_gemm_workspace_bytes(&w->desc, M);
        w->workspace.ensure(need);
        abi_check(mfq_hip_nvq_gemm(&w->desc, w->data.get(), x, x_dtype, ldx, M, y + (w == &second ? first.desc.out : 0), N,
                                   w->workspace.get(), need, stream));
    }
}
void nvq_matmul_swiglu(const NvqWeight &gate, const NvqWeight &up, const void *x, int x_dtype, int64_t ldx, int M, void *hidden,
                       float *scratch, mfq_stream_t stream) {
    if (gate.neuron_len() != up.neuron_len() || gate.out() != up.out())
        fail("NVQ SwiGLU requires compatible equal-width gate/up weights");
    if (!scratch) fail("nvq_matmul_swiglu: needs a [M, 2W] fp32 scratch buffer");
    const int W = static_cast<int>(gate.out());
    nvq_matmul_multi2(gate, up, x, x_dtype, ldx, M, scratch, stream);
    abi_check(mfq_hip_moe_swiglu(scratch, 2 * W, M, W, hidden, MFQ_X_F16, W, stream));
}
void nvq_ffn_swiglu_down(const NvqWeight &gate, const NvqWeight &up, const NvqWeight &down, const void *x, int x_dtype,
                         int64_t ldx, int M, float *y, void *hidden, float *scratch, mfq_stream_t stream) {
    if (gate.neuron_len() != up.neuron_len() || gate.out() != up.out() || gate.out() != down.neuron_len())
        fail("NVQ fused FFN weight layouts are incompatible");
    if (!hidden) fail("nvq_ffn_swiglu_down: needs a [M, W] fp16 buffer for the hidden rows");
    nvq_matmul_swiglu(gate, up, x, x_dtype, ldx, M, hidden, scratch, stream);
    nvq_matmul(down, hidden, MFQ_X_F16, gate.out(), M, y, stream);
}
void nepq_matmul(const NepqWeight &w, int expert, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                 mfq_stream_t stream) {
    if (expert < 0 || expert >= w.n_experts) fail("expert outside the NEPQ tensor");
    const int K = static_cast<int>(w.neuron_len());
    if (w.rotation_block) {
        w.rotated.ensure(static_cast<size_t>(M) * K * 2);
        abi_check(mfq_hip_nepq_hadamard(x, x_dtype, ldx, M, K, w.rotation_block, static_cast<const int8_t *>(w.signs.get()),
                                        w.rotated.get(), K, stream));
        x = w.rotated.get();
        ldx = K;
    }
    if (w.streams) {
        const size_t need = mfq_hip_nvqs_gemm_rows_workspace_bytes(&w.sdesc, w.out_per_expert, M);
        w.workspace.ensure(need);
        abi_check(mfq_hip_nvqs_gemm_rows(&w.sdesc, w.data.get(), expert * w.out_per_expert, w.out_per_expert, x, x_dtype, ldx, M,
                                         y, w.out_per_expert, w.workspace.get(), need, stream));
        return;
    }
    const size_t need = mfq_hip_nepq_gemm_workspace_bytes(&w.desc, w.out_per_expert, M);
    w.workspace.ensure(need);
    abi_check(mfq_hip_nepq_gemm(&w.desc, w.data.get(), expert * w.out_per_expert, w.out_per_expert, x, x_dtype, ldx, M, y,
                                w.out_per_expert, w.workspace.get(), need, stream));
}
void nint_dequantize(const NintWeight &w, float *out, mfq_stream_t stream) {
    abi_check(mfq_hip_nint_dequant_f32(&w.desc, w.data.get(), out, w.desc.neuron_len, stream));
}
void nint8_zero_matmul(const Nint8ZeroWeight &w, const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) {
    const size_t need = mfq_hip_nint8z_gemm_workspace_bytes(&w.desc, M);
    w.workspace.ensure(need);
    abi_check(mfq_hip_nint8z_gemm(&w.desc, w.data.get(), x, x_dtype, ldx, M, y, w.desc.out, w.workspace.get(), need, stream));
}
void nint8_zero_dequantize(const Nint8ZeroWeight &w, float *out, mfq_stream_t stream) {
    abi_check(mfq_hip_nint8z_dequant_f32(&w.desc, w.data.get(), out, w.desc.neuron_len, stream));
}
void mx_matmul(const MxWeight &w, int expert, const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) {
    if (expert < 0 || expert >= w.n_experts()) fail(w.dtype + ": expert index out of range");
    const int nrows = static_cast<int>(w.out_per_expert), row0 = expert * nrows;
    const size_t need = mfq_hip_mx_gemm_rows_workspace_bytes(static_cast<int>(w.cols), nrows, M);
    w.workspace.ensure(need);
    abi_check(mfq_hip_mx_gemm_rows(w.kind, w.values.get(), w.scales.get(), static_cast<int>(w.rows), static_cast<int>(w.cols), row0,
                                   nrows, x, x_dtype, ldx, M, y, nrows, w.workspace.get(), need, stream));
}
void mx_dequantize(const MxWeight &w, int expert, float *out, mfq_stream_t stream) {
    if (expert < 0 || expert >= w.n_experts()) fail(w.dtype + ": expert index out of range");
    const int nrows = static_cast<int>(w.out_per_expert), row0 = expert * nrows;
    abi_check(mfq_hip_mx_dequant_rows(w.kind, w.values.get(), w.scales.get(), static_cast<int>(w.rows), static_cast<int>(w.cols),
                                      row0, nrows, MFQ_X_F32, out, w.cols, stream));
}
void nvq_dequantize(const NvqWeight &w, float *out, mfq_stream_t stream) {
    if (w.streams) {
        abi_check(mfq_hip_nvqs_dequant_f32(&w.sdesc, w.data.get(), out, w.sdesc.neuron_len, stream));
        return;
    }
    abi_check(mfq_hip_nvq_dequant_f32(&w.desc, w.data.get(), out, w.desc.neuron_len, stream));
}
void nepq_dequantize(const NepqWeight &w, float *out, mfq_stream_t stream) {
    if (w.streams) {
        abi_check(mfq_hip_nvqs_dequant_rows_f32(&w.sdesc, w.data.get(), 0, w.sdesc.out, out, w.sdesc.neuron_len, stream));
        return;
    }
    abi_check(mfq_hip_nepq_dequant_f32(&w.desc, w.data.get(), out, w.desc.neuron_len, stream));
}

// ---- registry -------------------------------------------------------------------------------------------
bool is_nint_linear_dtype(const std::string &d) {
    if (d.size() <= 4 || d.compare(0, 4, "NINT") != 0) return false;
    return std::all_of(d.begin() + 4, d.end(), [](char c) { return c >= '0' && c <= '9'; });
}
bool is_nvq_linear_dtype(const std::string &d) {
    return d == "NVQ3" || d == "NVQ3J" || d == "NVQ3J-512" || d == "NVQ3J-L" || d == "NVQ2" || d == "NVQ2J" || d == "NVQ2J-L" ||
           d == "NVQ2J-XL" || d == "NIQ3" || d == "NIQ2" || d == "NIQ2J";
}
bool is_nepq_linear_dtype(const std::string &d) { return d == "NEPQ1-S" || d == "NEPQ1-L" || d == "NEPQ0-S" || d == "NEPQ0-L"; }
bool is_lowbit_linear_dtype(const std::string &d) { return d == "NVQ1-L" || d == "NVQ1-S" || d == "NPQ0-L" || d == "NPQ0-S"; }
bool is_mx_linear_dtype(const std::string &d) { return d == "MXFP4" || d == "MXFP8"; }

int64_t QuantLinear::out() const {
    return kind == QuantLinearKind::Nint ? nint->out() : kind == QuantLinearKind::Nvq ? nvq->out()
         : kind == QuantLinearKind::Nepq ? nepq->out() : kind == QuantLinearKind::Mx ? mx->out() : nint8z->out();
}
int64_t QuantLinear::neuron_len() const {
    return kind == QuantLinearKind::Nint ? nint->neuron_len() : kind == QuantLinearKind::Nvq ? nvq->neuron_len()
         : kind == QuantLinearKind::Nepq ? nepq->neuron_len() : kind == QuantLinearKind::Mx ? mx->neuron_len() : nint8z->neuron_len();
}
int64_t QuantLinear::payload_bytes() const {
    return kind == QuantLinearKind::Nint ? nint->desc.payload_bytes : kind == QuantLinearKind::Nvq ? nvq->payload_bytes()
         : kind == QuantLinearKind::Nepq ? nepq->payload_bytes() : kind == QuantLinearKind::Mx ? mx->payload_bytes()
         : nint8z->desc.payload_bytes;
}
void QuantLinear::forward(const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) const {
    if (M == 0) return;  // an empty batch: no rows to write
    if (kind == QuantLinearKind::Nint) nint_matmul(*nint, x, x_dtype, ldx, M, y, stream);
    else if (kind == QuantLinearKind::Nvq) nvq_matmul(*nvq, x, x_dtype, ldx, M, y, stream);
    else if (kind == QuantLinearKind::Nepq) nepq_matmul(*nepq, 0, x, x_dtype, ldx, M, y, stream);
    else if (kind == QuantLinearKind::Mx) mx_matmul(*mx, 0, x, x_dtype, ldx, M, y, stream);
    else nint8_zero_matmul(*nint8z, x, x_dtype, ldx, M, y, stream);
}
void QuantLinear::reserve(int max_M) const {
    // the need is not monotonic in M (the kernels change with the batch): take the largest over every batch size up to 512
    // rows, every multiple of 64 beyond, and max_M itself
    size_t need = 0, rot = 0;
    auto one = [&](int M) {
        size_t n = 0;
        if (kind == QuantLinearKind::Nint) n = mfq_hip_nint_gemm_workspace_bytes(&nint->desc, M);
        else if (kind == QuantLinearKind::Nvq)
            n = nvq->streams ? mfq_hip_nvqs_gemm_workspace_bytes(&nvq->sdesc, M) : mfq_hip_nvq_gemm_workspace_bytes(&nvq->desc, M);
        else if (kind == QuantLinearKind::Nepq)
            n = nepq->streams ? mfq_hip_nvqs_gemm_rows_workspace_bytes(&nepq->sdesc, nepq->out_per_expert, M)
                              : mfq_hip_nepq_gemm_workspace_bytes(&nepq->desc, nepq->out_per_expert, M);
        else if (kind == QuantLinearKind::Mx)
            n = mfq_hip_mx_gemm_rows_workspace_bytes(static_cast<int>(mx->cols), static_cast<int>(mx->out_per_expert), M);
        else n = mfq_hip_nint8z_gemm_workspace_bytes(&nint8z->desc, M);
        need = std::max(need, n);
    };
    for (int M = 1; M <= std::min(max_M, 512); ++M) one(M);
    for (int M = 576; M < max_M; M += 64) one(M);
    if (max_M > 0) one(max_M);
    if (kind == QuantLinearKind::Nint) nint->workspace.ensure(need);
    else if (kind == QuantLinearKind::Nvq) nvq->workspace.ensure(need);
    else if (kind == QuantLinearKind::Nepq) {
        nepq->workspace.ensure(need);
        if (nepq->rotation_block) rot = static_cast<size_t>(std::max(max_M, 0)) * nepq->neuron_len() * 2;
        nepq->rotated.ensure(rot);
    } else if (kind == QuantLinearKind::Mx) mx->workspace.ensure(need);
    else nint8z->workspace.ensure(need);
}
void QuantLinear::dequantize(float *out, mfq_stream_t stream) const {
    if (kind == QuantLinearKind::Nint) nint_dequantize(*nint, out, stream);
    else if (kind == QuantLinearKind::Nvq) nvq_dequantize(*nvq, out, stream);
    else if (kind == QuantLinearKind::Nepq) nepq_dequantize(*nepq, out, stream);
    else if (kind == QuantLinearKind::Mx) mx_dequantize(*mx, 0, out, stream);
    else nint8_zero_dequantize(*nint8z, out, stream);
}

void QuantLinear::embedding(const int64_t *ids, int n_ids, void *out, int out_dtype, mfq_stream_t stream) const {
    if (kind == QuantLinearKind::Nint) nint_embedding(*nint, ids, n_ids, out, out_dtype, stream);
    else if (kind == QuantLinearKind::Nint8Zero) nint8_zero_embedding(*nint8z, ids, n_ids, out, out_dtype, stream);
    else if (kind == QuantLinearKind::Nvq) nvq_embedding(*nvq, ids, n_ids, out, out_dtype, stream);
    else fail("token embeddings need a NINT, NINT8-0 or NVQ table");
}

QuantLinear load_quant_linear(const std::string &dtype_in, const uint8_t *blob, size_t n, mfq_stream_t stream) {
    const std::string dtype = dtype_in == "NIQ3" ? "NVQ3" : dtype_in == "NIQ2" ? "NVQ2" : dtype_in == "NIQ2J" ? "NVQ2J" : dtype_in;
    QuantLinear q;
    if (is_nint_linear_dtype(dtype)) {
        q.kind = QuantLinearKind::Nint;
        q.nint = std::make_shared<NintWeight>(NintWeight::from_blob(blob, n, stream));
        if ("NINT" + std::to_string(q.nint->desc.bits) != dtype)
            fail("MFQ dtype/blob mismatch: " + dtype + " contains NINT" + std::to_string(q.nint->desc.bits));
        return q;
    }
    if (dtype == "NINT8-0") {
        q.kind = QuantLinearKind::Nint8Zero;
        q.nint8z = std::make_shared<Nint8ZeroWeight>(Nint8ZeroWeight::from_blob(blob, n, stream));
        return q;
    }
    if (is_nvq_linear_dtype(dtype)) {
        q.kind = QuantLinearKind::Nvq;
        q.nvq = std::make_shared<NvqWeight>(NvqWeight::from_blob(blob, n, nullptr, stream));
        if (q.nvq->dtype != dtype) fail("MFQ dtype/blob mismatch: " + dtype + " contains " + q.nvq->dtype);
        return q;
    }
    if (is_lowbit_linear_dtype(dtype)) {
        q.kind = QuantLinearKind::Nvq;
        q.nvq = std::make_shared<NvqWeight>(NvqWeight::from_lowbit_blob(dtype, blob, n, nullptr, stream));
        return q;
    }
    if (is_nepq_linear_dtype(dtype)) {
        q.kind = QuantLinearKind::Nepq;
        q.nepq = std::make_shared<NepqWeight>(NepqWeight::from_blob(blob, n, nullptr, stream));
        if (q.nepq->label != dtype) fail("MFQ dtype/blob mismatch: " + dtype + " contains " + q.nepq->label);
        if (q.nepq->n_experts != 1)
            fail("a " + dtype + " linear must hold one expert, the blob holds " + std::to_string(q.nepq->n_experts) +
                 " (multi-expert NEPQ tensors are NINTM cohorts)");
        return q;
    }
    if (is_mx_linear_dtype(dtype)) {
        q.kind = QuantLinearKind::Mx;
        q.mx = std::make_shared<MxWeight>(MxWeight::from_blob(dtype, blob, n, 0, stream));
        return q;
    }
    fail("unsupported quantized linear dtype: " + dtype);
}

// ---- MoE ---------------------------------------------------------------------------------------------------
void MoeRoutePlan::reserve(int max_tokens, int routes_, int n_experts_) {
    if (max_tokens <= 8 || routes_ <= 0 || n_experts_ <= 0) return;
    const int n_pairs = max_tokens * routes_, tile_m = mfq_hip_moe_tile_m();
    const int max_tiles = static_cast<int>(cdiv(n_pairs, tile_m)) + n_experts_;
    counts.ensure(4ull * n_experts_);
    expert_bounds.ensure(4ull * (n_experts_ + 1));
    tile_bounds.ensure(4ull * (n_experts_ + 1));
    tile_experts.ensure(4ull * max_tiles);
    ids_dst.ensure(4ull * n_pairs);
}

void build_moe_route_plan(MoeRoutePlan &p, const int32_t *ids, int tokens, int routes, int n_experts, mfq_stream_t stream) {
    if (!ids || tokens <= 0 || routes <= 0) fail("MoE ids must be device int32 [tokens, routes]");
    p.ids = ids; p.tokens = tokens; p.routes = routes; p.n_experts = n_experts;
    p.has_map = tokens > 8;
    if (p.has_map) {
        const int n_pairs = tokens * routes, tile_m = mfq_hip_moe_tile_m();
        const int max_tiles = static_cast<int>(cdiv(n_pairs, tile_m)) + n_experts;
        p.reserve(tokens, routes, n_experts);
        abi_check(mfq_hip_moe_route_map(ids, n_pairs, n_experts, tile_m, static_cast<int32_t *>(p.counts.get()),
                                        static_cast<int32_t *>(p.expert_bounds.get()),
                                        static_cast<int32_t *>(p.tile_bounds.get()),
                                        static_cast<int32_t *>(p.tile_experts.get()), max_tiles,
                                        static_cast<int32_t *>(p.ids_dst.get()), stream));
    }
    p.map_ready = true;
}

MoeRoutePlan build_moe_route_plan(const int32_t *ids, int tokens, int routes, int n_experts, mfq_stream_t stream) {
    MoeRoutePlan p;
    build_moe_route_plan(p, ids, tokens, routes, n_experts, stream);
    return p;
}

NintMoeWeight NintMoeWeight::from_blob(const uint8_t *base_blob, size_t n, mfq_stream_t stream, const uint8_t *overlay,
                                       size_t overlay_n) {
    const NintmHeader h = parse_nintm(base_blob, n);
    NintMoeWeight w;
    w.n_experts = h.n_experts; w.out_per_expert = h.out_per_expert; w.neuron_len = h.neuron_len;
    // the cohorts of an expert overlay follow the tensor's own; the last cohort that lists an expert owns it
    struct Cohort { const uint8_t *blob; const NintmPool *pool; };
    std::vector<Cohort> cohorts;
    for (const NintmPool &p : h.pools) cohorts.push_back({base_blob, &p});
    NintmHeader d;
    if (overlay) {
        d = parse_nintm(overlay, overlay_n, true);
        if (d.n_experts != h.n_experts || d.out_per_expert != h.out_per_expert || d.neuron_len != h.neuron_len)
            fail("expert overlay shape mismatch");
        for (const NintmPool &p : d.pools) cohorts.push_back({overlay, &p});
    }
    std::vector<int> owner(static_cast<size_t>(h.n_experts), -1);
    for (size_t ci = 0; ci < cohorts.size(); ++ci)
        for (int32_t e : cohorts[ci].pool->expert_ids) owner[static_cast<size_t>(e)] = static_cast<int>(ci);
    std::vector<int32_t> ep(h.n_experts, -1), el(h.n_experts, -1);
    for (size_t pi = 0; pi < cohorts.size(); ++pi) {
        const NintmPool &p = *cohorts[pi].pool;
        const uint8_t *blob = cohorts[pi].blob;
        std::vector<uint8_t> live;
        for (int32_t e : p.expert_ids) live.push_back(owner[static_cast<size_t>(e)] == static_cast<int>(pi) ? 1 : 0);
        if (p.runtime_bytes) fail("unexpected NINTM cohort runtime metadata");
        const std::string shape_error = "NINTM pool " + std::to_string(pi) + " tensor shape does not match its expert count";
        if (!is_nint_linear_dtype(p.dtype)) {
            MoeForeignCohort c;
            c.dtype = p.dtype; c.expert_ids = p.expert_ids; c.live = live;
            const int parts = static_cast<int>(p.expert_ids.size());
            if (is_nepq_linear_dtype(p.dtype)) {
                c.nepq = std::make_shared<NepqWeight>(NepqWeight::from_blob(blob + p.payload_off, p.payload_bytes, nullptr, stream));
                if (c.nepq->label != p.dtype) fail("MFQ dtype/blob mismatch: " + p.dtype + " contains " + c.nepq->label);
                if (c.nepq->n_experts != parts || c.nepq->out_per_expert != h.out_per_expert || c.nepq->neuron_len() != h.neuron_len)
                    fail(shape_error);
            } else if (is_nvq_linear_dtype(p.dtype) || is_lowbit_linear_dtype(p.dtype) || p.dtype == "NINT8-0") {
                for (const auto &piece : split_rows(p.dtype, blob + p.payload_off, p.payload_bytes, parts)) {
                    c.linears.push_back(load_quant_linear(p.dtype, piece.data(), piece.size(), stream));
                    if (c.linears.back().out() != h.out_per_expert || c.linears.back().neuron_len() != h.neuron_len) fail(shape_error);
                }
            } else if (p.dtype == "MXFP4") {  // mfq/formats/moe.py:122-124: one [experts * out, K] tensor
                c.mx = std::make_shared<MxWeight>(MxWeight::from_blob(p.dtype, blob + p.payload_off, p.payload_bytes, h.out_per_expert, stream));
                if (c.mx->rows != static_cast<int64_t>(parts) * h.out_per_expert || c.mx->cols != h.neuron_len) fail(shape_error);
            } else if (p.dtype == "MXFP8") {  // expert_tensor_family, mfq/formats/moe.py:38-47
                fail("NINTM supports native MXFP4 expert pools, got " + p.dtype);
            } else {
                fail("NINTM cohort family " + p.dtype + " is not supported");
            }
            c.prepare_pairs(h.n_experts, h.out_per_expert, stream);
            w.foreign.push_back(std::move(c));
            continue;
        }
        auto pw = std::make_shared<NintWeight>(NintWeight::from_blob(blob + p.payload_off, p.payload_bytes, stream));
        if (pw->out() != static_cast<int64_t>(p.expert_ids.size()) * h.out_per_expert || pw->neuron_len() != h.neuron_len)
            fail(shape_error);
        for (size_t i = 0; i < p.expert_ids.size(); ++i) {
            if (!live[i]) continue;
            ep[p.expert_ids[i]] = static_cast<int32_t>(w.pool_table.size());
            el[p.expert_ids[i]] = static_cast<int32_t>(i);
        }
        w.pool_table.push_back(mfq_moe_pool{pw->desc, pw->data.get()});
        w.pools.push_back(std::move(pw));
        w.pool_expert_ids.push_back(p.expert_ids);
    }
    w.expert_pool = DeviceBuffer::from_host(ep.data(), 4ull * ep.size());
    w.expert_local = DeviceBuffer::from_host(el.data(), 4ull * el.size());
    return w;
}

int64_t MoeForeignCohort::payload_bytes() const {
    if (mx) return mx->payload_bytes();
    if (nepq) return nepq->payload_bytes();
    int64_t n = 0;
    for (const QuantLinear &q : linears) n += q.payload_bytes();
    return n;
}
void MoeForeignCohort::matmul(int local, const void *x, int x_dtype, int64_t ldx, int M, float *y, mfq_stream_t stream) const {
    if (mx) mx_matmul(*mx, local, x, x_dtype, ldx, M, y, stream);
    else if (nepq) nepq_matmul(*nepq, local, x, x_dtype, ldx, M, y, stream);
    else linears[static_cast<size_t>(local)].forward(x, x_dtype, ldx, M, y, stream);
}
void MoeForeignCohort::dequantize(int local, float *out, mfq_stream_t stream) const {
    if (mx) { mx_dequantize(*mx, local, out, stream); return; }
    if (!nepq) { linears[static_cast<size_t>(local)].dequantize(out, stream); return; }
    // the cohort dequantizes as a whole: take the expert's rows out of it
    const size_t rows = static_cast<size_t>(nepq->out_per_expert), K = static_cast<size_t>(nepq->neuron_len());
    DeviceBuffer all(static_cast<size_t>(nepq->n_experts) * rows * K * 4);
    nepq_dequantize(*nepq, static_cast<float *>(all.get()), stream);
    hip_check(hipMemcpyAsync(out, static_cast<const float *>(all.get()) + static_cast<size_t>(local) * rows * K, rows * K * 4,
                             hipMemcpyDeviceToDevice, hs(stream)), "foreign cohort dequantize");
    hip_check(hipStreamSynchronize(hs(stream)), "foreign cohort dequantize");
}

void MoeForeignCohort::prepare_pairs(int n_experts, int out_per_expert, mfq_stream_t stream) {
    if (nepq && !nepq->streams && out_per_expert % 16) return;  // NEPQ1 experts must be whole row-blocks
    std::vector<int32_t> slot(static_cast<size_t>(n_experts), -1);
    for (size_t i = 0; i < expert_ids.size(); ++i)
        if (live.empty() || live[i]) slot[static_cast<size_t>(expert_ids[i])] = static_cast<int32_t>(i);
    pair_slot.ensure(slot.size() * 4);
    hip_check(hipMemcpyAsync(pair_slot.get(), slot.data(), slot.size() * 4, hipMemcpyHostToDevice, hs(stream)), "NINTM cohort tables");
    std::vector<const void *> ptrs;
    if (!linears.empty()) {
        for (const QuantLinear &q : linears) ptrs.push_back(q.kind == QuantLinearKind::Nint8Zero ? q.nint8z->data.get() : q.nvq->data.get());
        pair_weights.ensure(ptrs.size() * sizeof(void *));
        hip_check(hipMemcpyAsync(pair_weights.get(), ptrs.data(), ptrs.size() * sizeof(void *), hipMemcpyHostToDevice, hs(stream)),
                  "NINTM cohort tables");
    }
    hip_check(hipStreamSynchronize(hs(stream)), "NINTM cohort tables");  // the host vectors go out of scope
}

bool MoeForeignCohort::matmul_pairs(int n_experts, int out_per_expert, const void *x, int x_dtype, int64_t ldx, bool routed_input,
                                    const int32_t *ids, int T, int R, float *out, mfq_stream_t stream) const {
    if (!pair_slot.get()) return false;
    const int32_t *slot = static_cast<const int32_t *>(pair_slot.get());
    if (mx) {
        abi_check(mfq_hip_mx_gemv_pairs(mx->kind, mx->values.get(), mx->scales.get(), static_cast<int>(mx->rows),
                                        static_cast<int>(mx->cols), out_per_expert, slot, n_experts, x, x_dtype, ldx,
                                        routed_input ? 1 : 0, ids, T, R, out, out_per_expert, stream));
        return true;
    }
    if (nepq) {
        const NepqWeight &w = *nepq;
        const int K = static_cast<int>(w.neuron_len());
        if (w.rotation_block) {
            const int rows = routed_input ? T * R : T;
            w.rotated.ensure(static_cast<size_t>(rows) * K * 2);
            abi_check(mfq_hip_nepq_hadamard(x, x_dtype, ldx, rows, K, w.rotation_block, static_cast<const int8_t *>(w.signs.get()),
                                            w.rotated.get(), K, stream));
            x = w.rotated.get();
            ldx = K;
        }
        if (w.streams)
            abi_check(mfq_hip_nvqs_gemv_pairs(&w.sdesc, nullptr, w.data.get(), out_per_expert, slot, n_experts, x, x_dtype, ldx,
                                              routed_input ? 1 : 0, ids, T, R, out, out_per_expert, stream));
        else
            abi_check(mfq_hip_nepq_gemv_pairs(&w.desc, w.data.get(), out_per_expert, slot, n_experts, x, x_dtype, ldx,
                                              routed_input ? 1 : 0, ids, T, R, out, out_per_expert, stream));
        return true;
    }
    const void *const *ptrs = static_cast<const void *const *>(pair_weights.get());
    if (linears[0].kind == QuantLinearKind::Nint8Zero) {
        abi_check(mfq_hip_nint8z_gemv_pairs(&linears[0].nint8z->desc, ptrs, slot, n_experts, x, x_dtype, ldx, routed_input ? 1 : 0,
                                            ids, T, R, out, out_per_expert, stream));
        return true;
    }
    const NvqWeight &w0 = *linears[0].nvq;
    if (w0.streams)
        abi_check(mfq_hip_nvqs_gemv_pairs(&w0.sdesc, ptrs, nullptr, out_per_expert, slot, n_experts, x, x_dtype, ldx,
                                          routed_input ? 1 : 0, ids, T, R, out, out_per_expert, stream));
    else
        abi_check(mfq_hip_nvq_gemv_pairs(&w0.desc, ptrs, slot, n_experts, x, x_dtype, ldx, routed_input ? 1 : 0, ids, T, R, out,
                                         out_per_expert, stream));
    return true;
}

void NintMoeWeight::add_foreign(const void *x, int x_dtype, int64_t ldx, bool routed_input, const MoeRoutePlan &r, float *out,
                                mfq_stream_t stream) const {
    if (foreign.empty()) return;
    if (neuron_len % 2 || ldx % 2) fail("mixed NINTM cohorts need activation rows of whole 32-bit words");
    const int T = r.tokens, R = r.routes;
    // a decode step: one launch per cohort over all pairs, nothing read back; the cohorts without such a launch (and
    // every cohort of a larger batch) take the walk below
    std::vector<const MoeForeignCohort *> walk;
    for (const MoeForeignCohort &c : foreign)
        if (T * R > MoeForeignCohort::kPairsMax ||
            !c.matmul_pairs(n_experts, out_per_expert, x, x_dtype, ldx, routed_input, r.ids, T, R, out, stream))
            walk.push_back(&c);
    if (walk.empty()) return;
    std::vector<int32_t> ids(static_cast<size_t>(T) * R);
    hip_check(hipStreamSynchronize(hs(stream)), "mixed NINTM: routing table");
    hip_check(hipMemcpy(ids.data(), r.ids, 4 * ids.size(), hipMemcpyDeviceToHost), "mixed NINTM: routing table");
    std::vector<int32_t> index;  // per expert: n pair rows, then n source rows
    for (const MoeForeignCohort *cp : walk) {
        const MoeForeignCohort &c = *cp;
        for (size_t local = 0; local < c.expert_ids.size(); ++local) {
            if (!c.live.empty() && !c.live[local]) continue;  // an expert overlay gave this expert to a later cohort
            const int32_t e = c.expert_ids[local];
            std::vector<int32_t> pair_rows, src_rows;
            for (int t = 0; t < T; ++t)
                for (int k = 0; k < R; ++k)
                    if (ids[static_cast<size_t>(t) * R + k] == e) {
                        pair_rows.push_back(t * R + k);
                        src_rows.push_back(routed_input ? t * R + k : t);
                    }
            const int n = static_cast<int>(pair_rows.size());
            if (!n) continue;
            index = pair_rows;
            index.insert(index.end(), src_rows.begin(), src_rows.end());
            f_index.ensure(8ull * n);
            f_x.ensure(2ull * n * neuron_len);
            f_y.ensure(4ull * n * out_per_expert);
            // the three buffers are reused by the next expert: the copy below waits for the previous expert's kernels
            hip_check(hipStreamSynchronize(hs(stream)), "mixed NINTM: expert walk");
            hip_check(hipMemcpy(f_index.get(), index.data(), 8ull * n, hipMemcpyHostToDevice), "mixed NINTM: row lists");
            const int32_t *d_pairs = static_cast<const int32_t *>(f_index.get()), *d_src = d_pairs + n;
            abi_check(mfq_hip_moe_move_rows(x, 2 * ldx, d_src, n, 2 * neuron_len, 0, f_x.get(), 2ll * neuron_len, stream));
            c.matmul(static_cast<int>(local), f_x.get(), x_dtype, neuron_len, n, static_cast<float *>(f_y.get()), stream);
            abi_check(mfq_hip_moe_move_rows(f_y.get(), 4ll * out_per_expert, d_pairs, n, 4 * out_per_expert, 1, out,
                                            4ll * out_per_expert, stream));
        }
    }
}

void NintMoeWeight::forward(const void *x, int x_dtype, int64_t ldx, bool routed_input, const MoeRoutePlan &r, float *out,
                            mfq_stream_t stream) const {
    if (pools.empty()) {  // no NINT cohort at all: every row comes from the host's walk
        abi_check(mfq_hip_fill_zero(out, 4ull * r.tokens * r.routes * out_per_expert, stream));
        add_foreign(x, x_dtype, ldx, routed_input, r, out, stream);
        return;
    }
    const bool mapped = r.mapped();
    // a workspace lets the library take the prefill kernel when a mapped call has many pairs per expert
    const int x_rows = routed_input ? r.tokens * r.routes : r.tokens;
    size_t need = 0;
    if (mapped)
        need = mfq_hip_moe_grouped_workspace_bytes(pool_table.data(), static_cast<int>(pool_table.size()), neuron_len, x_rows);
    if (need) workspace.ensure(need);
    abi_check(mfq_hip_moe_grouped_matmul_ws(
        pool_table.data(), static_cast<int>(pool_table.size()), static_cast<const int32_t *>(expert_pool.get()),
        static_cast<const int32_t *>(expert_local.get()), n_experts, out_per_expert, neuron_len, x, x_dtype, ldx,
        routed_input ? 1 : 0, r.ids, r.tokens, r.routes, mapped ? static_cast<const int32_t *>(r.ids_dst.get()) : nullptr,
        mapped ? static_cast<const int32_t *>(r.expert_bounds.get()) : nullptr,
        mapped ? static_cast<const int32_t *>(r.tile_bounds.get()) : nullptr,
        mapped ? static_cast<const int32_t *>(r.tile_experts.get()) : nullptr, out, out_per_expert,
        need ? workspace.get() : nullptr, need, stream));
    add_foreign(x, x_dtype, ldx, routed_input, r, out, stream);
}

void NintMoeWeight::forward_glu(const void *x, int x_dtype, int64_t ldx, bool routed_input, const MoeRoutePlan &r, bool gelu,
                                void *hidden, float *scratch, mfq_stream_t stream) const {
    const int W = out_per_expert / 2, pairs = r.tokens * r.routes;
    const int activation = gelu ? MFQ_GLU_GELU : MFQ_GLU_SILU;
    if (r.mapped() && out_per_expert % 32 == 0 && foreign.empty()) {
        const int x_rows = routed_input ? pairs : r.tokens;
        const size_t need =
            mfq_hip_moe_grouped_workspace_bytes(pool_table.data(), static_cast<int>(pool_table.size()), neuron_len, x_rows);
        if (need) {
            workspace.ensure(need);
            const int rc = mfq_hip_moe_grouped_glu_ws(
                pool_table.data(), static_cast<int>(pool_table.size()), static_cast<const int32_t *>(expert_pool.get()),
                static_cast<const int32_t *>(expert_local.get()), n_experts, out_per_expert, neuron_len, x, x_dtype, ldx,
                routed_input ? 1 : 0, r.ids, r.tokens, r.routes, static_cast<const int32_t *>(r.ids_dst.get()),
                static_cast<const int32_t *>(r.expert_bounds.get()), activation, hidden, MFQ_X_F16, W, workspace.get(), need,
                stream);
            if (rc == MFQ_OK) return;
            if (rc != MFQ_ERR_UNSUPPORTED) abi_check(rc);
        }
    }
    forward(x, x_dtype, ldx, routed_input, r, scratch, stream);
    abi_check(mfq_hip_moe_glu(scratch, out_per_expert, pairs, W, hidden, MFQ_X_F16, W, activation, stream));
}

bool NintMoeWeight::decode_capable(const NintWeight *shared, int tokens, int routes, bool swiglu) const {
    if (!foreign.empty() || (shared && shared->desc.neuron_len != neuron_len)) return false;
    return mfq_hip_moe_decode_capable(pool_table.data(), static_cast<int>(pool_table.size()), out_per_expert, neuron_len,
                                      shared ? &shared->desc : nullptr, tokens, routes, swiglu ? 1 : 0) != 0;
}

void NintMoeWeight::forward_decode(const void *x, int x_dtype, int64_t ldx, bool routed_input, const int32_t *ids, int T,
                                   int R, const NintWeight *shared, bool swiglu, void *out, mfq_stream_t stream) const {
    abi_check(mfq_hip_moe_decode_matmul(pool_table.data(), static_cast<int>(pool_table.size()),
                                        static_cast<const int32_t *>(expert_pool.get()),
                                        static_cast<const int32_t *>(expert_local.get()), n_experts, out_per_expert,
                                        neuron_len, x, x_dtype, ldx, routed_input ? 1 : 0, ids, T, R,
                                        shared ? &shared->desc : nullptr, shared ? shared->data.get() : nullptr,
                                        swiglu ? 1 : 0, out, MFQ_X_F16, swiglu ? out_per_expert / 2 : out_per_expert, stream));
}

void nint_moe_ffn_forward(const NintMoeWeight &gate_up, const NintMoeWeight &down, const void *x, int x_dtype, int64_t ldx,
                          int T, const float *router_logits, int top_k, int topk_mode, bool normalize,
                          const float *router_bias, float router_scale, const NintWeight *shared_gate_up,
                          const NintWeight *shared_down, MoeFfnScratch &s, float *out, mfq_stream_t stream) {
    if (gate_up.n_experts != down.n_experts || gate_up.out_per_expert != 2 * down.neuron_len ||
        down.out_per_expert != gate_up.neuron_len)
        fail("incompatible fused gate_up/down NINTM tensors");
    const int E = gate_up.n_experts, W = down.neuron_len, H = down.out_per_expert;
    const size_t pairs = static_cast<size_t>(T) * top_k;
    s.ids.ensure(4 * pairs); s.weights.ensure(4 * pairs);
    int32_t *ids = static_cast<int32_t *>(s.ids.get());
    float *wts = static_cast<float *>(s.weights.get());
    abi_check(mfq_hip_moe_topk(router_logits, router_bias, T, E, top_k, topk_mode, normalize ? 1 : 0, 1e-20f, router_scale, ids,
                               wts, stream));
    const bool with_shared = shared_gate_up && shared_down;
    if (T <= 8 && gate_up.decode_capable(with_shared ? shared_gate_up : nullptr, T, top_k, true) &&
        down.decode_capable(with_shared ? shared_down : nullptr, T, top_k, false)) {
        // decode step: gate/up + SwiGLU of the routes and the shared expert in one launch, the down projections in a
        // second one; rows pairs .. pairs + T - 1 of both buffers belong to the shared expert
        const size_t rows = pairs + (with_shared ? T : 0);
        s.hidden.ensure(2 * rows * W); s.down.ensure(4 * rows * H);
        gate_up.forward_decode(x, x_dtype, ldx, false, ids, T, top_k, with_shared ? shared_gate_up : nullptr, true,
                               s.hidden.get(), stream);
        float *dn = static_cast<float *>(s.down.get());
        down.forward_decode(s.hidden.get(), MFQ_X_F16, W, true, ids, T, top_k, with_shared ? shared_down : nullptr, false, dn,
                            stream);
        abi_check(mfq_hip_moe_weighted_reduce(dn, wts, T, top_k, H, with_shared ? dn + pairs * H : nullptr, nullptr, out, stream));
        return;
    }
    MoeRoutePlan &route = s.route;  // lives in the scratch: nothing is freed on return, so nothing has to be waited for
    build_moe_route_plan(route, ids, T, top_k, E, stream);
    s.gate_up.ensure(4 * pairs * 2 * W); s.hidden.ensure(2 * pairs * W); s.down.ensure(4 * pairs * H);
    float *gu = static_cast<float *>(s.gate_up.get());
    gate_up.forward_glu(x, x_dtype, ldx, false, route, false, s.hidden.get(), gu, stream);
    float *dn = static_cast<float *>(s.down.get());
    down.forward(s.hidden.get(), MFQ_X_F16, W, true, route, dn, stream);
    const float *shared = nullptr;
    if (shared_gate_up && shared_down) {
        s.shared_gu.ensure(4ull * T * 2 * W); s.shared_h.ensure(2ull * T * W); s.shared_out.ensure(4ull * T * H);
        nint_matmul(*shared_gate_up, x, x_dtype, ldx, T, static_cast<float *>(s.shared_gu.get()), stream);
        abi_check(mfq_hip_moe_swiglu(static_cast<float *>(s.shared_gu.get()), 2 * W, T, W, s.shared_h.get(), MFQ_X_F16, W, stream));
        nint_matmul(*shared_down, s.shared_h.get(), MFQ_X_F16, W, T, static_cast<float *>(s.shared_out.get()), stream);
        shared = static_cast<const float *>(s.shared_out.get());
    }
    abi_check(mfq_hip_moe_weighted_reduce(dn, wts, T, top_k, H, shared, nullptr, out, stream));
}

void MoeFfnScratch::reserve(const NintMoeWeight &wgu, const NintMoeWeight &wdn, int max_tokens, int top_k,
                            const NintWeight *shared_gate_up, const NintWeight *shared_down) {
    if (max_tokens <= 0 || top_k <= 0) return;
    const size_t T = static_cast<size_t>(max_tokens), pairs = T * top_k;
    const size_t W = static_cast<size_t>(wdn.neuron_len), H = static_cast<size_t>(wdn.out_per_expert);
    const bool with_shared = shared_gate_up && shared_down;
    const size_t rows = pairs + (with_shared ? T : 0);  // the decode form keeps the shared expert's rows behind the pairs
    ids.ensure(4 * pairs); weights.ensure(4 * pairs);
    hidden.ensure(2 * rows * W); down.ensure(4 * rows * H);
    if (max_tokens > 8) {
        gate_up.ensure(4 * pairs * 2 * W);
        route.reserve(max_tokens, top_k, wgu.n_experts);
        // the tensors' prefill workspaces: the need grows with the rows of the call
        auto grouped = [](const NintMoeWeight &w, int x_rows) {
            if (w.pool_table.empty()) return;
            const size_t need = mfq_hip_moe_grouped_workspace_bytes(w.pool_table.data(), static_cast<int>(w.pool_table.size()),
                                                                    w.neuron_len, x_rows);
            w.workspace.ensure(need);
        };
        for (int t = 9; t <= max_tokens; t = t < 64 ? t + 1 : t + 64) { grouped(wgu, t); grouped(wdn, t * top_k); }
        grouped(wgu, max_tokens); grouped(wdn, max_tokens * top_k);
        if (with_shared) {
            shared_gu.ensure(4 * T * 2 * W); shared_h.ensure(2 * T * W); shared_out.ensure(4 * T * H);
            for (const NintWeight *w : {shared_gate_up, shared_down}) {
                size_t need = 0;
                for (int M = 1; M <= std::min(max_tokens, 512); ++M) need = std::max(need, mfq_hip_nint_gemm_workspace_bytes(&w->desc, M));
                for (int M = 576; M < max_tokens; M += 64) need = std::max(need, mfq_hip_nint_gemm_workspace_bytes(&w->desc, M));
                need = std::max(need, mfq_hip_nint_gemm_workspace_bytes(&w->desc, max_tokens));
                w->workspace.ensure(need);
            }
        }
    }
}

// ---- expert residency -----------------------------------------------------------------------------------------
MoeExpertCache::MoeExpertCache(int64_t budget_bytes) : budget_bytes_(budget_bytes) {
    if (budget_bytes <= 0) fail("MoE GPU cache budget must be positive");
}
MoeExpertCache::~MoeExpertCache() {
    for (auto &s : sources_)
        for (auto &c : s->cohorts)
            if (c.host) (void)hipHostFree(c.host);
    if (stage_host_) (void)hipHostFree(stage_host_);
}

MoeCachedSource *MoeExpertCache::register_source(const uint8_t *blob, size_t n, int minimum_slots) {
    if (finalized_) fail("cannot register a MoE source after cache finalization");
    NintMoeWeight full = NintMoeWeight::from_blob(blob, n);
    if (!full.foreign.empty())
        fail("expert residency holds NINT cohorts only; this tensor has a " + full.foreign[0].dtype + " cohort");
    auto src = std::make_unique<MoeCachedSource>();
    src->n_experts = full.n_experts; src->out_per_expert = full.out_per_expert; src->neuron_len = full.neuron_len;
    src->cohort_of.assign(full.n_experts, -1);
    src->local_of.assign(full.n_experts, -1);
    for (size_t pi = 0; pi < full.pools.size(); ++pi) {
        MoeCachedSource::Cohort c;
        c.src = full.pools[pi]->desc;
        c.expert_ids = full.pool_expert_ids[pi];
        c.host_bytes = static_cast<size_t>(c.src.total_bytes);
        hip_check(hipHostMalloc(&c.host, c.host_bytes, hipHostMallocDefault), "hipHostMalloc");
        hip_check(hipMemcpy(c.host, full.pools[pi]->data.get(), c.host_bytes, hipMemcpyDeviceToHost), "expert cache: copy to host");
        c.body_bytes = static_cast<int64_t>(full.out_per_expert / 16) * c.src.rowblock_bytes;
        c.slot_bytes = c.body_bytes + 2ll * full.out_per_expert * 4;
        c.minimum_slots = std::min<int>(minimum_slots, static_cast<int>(c.expert_ids.size()));
        for (size_t l = 0; l < c.expert_ids.size(); ++l) {
            src->cohort_of[c.expert_ids[l]] = static_cast<int32_t>(pi);
            src->local_of[c.expert_ids[l]] = static_cast<int32_t>(l);
        }
        src->cohorts.push_back(std::move(c));
    }
    sources_.push_back(std::move(src));
    return sources_.back().get();  // `full` (the device copies of the pools) goes away here; the host copies stay
}

void MoeExpertCache::finalize() {
    if (finalized_) return;
    int64_t need = 0;
    double total = 0;
    for (auto &s : sources_)
        for (auto &c : s->cohorts) {
            need += c.minimum_slots * c.slot_bytes;
            total += static_cast<double>(c.expert_ids.size()) * c.slot_bytes;
        }
    if (need > budget_bytes_)
        fail("MoE GPU cache budget " + std::to_string(budget_bytes_) + " is below the minimum working set " + std::to_string(need));
    const int64_t spare = budget_bytes_ - need;
    for (auto &s : sources_) {
        NintMoeWeight &w = s->weight;
        w.n_experts = s->n_experts; w.out_per_expert = s->out_per_expert; w.neuron_len = s->neuron_len;
        for (auto &c : s->cohorts) {
            const double share = static_cast<double>(c.expert_ids.size()) * c.slot_bytes / total;
            const int extra = static_cast<int>(static_cast<int64_t>(spare * share) / c.slot_bytes);
            const int slots = std::min<int>(static_cast<int>(c.expert_ids.size()), c.minimum_slots + extra);
            c.arena = std::make_shared<NintWeight>();
            abi_check(mfq_hip_nint_plan(c.src.bits, c.src.sub_bits, c.src.gs, slots * s->out_per_expert, c.src.neuron_len,
                                        &c.arena->desc));
            c.arena->data = DeviceBuffer(static_cast<size_t>(c.arena->desc.total_bytes));
            hip_check(hipMemset(c.arena->data.get(), 0, static_cast<size_t>(c.arena->desc.total_bytes)), "hipMemset");
            allocated_bytes_ += c.arena->desc.total_bytes;
            for (int i = slots - 1; i >= 0; --i) c.free_slots.push_back(i);
            w.pools.push_back(c.arena);
            w.pool_expert_ids.emplace_back();
            mfq_moe_pool entry;
            entry.desc = c.arena->desc;
            entry.weight = c.arena->data.get();
            w.pool_table.push_back(entry);
        }
        std::vector<int32_t> none(static_cast<size_t>(s->n_experts), -1);
        w.expert_pool = DeviceBuffer::from_host(s->cohort_of.data(), 4 * s->cohort_of.size());
        w.expert_local = DeviceBuffer::from_host(none.data(), 4 * none.size());
    }
    finalized_ = true;
}

void MoeExpertCache::prepare(MoeCachedSource &source, const int32_t *experts, size_t count, mfq_stream_t stream) {
    if (!finalized_) fail("MoE cache must be finalized before inference");
    std::vector<std::vector<int>> wanted(source.cohorts.size());
    {
        std::vector<int32_t> uniq(experts, experts + count);
        std::sort(uniq.begin(), uniq.end());
        uniq.erase(std::unique(uniq.begin(), uniq.end()), uniq.end());
        for (int32_t e : uniq)
            if (e >= 0 && e < source.n_experts) wanted[source.cohort_of[e]].push_back(e);
    }
    struct Copy { const uint8_t *src; uint64_t dst; int64_t nbytes; };
    std::vector<Copy> copies;
    std::vector<std::pair<int32_t, int32_t>> table;  // (expert, slot or -1)
    const int out = source.out_per_expert;
    for (size_t ci = 0; ci < wanted.size(); ++ci) {
        auto &c = source.cohorts[ci];
        const size_t capacity = c.free_slots.size() + c.slot_of.size();
        if (wanted[ci].size() > capacity)
            fail("MoE route needs " + std::to_string(wanted[ci].size()) + " experts of one cohort, its arena holds " + std::to_string(capacity));
        std::vector<bool> keep(c.expert_ids.size(), false);
        for (int e : wanted[ci]) keep[source.local_of[e]] = true;
        for (int e : wanted[ci]) {
            const int local = source.local_of[e];
            auto hit = c.slot_of.find(local);
            if (hit != c.slot_of.end()) {
                ++stats_.hits;
                c.lru.erase(std::find(c.lru.begin(), c.lru.end(), local));
                c.lru.push_back(local);
                continue;
            }
            ++stats_.misses;
            int slot;
            if (!c.free_slots.empty()) {
                slot = c.free_slots.back();
                c.free_slots.pop_back();
            } else {
                auto victim = std::find_if(c.lru.begin(), c.lru.end(), [&](int v) { return !keep[v]; });
                slot = c.slot_of[*victim];
                table.emplace_back(c.expert_ids[*victim], -1);
                c.slot_of.erase(*victim);
                c.lru.erase(victim);
                ++stats_.evictions;
            }
            c.slot_of[local] = slot;
            c.lru.push_back(local);
            const uint8_t *h = static_cast<const uint8_t *>(c.host);
            const uint64_t base = reinterpret_cast<uint64_t>(c.arena->data.get());
            const mfq_nint_desc &a = c.arena->desc;
            copies.push_back({h + static_cast<int64_t>(local) * c.body_bytes, base + static_cast<uint64_t>(slot) * c.body_bytes, c.body_bytes});
            copies.push_back({h + c.src.anchors_off + static_cast<int64_t>(local) * out * 4,
                              base + a.anchors_off + static_cast<uint64_t>(slot) * out * 4, out * 4ll});
            copies.push_back({h + c.src.anchors_off + 16ll * c.src.n_rowblocks * 4 + static_cast<int64_t>(local) * out * 4,
                              base + a.anchors_off + 16ull * a.n_rowblocks * 4 + static_cast<uint64_t>(slot) * out * 4, out * 4ll});
            table.emplace_back(e, slot);
        }
    }
    if (copies.empty() && table.empty()) return;
    // staging image: byte ranges (16-byte aligned), table words, descriptors
    size_t off = 0;
    std::vector<size_t> at(copies.size());
    int64_t biggest = 4;
    for (size_t i = 0; i < copies.size(); ++i) {
        at[i] = off;
        off += (static_cast<size_t>(copies[i].nbytes) + 15) & ~size_t(15);
        biggest = std::max(biggest, copies[i].nbytes);
    }
    const size_t words_off = off;
    off += (4 * table.size() + 15) & ~size_t(15);
    const size_t desc_off = off, n = copies.size() + table.size(), total = desc_off + sizeof(mfq_scatter_desc) * n;
    hipStream_t st = hs(stream);
    if (total > stage_bytes_) {
        hip_check(hipStreamSynchronize(st), "expert cache: sync");
        if (stage_host_) hip_check(hipHostFree(stage_host_), "hipHostFree");
        stage_bytes_ = std::max<size_t>(total, size_t(1) << 20);
        hip_check(hipHostMalloc(&stage_host_, stage_bytes_, hipHostMallocDefault), "hipHostMalloc");
        stage_dev_ = DeviceBuffer(stage_bytes_);
    } else {
        hip_check(hipStreamSynchronize(st), "expert cache: sync");  // the previous batch has left the pinned buffer
    }
    uint8_t *img = static_cast<uint8_t *>(stage_host_);
    auto *descs = reinterpret_cast<mfq_scatter_desc *>(img + desc_off);
    for (size_t i = 0; i < copies.size(); ++i) {
        std::memcpy(img + at[i], copies[i].src, static_cast<size_t>(copies[i].nbytes));
        descs[i] = {copies[i].dst, at[i], static_cast<uint64_t>(copies[i].nbytes)};
        stats_.bytes += copies[i].nbytes;
    }
    const uint64_t local_ptr = reinterpret_cast<uint64_t>(source.weight.expert_local.get());
    for (size_t j = 0; j < table.size(); ++j) {
        std::memcpy(img + words_off + 4 * j, &table[j].second, 4);
        descs[copies.size() + j] = {local_ptr + 4ull * table[j].first, words_off + 4 * j, 4};
    }
    hip_check(hipMemcpyAsync(stage_dev_.get(), stage_host_, total, hipMemcpyHostToDevice, st), "expert cache: staged copy");
    abi_check(mfq_hip_cache_scatter(stage_dev_.get(), static_cast<int64_t>(desc_off), static_cast<int>(n), biggest, stream));
    ++stats_.launches;
}

void MoeExpertCache::forward(MoeCachedSource &source, const void *x, int x_dtype, int64_t ldx, bool routed_input,
                             const MoeRoutePlan &route, float *out, mfq_stream_t stream) {
    std::vector<int32_t> ids(static_cast<size_t>(route.tokens) * route.routes);
    hip_check(hipMemcpyAsync(ids.data(), route.ids, 4 * ids.size(), hipMemcpyDeviceToHost, hs(stream)), "route readback");
    hip_check(hipStreamSynchronize(hs(stream)), "route readback");
    prepare(source, ids.data(), ids.size(), stream);
    source.weight.forward(x, x_dtype, ldx, routed_input, route, out, stream);
}

// ---- MFQ1 container ---------------------------------------------------------------------------------------
namespace {
struct MfqHeaderInfo {
    uint32_t version = 0, record_count = 0;
    std::string architecture;
    std::unordered_map<std::string, std::string> extra;
};
const uint64_t kNoCount = std::numeric_limits<uint64_t>::max();

// integer metadata value (JSON text of a non-negative integer); `dflt` when the key is absent
uint64_t json_uint(const std::unordered_map<std::string, std::string> &extra, const std::string &key, uint64_t dflt) {
    auto it = extra.find(key);
    if (it == extra.end()) return dflt;
    const std::string &t = it->second;
    size_t i = 0;
    uint64_t v = 0;
    bool digits = false;
    for (; i < t.size() && t[i] >= '0' && t[i] <= '9'; ++i) {
        if (v > (kNoCount - static_cast<uint64_t>(t[i] - '0')) / 10) fail("invalid MFQ integer metadata " + key + ": " + t);
        v = v * 10 + static_cast<uint64_t>(t[i] - '0');
        digits = true;
    }
    while (i < t.size() && std::isspace(static_cast<unsigned char>(t[i]))) ++i;
    if (!digits || i != t.size()) fail("invalid MFQ integer metadata " + key + ": " + t);
    return v;
}

// "<stem>-NNNNN-of-NNNNN.mfq": stem, 1-based index and count, or false
bool parse_shard_name(const std::string &filename, std::string &stem, uint64_t &index, uint64_t &count) {
    const size_t n = filename.size();  // tail: -ddddd-of-ddddd.mfq = 19 characters
    if (n < 20 || filename.compare(n - 4, 4, ".mfq") != 0 || filename[n - 19] != '-' || filename.compare(n - 13, 4, "-of-") != 0)
        return false;
    index = count = 0;
    for (size_t i = n - 18; i < n - 13; ++i) {
        if (filename[i] < '0' || filename[i] > '9') return false;
        index = index * 10 + static_cast<uint64_t>(filename[i] - '0');
    }
    for (size_t i = n - 9; i < n - 4; ++i) {
        if (filename[i] < '0' || filename[i] > '9') return false;
        count = count * 10 + static_cast<uint64_t>(filename[i] - '0');
    }
    stem = filename.substr(0, n - 19);
    return !stem.empty();
}

std::vector<std::string> shard_paths(const std::string &path_value, uint64_t split_no, uint64_t split_count) {
    const size_t slash = path_value.find_last_of('/');
    const std::string dir = slash == std::string::npos ? "" : path_value.substr(0, slash + 1);
    const std::string filename = slash == std::string::npos ? path_value : path_value.substr(slash + 1);
    std::string stem;
    uint64_t file_no = 0, file_count = 0;
    if (!parse_shard_name(filename, stem, file_no, file_count))
        fail("sharded MFQ path lacks -00001-of-00000 suffix: " + path_value);
    if (file_no != split_no + 1 || file_count != split_count) fail("MFQ shard filename/metadata mismatch: " + path_value);
    std::vector<std::string> result;
    for (uint64_t i = 1; i <= split_count; ++i) {
        char tail[32];
        std::snprintf(tail, sizeof(tail), "-%05llu-of-%05llu.mfq", static_cast<unsigned long long>(i),
                      static_cast<unsigned long long>(split_count));
        const std::string shard = dir + stem + tail;
        struct stat sb;
        if (::stat(shard.c_str(), &sb) != 0 || !S_ISREG(sb.st_mode)) fail("missing MFQ shard: " + shard);
        result.push_back(shard);
    }
    return result;
}
}  // namespace

int MfqFile::map_file(const std::string &source) {
    const int fd = ::open(source.c_str(), O_RDONLY);
    if (fd < 0) fail("cannot open MFQ file: " + source);
    struct stat sb;
    if (::fstat(fd, &sb) != 0) {
        ::close(fd);
        fail("cannot stat MFQ file: " + source);
    }
    Mapping m;
    m.size = static_cast<size_t>(sb.st_size);
    if (m.size) {
        void *p = ::mmap(nullptr, m.size, PROT_READ, MAP_PRIVATE, fd, 0);
        if (p == MAP_FAILED) {
            ::close(fd);
            fail("cannot map MFQ file: " + source);
        }
        m.base = static_cast<const uint8_t *>(p);
    }
    ::close(fd);  // the mapping keeps the file
    maps_.push_back(std::move(m));
    source_paths.push_back(source);
    return static_cast<int>(maps_.size()) - 1;
}

MfqFile::Mapping::~Mapping() {
    if (base) ::munmap(const_cast<uint8_t *>(base), size);
}
MfqFile::Mapping &MfqFile::Mapping::operator=(Mapping &&o) noexcept {
    if (this != &o) {
        if (base) ::munmap(const_cast<uint8_t *>(base), size);
        base = o.base;
        size = o.size;
        o.base = nullptr;
        o.size = 0;
    }
    return *this;
}

MfqFile::MfqFile(const std::string &path_in, const std::string &tensor_overlay, const std::string &expert_overlay)
    : path(path_in) {
    // header + record table of one file into `out` (its records appended in file order)
    auto load_records = [this](const std::string &source, std::vector<MfqRecord> &out) {
        const int src = map_file(source);
        const uint8_t *b = maps_[static_cast<size_t>(src)].base;
        const size_t n = maps_[static_cast<size_t>(src)].size;
        if (n < 12 || std::memcmp(b, "MFQ1", 4) != 0) fail("invalid MFQ magic: " + source);
        MfqHeaderInfo h;
        h.version = rd<uint32_t>(b, 4);
        size_t off = 8;
        auto str = [&](std::string &s) {
            if (off + 4 > n) fail("truncated MFQ header: " + source);
            const uint32_t len = rd<uint32_t>(b, off);
            off += 4;
            if (len > n - off) fail("truncated MFQ header: " + source);
            s.assign(reinterpret_cast<const char *>(b + off), len);
            off += len;
        };
        str(h.architecture);
        if (h.version >= 2) {
            if (off + 4 > n) fail("truncated MFQ header: " + source);
            const uint32_t n_extra = rd<uint32_t>(b, off);
            off += 4;
            for (uint32_t i = 0; i < n_extra; ++i) {
                std::string key, value;
                str(key);
                str(value);
                if (!h.extra.emplace(key, value).second) fail("duplicate MFQ metadata key: " + key + ": " + source);
            }
        }
        if (off + 4 > n) fail("truncated MFQ header: " + source);
        h.record_count = rd<uint32_t>(b, off);
        off += 4;
        const size_t first = out.size();
        for (uint32_t i = 0; i < h.record_count; ++i) {
            MfqRecord r;
            str(r.name);
            str(r.dtype);
            if (off + 8 > n) fail("truncated MFQ directory: " + source);
            r.nbytes = static_cast<size_t>(rd<uint64_t>(b, off));
            off += 8;
            r.source = src;
            out.push_back(std::move(r));
        }
        for (size_t i = first; i < out.size(); ++i) {
            MfqRecord &r = out[i];
            if (r.nbytes > n - off) fail("truncated MFQ blob for " + r.name + ": " + source);  // compared with what is left: cannot wrap
            r.offset = off;
            off += r.nbytes;
        }
        if (off != n)
            fail("MFQ file length mismatch: records end=" + std::to_string(off) + ", file size=" + std::to_string(n) + ": " + source);
        return h;
    };
    auto reject_duplicates = [](const std::vector<MfqRecord> &recs, const std::string &what) {
        std::unordered_map<std::string, int> seen;
        for (const MfqRecord &r : recs)
            if (!seen.emplace(r.name, 1).second) fail("duplicate MFQ tensor record: " + r.name + ": " + what);
    };

    MfqHeaderInfo probe = load_records(path, records);
    const uint64_t split_no = json_uint(probe.extra, "split.no", 0);
    const uint64_t split_count = json_uint(probe.extra, "split.count", 1);
    if (split_count < 1 || split_count > 99999 || split_no >= split_count) fail("invalid MFQ split metadata: " + path);
    model_arch = probe.architecture;
    version = probe.version;
    extra = probe.extra;
    if (split_count > 1) {
        const std::vector<std::string> paths = shard_paths(path, split_no, split_count);
        // start over in shard order
        records.clear();
        maps_.clear();
        source_paths.clear();
        uint64_t expected_records = kNoCount, expected_tensors = kNoCount;
        for (uint64_t i = 0; i < split_count; ++i) {
            const std::string &shard = paths[static_cast<size_t>(i)];
            const MfqHeaderInfo cur = load_records(shard, records);
            if (json_uint(cur.extra, "split.no", split_count) != i || json_uint(cur.extra, "split.count", 0) != split_count)
                fail("MFQ shard metadata mismatch: " + shard);
            if (cur.version != probe.version || cur.architecture != probe.architecture)
                fail("MFQ shard architecture/version mismatch: " + shard);
            const uint64_t cr = json_uint(cur.extra, "split.records.count", kNoCount);
            const uint64_t ct = json_uint(cur.extra, "split.tensors.count", kNoCount);
            if (expected_records == kNoCount) expected_records = cr;
            else if (cr != kNoCount && cr != expected_records) fail("MFQ shard record count mismatch: " + shard);
            if (expected_tensors == kNoCount) expected_tensors = ct;
            else if (ct != kNoCount && ct != expected_tensors) fail("MFQ shard tensor count mismatch: " + shard);
            if (i == 0) extra = cur.extra;  // model metadata lives in the first shard
        }
        reject_duplicates(records, "across shards");
        if (expected_records != kNoCount && records.size() != expected_records) fail("MFQ shard record total mismatch");
        if (expected_tensors != kNoCount && tensor_count() != expected_tensors) fail("MFQ shard tensor total mismatch");
        path = paths.front();
    } else {
        std::string stem;
        uint64_t file_no = 0, file_count = 0;
        const size_t slash = path.find_last_of('/');
        if (parse_shard_name(slash == std::string::npos ? path : path.substr(slash + 1), stem, file_no, file_count) &&
            file_count != 1)
            fail("MFQ filename claims multiple shards but metadata does not: " + path);
        reject_duplicates(records, path);
    }

    auto overlay_path = [](const std::string &given, const char *env) -> std::string {
        if (given == "-") return "";
        if (!given.empty()) return given;
        const char *v = std::getenv(env);
        return v ? std::string(v) : std::string();
    };
    const std::string tensor_src = overlay_path(tensor_overlay, "MFQ_TENSOR_OVERLAY");
    if (!tensor_src.empty()) {
        std::vector<MfqRecord> over;
        const MfqHeaderInfo oh = load_records(tensor_src, over);
        if (json_uint(oh.extra, "split.count", 1) != 1) fail("sharded MFQ tensor overlays are not supported");
        reject_duplicates(over, tensor_src);
        for (MfqRecord &o : over) {
            bool found = false;
            for (MfqRecord &base : records)
                if (base.name == o.name) {
                    base = o;
                    found = true;
                }
            if (!found) fail("tensor overlay replaces an unknown record: " + o.name);
            tensor_overlays.emplace(o.name, o);
        }
    }
    const std::string expert_src = overlay_path(expert_overlay, "MFQ_EXPERT_OVERLAY");
    if (!expert_src.empty()) {
        std::vector<MfqRecord> over;
        const MfqHeaderInfo oh = load_records(expert_src, over);
        if (json_uint(oh.extra, "split.count", 1) != 1) fail("sharded MFQ expert overlays are not supported");
        reject_duplicates(over, expert_src);
        for (MfqRecord &o : over) {
            if (o.dtype != "NINTMD" || !has_record(o.name) || find(o.name).dtype != "NINTM")
                fail("invalid expert overlay record: " + o.name);
            expert_overlays.emplace(o.name, o);
        }
    }
}
const MfqRecord &MfqFile::find(const std::string &name) const {
    for (const auto &r : records)
        if (r.name == name) return r;
    fail("missing tensor: " + name);
}
bool MfqFile::has_record(const std::string &name) const {
    for (const auto &r : records)
        if (r.name == name) return true;
    return false;
}
const uint8_t *MfqFile::data(const MfqRecord &r) const { return maps_.at(static_cast<size_t>(r.source)).base + r.offset; }
size_t MfqFile::tensor_count() const {
    size_t n = 0;
    for (const auto &r : records) n += r.name.rfind("__mfq_asset__/", 0) != 0;
    return n;
}
std::string MfqFile::read_asset_text(const std::string &name) const {
    const MfqRecord &r = find(name);
    if (r.dtype != "BLOB") fail("MFQ runtime asset has non-BLOB dtype: " + name);
    return std::string(reinterpret_cast<const char *>(data(r)), r.nbytes);
}

// ---- --check-linear -------------------------------------------------------------------------------------------
LinearCheckResult run_linear_check(const QuantLinear &lin, int M, int reps) {
    const int64_t N = lin.out(), K = lin.neuron_len();
    std::vector<uint16_t> x(static_cast<size_t>(M) * K);
    std::vector<float> xf(x.size());
    for (size_t i = 0; i < x.size(); ++i) {
        const float v = (static_cast<float>(static_cast<int>(i % 97) - 48)) / 512.f;  // exact in bf16
        uint32_t u;
        std::memcpy(&u, &v, 4);
        x[i] = static_cast<uint16_t>(u >> 16);
        xf[i] = v;
    }
    DeviceBuffer dx = DeviceBuffer::from_host(x.data(), x.size() * 2);
    DeviceBuffer dy(static_cast<size_t>(M) * N * 4), dw(static_cast<size_t>(N) * K * 4);
    hipStream_t st;
    hip_check(hipStreamCreate(&st), "hipStreamCreate");
    for (int i = 0; i < std::min(30, reps); ++i) lin.forward(dx.get(), MFQ_X_BF16, K, M, static_cast<float *>(dy.get()), st);
    hipEvent_t e0, e1;
    hip_check(hipEventCreate(&e0), "hipEventCreate");
    hip_check(hipEventCreate(&e1), "hipEventCreate");
    hip_check(hipEventRecord(e0, st), "hipEventRecord");
    for (int i = 0; i < reps; ++i) lin.forward(dx.get(), MFQ_X_BF16, K, M, static_cast<float *>(dy.get()), st);
    hip_check(hipEventRecord(e1, st), "hipEventRecord");
    hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
    float ms = 0.f;
    hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    lin.dequantize(static_cast<float *>(dw.get()), st);
    hip_check(hipStreamSynchronize(st), "sync");
    std::vector<float> y(static_cast<size_t>(M) * N), W(static_cast<size_t>(N) * K);
    hip_check(hipMemcpy(y.data(), dy.get(), y.size() * 4, hipMemcpyDeviceToHost), "copy y");
    hip_check(hipMemcpy(W.data(), dw.get(), W.size() * 4, hipMemcpyDeviceToHost), "copy W");
    double num = 0, den = 0, sum_abs = 0, max_abs = 0;
    for (int m = 0; m < M; ++m)
        for (int64_t r = 0; r < N; ++r) {
            double acc = 0;
            for (int64_t k = 0; k < K; ++k) acc += static_cast<double>(xf[m * K + k]) * W[r * K + k];
            const double d = y[m * N + r] - acc;
            num += d * d; den += acc * acc; sum_abs += std::fabs(d); max_abs = std::max(max_abs, std::fabs(d));
        }
    LinearCheckResult res;
    res.production_ms = ms / reps;
    res.payload_bytes = lin.payload_bytes();
    res.weight_bytes = lin.kind == QuantLinearKind::Nint ? lin.nint->desc.total_bytes
                     : lin.kind == QuantLinearKind::Nvq ? lin.nvq->total_bytes()
                     : lin.kind == QuantLinearKind::Nepq ? lin.nepq->total_bytes()
                     : lin.kind == QuantLinearKind::Mx ? lin.mx->payload_bytes() : lin.nint8z->desc.total_bytes;
    res.production_weight_gbps = res.weight_bytes / (res.production_ms * 1e6);
    res.payload_gbps = res.payload_bytes / (res.production_ms * 1e6);
    res.production_rel = den > 0 ? std::sqrt(num / den) : std::sqrt(num);
    res.production_mean_abs = sum_abs / (static_cast<double>(M) * N);
    res.production_max_abs = max_abs;
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); (void)hipStreamDestroy(st);
    return res;
}

}  // namespace mfq_rt

// ---- flat C wrappers, for bindings and tests ----------------------------------------------------------------------
using namespace mfq_rt;
namespace {
thread_local std::string g_err;
template <typename F>
int guard(F &&f) {
    try {
        f();
        return 0;
    } catch (const std::exception &e) {
        g_err = e.what();
        return 1;
    }
}
}  // namespace

extern "C" {
const char *mfq_rt_last_error(void) { return g_err.c_str(); }

int mfq_rt_load_quant_linear(const char *dtype, const void *blob, size_t n, void **handle) {
    return guard([&] { *handle = new QuantLinear(load_quant_linear(dtype, static_cast<const uint8_t *>(blob), n)); });
}
void mfq_rt_free_quant_linear(void *handle) { delete static_cast<QuantLinear *>(handle); }
int64_t mfq_rt_linear_out(void *h) { return static_cast<QuantLinear *>(h)->out(); }
int64_t mfq_rt_linear_neuron_len(void *h) { return static_cast<QuantLinear *>(h)->neuron_len(); }
int mfq_rt_linear_reserve(void *h, int max_M) {
    return guard([&] { static_cast<QuantLinear *>(h)->reserve(max_M); });
}
int mfq_rt_linear_forward(void *h, const void *x, int x_dtype, int64_t ldx, int M, float *y, void *stream) {
    return guard([&] { static_cast<QuantLinear *>(h)->forward(x, x_dtype, ldx, M, y, stream); });
}
int mfq_rt_linear_forward_glu(void *h, const void *x, int x_dtype, int64_t ldx, int M, int gelu, void *hidden, float *scratch,
                              void *stream) {
    return guard([&] {
        const QuantLinear *q = static_cast<QuantLinear *>(h);
        if (!q->nint) fail("the fused gate/up projection needs a NINT tensor");
        if (gelu) nint_matmul_geglu(*q->nint, x, x_dtype, ldx, M, hidden, scratch, stream);
        else nint_matmul_swiglu(*q->nint, x, x_dtype, ldx, M, hidden, scratch, stream);
    });
}
int mfq_rt_linear_dequantize(void *h, float *out, void *stream) {
    return guard([&] { static_cast<QuantLinear *>(h)->dequantize(out, stream); });
}
int mfq_rt_linear_embedding(void *h, const int64_t *ids, int n_ids, void *out, int out_dtype, void *stream) {
    return guard([&] {
        const QuantLinear *q = static_cast<QuantLinear *>(h);
        q->embedding(ids, n_ids, out, out_dtype, stream);
    });
}
int mfq_rt_linear_argmax(void *h, const void *x, int x_dtype, int64_t ldx, int M, int64_t *token, float *logits, void *stream) {
    return guard([&] {
        const QuantLinear *q = static_cast<QuantLinear *>(h);
        if (!q->nint) fail("the arg-max LM head needs a NINT tensor");
        nint_matmul_argmax(*q->nint, x, x_dtype, ldx, M, token, logits, stream);
    });
}
int mfq_rt_linear_check(void *h, int M, int reps, double *out6) {
    return guard([&] {
        const LinearCheckResult r = run_linear_check(*static_cast<QuantLinear *>(h), M, reps);
        out6[0] = r.production_ms; out6[1] = r.production_weight_gbps; out6[2] = r.payload_gbps;
        out6[3] = r.production_rel; out6[4] = r.production_mean_abs; out6[5] = r.production_max_abs;
    });
}

// Feed-forward block of three NVQ linears (handles from mfq_rt_load_quant_linear); the hidden rows and the joint
// gate/up output live in buffers of this call, so the stream is synchronised before they go.
int mfq_rt_nvq_ffn_swiglu_down(void *gate, void *up, void *down, const void *x, int x_dtype, int64_t ldx, int M, float *y,
                               void *stream) {
    return guard([&] {
        const QuantLinear *g = static_cast<QuantLinear *>(gate), *u = static_cast<QuantLinear *>(up),
                          *d = static_cast<QuantLinear *>(down);
        if (g->kind != QuantLinearKind::Nvq || u->kind != QuantLinearKind::Nvq || d->kind != QuantLinearKind::Nvq)
            throw std::runtime_error("nvq_ffn_swiglu_down takes three NVQ linears");
        const size_t W = static_cast<size_t>(g->out());
        DeviceBuffer hidden(static_cast<size_t>(M) * W * 2), scratch(static_cast<size_t>(M) * W * 8);
        nvq_ffn_swiglu_down(*g->nvq, *u->nvq, *d->nvq, x, x_dtype, ldx, M, y, hidden.get(),
                            static_cast<float *>(scratch.get()), static_cast<mfq_stream_t>(stream));
        hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "sync");
    });
}

// expert residency: cache handle, source handle (owned by the cache)
int mfq_rt_moe_cache_create(int64_t budget_bytes, void **cache) {
    return guard([&] { *cache = new MoeExpertCache(budget_bytes); });
}
void mfq_rt_moe_cache_free(void *cache) { delete static_cast<MoeExpertCache *>(cache); }
int mfq_rt_moe_cache_register(void *cache, const void *blob, size_t n, int minimum_slots, void **source) {
    return guard([&] {
        *source = static_cast<MoeExpertCache *>(cache)->register_source(static_cast<const uint8_t *>(blob), n, minimum_slots);
    });
}
int mfq_rt_moe_cache_finalize(void *cache) {
    return guard([&] { static_cast<MoeExpertCache *>(cache)->finalize(); });
}
int mfq_rt_moe_cache_forward(void *cache, void *source, const void *x, int x_dtype, int64_t ldx, int routed_input,
                             const int32_t *ids, int T, int R, float *out, void *stream) {
    return guard([&] {
        auto *src = static_cast<MoeCachedSource *>(source);
        MoeRoutePlan route = build_moe_route_plan(ids, T, R, src->n_experts, static_cast<mfq_stream_t>(stream));
        static_cast<MoeExpertCache *>(cache)->forward(*src, x, x_dtype, ldx, routed_input != 0, route, out,
                                                      static_cast<mfq_stream_t>(stream));
        hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "sync");  // the route plan's buffers go away
    });
}
int mfq_rt_moe_cache_stats(void *cache, int64_t *out5) {
    return guard([&] {
        const MoeCacheStats &s = static_cast<MoeExpertCache *>(cache)->stats();
        out5[0] = s.hits; out5[1] = s.misses; out5[2] = s.evictions; out5[3] = s.bytes; out5[4] = s.launches;
    });
}

int mfq_rt_load_nint_moe(const void *blob, size_t n, void **handle) {
    return guard([&] { *handle = new NintMoeWeight(NintMoeWeight::from_blob(static_cast<const uint8_t *>(blob), n)); });
}
int mfq_rt_load_nint_moe_overlay(const void *blob, size_t n, const void *overlay, size_t overlay_n, void **handle) {
    return guard([&] {
        *handle = new NintMoeWeight(NintMoeWeight::from_blob(static_cast<const uint8_t *>(blob), n, nullptr,
                                                             static_cast<const uint8_t *>(overlay), overlay_n));
    });
}
void mfq_rt_free_nint_moe(void *handle) { delete static_cast<NintMoeWeight *>(handle); }
int mfq_rt_file_open(const char *path, const char *tensor_overlay, const char *expert_overlay, void **handle) {
    return guard([&] {
        *handle = new MfqFile(path ? path : "", tensor_overlay ? tensor_overlay : "", expert_overlay ? expert_overlay : "");
    });
}
void mfq_rt_file_close(void *handle) { delete static_cast<MfqFile *>(handle); }
int64_t mfq_rt_file_record_count(void *handle) { return static_cast<int64_t>(static_cast<MfqFile *>(handle)->records.size()); }
int64_t mfq_rt_file_tensor_count(void *handle) { return static_cast<int64_t>(static_cast<MfqFile *>(handle)->tensor_count()); }
int64_t mfq_rt_file_source_count(void *handle) { return static_cast<int64_t>(static_cast<MfqFile *>(handle)->source_paths.size()); }
const char *mfq_rt_file_arch(void *handle) { return static_cast<MfqFile *>(handle)->model_arch.c_str(); }
const char *mfq_rt_file_extra(void *handle, const char *key) {
    const MfqFile *f = static_cast<MfqFile *>(handle);
    auto it = f->extra.find(key ? key : "");
    return it == f->extra.end() ? nullptr : it->second.c_str();
}
int mfq_rt_file_record(void *handle, int64_t index, const char **name, const char **dtype, int *source, const void **data,
                       size_t *nbytes) {
    return guard([&] {
        const MfqFile *f = static_cast<MfqFile *>(handle);
        if (index < 0 || index >= static_cast<int64_t>(f->records.size())) fail("MFQ record index out of range");
        const MfqRecord &r = f->records[static_cast<size_t>(index)];
        if (name) *name = r.name.c_str();
        if (dtype) *dtype = r.dtype.c_str();
        if (source) *source = r.source;
        if (data) *data = f->data(r);
        if (nbytes) *nbytes = r.nbytes;
    });
}
int mfq_rt_file_find(void *handle, const char *name, int64_t *index) {
    return guard([&] {
        const MfqFile *f = static_cast<MfqFile *>(handle);
        const MfqRecord &r = f->find(name ? name : "");
        *index = &r - f->records.data();
    });
}
int mfq_rt_file_load_quant_linear(void *handle, const char *name, void **linear) {
    return guard([&] {
        const MfqFile *f = static_cast<MfqFile *>(handle);
        const MfqRecord &r = f->find(name ? name : "");
        *linear = new QuantLinear(load_quant_linear(r.dtype, f->data(r), r.nbytes));
    });
}

int mfq_rt_moe_ffn_forward(void *gate_up, void *down, const void *x, int x_dtype, int64_t ldx, int T,
                           const float *router_logits, int top_k, int topk_mode, int normalize, void *shared_gate_up,
                           void *shared_down, float *out, int32_t *ids_out, float *weights_out, void *stream) {
    return guard([&] {
        MoeFfnScratch s;
        const NintWeight *sg = shared_gate_up ? static_cast<QuantLinear *>(shared_gate_up)->nint.get() : nullptr;
        const NintWeight *sd = shared_down ? static_cast<QuantLinear *>(shared_down)->nint.get() : nullptr;
        nint_moe_ffn_forward(*static_cast<NintMoeWeight *>(gate_up), *static_cast<NintMoeWeight *>(down), x, x_dtype, ldx, T,
                             router_logits, top_k, topk_mode, normalize != 0, nullptr, 1.f, sg, sd, s, out, stream);
        const size_t pairs = static_cast<size_t>(T) * top_k;
        // the scratch is freed on return: wait for the kernels that use it (the copies below are synchronous anyway)
        if (hipStreamSynchronize(static_cast<hipStream_t>(stream)) != hipSuccess) throw std::runtime_error("nint_moe_ffn_forward");
        if (ids_out && hipMemcpy(ids_out, s.ids.get(), 4 * pairs, hipMemcpyDeviceToDevice) != hipSuccess)
            throw std::runtime_error("copy ids");
        if (weights_out && hipMemcpy(weights_out, s.weights.get(), 4 * pairs, hipMemcpyDeviceToDevice) != hipSuccess)
            throw std::runtime_error("copy weights");
    });
}

int mfq_rt_moe_scratch_create(void **scratch) {
    return guard([&] { *scratch = new MoeFfnScratch(); });
}
void mfq_rt_moe_scratch_free(void *scratch) { delete static_cast<MoeFfnScratch *>(scratch); }
int mfq_rt_moe_scratch_reserve(void *scratch, void *gate_up, void *down, int max_tokens, int top_k, void *shared_gate_up,
                               void *shared_down) {
    return guard([&] {
        const NintWeight *sg = shared_gate_up ? static_cast<QuantLinear *>(shared_gate_up)->nint.get() : nullptr;
        const NintWeight *sd = shared_down ? static_cast<QuantLinear *>(shared_down)->nint.get() : nullptr;
        static_cast<MoeFfnScratch *>(scratch)->reserve(*static_cast<NintMoeWeight *>(gate_up), *static_cast<NintMoeWeight *>(down),
                                                       max_tokens, top_k, sg, sd);
    });
}
int mfq_rt_moe_scratch_topk(void *scratch, const int32_t **ids, const float **weights) {
    return guard([&] {
        const MoeFfnScratch *s = static_cast<const MoeFfnScratch *>(scratch);
        if (ids) *ids = static_cast<const int32_t *>(s->ids.get());
        if (weights) *weights = static_cast<const float *>(s->weights.get());
    });
}
int mfq_rt_moe_ffn_forward_scratch(void *scratch, void *gate_up, void *down, const void *x, int x_dtype, int64_t ldx, int T,
                                   const float *router_logits, int top_k, int topk_mode, int normalize, void *shared_gate_up,
                                   void *shared_down, float *out, void *stream) {
    return guard([&] {
        const NintWeight *sg = shared_gate_up ? static_cast<QuantLinear *>(shared_gate_up)->nint.get() : nullptr;
        const NintWeight *sd = shared_down ? static_cast<QuantLinear *>(shared_down)->nint.get() : nullptr;
        nint_moe_ffn_forward(*static_cast<NintMoeWeight *>(gate_up), *static_cast<NintMoeWeight *>(down), x, x_dtype, ldx, T,
                             router_logits, top_k, topk_mode, normalize != 0, nullptr, 1.f, sg, sd,
                             *static_cast<MoeFfnScratch *>(scratch), out, stream);
    });
}
}
