// Measurement probes: what this part sustains on plain streaming and on back-to-back MFMAs, so that
// roofline fractions can be stated against measured figures as well as against the published peaks.
// Not part of the codec; the callers time the launches themselves.
// Built into its own library (libtq_probe.so, header tq_probe.h): the codec's C ABI does not carry it.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "tq_probe.h"

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// mode 0: read, 1: write, 2: copy, 3 / 4 / 5: write / read / copy with the non-temporal hint; 16 bytes per lane and step.  CHUNKED: every workgroup a contiguous slice,
// else all lanes of the grid stride over the buffer.
template <int MODE, bool CHUNKED>
__global__ __launch_bounds__(512) void k_probe_stream(const uint4 *src, uint4 *dst, int64_t n16) {
    const int64_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const int64_t lo = CHUNKED ? (int64_t)blockIdx.x * per : (int64_t)blockIdx.x * 512;
    const int64_t hi = CHUNKED ? (lo + per < n16 ? lo + per : n16) : n16;
    const int64_t step = CHUNKED ? 512 : (int64_t)gridDim.x * 512;
    uint4 acc = make_uint4(0, 0, 0, 0);
    const uint4 fill = make_uint4(threadIdx.x, 1u, 2u, 3u);
    for (int64_t i = lo + threadIdx.x; i < hi; i += step) {
        if constexpr (MODE == 0) {
            const uint4 v = src[i];
            acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
        } else if constexpr (MODE == 1) {
            dst[i] = fill;
        } else if constexpr (MODE == 2) {
            dst[i] = src[i];
        } else if constexpr (MODE == 3) {
            __builtin_nontemporal_store(u32x4_t{fill.x, fill.y, fill.z, fill.w}, reinterpret_cast<u32x4_t *>(dst + i));
        } else if constexpr (MODE == 4) {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(src + i));
            acc.x ^= v[0]; acc.y ^= v[1]; acc.z ^= v[2]; acc.w ^= v[3];
        } else {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(src + i));
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t *>(dst + i));
        }
    }
    // keeps the reads alive; the condition does not hold for any data a caller would pass
    if constexpr (MODE == 0 || MODE == 4) {
        if ((acc.x & acc.y & acc.z & acc.w) == 0xFFFFFFFFu && dst) dst[0] = acc;
    }
}

// Short-lived workgroups in dispatch order: workgroup u reads the 16 KB unit u of src (four 16-byte loads per
// lane, when READS) and writes 16 * W chunks of 16 bytes at dst + u * 16 * W chunks (the first lanes, when W > 0).
// The memory side sees one compact window that moves through both buffers, which this part serves faster than
// the strided sweeps of long-lived workgroups above (writes above all).
template <bool READS, bool NT>
__global__ __launch_bounds__(256) void k_probe_flat(const u32x4_t *src, u32x4_t *dst, int w64) {
    const int64_t u = blockIdx.x;
    u32x4_t acc = {threadIdx.x, 1u, 2u, 3u};
    if constexpr (READS) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u32x4_t *p = src + u * 1024 + j * 256 + threadIdx.x;
            acc ^= NT ? __builtin_nontemporal_load(p) : *p;
        }
    }
    for (int c = threadIdx.x; c < 16 * w64; c += 256) {
        u32x4_t *q = dst + u * 16 * w64 + c;
        if (NT) __builtin_nontemporal_store(acc, q);
        else *q = acc;
    }
    // keeps the reads alive when nothing is written; the condition does not hold for any data a caller would pass
    if (READS && w64 == 0 && dst && (acc[0] & acc[1] & acc[2] & acc[3]) == 0xFFFFFFFFu) dst[0] = acc;
}

// 8 independent accumulator tiles per wavefront, `iters` rounds of one MFMA on each
__global__ __launch_bounds__(256) void k_probe_mfma(int64_t iters, float *sink) {
    const int lane = threadIdx.x & 63;
    half8_t a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (_Float16)(0.001f * (float)((lane + e) & 7));
        b[e] = (_Float16)(0.002f * (float)((lane * 3 + e) & 7));
    }
    float16_t acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.0f;
    for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[t], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[t][e];
    if (s == -1.0f) sink[0] = s;  // sums of non-negative products: never taken, keeps the MFMAs alive
}

constexpr int PROBE_MFMA_WGS = 2048;  // 8 workgroups of 4 wavefronts per CU

}  // namespace

extern "C" int tq_probe_stream(int mode, int chunked, const void *src, void *dst, int64_t bytes, void *stream) {
    hipStream_t s = (hipStream_t)stream;
    const bool reads = mode == 0 || mode == 2 || mode == 4 || mode == 5, writes = mode == 1 || mode == 2 || mode == 3 || mode == 5;
    if (mode < 0 || mode > 5 || bytes < 16 || (bytes & 15) || (reads && !src) || (writes && !dst)) return TQ_PROBE_ERR_ARG;
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) return TQ_PROBE_ERR_ARG;
    const int64_t n16 = bytes / 16;
    const unsigned grid = 256 * 4;
    const uint4 *s4 = reads ? (const uint4 *)src : nullptr;
    uint4 *d4 = writes ? (uint4 *)dst : nullptr;
#define TQ_PROBE_MODE(M)                                                              \
    case M:                                                                           \
        if (chunked) k_probe_stream<M, true><<<grid, 512, 0, s>>>(s4, d4, n16);       \
        else k_probe_stream<M, false><<<grid, 512, 0, s>>>(s4, d4, n16);              \
        break
    switch (mode) {
        TQ_PROBE_MODE(0); TQ_PROBE_MODE(1); TQ_PROBE_MODE(2); TQ_PROBE_MODE(3); TQ_PROBE_MODE(4);
        default: TQ_PROBE_MODE(5);
    }
#undef TQ_PROBE_MODE
    return hipGetLastError() == hipSuccess ? 0 : TQ_PROBE_ERR_HIP;
}

extern "C" int tq_probe_flat(const void *src, void *dst, int64_t units, int write_64ths, int nontemporal, void *stream) {
    if (units < 1 || units > 0x7FFFFFFF || write_64ths < 0 || write_64ths > 64 || (!src && write_64ths == 0) || (write_64ths > 0 && !dst))
        return TQ_PROBE_ERR_ARG;
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) return TQ_PROBE_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const u32x4_t *s4 = (const u32x4_t *)src;
    u32x4_t *d4 = (u32x4_t *)dst;
    const unsigned grid = (unsigned)units;
    if (src && nontemporal) k_probe_flat<true, true><<<grid, 256, 0, s>>>(s4, d4, write_64ths);
    else if (src) k_probe_flat<true, false><<<grid, 256, 0, s>>>(s4, d4, write_64ths);
    else if (nontemporal) k_probe_flat<false, true><<<grid, 256, 0, s>>>(s4, d4, write_64ths);
    else k_probe_flat<false, false><<<grid, 256, 0, s>>>(s4, d4, write_64ths);
    return hipGetLastError() == hipSuccess ? 0 : TQ_PROBE_ERR_HIP;
}

extern "C" int64_t tq_probe_mfma_f16(int64_t iters, float *sink, void *stream) {
    // one launch keeps every CU busy for about iters * 0.13 us: the cap bounds a single launch at about 0.13 s
    if (iters < 1 || iters > TQ_PROBE_MAX_ITERS || !sink) return (int64_t)TQ_PROBE_ERR_ARG;
    k_probe_mfma<<<PROBE_MFMA_WGS, 256, 0, (hipStream_t)stream>>>(iters, sink);
    if (hipGetLastError() != hipSuccess) return (int64_t)TQ_PROBE_ERR_HIP;
    return (int64_t)PROBE_MFMA_WGS * 4 * iters * 8 * (2ll * 32 * 32 * 16);
}
