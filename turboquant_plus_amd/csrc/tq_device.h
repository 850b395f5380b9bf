// Device-side helpers: cross-lane exchanges for wave64, Walsh-Hadamard
// butterflies, and the packed "pair container" row format.
#pragma once
#include "tq_internal.h"
#include "tq_layout.h"
#include "tq_measure.h"

namespace tqd {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// ---- streaming stores -----------------------------------------------------------
// Output that a launch writes once and never reads back goes out with the non-temporal hint: the lines do not
// wait in the L2 for the end-of-kernel write-back, so the writes overlap the rest of the launch.
// TQ_STREAM_SITES (bit mask, tq_measure.h: measurement builds only) switches the hint off per family of kernels.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <int SITE> __device__ __forceinline__ void stream_store(uint32_t *p, uint32_t v) {
    if constexpr ((TQ_STREAM_SITES & SITE) != 0) __builtin_nontemporal_store(v, p);
    else *p = v;
}
template <int SITE> __device__ __forceinline__ void stream_store(float *p, float v) {
    if constexpr ((TQ_STREAM_SITES & SITE) != 0) __builtin_nontemporal_store(v, p);
    else *p = v;
}
template <int SITE> __device__ __forceinline__ void stream_store(uint4 *p, uint4 v) {
    if constexpr ((TQ_STREAM_SITES & SITE) != 0) {
        const u32x4_t u = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(u, reinterpret_cast<u32x4_t *>(p));
    } else {
        *p = v;
    }
}
constexpr int STREAM_STORE_CODES = 1, STREAM_LOAD_OUT = 2, STREAM_LOGITS = 4, STREAM_Q8 = 8, STREAM_ATTN_ROWS = 16,
              STREAM_STORE_V_IN = 32;
// 16 bytes of input that a launch reads exactly once, every 128-byte line whole within one instruction
template <int SITE> __device__ __forceinline__ float4 stream_load(const float4 *p) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    if constexpr ((TQ_STREAM_SITES & SITE) != 0) {
        const f32x4_t u = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(p));
        return make_float4(u[0], u[1], u[2], u[3]);
    } else {
        return *p;
    }
}
template <int SITE> __device__ __forceinline__ uint4 stream_load(const uint4 *p) {
    if constexpr ((TQ_STREAM_SITES & SITE) != 0) {
        const u32x4_t u = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
        return make_uint4(u[0], u[1], u[2], u[3]);
    } else {
        return *p;
    }
}

// ---- cross-lane exchange ------------------------------------------------------
// DPP control words (GCN3+/CDNA): quad_perm = 4 x 2-bit selectors, 0x12n =
// row_ror:n, 0x141 = row_half_mirror.  Every pattern used here reads a valid
// lane, so bound_ctrl / old are irrelevant.
template <int CTRL> __device__ inline float dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> __device__ inline uint32_t dpp(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL> __device__ inline double dpp(double v) {
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(b & 0xffffffffll), CTRL, 0xF, 0xF, true);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xF, 0xF, true);
    return __builtin_bit_cast(double, ((long long)hi << 32) | (unsigned)lo);
}

// value held by lane (lane ^ M); M in {1,2,4,8,16,32}
template <int M, typename T> __device__ inline T xor_lane(T v) {
    if constexpr (M == 1) return dpp<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (M == 2) return dpp<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (M == 4) return dpp<0x1B>(dpp<0x141>(v));  // half-mirror (^7) then quad reverse (^3)
    else if constexpr (M == 8) return dpp<0x128>(v);  // row_ror:8
    else if constexpr (M == 16) {
        if constexpr (sizeof(T) == 4) {
            return __builtin_bit_cast(T, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
        } else {
            const long long b = __builtin_bit_cast(long long, v);
            const int lo = __builtin_amdgcn_ds_swizzle((int)(b & 0xffffffffll), 0x401F);
            const int hi = __builtin_amdgcn_ds_swizzle((int)(b >> 32), 0x401F);
            return __builtin_bit_cast(T, ((long long)hi << 32) | (unsigned)lo);
        }
    } else {
        static_assert(M == 32, "unsupported xor mask");
        if constexpr (sizeof(T) == 4) {
            const unsigned u = __builtin_bit_cast(unsigned, v);
            // r[0] = lanes 0..31 duplicated into both halves, r[1] = lanes 32..63 duplicated
            auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
            const unsigned o = (__lane_id() < 32) ? r[1] : r[0];
            return __builtin_bit_cast(T, o);
        } else {
            return __shfl_xor(v, 32);
        }
    }
}

// sum over the 16 lanes of a DPP row (result in every lane of the row)
template <typename T> __device__ inline T row16_sum(T v) {
    v += xor_lane<1>(v);
    v += xor_lane<2>(v);
    v += dpp<0x124>(v);  // row_ror:4
    v += dpp<0x128>(v);  // row_ror:8
    return v;
}

// ---- Walsh-Hadamard butterflies ------------------------------------------------
// One cross-lane stage: lanes with bit M clear get own+partner, lanes with it
// set get partner-own.  `sgn` is +1 / -1 accordingly (precomputed per lane).
template <int M, typename T> __device__ inline T bfly(T v, T sgn) { return fma(sgn, v, xor_lane<M>(v)); }

// 8 values per lane, 16 lanes per vector: element index e = 8*(lane&15) + m.
// Unnormalised natural-order WHT of the 128 values held by a 16-lane row.
template <typename T> __device__ inline void wht128_row16(T (&x)[8], int lane) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if ((m & h) == 0) {
                const T a = x[m], b = x[m + h];
                x[m] = a + b;
                x[m + h] = a - b;
            }
        }
    }
    const T s1 = (lane & 1) ? T(-1) : T(1), s2 = (lane & 2) ? T(-1) : T(1);
    const T s4 = (lane & 4) ? T(-1) : T(1), s8 = (lane & 8) ? T(-1) : T(1);
#pragma unroll
    for (int m = 0; m < 8; ++m) x[m] = bfly<1>(x[m], s1);
#pragma unroll
    for (int m = 0; m < 8; ++m) x[m] = bfly<2>(x[m], s2);
#pragma unroll
    for (int m = 0; m < 8; ++m) x[m] = bfly<4>(x[m], s4);
#pragma unroll
    for (int m = 0; m < 8; ++m) x[m] = bfly<8>(x[m], s8);
}

// 2 values per lane, one 64-lane wavefront per vector: lane holds elements
// (2*lane, 2*lane+1).  Stage h=1 is in-lane, h=2..64 are lane xor 1..32.
__device__ inline void wht128_wave(float &a, float &b, int lane) {
    const float t = a + b;
    b = a - b;
    a = t;
#define TQ_STAGE(M)                                           \
    {                                                         \
        const float sg = (lane & M) ? -1.0f : 1.0f;           \
        a = bfly<M>(a, sg);                                   \
        b = bfly<M>(b, sg);                                   \
    }
    TQ_STAGE(1) TQ_STAGE(2) TQ_STAGE(4) TQ_STAGE(8) TQ_STAGE(16) TQ_STAGE(32)
#undef TQ_STAGE
}

// ---- packed rows: the index arithmetic lives in tq_layout.h (shared with the host checks) -------------
// 24-bit tail (pairs 12..15) of group g of a 3-bit row
__device__ __forceinline__ uint32_t tail24(const uint32_t *w, int g) {
    return (w[g] >> 24) | ((w[4 + g] >> 24) << 8) | ((w[8 + g] >> 24) << 16);
}

// field `width` bits wide at bit `sh` of x, scaled by 2^SCALE (a table byte offset)
template <int SCALE> __device__ __forceinline__ uint32_t field_offset(uint32_t x, int sh, int width) {
    const uint32_t mask = ((1u << width) - 1u) << SCALE;
    return sh >= SCALE ? ((x >> (sh - SCALE)) & mask) : ((x << (SCALE - sh)) & mask);
}

// byte offset (pair code * 4) into a 4-byte-entry LUT; p must fold to a constant
template <int BITS> __device__ __forceinline__ uint32_t pair_lut_offset(const uint32_t (&w)[4 * BITS], int p) {
    if (pair_in_tail(BITS, p)) return field_offset<2>(tail24(w, p >> 4), 6 * ((p & 15) - 12), 6);
    return field_offset<2>(w[pair_dword(BITS, p)], pair_shift(BITS, p), 2 * BITS);
}

// byte offset (quad code * 8) into an 8-byte-entry LUT of quad Q = pairs 2Q, 2Q+1;
// Q must fold to a constant
template <int BITS> __device__ __forceinline__ uint32_t quad_lut_offset(const uint32_t (&w)[4 * BITS], int Q) {
    if (pair_in_tail(BITS, 2 * Q)) return field_offset<3>(tail24(w, Q >> 3), 12 * ((Q & 7) - 6), 12);
    return field_offset<3>(w[pair_dword(BITS, 2 * Q)], pair_shift(BITS, 2 * Q), 4 * BITS);
}

// runtime pair extraction (slow path: unpack / load kernels)
__device__ inline uint32_t pair_code(const uint32_t *w, int bits, int p) {
    if (pair_in_tail(bits, p)) return (tail24(w, p >> 4) >> (6 * ((p & 15) - 12))) & 63u;
    return (w[pair_dword(bits, p)] >> pair_shift(bits, p)) & ((1u << (2 * bits)) - 1u);
}

}  // namespace tqd
