// Production-format kernels (d = 128, sign-diagonal WHT rotation, fp32
// arithmetic, corrected fp16 norm, 128-token blocks of packed pair codes).
//
//   k_wht128       one 64-lane wavefront per vector, two values per lane, the
//                  seven butterfly stages in registers (one in-lane, six through
//                  DPP / ds_swizzle / permlane32 exchanges).
//   k_store        norm -> D2 H D1 -> nearest centroid -> corrected norm -> pack.
//                  16 lanes per vector (8 values each): three in-lane stages and
//                  four DPP row stages; a workgroup owns one 128-token block,
//                  stages the codes in LDS and writes the block coalesced.
//   k_store_qjl_mfma  float64 variant that also sketches the residual (1-bit QJL), projection on fp64 MFMAs.
//   k_load         packed block -> values (rotated or original domain).
//   k_unpack_codes packed block -> uint8 indices + fp32 norms.
//   k_q8_0_store   32-value int8 blocks with fp16 scale, 128-token block layout.
#include <cstdlib>
#include <cstring>

#include "tq_device.h"
#include "tq_device64.h"

namespace {

using namespace tqd;

constexpr float RSQRT128 = 0.08838834764831845f;
constexpr int CODE_STRIDE = 136;  // bytes per token in the LDS code stage (8-byte aligned, odd multiple of 8)

// ---- typed 8-value loads / stores ---------------------------------------------
template <typename T> __device__ inline void load8(const T *p, float (&v)[8]);
template <> __device__ inline void load8<__half>(const __half *p, float (&v)[8]) {
    const uint4 u = *reinterpret_cast<const uint4 *>(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __half2float(__ushort_as_half((unsigned short)(w[i] & 0xffffu)));
        v[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(w[i] >> 16)));
    }
}
template <> __device__ inline void load8<float>(const float *p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4 *>(p);
    const float4 b = *reinterpret_cast<const float4 *>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <> __device__ inline void load8<double>(const double *p, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)p[i];
}
template <typename T> __device__ inline void store8(T *p, const float (&v)[8]);
template <> __device__ inline void store8<__half>(__half *p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        w[i] = (uint32_t)__half_as_ushort(__float2half_rn(v[2 * i])) |
               ((uint32_t)__half_as_ushort(__float2half_rn(v[2 * i + 1])) << 16);
    *reinterpret_cast<uint4 *>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}
template <> __device__ inline void store8<float>(float *p, const float (&v)[8]) {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <> __device__ inline void store8<double>(double *p, const float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) p[i] = (double)v[i];
}
template <typename T> __device__ inline float ld1(const T *p) { return (float)*p; }
template <> __device__ inline float ld1<__half>(const __half *p) { return __half2float(*p); }
template <typename T> __device__ inline void st1(T *p, float v) { *p = (T)v; }
template <> __device__ inline void st1<__half>(__half *p, float v) { *p = __float2half_rn(v); }

// ---- K1: standalone rotation, one wavefront per vector -------------------------
// y = sb * H(sa * x) / sqrt(128) with (sa, sb) = (s1, s2) forward, (s2, s1) transposed.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void k_wht128(const TI *x, TO *y, int64_t n, const float *sa, const float *sb) {
    const int lane = threadIdx.x & 63;
    const int64_t wave0 = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    const float a0 = sa[2 * lane], a1 = sa[2 * lane + 1];
    const float b0 = sb[2 * lane] * RSQRT128, b1 = sb[2 * lane + 1] * RSQRT128;
    for (int64_t v = wave0; v < n; v += nwaves) {
        float a = ld1(x + v * 128 + 2 * lane) * a0;
        float b = ld1(x + v * 128 + 2 * lane + 1) * a1;
        wht128_wave(a, b, lane);
        st1(y + v * 128 + 2 * lane, a * b0);
        st1(y + v * 128 + 2 * lane + 1, b * b1);
    }
}

// ---- block packer ----------------------------------------------------------------
// codes: LDS bytes [128 tokens][CODE_STRIDE]; norms: LDS float [128]; out: one block.
template <int BITS> __device__ inline uint32_t pair_from_stage(const uint8_t *codes, int kind, int row, int p) {
    uint32_t lo, hi;
    if (kind == TQ_KIND_K) {
        lo = codes[row * CODE_STRIDE + 2 * p];
        hi = codes[row * CODE_STRIDE + 2 * p + 1];
    } else {
        const int tok = (row & 64) + ((p & 60) | ((p & 1) << 1));
        const int dim = ((p & 2) << 5) | (row & 63);
        lo = codes[tok * CODE_STRIDE + dim];
        hi = codes[(tok + 1) * CODE_STRIDE + dim];
    }
    return lo | (hi << BITS);
}

// first_row > 0 (K rows only, where a row is a token): rows and norms below it are left as they are in memory.
template <int BITS, int NTHREADS>
__device__ inline void pack_block(const uint8_t *codes, const float *norms, uint8_t *out_block, int kind, int first_row = 0) {
    uint32_t *out = reinterpret_cast<uint32_t *>(out_block);
    constexpr int NDW = TQ_ROWS_PER_BLOCK * 4 * BITS;
    for (int o = threadIdx.x; o < NDW; o += NTHREADS) {
        const int c = o >> 9, r = (o & 511) >> 2, k = o & 3;
        if (r < first_row) continue;
        // chunk c, dword k of the row = dword j = c of group g = k
        constexpr int PER = pairs_per_dword(BITS);
        const int g = k, j = c;
        uint32_t word = 0;
        if (kind == TQ_KIND_K) {
            // a K row's pairs are neighbouring bytes of the stage: the dword's 2 PER codes (and the 3-bit tail's
            // eight) come in 8-byte reads, code i at bit BITS i
            const uint8_t *src = codes + r * CODE_STRIDE + 32 * g;
            auto gather8 = [](uint2 v) {
                uint32_t w = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    w |= ((v.x >> (8 * i)) & 0xFFu) << (BITS * i);
                    w |= ((v.y >> (8 * i)) & 0xFFu) << (BITS * (4 + i));
                }
                return w;
            };
            word = gather8(*reinterpret_cast<const uint2 *>(src + 2 * PER * j));
            if constexpr (BITS == 2) word |= gather8(*reinterpret_cast<const uint2 *>(src + 16 * j + 8)) << 16;
            if constexpr (BITS == 3) word |= ((gather8(*reinterpret_cast<const uint2 *>(src + 24)) >> (8 * j)) & 0xFFu) << 24;
        } else {
#pragma unroll
            for (int t = 0; t < PER; ++t) word |= pair_from_stage<BITS>(codes, kind, r, 16 * g + PER * j + t) << (2 * BITS * t);
            if constexpr (BITS == 3) {
                uint32_t tail = 0;
#pragma unroll
                for (int t = 0; t < 4; ++t) tail |= pair_from_stage<3>(codes, kind, r, 16 * g + 12 + t) << (6 * t);
                word |= ((tail >> (8 * j)) & 0xFFu) << 24;
            }
        }
        out[o] = word;
    }
    if (first_row == 0) {
        for (int t = threadIdx.x; t < 64; t += NTHREADS) {
            const uint32_t lo = __half_as_ushort(__float2half_rn(norms[2 * t]));
            const uint32_t hi = __half_as_ushort(__float2half_rn(norms[2 * t + 1]));
            out[NDW + t] = lo | (hi << 16);
        }
    } else {
        __half *nout = reinterpret_cast<__half *>(out + NDW);
        for (int t = first_row + (int)threadIdx.x; t < TQ_ROWS_PER_BLOCK; t += NTHREADS) nout[t] = __float2half_rn(norms[t]);
    }
}

struct StoreArgs {
    const float *s1, *s2, *bounds, *cent;
    int kind, norm_correction;
    int64_t tokens;       // per sequence
    int64_t blocks_per_seq;
};

// TQ_KNOCKOUT (tq_measure.h; measurement builds only, 0 in the product) removes one phase of the fp16 store kernels so
// that its share of the launch time and of the vector instructions can be read off (results are then meaningless).
// 1: quantiser compares (a value's code bits come from one xor of its raw bits); 2: four-point butterfly over the input
// slices; 4: level counts and sum c^2; 8: the sum-of-squares MFMAs (norm = 1); 16: the code stores; 32: the HBM reads
// (a wavefront re-reads the first units of its share).
// 16 bytes of input (read with the default cache policy: the four loads of a K unit touch every 128-byte line of
// the unit four times, and with the non-temporal hint each touch went to memory: 20.7 -> 29.8 us for 262 144 K rows)
__device__ __forceinline__ uint4 load_input16(const uint4 *p) { return *p; }
__device__ __forceinline__ uint32_t ko_append4(uint32_t w, float y0, float y1, float y2, float y3) {
    return ((w << 4) ^ __float_as_uint(y0)) + ((__float_as_uint(y1) ^ __float_as_uint(y2)) + __float_as_uint(y3));
}

// ---- K2, fp16 input: rotation on the matrix cores ------------------------------------
// R' = D2 H D1 has entries +-1, so with fp16 inputs every product of X R'^T is exact and
// only the fp32 accumulation rounds (same error class as the butterfly).  Quantisation uses
// the sign symmetry of the codebook (checked when the handle is built): index = mid+1+m for
// a positive rotated value, mid-m otherwise, with m = #{positive boundaries < |y|}.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// a * s + b per element (the table path of 4-bit codes normalises inside the last butterfly stage: two products and
// four fused multiply-adds per four outputs instead of four additions and four products)
__device__ __forceinline__ float4_t fma4(float4_t a, float4_t s, float4_t b) {
    float4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __builtin_fmaf(a[i], s[i], b[i]);
    return r;
}

// ---- K2, fp16 input, K rows: codes packed in registers ---------------------------------
// Index bits of H128[m][k] = (-1)^popcount(m & k) pair up, so the transform splits as
//   m = 32c + 8fh + 4f0 + i  (c = lane quarter, fh/f0 = fragment, i = row in the lane)
//   k = 32kb + 8ks + e       (kb = operand lane quarter, ks = input slice, e = element)
//   y'[m] = s2[m] * sum_ks (-1)^popcount(fh & ks) * Q[f0][ks][4c + i],
//   Q[f0][ks] = A[f0][ks] (16 x 32) * X[ks] (32 x 16 tokens),
//   A[f0][ks][4c + i][8kb + e] = s1[k] * H[32c + 4f0 + i][k]:
// eight MFMAs with +-1 operands (exact products, fp32 accumulation) and a four-point
// butterfly over ks per (f0, i) replace a dense 128 x 128 product.  Lane quarter c of token
// lane%16 ends up with dims 32c .. 32c+31 of that token, which is pair group c of the
// token's row: BITS dwords that no other lane touches.  Code bits come from compares whose
// lane masks are shifted into the dword with one add-with-carry each (w = 2w + bit, most
// significant bit first) in unfolded form [sign, level bits]; one xor per dword turns the
// appended sign bits into "positive after s2", sum c^2 comes from population counts on the
// unfolded dwords and the final codes from one in-word fold (level bits are complemented
// where the value is not positive).
// Code bits are appended by hand-scheduled groups: every compare result (a lane mask in an
// SGPR pair) is consumed at least three instructions after the compare that wrote it, which
// is what the hardware needs between a vector instruction writing a scalar register and a
// vector instruction reading it; the carry-out of each add goes to vcc and is never read.
// The scalar registers named in the text are listed as clobbers.

// The sign bit of the value itself is appended with one funnel shift (so the sign field of
// the unfolded code is 1 for negative values).  t[0] is not used: the middle boundary is 0.

// 3-bit: values y0..y3 in append order; t[1..3] magnitude boundaries
__device__ __forceinline__ uint32_t append4_b3(uint32_t w, float y0, float y1, float y2, float y3, const float (&t)[4]) {
    float u0, u1, u2, u3;
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t2]\n\t"
        "v_cndmask_b32_e64 %[u0], %[t1], %[t3], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[u1], %[t1], %[t3], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[u2], %[t1], %[t3], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[u3], %[t1], %[t3], s[66:67]\n\t"
        "v_cmp_gt_f32_e64 s[70:71], |%[y0]|, %[u0]\n\t"
        "v_cmp_gt_f32_e64 s[72:73], |%[y1]|, %[u1]\n\t"
        "v_cmp_gt_f32_e64 s[74:75], |%[y2]|, %[u2]\n\t"
        "v_cmp_gt_f32_e64 s[76:77], |%[y3]|, %[u3]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y0], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[60:61]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[70:71]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y1], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[62:63]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[72:73]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y2], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[64:65]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[74:75]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y3], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[66:67]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[76:77]\n\t"
        : [w] "+v"(w), [u0] "=&v"(u0), [u1] "=&v"(u1), [u2] "=&v"(u2), [u3] "=&v"(u3)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t1] "v"(t[1]), [t2] "v"(t[2]), [t3] "v"(t[3])
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77", "vcc");
    return w;
}

// 4-bit: binary search over t[1..7] (t[4] first), values y0..y3 in append order
__device__ __forceinline__ uint32_t append4_b4(uint32_t w, float y0, float y1, float y2, float y3, const float (&t)[8]) {
    float a0, a1, a2, a3, b0, b1, b2, b3;
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t4]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t4]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t4]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t4]\n\t"
        "v_cndmask_b32_e64 %[a0], %[t2], %[t6], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[a1], %[t2], %[t6], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[a2], %[t2], %[t6], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[a3], %[t2], %[t6], s[66:67]\n\t"
        "v_cmp_gt_f32_e64 s[68:69], |%[y0]|, %[a0]\n\t"
        "v_cmp_gt_f32_e64 s[70:71], |%[y1]|, %[a1]\n\t"
        "v_cmp_gt_f32_e64 s[72:73], |%[y2]|, %[a2]\n\t"
        "v_cmp_gt_f32_e64 s[74:75], |%[y3]|, %[a3]\n\t"
        "v_cndmask_b32_e64 %[b0], %[t1], %[t5], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[b1], %[t1], %[t5], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[b2], %[t1], %[t5], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[b3], %[t1], %[t5], s[66:67]\n\t"
        "v_cndmask_b32_e64 %[a0], %[t3], %[t7], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[a1], %[t3], %[t7], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[a2], %[t3], %[t7], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[a3], %[t3], %[t7], s[66:67]\n\t"
        "v_cndmask_b32_e64 %[b0], %[b0], %[a0], s[68:69]\n\t"
        "v_cndmask_b32_e64 %[b1], %[b1], %[a1], s[70:71]\n\t"
        "v_cndmask_b32_e64 %[b2], %[b2], %[a2], s[72:73]\n\t"
        "v_cndmask_b32_e64 %[b3], %[b3], %[a3], s[74:75]\n\t"
        "v_cmp_gt_f32_e64 s[76:77], |%[y0]|, %[b0]\n\t"
        "v_cmp_gt_f32_e64 s[78:79], |%[y1]|, %[b1]\n\t"
        "v_cmp_gt_f32_e64 s[80:81], |%[y2]|, %[b2]\n\t"
        "v_cmp_gt_f32_e64 s[82:83], |%[y3]|, %[b3]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y0], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[60:61]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[68:69]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[76:77]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y1], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[62:63]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[70:71]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[78:79]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y2], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[64:65]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[72:73]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[80:81]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y3], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[66:67]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[74:75]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[82:83]\n\t"
        : [w] "+v"(w), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3), [b0] "=&v"(b0), [b1] "=&v"(b1),
          [b2] "=&v"(b2), [b3] "=&v"(b3)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t1] "v"(t[1]), [t2] "v"(t[2]),
          [t3] "v"(t[3]), [t4] "v"(t[4]), [t5] "v"(t[5]), [t6] "v"(t[6]), [t7] "v"(t[7])
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "vcc");
    return w;
}

__device__ __forceinline__ uint32_t append4_b2(uint32_t w, float y0, float y1, float y2, float y3, const float (&t)[2]) {
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t1]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y0], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[60:61]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y1], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[62:63]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y2], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[64:65]\n\t"
        "v_alignbit_b32 %[w], %[w], %[y3], 31\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[w], s[66:67]\n\t"
        : [w] "+v"(w)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t1] "v"(t[1])
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "vcc");
    return w;
}

// 4-bit codes by table: entry e of a value (tq_handle::quant_lut, indexed by the value's top 12 bits) holds in
// .x the unfolded field [sign, boundaries below the bin] and in .y the one boundary inside the bin, so
// field = e.x + (|y| > e.y): one compare and one add-with-carry per value instead of a three-level search.
// DUP: the table holds every entry twice (8192 x 8 B, load_quant_lut_dup), so that the byte offset is a plain mask of the
// value's upper half - one instruction with sub-dword operand selection instead of a shift and a mask.
template <bool DUP> __device__ __forceinline__ uint32_t quant_lut_offset(float y) {
    if constexpr (DUP) {
        uint32_t off;
        asm("v_and_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"
            : "=v"(off)
            : "v"(0xfff8u), "v"(y));
        return off;
    } else {
        return (__float_as_uint(y) >> 17) & 0x7ff8u;
    }
}

__device__ __forceinline__ uint32_t append4_lut(uint32_t w, float y0, float y1, float y2, float y3, uint2 e0, uint2 e1, uint2 e2,
                                                uint2 e3) {
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t0]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t3]\n\t"
        "v_lshlrev_b32_e32 %[w], 4, %[w]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[b0], s[60:61]\n\t"
        "v_lshlrev_b32_e32 %[w], 4, %[w]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[b1], s[62:63]\n\t"
        "v_lshlrev_b32_e32 %[w], 4, %[w]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[b2], s[64:65]\n\t"
        "v_lshlrev_b32_e32 %[w], 4, %[w]\n\t"
        "v_addc_co_u32_e64 %[w], vcc, %[w], %[b3], s[66:67]\n\t"
        : [w] "+v"(w)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t0] "v"(e0.y), [t1] "v"(e1.y), [t2] "v"(e2.y), [t3] "v"(e3.y),
          [b0] "v"(e0.x), [b1] "v"(e1.x), [b2] "v"(e2.x), [b3] "v"(e3.x)
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "vcc");
    return w;
}

// the same for four rows at once (V kernel): w_d = 16 w_d + field_d
__device__ __forceinline__ void append_rows_lut(uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &w3, float y0, float y1, float y2,
                                                float y3, uint2 e0, uint2 e1, uint2 e2, uint2 e3) {
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t0]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t3]\n\t"
        "v_lshlrev_b32_e32 %[w0], 4, %[w0]\n\t"
        "v_lshlrev_b32_e32 %[w1], 4, %[w1]\n\t"
        "v_lshlrev_b32_e32 %[w2], 4, %[w2]\n\t"
        "v_lshlrev_b32_e32 %[w3], 4, %[w3]\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[b0], s[60:61]\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[b1], s[62:63]\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[b2], s[64:65]\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[b3], s[66:67]\n\t"
        : [w0] "+v"(w0), [w1] "+v"(w1), [w2] "+v"(w2), [w3] "+v"(w3)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t0] "v"(e0.y), [t1] "v"(e1.y), [t2] "v"(e2.y), [t3] "v"(e3.y),
          [b0] "v"(e0.x), [b1] "v"(e1.x), [b2] "v"(e2.x), [b3] "v"(e3.x)
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "vcc");
}

// The same counts for the four unfolded 4-bit dwords of a lane (32 values) at once: level-bit plane k of dword d is
// moved to bit 4 i + d of one word per plane, so the products and the population counts run once per 32 values
// instead of once per 8 (32 instructions instead of 64).
__device__ __forceinline__ void count_levels4_merged(const uint32_t (&w)[4], uint32_t (&n)[8]) {
    constexpr uint32_t K0 = 0x11111111u;
    uint32_t plane[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        plane[k] = 0u;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t t = d >= k ? w[d] << (d - k) : w[d] >> (k - d);
            plane[k] |= t & (K0 << d);
        }
    }
    const uint32_t b01 = plane[0] & plane[1];
    n[1] += __builtin_popcount(plane[0]);
    n[2] += __builtin_popcount(plane[1]);
    n[3] += __builtin_popcount(b01);
    n[4] += __builtin_popcount(plane[2]);
    n[5] += __builtin_popcount(plane[0] & plane[2]);
    n[6] += __builtin_popcount(plane[1] & plane[2]);
    n[7] += __builtin_popcount(b01 & plane[2]);
}

// n[S] += number of fields of the unfolded dword whose level bits include the set S
template <int BITS> __device__ __forceinline__ void count_levels(uint32_t w, uint32_t (&n)[1 << (BITS - 1)]) {
    if constexpr (BITS == 2) {
        n[1] += __builtin_popcount(w & 0x55555555u);
    } else if constexpr (BITS == 3) {
        constexpr uint32_t K0 = 0x00249249u;  // bit 0 of the eight 3-bit fields
        const uint32_t b0 = w & K0, b1 = (w >> 1) & K0;
        n[1] += __builtin_popcount(b0);
        n[2] += __builtin_popcount(b1);
        n[3] += __builtin_popcount(b0 & b1);
    } else {
        constexpr uint32_t K0 = 0x11111111u;
        const uint32_t b0 = w & K0, b1 = (w >> 1) & K0, b2 = (w >> 2) & K0;
        const uint32_t b01 = b0 & b1;
        n[1] += __builtin_popcount(b0);
        n[2] += __builtin_popcount(b1);
        n[3] += __builtin_popcount(b01);
        n[4] += __builtin_popcount(b2);
        n[5] += __builtin_popcount(b0 & b2);
        n[6] += __builtin_popcount(b1 & b2);
        n[7] += __builtin_popcount(b01 & b2);
    }
}

// unfolded [sign, level] fields -> codes: level bits complemented where the sign bit is 0
template <int BITS> __device__ __forceinline__ uint32_t fold_codes(uint32_t w) {
    if constexpr (BITS == 2) {
        return w ^ ((~w & 0xAAAAAAAAu) >> 1);
    } else if constexpr (BITS == 3) {
        const uint32_t np = ~w & 0x00924924u;  // sign bits of the eight fields
        return w ^ (np - (np >> 2));
    } else {
        const uint32_t np = ~w & 0x88888888u;
        return w ^ (np - (np >> 3));
    }
}

// TQ_TIMELINE (tq_measure.h; measurement builds only): per-wavefront timestamps (100 MHz wall clock) of the fused K+V
// store; reading the clock costs about a microsecond per stamp, so deltas between neighbouring stamps are upper bounds
#ifdef TQ_TIMELINE
__device__ unsigned long long g_tl[4096 * 16];
#define TQ_TL(slot)                                                                                              \
    do {                                                                                                         \
        const unsigned tlw = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);                                \
        if ((threadIdx.x & 63) == 0 && tlw < 4096) g_tl[tlw * 16 + (slot)] = wall_clock64();                      \
    } while (0)
#define TQ_TL_VAL(slot, v)                                                                                       \
    do {                                                                                                         \
        const unsigned tlw = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);                                \
        if ((threadIdx.x & 63) == 0 && tlw < 4096) g_tl[tlw * 16 + (slot)] = (v);                                 \
    } while (0)
#else
#define TQ_TL(slot) do {} while (0)
#define TQ_TL_VAL(slot, v) do {} while (0)
#endif

// The compiler pads the distance between a matrix instruction and the first vector instruction that reads its result
// with s_nop, but only along straight-line code: where a branch follows the matrix instructions, the path that takes the
// branch arrives at the reader with no padding (observed: a wavefront that skipped a conditional block read the first
// element of a 16x16x32 result too early).  Conditional blocks behind matrix instructions are therefore preceded by this
// pause, pinned in place: 16 wait states, the longest such distance on this part.
__device__ __forceinline__ void settle_matrix_results() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 7\n\ts_nop 7");
    __builtin_amdgcn_sched_barrier(0);
}

// ---- fp32 rows on the fp16 matrix cores ---------------------------------------------------------
// A row is scaled by a power of two to 512 <= ||x|| < 1024 (exact; every element then lies inside fp16's normal range or is
// negligible against the row) and every scaled element is split into two fp16 terms, hi = rn(x), mid = rn(x - hi): hi +
// mid equals x up to 2^-22 |x|.  The +-1 transform is applied to both terms into one accumulator, so the products are
// exact and the rotated value differs from the fp32 butterfly's only by roundings of the same size (the codes are held
// to the float64 oracle outside the 1e-6 boundary band, as for fp16 rows).  The norm comes from the fp32 values.
typedef float float2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float row_pow2_scale(float norm) {
    const uint32_t e = (__float_as_uint(norm) >> 23) & 0xFFu;  // biased exponent: norm = m 2^(e - 127), 1 <= m < 2
    const uint32_t se = 263u - e;                              // 2^(9 - (e - 127)), biased
    return (e == 0u || e == 255u) ? 1.0f : __uint_as_float((se > 254u ? 254u : se) << 23);
}
__device__ __forceinline__ float pow2_reciprocal(float p) { return __uint_as_float(0x7F000000u - __float_as_uint(p)); }  // p = 2^k, |k| < 127
// eight consecutive fp32 inputs (two 16-byte pieces) times sc -> their hi and mid terms as MFMA operands
__device__ __forceinline__ void split8(uint4 a, uint4 b, float sc, half8_t &hi, half8_t &mid) {
    const float v[8] = {__uint_as_float(a.x), __uint_as_float(a.y), __uint_as_float(a.z), __uint_as_float(a.w),
                        __uint_as_float(b.x), __uint_as_float(b.y), __uint_as_float(b.z), __uint_as_float(b.w)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float2_t xs = {v[2 * i] * sc, v[2 * i + 1] * sc};
        const half2_t h = __builtin_convertvector(xs, half2_t);
        const float2_t r = xs - __builtin_convertvector(h, float2_t);
        const half2_t m = __builtin_convertvector(r, half2_t);
        hi[2 * i] = h[0]; hi[2 * i + 1] = h[1];
        mid[2 * i] = m[0]; mid[2 * i + 1] = m[1];
    }
}
__device__ __forceinline__ float sumsq8(uint4 a, uint4 b, float acc) {
    acc = fmaf(__uint_as_float(a.x), __uint_as_float(a.x), acc); acc = fmaf(__uint_as_float(a.y), __uint_as_float(a.y), acc);
    acc = fmaf(__uint_as_float(a.z), __uint_as_float(a.z), acc); acc = fmaf(__uint_as_float(a.w), __uint_as_float(a.w), acc);
    acc = fmaf(__uint_as_float(b.x), __uint_as_float(b.x), acc); acc = fmaf(__uint_as_float(b.y), __uint_as_float(b.y), acc);
    acc = fmaf(__uint_as_float(b.z), __uint_as_float(b.z), acc); acc = fmaf(__uint_as_float(b.w), __uint_as_float(b.w), acc);
    return acc;
}

struct StoreKArgs {
    const uint4 *afrag;      // [8 fragments f0*4+ks][64 lanes] 8 halves (+-1)
    const uint32_t *s2flip;  // [4 lane quarters][4]: sign-field positions of the dims with s2 = +1, per output dword
                             // (3-bit: entry 3 is for the tail word): appended sign bit ^ this = "positive"
    const float *symthr;     // [0] middle boundary, [1..] positive boundaries
    const float *sqcoef;     // multilinear coefficients of c^2 over the level bits
    const uint2 *quant_lut;  // tq_handle::quant_lut (4-bit codes)
    int norm_correction;
    int64_t tokens;
    uint32_t blocks_per_seq, n_units;  // unit = 16 tokens
    FastDiv bps_div;                   // division by blocks_per_seq
    uint32_t out_blocks_per_seq;       // blocks between two sequences in `packed` (RAGGED kernels; a cache laid out for more tokens)
    // the same constants by value (REG kernels: nothing is fetched before the first input): bit k of s1neg = s1[k] < 0
    uint32_t s1neg[4], flipw[16];
    float thr[8], coef[8];
};

// ---- the +-1 operand fragments built in registers -------------------------------------------------
// bit e of row hm of the 8 x 8 Hadamard sign pattern: parity(hm & e)
__device__ __forceinline__ uint32_t h8_row(uint32_t hm) {
    const uint64_t rows = 0x963C5AF066CCAA00ull;  // rows 0..7, one byte each
    return (uint32_t)(rows >> (8u * hm)) & 0xFFu;
}
// eight sign bits (1 = negative) -> eight halves +-1.0
__device__ __forceinline__ half8_t signs_to_half8(uint32_t bits) {
    uint4 v;
    v.x = 0x3C003C00u | ((bits << 15) & 0x8000u) | ((bits << 30) & 0x80000000u);
    v.y = 0x3C003C00u | ((bits << 13) & 0x8000u) | ((bits << 28) & 0x80000000u);
    v.z = 0x3C003C00u | ((bits << 11) & 0x8000u) | ((bits << 26) & 0x80000000u);
    v.w = 0x3C003C00u | ((bits << 9) & 0x8000u) | ((bits << 24) & 0x80000000u);
    return __builtin_bit_cast(half8_t, v);
}
// K rows (tq_handle::rfrag16k): fragment f0*4+ks, lane l, element e = s1[k] H[m][k], m = 32(l%16/4) + 4 f0 + l%4,
// k = 32(l/16) + 8 ks + e.  m and k share the bits of e with 4 f0 + l%4 and the bits of l/16 with l%16/4.
__device__ __forceinline__ void build_k_fragments(half8_t (&af)[8], const uint32_t (&s1neg)[4], int lane) {
    const uint32_t r = lane & 15, kb = lane >> 4;
    const uint32_t hi = (uint32_t)__builtin_popcount((r >> 2) & kb) & 1u ? 0xFFu : 0u;
    const uint32_t w = kb == 0 ? s1neg[0] : kb == 1 ? s1neg[1] : kb == 2 ? s1neg[2] : s1neg[3];
#pragma unroll
    for (int f0 = 0; f0 < 2; ++f0) {
        const uint32_t pat = h8_row(4u * f0 + (r & 3u)) ^ hi;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) af[f0 * 4 + ks] = signs_to_half8((pat ^ (w >> (8 * ks))) & 0xFFu);
    }
}
// V rows (tq_handle::rfrag16v): fragment d0*4+ks, lane l, element e = s1[k] H[16 d0 + l%16][k], k = 32 ks + 8(l/16) + e
__device__ __forceinline__ void build_v_fragments(half8_t (&bf)[8], const uint32_t (&s1neg)[4], int lane) {
    const uint32_t n = lane & 15, kb = lane >> 4;
    const uint32_t base = h8_row(n & 7u) ^ ((n >> 3) & kb & 1u ? 0xFFu : 0u);
#pragma unroll
    for (int d0 = 0; d0 < 2; ++d0) {
        const uint32_t pat = base ^ (d0 && (kb >> 1) ? 0xFFu : 0u);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) bf[d0 * 4 + ks] = signs_to_half8((pat ^ (s1neg[ks] >> (8u * kb))) & 0xFFu);
    }
}

// copy a handle's quantiser table (4096 x 8 B) into LDS with NT threads; every load is issued before the
// first LDS write
template <int NT> __device__ __forceinline__ void load_quant_lut(uint2 *dst, const uint2 *src) {
    constexpr int N16 = 2048, PER = (N16 + NT - 1) / NT;  // 16-byte pieces
    const uint4 *s4 = reinterpret_cast<const uint4 *>(src);
    uint4 *d4 = reinterpret_cast<uint4 *>(dst);
    uint4 v[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = (int)threadIdx.x + i * NT;
        v[i] = s4[e < N16 ? e : N16 - 1];
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = (int)threadIdx.x + i * NT;
        if (e < N16) d4[e] = v[i];
    }
}

// the same table with every entry twice (entry i at 2i and 2i + 1): 64 KB, indexed by the value's top 13 bits
template <int NT> __device__ __forceinline__ void load_quant_lut_dup(uint2 *dst, const uint2 *src) {
    constexpr int N16 = 2048, PER = (N16 + NT - 1) / NT;  // 16-byte pieces of the source = pairs of entries
    const uint4 *s4 = reinterpret_cast<const uint4 *>(src);
    uint4 *d4 = reinterpret_cast<uint4 *>(dst);
    uint4 v[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = (int)threadIdx.x + i * NT;
        v[i] = s4[e < N16 ? e : N16 - 1];
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = (int)threadIdx.x + i * NT;
        if (e < N16) {
            d4[2 * e] = make_uint4(v[i].x, v[i].y, v[i].x, v[i].y);
            d4[2 * e + 1] = make_uint4(v[i].z, v[i].w, v[i].z, v[i].w);
        }
    }
}

// RAGGED: sequences whose token count is not a multiple of the block size (rows past the
// end are quantised as zeros, and the block index needs a division by blocks per sequence).
// Units lo, lo + step, .. below end are handed out through a ticket counter in LDS (zero on
// entry).  A counter shared by the wavefronts of a workgroup makes them a work queue (the
// hardware favours the oldest wavefronts of a SIMD, and with a fixed share per wavefront the
// youngest are left to finish alone at a fraction of the SIMD's issue rate); a counter per
// wavefront gives a fixed strided share.
__device__ __forceinline__ uint32_t take_ticket(uint32_t *counter, int lane) {
    uint32_t t = 0;
    if (lane == 0) t = atomicAdd(counter, 1u);
    return __builtin_amdgcn_readfirstlane(t);
}

constexpr uint32_t DRAW_TICKET = 0xFFFFFFFFu;
constexpr int K_UNITS_AHEAD = 1;
// first_ticket: the wavefront's first two tickets are first_ticket and first_ticket + 1 (the counter starts past
// them), or DRAW_TICKET to draw them.  `stage` makes the workgroup's LDS copy of the constant operands (frag,
// flips) readable; it runs after the first inputs have been requested.
// REG: the constants come from the argument block (fragments built in registers, frag and flips unused).
// TI = float: fp32 rows, split into two fp16 terms (see row_pow2_scale).
template <int BITS, bool RAGGED, bool DUP_LUT, bool REG, typename Stage, typename TI>
__device__ __forceinline__ void store_k_units(const TI *x, uint8_t *packed, const StoreKArgs &a, uint32_t lo, uint32_t step,
                                              uint32_t end, uint32_t *counter, const uint2 *qlut, const uint4 *frag,
                                              const uint32_t *flips, uint32_t first_ticket, Stage &&stage) {
    constexpr int NT = 1 << (BITS - 1);
    constexpr bool F32 = sizeof(TI) == 4;
    constexpr int NX = F32 ? 8 : 4;  // 16-byte pieces of a lane's 32 inputs
    const int tid = threadIdx.x, lane = tid & 63;
    const int n16 = lane & 15, kc = lane >> 4;
    float thr0[NT], coef[NT];
#pragma unroll
    for (int k = 0; k < NT; ++k) {
        thr0[k] = REG ? a.thr[k] : a.symthr[k];
        coef[k] = REG ? a.coef[k] : a.sqcoef[k];
    }

    const uint32_t bps = a.blocks_per_seq, last_unit = end ? end - 1 : 0;  // prefetches past the share re-read its last unit
    // This lane's 64 contiguous bytes of its token (inputs 32kc .. 32kc+31; slice ks = 16 B; twice that for fp32 rows).
    // The address is always valid: units past the end and rows past a sequence's last token
    // are clamped, and `valid` says whether the data is to be used.
    auto fetch = [&](uint32_t unit, uint4 (&xb)[NX], bool &valid) {
        // A prefetch past the share (its data is never used) reads the tensor's first bytes, every lane the same
        // ones: a clamped re-read of the last unit would go to memory again where rows are read with the
        // non-temporal hint, and a branch around the loads costs registers.
        const bool beyond = unit > last_unit;
        unit = unit < last_unit ? unit : last_unit;
#if TQ_KNOCKOUT & 32
        unit = lo + (((unit - lo) / step) & 7u) * step;  // the first eight units of the share over and over: no HBM reads
#endif
        const uint4 *p;
        if constexpr (RAGGED) {
            const uint32_t blk = unit >> 3, seq = a.bps_div.div(blk), bis = blk - seq * bps;
            int64_t tok = (int64_t)bis * TQ_ROWS_PER_BLOCK + (unit & 7) * 16 + n16;
            valid = tok < a.tokens;
            tok = valid ? tok : a.tokens - 1;
            p = reinterpret_cast<const uint4 *>(x + (beyond ? (int64_t)0 : ((int64_t)seq * a.tokens + tok) * 128 + 32 * kc));
        } else {
            valid = true;
            p = reinterpret_cast<const uint4 *>(x + (beyond ? (int64_t)0 : ((int64_t)unit * 16 + n16) * 128 + 32 * kc));
        }
#pragma unroll
        for (int ks = 0; ks < NX; ++ks) xb[ks] = load_input16(p + ks);
    };

    // an exact zero counts as positive only if the middle boundary is below zero
    const uint32_t zero_word = thr0[0] < 0.0f ? 0xFFFFFFFFu : 0u;
    const int diag_sel = n16 & 3;
    const bool diag_here = kc == (n16 >> 2);

    // units of input in flight per wavefront: one ahead measures faster than two (262 144 rows of 3-bit K alone
    // 16.9 against 18.2 us, the fused K+V launch 34.4 against 36.0 us)
    constexpr int DEPTH = K_UNITS_AHEAD;
    uint4 xq[DEPTH][NX];
    bool xvalid[DEPTH];
    uint32_t cur[DEPTH];
#pragma unroll
    for (int r = 0; r < DEPTH; ++r) {
        cur[r] = lo + step * (first_ticket == DRAW_TICKET ? take_ticket(counter, lane) : first_ticket + r);
        fetch(cur[r], xq[r], xvalid[r]);
    }
    stage();
    half8_t af[8];
    uint32_t flip[4];
    if constexpr (REG) {
        build_k_fragments(af, a.s1neg, lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) flip[j] = kc == 0 ? a.flipw[j] : kc == 1 ? a.flipw[4 + j] : kc == 2 ? a.flipw[8 + j] : a.flipw[12 + j];
    } else {
#pragma unroll
        for (int f = 0; f < 8; ++f) af[f] = __builtin_bit_cast(half8_t, frag[f * 64 + lane]);
#pragma unroll
        for (int j = 0; j < 4; ++j) flip[j] = flips[kc * 4 + j];
    }

    [[maybe_unused]] unsigned tl_n = 0;
    // The codes and the norm of a unit leave one unit later, right after the next unit's matrix instructions have been
    // issued: loads and stores share one counter of outstanding operations, so a wait for input also waits for all
    // but a few of the stores issued after that input was requested - stores issued at the end of a unit were waited
    // for, with their full latency, at the top of the next one.
    static_assert(DEPTH == 1, "the deferred stores assume one unit in flight");
    uint32_t pend_g[BITS];
    float pend_gn = 0.0f;
    uint32_t pend_unit = 0;
    bool pending = false;
#pragma unroll
    for (int j = 0; j < BITS; ++j) pend_g[j] = 0;
    auto flush = [&] {
        const uint32_t blk = pend_unit >> 3;
        const int row = (int)(pend_unit & 7) * 16 + n16;
        const uint32_t oseq = RAGGED ? a.bps_div.div(blk) : 0u;
        const uint32_t oblk = RAGGED ? oseq * a.out_blocks_per_seq + (blk - oseq * bps) : blk;
        uint8_t *block = packed + (int64_t)oblk * block_bytes(BITS);
#if TQ_KNOCKOUT & 16
        if (pend_g[0] == 0x12345678u && pend_g[BITS - 1] == 0x9abcdef0u)   // keeps the codes alive; not taken for real data
#endif
#pragma unroll
        for (int j = 0; j < BITS; ++j)
            stream_store<STREAM_STORE_CODES>(reinterpret_cast<uint32_t *>(block + j * 2048 + row * 16 + kc * 4), pend_g[j]);
        if (kc == 0) reinterpret_cast<__half *>(block + block_code_bytes(BITS))[row] = __float2half_rn(pend_gn);
    };
#pragma unroll 1
    for (bool more = true; more;) {
#pragma unroll
        for (int r = 0; r < DEPTH; ++r) {
            const uint32_t unit = cur[r];
            if (unit >= end) {  // tickets only grow: nothing is left for this wavefront
                more = false;
                break;
            }
            if (tl_n == 1) TQ_TL(4);
            ++tl_n;
            const uint32_t next = lo + step * take_ticket(counter, lane);
            uint4 (&xb)[NX] = xq[r];
            if constexpr (RAGGED) {
                if (!xvalid[r]) {
#pragma unroll
                    for (int ks = 0; ks < NX; ++ks) xb[ks] = make_uint4(0, 0, 0, 0);
                }
            }

            float4_t q[2][4];
            float ss, rowscale = 1.0f;  // rowscale: the power of two an fp32 row was multiplied by
            if constexpr (F32) {
                // norm first (the split needs the row's scale), from the fp32 values
                float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
                for (int ks = 0; ks < 4; ks += 2) {
                    s0 = sumsq8(xb[2 * ks], xb[2 * ks + 1], s0);
                    s1 = sumsq8(xb[2 * ks + 2], xb[2 * ks + 3], s1);
                }
                ss = s0 + s1;
                ss += xor_lane<16>(ss);
                ss += xor_lane<32>(ss);
                rowscale = row_pow2_scale(__builtin_amdgcn_sqrtf(ss));
                half8_t hi[4], mid[4];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) split8(xb[2 * ks], xb[2 * ks + 1], rowscale, hi[ks], mid[ks]);
#pragma unroll
                for (int f0 = 0; f0 < 2; ++f0)
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) {
                        q[f0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[f0 * 4 + ks], mid[ks], float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        q[f0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[f0 * 4 + ks], hi[ks], q[f0][ks], 0, 0, 0);
                    }
                cur[r] = next;
                settle_matrix_results();
                if (pending) flush();  // the previous unit's codes, behind this unit's wait for its input
                fetch(next, xb, xvalid[r]);
            } else {
#pragma unroll
                for (int f0 = 0; f0 < 2; ++f0)
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks)
                        q[f0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[f0 * 4 + ks], __builtin_bit_cast(half8_t, xb[ks]),
                                                                           float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                // ||x||^2 on the matrix cores as well: the diagonal of X X^T (the same registers serve as
                // both operands); token n16's entry is element n16 % 4 of lane quarter n16 / 4
                float4_t gram = float4_t{0.f, 0.f, 0.f, 0.f};
#if TQ_KNOCKOUT & 8
                gram[0] = gram[1] = gram[2] = gram[3] = 1.0f;
#else
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
                    gram = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xb[ks]), __builtin_bit_cast(half8_t, xb[ks]),
                                                                  gram, 0, 0, 0);
#endif
                ss = diag_sel == 0 ? gram[0] : diag_sel == 1 ? gram[1] : diag_sel == 2 ? gram[2] : gram[3];
                ss = diag_here ? ss : 0.0f;
                cur[r] = next;
                settle_matrix_results();
                if (pending) flush();  // the previous unit's codes, behind this unit's wait for its input
                fetch(next, xb, xvalid[r]);
                ss += xor_lane<16>(ss);
                ss += xor_lane<32>(ss);
            }
            const float norm = __builtin_amdgcn_sqrtf(ss);  // 1 ulp: scales boundaries (1e-7 relative) and the stored fp16 norm
            const float scale = norm > 0.0f ? norm * rowscale * 11.313708498984761f : 1.0f;  // y' = sqrt(128) ||x|| y
            float thr[NT];
#pragma unroll
            for (int k = 0; k < NT; ++k) thr[k] = thr0[k] * scale;
            // table path (4 bits): values are normalised instead of the boundaries being scaled
            const float inv = norm > 0.0f ? __builtin_amdgcn_rsqf(ss) * (0.08838834764831845f * pow2_reciprocal(rowscale)) : 1.0f;

            // butterfly over the input slices: fragment 2*fh + f0 holds dims 32kc + 8fh + 4f0 + i
            float4_t y[8];
#pragma unroll
            for (int f0 = 0; f0 < 2; ++f0) {
#if TQ_KNOCKOUT & 2
                const float ko_s = BITS == 4 ? inv : 1.0f;  // the table path expects normalised values
                y[0 + f0] = q[f0][0] * ko_s; y[2 + f0] = q[f0][1] * ko_s; y[4 + f0] = q[f0][2] * ko_s; y[6 + f0] = q[f0][3] * ko_s;
#else
                const float4_t s01 = q[f0][0] + q[f0][1], d01 = q[f0][0] - q[f0][1];
                const float4_t s23 = q[f0][2] + q[f0][3], d23 = q[f0][2] - q[f0][3];
                if constexpr (BITS == 4) {  // the table is indexed by the normalised value
                    const float4_t iv = {inv, inv, inv, inv};
                    const float4_t s23i = s23 * iv, d23i = d23 * iv;
                    y[0 + f0] = fma4(s01, iv, s23i);
                    y[2 + f0] = fma4(d01, iv, d23i);
                    y[4 + f0] = fma4(s01, iv, -s23i);
                    y[6 + f0] = fma4(d01, iv, -d23i);
                } else {
                    y[0 + f0] = s01 + s23;
                    y[2 + f0] = d01 + d23;
                    y[4 + f0] = s01 - s23;
                    y[6 + f0] = d01 - d23;
                }
#endif
            }
            // value v = 0..31 of this lane (dim 32*kc + v) up to the sign s2
            auto val = [&](int v) -> float { return y[v >> 2][v & 3]; };
            const bool nonzero = norm > 0.0f;  // all-zero rows get the code of an exact 0 everywhere
            uint32_t g[BITS];
            uint32_t n[NT];
#pragma unroll
            for (int k = 0; k < NT; ++k) n[k] = 0;
            if constexpr (BITS == 3) {
                // four words of eight values: dwords 0..2 and the tail, whose byte j rides on top of dword j
                uint32_t w4[4];
#pragma unroll
                for (int j = 3; j >= 0; --j) {
                    const int v = 8 * j;
#if TQ_KNOCKOUT & 1
                    uint32_t w = ko_append4(thr[1] > 0.f ? 0u : 1u, val(v + 7), val(v + 6), val(v + 5), val(v + 4));
                    w = ko_append4(w, val(v + 3), val(v + 2), val(v + 1), val(v));
#else
                    uint32_t w = append4_b3(0u, val(v + 7), val(v + 6), val(v + 5), val(v + 4), thr);
                    w = append4_b3(w, val(v + 3), val(v + 2), val(v + 1), val(v), thr);
#endif
#if !(TQ_KNOCKOUT & 4)
                    count_levels<3>(w, n);
#endif
                    w4[j] = fold_codes<3>(nonzero ? w ^ flip[j] : (zero_word & 0x00924924u));
                }
                g[0] = __builtin_amdgcn_perm(w4[3], w4[0], 0x04020100u);
                g[1] = __builtin_amdgcn_perm(w4[3], w4[1], 0x05020100u);
                g[2] = __builtin_amdgcn_perm(w4[3], w4[2], 0x06020100u);
            } else if constexpr (BITS == 4) {
                uint32_t unfolded[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // eight values into one unfolded dword through the table, highest value first
                    const int v = 8 * j;
                    float yn[8];
                    uint2 e[8];
#pragma unroll
                    for (int m = 0; m < 8; ++m) {
                        yn[m] = val(v + m);  // normalised in the butterfly
#if TQ_KNOCKOUT & 1
                        if (m == 0)
#endif
                        e[m] = *reinterpret_cast<const uint2 *>(reinterpret_cast<const char *>(qlut) + quant_lut_offset<DUP_LUT>(yn[m]));
                    }
#if TQ_KNOCKOUT & 1
                    uint32_t w = ko_append4(e[0].x & 1u, yn[7], yn[6], yn[5], yn[4]);
                    w = ko_append4(w, yn[3], yn[2], yn[1], yn[0]);
#else
                    uint32_t w = append4_lut(0u, yn[7], yn[6], yn[5], yn[4], e[7], e[6], e[5], e[4]);
                    w = append4_lut(w, yn[3], yn[2], yn[1], yn[0], e[3], e[2], e[1], e[0]);
#endif
                    unfolded[j] = w;
                    g[j] = fold_codes<4>(nonzero ? w ^ flip[j] : (zero_word & 0x88888888u));
                }
#if !(TQ_KNOCKOUT & 4)
                count_levels4_merged(unfolded, n);
#endif
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    uint32_t w = 0;
#pragma unroll
                    for (int v = 16 * j + 12; v >= 16 * j; v -= 4) w = append4_b2(w, val(v + 3), val(v + 2), val(v + 1), val(v), thr);
                    count_levels<2>(w, n);
                    g[j] = fold_codes<2>(nonzero ? w ^ flip[j] : (zero_word & 0xAAAAAAAAu));
                }
            }
            float gn = norm;
            if (a.norm_correction) {
                float cs = 32.0f * coef[0];
#pragma unroll
                for (int k = 1; k < NT; ++k) cs = fmaf(coef[k], (float)n[k], cs);
                cs += xor_lane<16>(cs);
                cs += xor_lane<32>(cs);
                gn = norm * __builtin_amdgcn_rsqf(cs);  // cs >= 128 min c^2 > 0
            }
#pragma unroll
            for (int j = 0; j < BITS; ++j) pend_g[j] = g[j];
            pend_gn = gn;
            pend_unit = unit;
            pending = true;
        }
    }
    if (pending) flush();
    TQ_TL(5);
    TQ_TL_VAL(7, (unsigned long long)tl_n);
}

// ---- K2, fp16 input, V rows ---------------------------------------------------------------
// V rows are dim-major, so here the tokens are the MFMA rows (A = X, B = the +-1 factor): lane
// quarter q, column n = lane mod 16 holds, per 16-token sub-tile u of a 64-token tile, tokens
// 16q + 4u + i (i = 0..3) of dim 16*dd + 64*hf + n for the four rows dd and both dim halves.
// A group of appends takes one token (u, i) and one dim half and adds its code to the current
// dword of each of the four rows; sub-tiles run u = 3..0 so that pairs arrive in descending
// order.  2- and 3-bit codes compare against the token's scaled boundaries; 4-bit codes normalise the values
// by the token's norm first (the table is indexed by the normalised value).
//   m = 64hf + 32d1 + 16d0 + n,  k = 32ks + 8kb + e,  dd = 2 d1 + d0
//   y'[m] = s2[m] * sum_ks (-1)^popcount((d1 + 2hf) & ks) * Q[d0][ks],  Q[d0][ks] = X[ks] B[d0][ks],
//   B[d0][ks][8kb + e][n] = s1[k] * H[16 d0 + n][k]

// one 3-bit code per row: w_d = 8 w_d + [sign, level]; the per-token level counts come from field-wise sums
// over the rows afterwards
__device__ __forceinline__ void append_rows_b3(uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &w3, float y0, float y1,
                                                     float y2, float y3, const float (&t)[4]) {
    float u0, u1, u2, u3;
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t2]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t2]\n\t"
        "v_cndmask_b32_e64 %[u0], %[t1], %[t3], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[u1], %[t1], %[t3], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[u2], %[t1], %[t3], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[u3], %[t1], %[t3], s[66:67]\n\t"
        "v_cmp_gt_f32_e64 s[68:69], |%[y0]|, %[u0]\n\t"
        "v_cmp_gt_f32_e64 s[70:71], |%[y1]|, %[u1]\n\t"
        "v_cmp_gt_f32_e64 s[72:73], |%[y2]|, %[u2]\n\t"
        "v_cmp_gt_f32_e64 s[74:75], |%[y3]|, %[u3]\n\t"
        "v_alignbit_b32 %[w0], %[w0], %[y0], 31\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[w0], s[60:61]\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[w0], s[68:69]\n\t"
        "v_alignbit_b32 %[w1], %[w1], %[y1], 31\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[w1], s[62:63]\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[w1], s[70:71]\n\t"
        "v_alignbit_b32 %[w2], %[w2], %[y2], 31\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[w2], s[64:65]\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[w2], s[72:73]\n\t"
        "v_alignbit_b32 %[w3], %[w3], %[y3], 31\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[w3], s[66:67]\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[w3], s[74:75]\n\t"
        : [w0] "+v"(w0), [w1] "+v"(w1), [w2] "+v"(w2), [w3] "+v"(w3), [u0] "=&v"(u0), [u1] "=&v"(u1), [u2] "=&v"(u2), [u3] "=&v"(u3)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t1] "v"(t[1]), [t2] "v"(t[2]), [t3] "v"(t[3])
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "vcc");
}

__device__ __forceinline__ void append_rows_b2(uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &w3, uint32_t &n1, float y0,
                                               float y1, float y2, float y3, const float (&t)[2]) {
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t1]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t1]\n\t"
        "v_alignbit_b32 %[w0], %[w0], %[y0], 31\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[w0], s[60:61]\n\t"
        "v_alignbit_b32 %[w1], %[w1], %[y1], 31\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[w1], s[62:63]\n\t"
        "v_alignbit_b32 %[w2], %[w2], %[y2], 31\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[w2], s[64:65]\n\t"
        "v_alignbit_b32 %[w3], %[w3], %[y3], 31\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[w3], s[66:67]\n\t"
        "v_addc_co_u32_e64 %[n1], vcc, %[n1], 0, s[60:61]\n\t"
        "v_addc_co_u32_e64 %[n1], vcc, %[n1], 0, s[62:63]\n\t"
        "v_addc_co_u32_e64 %[n1], vcc, %[n1], 0, s[64:65]\n\t"
        "v_addc_co_u32_e64 %[n1], vcc, %[n1], 0, s[66:67]\n\t"
        : [w0] "+v"(w0), [w1] "+v"(w1), [w2] "+v"(w2), [w3] "+v"(w3), [n1] "+v"(n1)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t1] "v"(t[1])
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "vcc");
}

__device__ __forceinline__ void append_rows_b4(uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &w3, float y0, float y1, float y2,
                                               float y3, const float (&t)[8]) {
    float a0, a1, a2, a3, b0, b1, b2, b3;
    asm("v_cmp_gt_f32_e64 s[60:61], |%[y0]|, %[t4]\n\t"
        "v_cmp_gt_f32_e64 s[62:63], |%[y1]|, %[t4]\n\t"
        "v_cmp_gt_f32_e64 s[64:65], |%[y2]|, %[t4]\n\t"
        "v_cmp_gt_f32_e64 s[66:67], |%[y3]|, %[t4]\n\t"
        "v_cndmask_b32_e64 %[a0], %[t2], %[t6], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[a1], %[t2], %[t6], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[a2], %[t2], %[t6], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[a3], %[t2], %[t6], s[66:67]\n\t"
        "v_cmp_gt_f32_e64 s[68:69], |%[y0]|, %[a0]\n\t"
        "v_cmp_gt_f32_e64 s[70:71], |%[y1]|, %[a1]\n\t"
        "v_cmp_gt_f32_e64 s[72:73], |%[y2]|, %[a2]\n\t"
        "v_cmp_gt_f32_e64 s[74:75], |%[y3]|, %[a3]\n\t"
        "v_cndmask_b32_e64 %[b0], %[t1], %[t5], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[b1], %[t1], %[t5], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[b2], %[t1], %[t5], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[b3], %[t1], %[t5], s[66:67]\n\t"
        "v_cndmask_b32_e64 %[a0], %[t3], %[t7], s[60:61]\n\t"
        "v_cndmask_b32_e64 %[a1], %[t3], %[t7], s[62:63]\n\t"
        "v_cndmask_b32_e64 %[a2], %[t3], %[t7], s[64:65]\n\t"
        "v_cndmask_b32_e64 %[a3], %[t3], %[t7], s[66:67]\n\t"
        "v_cndmask_b32_e64 %[b0], %[b0], %[a0], s[68:69]\n\t"
        "v_cndmask_b32_e64 %[b1], %[b1], %[a1], s[70:71]\n\t"
        "v_cndmask_b32_e64 %[b2], %[b2], %[a2], s[72:73]\n\t"
        "v_cndmask_b32_e64 %[b3], %[b3], %[a3], s[74:75]\n\t"
        "v_cmp_gt_f32_e64 s[76:77], |%[y0]|, %[b0]\n\t"
        "v_cmp_gt_f32_e64 s[78:79], |%[y1]|, %[b1]\n\t"
        "v_cmp_gt_f32_e64 s[80:81], |%[y2]|, %[b2]\n\t"
        "v_cmp_gt_f32_e64 s[82:83], |%[y3]|, %[b3]\n\t"
        "v_alignbit_b32 %[w0], %[w0], %[y0], 31\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[w0], s[60:61]\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[w0], s[68:69]\n\t"
        "v_addc_co_u32_e64 %[w0], vcc, %[w0], %[w0], s[76:77]\n\t"
        "v_alignbit_b32 %[w1], %[w1], %[y1], 31\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[w1], s[62:63]\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[w1], s[70:71]\n\t"
        "v_addc_co_u32_e64 %[w1], vcc, %[w1], %[w1], s[78:79]\n\t"
        "v_alignbit_b32 %[w2], %[w2], %[y2], 31\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[w2], s[64:65]\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[w2], s[72:73]\n\t"
        "v_addc_co_u32_e64 %[w2], vcc, %[w2], %[w2], s[80:81]\n\t"
        "v_alignbit_b32 %[w3], %[w3], %[y3], 31\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[w3], s[66:67]\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[w3], s[74:75]\n\t"
        "v_addc_co_u32_e64 %[w3], vcc, %[w3], %[w3], s[82:83]\n\t"
        : [w0] "+v"(w0), [w1] "+v"(w1), [w2] "+v"(w2), [w3] "+v"(w3), [a0] "=&v"(a0), [a1] "=&v"(a1), [a2] "=&v"(a2), [a3] "=&v"(a3), [b0] "=&v"(b0), [b1] "=&v"(b1),
          [b2] "=&v"(b2), [b3] "=&v"(b3)
        : [y0] "v"(y0), [y1] "v"(y1), [y2] "v"(y2), [y3] "v"(y3), [t1] "v"(t[1]), [t2] "v"(t[2]), [t3] "v"(t[3]), [t4] "v"(t[4]), [t5] "v"(t[5]), [t6] "v"(t[6]), [t7] "v"(t[7])
        : "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "vcc");
}

// pair k = 0..15 of a 16-pair group -> dword inside the group (3-bit: 3 = the tail word) and shift
__host__ __device__ constexpr int grp_word(int bits, int k) { return k / pairs_per_dword(bits); }
__host__ __device__ constexpr int grp_shift(int bits, int k) { return 2 * bits * (k % pairs_per_dword(bits)); }
// V rows: sign-field bits of group dword j that belong to dim half hf (pairs with (k / 2) % 2 == hf) and to the
// tokens of the 16-token group named by tokmask (pair k = tokens 4(k/4) + 2(k%2), +1 as low and high code)
__host__ __device__ constexpr uint32_t v_sign_mask(int bits, int j, int hf, uint32_t tokmask) {
    uint32_t m = 0;
    for (int k = 0; k < 16; ++k) {
        if (((k >> 1) & 1) != hf || grp_word(bits, k) != j) continue;
        for (int h = 0; h < 2; ++h)
            if ((tokmask >> (4 * (k >> 2) + 2 * (k & 1) + h)) & 1) m |= 1u << (grp_shift(bits, k) + bits * h + bits - 1);
    }
    return m;
}

struct StoreVArgs {
    const uint4 *bfrag;   // [8 fragments d0*4+ks][64 lanes] 8 halves (+-1)
    const float *s2;      // [128] output signs
    const float *symthr;  // [0] middle boundary, [1..] positive boundaries
    const float *sqcoef;  // multilinear coefficients of c^2 over the level bits
    const uint2 *quant_lut;  // tq_handle::quant_lut (4-bit codes)
    int norm_correction;
    int share_k_lut;      // fused K+V store: V's 4-bit table equals K's, which is already in LDS
    int64_t tokens;
    uint32_t blocks_per_seq, n_units;  // unit = 64-token tile (half a block)
    FastDiv bps_div;                   // division by blocks_per_seq
    uint32_t out_blocks_per_seq;       // blocks between two sequences in `packed` (RAGGED kernels; a cache laid out for more tokens)
    uint32_t s1neg[4], s2neg[4];       // the constants by value (REG kernels): bit k = s1[k] < 0, s2[k] < 0
    float thr[8], coef[8];
};

// Tiles lo, lo + step, .. below end through a ticket counter in LDS, as for the K units.  The first
// ticket is the caller's (the counter starts past the tickets given out this way), so the first tile's
// input is requested before anything is waited for; `stage` then makes the workgroup's copy of the
// constant operands (frag, s2: LDS) readable.
// STREAM_IN: the input is read with the non-temporal hint (every 128-byte line is touched by two instructions of one
// wavefront, back to back).  It gains 2 us in the fused K+V launch and loses 1 us in the V-only kernel (measured).
// REG: the constants come from the argument block (fragments built in registers, frag and s2 unused), the first tile is
// requested before anything else and `stage` runs while it is in flight.
template <int BITS, bool RAGGED, bool STREAM_IN, bool DUP_LUT, bool REG, typename Stage, typename TI>
__device__ __forceinline__ void store_v_units(const TI *x, uint8_t *packed, const StoreVArgs &a, uint32_t lo, uint32_t step,
                                              uint32_t end, uint32_t *counter, const uint2 *qlut, const uint4 *frag,
                                              const float *s2, uint32_t first_ticket, Stage &&stage) {
    constexpr int NT = 1 << (BITS - 1);
    constexpr int NW = BITS == 3 ? 4 : BITS;  // dwords of a row group while it is built (3-bit: + the tail word)
    constexpr bool F32 = sizeof(TI) == 4;     // fp32 rows: two fp16 terms per value (see row_pow2_scale)
    constexpr int NX = F32 ? 8 : 4;           // 16-byte pieces of a lane's 32 inputs of one sub-tile
    const int tid = threadIdx.x, lane = tid & 63;
    const int n16 = lane & 15, kq = lane >> 4;
    float thr0[NT], coef[NT];
#pragma unroll
    for (int k = 0; k < NT; ++k) {
        thr0[k] = REG ? a.thr[k] : a.symthr[k];
        coef[k] = REG ? a.coef[k] : a.sqcoef[k];
    }
    // an exact zero counts as positive only if the middle boundary is below zero
    const uint32_t zero_word = thr0[0] < 0.0f ? 0xFFFFFFFFu : 0u;

    const uint32_t bps = a.blocks_per_seq, last_unit = end ? end - 1 : 0;  // prefetches past the share re-read its last unit
    // A operand of sub-tile u: row r = lane%16 is token 16(r/4) + 4u + r%4 of the tile, this lane
    // supplies inputs 32ks + 8kq .. +7.  The address is always valid (clamped); `valid` says
    // whether the row exists.
    auto row_ptr = [&](uint32_t unit, int u, bool &valid) -> const uint4 * {
        const bool beyond = unit > last_unit;  // past the share: every lane reads the tensor's first bytes (see the K units)
        unit = unit < last_unit ? unit : last_unit;
#if TQ_KNOCKOUT & 32
        unit = lo + (((unit - lo) / step) & 1u) * step;  // the first two tiles of the share over and over: no HBM reads
#endif
        const uint32_t blk = unit >> 1;
        const int tb = (int)(unit & 1) * 64 + 16 * (n16 >> 2) + 4 * u + (n16 & 3);
        if constexpr (RAGGED) {
            const uint32_t seq = a.bps_div.div(blk), bis = blk - seq * bps;
            int64_t tok = (int64_t)bis * TQ_ROWS_PER_BLOCK + tb;
            valid = tok < a.tokens;
            tok = valid ? tok : a.tokens - 1;
            return reinterpret_cast<const uint4 *>(x + (beyond ? (int64_t)0 : ((int64_t)seq * a.tokens + tok) * 128 + 8 * kq));
        } else {
            valid = true;
            return reinterpret_cast<const uint4 *>(x + (beyond ? (int64_t)0 : ((int64_t)blk * TQ_ROWS_PER_BLOCK + tb) * 128 + 8 * kq));
        }
    };
    auto fetch = [&](uint32_t unit, int u, uint4 (&xb)[NX], bool &valid) {
        const uint4 *p = row_ptr(unit, u, valid);
        if constexpr (F32) {  // inputs 32 ks + 8 kq .. + 7: 32 bytes at a 128-byte stride
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                xb[2 * ks] = STREAM_IN ? stream_load<STREAM_STORE_V_IN>(p + 8 * ks) : p[8 * ks];
                xb[2 * ks + 1] = STREAM_IN ? stream_load<STREAM_STORE_V_IN>(p + 8 * ks + 1) : p[8 * ks + 1];
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) xb[ks] = STREAM_IN ? stream_load<STREAM_STORE_V_IN>(p + 4 * ks) : p[4 * ks];
        }
    };
    // sub-tiles of input in flight: two of fp16 rows, one of fp32 rows (which take twice the registers; two of them
    // leave room for two wavefronts per SIMD only: 41 against 30 us for 262 144 rows)
    constexpr int VD = F32 ? 1 : 2;
    uint4 xq[VD][NX];
    bool xvalid[VD];
    uint32_t unit = lo + step * first_ticket;
    // The first tile is requested behind the barrier that makes the constants readable: when the wavefronts of the
    // chip ask for their first input at once, ahead of the constants, the burst takes several microseconds to serve and
    // the constants queue behind it (measured: no wavefront asking early 32.3 us, one per SIMD 32.9 us, two 33.1 us,
    // all 33.0 us for the 3-bit K+V launch; 4-bit alike within its run-to-run spread).
    half8_t bf[8];
    bool s2pos[4][2];
    if constexpr (REG) {
        // nothing has to come from memory before the first input: the constants are kernel arguments.  Only the
        // first sub-tile is requested ahead of the barrier: with both in flight at once the chip-wide burst is twice
        // as long and every wavefront's first data arrives later (measured: 33.2 against 32.2 us for the 3-bit launch)
        fetch(unit, 3, xq[0], xvalid[0]);
        TQ_TL(8);
        build_v_fragments(bf, a.s1neg, lane);
#pragma unroll
        for (int dd = 0; dd < 4; ++dd)
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) s2pos[dd][hf] = ((a.s2neg[2 * hf + (dd >> 1)] >> (16 * (dd & 1) + n16)) & 1u) == 0u;
        TQ_TL(9);
        stage();
        TQ_TL(10);
        if constexpr (VD == 2) fetch(unit, 2, xq[1], xvalid[1]);
    } else {
        stage();
        fetch(unit, 3, xq[0], xvalid[0]);
        if constexpr (VD == 2) fetch(unit, 2, xq[1], xvalid[1]);
#pragma unroll
        for (int f = 0; f < 8; ++f) bf[f] = __builtin_bit_cast(half8_t, frag[f * 64 + lane]);
#pragma unroll
        for (int dd = 0; dd < 4; ++dd)
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) s2pos[dd][hf] = s2[64 * hf + 16 * dd + n16] > 0.0f;
    }

    [[maybe_unused]] unsigned tl_n = 0;
    TQ_TL(1);
    // DEFER: codes and norms leave one sub-tile after they are complete, right behind the next sub-tile's matrix
    // instructions (loads and stores share one counter of outstanding operations, so a wait for input also waits for all
    // but a few of the stores issued after that input was requested; stores issued at the end of a sub-tile were waited
    // for, with their full latency, at the top of the next one).  A sub-tile completes one dword of each of the lane's
    // four rows (2-bit codes: every second sub-tile), which is finished - signs, zero tokens, fold - and parked in `park`;
    // the last one of a tile crosses into the next tile (pend_unit) or is flushed after the loop.
    constexpr bool DEFER = REG;
    uint32_t park[4] = {0, 0, 0, 0};
    float park_norm = 0.0f;
    uint32_t pend_unit = 0;
    bool pending = false;
    auto block_of = [&](uint32_t un) -> uint8_t * {
        const uint32_t oseq = RAGGED ? a.bps_div.div(un >> 1) : 0u;
        const uint32_t oblk = RAGGED ? oseq * a.out_blocks_per_seq + ((un >> 1) - oseq * bps) : un >> 1;
        return packed + (int64_t)oblk * block_bytes(BITS);
    };
    // the parked dword j of the four rows and the parked norms of sub-tile u, tile `un`
    auto flush_park = [&](uint32_t un, int j, int u, bool with_codes) {
        uint8_t *blockp = block_of(un);
        const int hlf = (int)(un & 1);
        if (with_codes) {
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const int row = hlf * 64 + 16 * dd + n16;
#if TQ_KNOCKOUT & 16
                if (park[dd] == 0x12345678u)   // keeps the codes alive; practically never taken
#endif
                stream_store<STREAM_STORE_CODES>(reinterpret_cast<uint32_t *>(blockp + j * 2048 + row * 16 + kq * 4), park[dd]);
            }
        }
        __half *no = reinterpret_cast<__half *>(blockp + block_code_bytes(BITS)) + hlf * 64 + 16 * kq;
        if (n16 < 4) no[4 * u + n16] = __float2half_rn(park_norm);
    };
    // does sub-tile u complete its dword?  (2-bit codes: two sub-tiles share a dword)
    auto completes = [](int u) { return u == 0 || grp_word(BITS, 4 * (u - 1)) != grp_word(BITS, 4 * u); };
    // the dword that sub-tile u's completed word makes storable (-1: none; 3-bit: the tail word only rides on the others)
    auto storable = [&](int u) { const int j = grp_word(BITS, 4 * u); return !completes(u) || (BITS == 3 && j == 3) ? -1 : j; };
#pragma unroll 1
    for (; unit < end;) {
        if (tl_n == 1) TQ_TL(2);
        ++tl_n;
        const uint32_t next = lo + step * take_ticket(counter, lane);
        const uint32_t oseq = RAGGED ? a.bps_div.div(unit >> 1) : 0u;
        const uint32_t oblk = RAGGED ? oseq * a.out_blocks_per_seq + ((unit >> 1) - oseq * bps) : unit >> 1;
        uint8_t *block = packed + (int64_t)oblk * block_bytes(BITS);
        const int half = (int)(unit & 1);
        __half *norms_out = reinterpret_cast<__half *>(block + block_code_bytes(BITS)) + half * 64 + 16 * kq;
        uint32_t w[4][NW];
#pragma unroll
        for (int dd = 0; dd < 4; ++dd)
#pragma unroll
            for (int j = 0; j < NW; ++j) w[dd][j] = 0;
        uint32_t zbits = 0;  // bit 4u+i: token 16kq + 4u + i is all zero

#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int u = 3 - q;
            const int xsel = VD == 2 ? (q & 1) : 0;
            uint4 (&xb)[NX] = xq[xsel];
            if constexpr (RAGGED) {
                if (!xvalid[xsel]) {
#pragma unroll
                    for (int ks = 0; ks < NX; ++ks) xb[ks] = make_uint4(0, 0, 0, 0);
                }
            }
            float4_t qq[2][4];
            // ||x||^2 of the four tokens whose values this lane ends up with, as gram[i] of the lane that holds it
            // (row 4kq + i, column n16: the diagonal of X X^T)
            float4_t gram = float4_t{0.f, 0.f, 0.f, 0.f};
            if constexpr (F32) {
                // this lane's 32 inputs belong to token row n16: its squared norm over the four lanes that share it, from
                // the fp32 values; then the two-term split at the row's scale
                float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
                for (int ks = 0; ks < 4; ks += 2) {
                    s0 = sumsq8(xb[2 * ks], xb[2 * ks + 1], s0);
                    s1 = sumsq8(xb[2 * ks + 2], xb[2 * ks + 3], s1);
                }
                float ssr = s0 + s1;
                ssr += xor_lane<16>(ssr);
                ssr += xor_lane<32>(ssr);
                gram[0] = gram[1] = gram[2] = gram[3] = ssr;  // picked where n16 == 4kq + i below
                const float rs = row_pow2_scale(__builtin_amdgcn_sqrtf(ssr));
                half8_t hi[4], mid[4];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) split8(xb[2 * ks], xb[2 * ks + 1], rs, hi[ks], mid[ks]);
#pragma unroll
                for (int d0 = 0; d0 < 2; ++d0)
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) {
                        qq[d0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mid[ks], bf[d0 * 4 + ks], float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        qq[d0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi[ks], bf[d0 * 4 + ks], qq[d0][ks], 0, 0, 0);
                    }
            } else {
#pragma unroll
                for (int d0 = 0; d0 < 2; ++d0)
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks)
                        qq[d0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xb[ks]), bf[d0 * 4 + ks],
                                                                            float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#if TQ_KNOCKOUT & 8
                gram[0] = gram[1] = gram[2] = gram[3] = 1.0f;
#else
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
                    gram = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xb[ks]), __builtin_bit_cast(half8_t, xb[ks]),
                                                                  gram, 0, 0, 0);
#endif
            }
            // (before this sub-tile's requests: the wait for a sub-tile's input lets only a few younger operations stay
            // outstanding, and these stores are then a whole sub-tile old when the next wait comes)
            if constexpr (DEFER) {
                if (q == 0) {
                    settle_matrix_results();
                    if (pending) flush_park(pend_unit, 0, 0, true);  // the previous tile's last dword and norms
                } else {
                    flush_park(unit, storable(u + 1) < 0 ? 0 : storable(u + 1), u + 1, storable(u + 1) >= 0);
                }
            }
            if constexpr (VD == 2) {
                if (q < 2) fetch(unit, 1 - q, xb, xvalid[xsel]);
                else fetch(next, 5 - q, xb, xvalid[xsel]);
            } else {
                if (q < 3) fetch(unit, 2 - q, xb, xvalid[xsel]);
                else fetch(next, 3, xb, xvalid[xsel]);
            }
#ifdef TQ_TIMELINE
            if (q == 0 && tl_n == 1 && gram[0] != 12345.678f) TQ_TL(11);   // the first sub-tile's input has arrived
            if (q == 1 && tl_n == 1 && gram[0] != 12345.678f) TQ_TL(12);
#endif

            float nrm[4];
            float4_t inv;
            float thr_tok[4][NT];  // 2- and 3-bit codes: this token's boundaries scaled by sqrt(128) ||x|| (as the K rows do)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float ss = row16_sum(n16 == 4 * kq + i ? gram[i] : 0.0f);
                nrm[i] = __builtin_amdgcn_sqrtf(ss);
                const bool nz = ss > 0.0f;
                const float rowscale = F32 ? row_pow2_scale(nrm[i]) : 1.0f;  // the power of two the token's fp32 row was multiplied by
                if constexpr (BITS == 4) {
                    inv[i] = nz ? __builtin_amdgcn_rsqf(ss) * (0.08838834764831845f * pow2_reciprocal(rowscale)) : 1.0f;  // 1 / (||x|| sqrt(128))
                } else {
                    inv[i] = 1.0f;
                    const float scale = nz ? nrm[i] * rowscale * 11.313708498984761f : 1.0f;
#pragma unroll
                    for (int k = 0; k < NT; ++k) thr_tok[i][k] = thr0[k] * scale;
                }
                zbits |= nz ? 0u : 1u << (4 * u + i);
            }
            // butterfly over the input slices, then normalise: y[fh][d0] is row dd = 2(fh % 2) + d0, dim half fh / 2
            float4_t y[4][2];
#pragma unroll
            for (int d0 = 0; d0 < 2; ++d0) {
#if TQ_KNOCKOUT & 2
                y[0][d0] = qq[d0][0] * inv; y[1][d0] = qq[d0][1] * inv; y[2][d0] = qq[d0][2] * inv; y[3][d0] = qq[d0][3] * inv;
#else
                const float4_t s01 = qq[d0][0] + qq[d0][1], d01 = qq[d0][0] - qq[d0][1];
                const float4_t s23 = qq[d0][2] + qq[d0][3], d23 = qq[d0][2] - qq[d0][3];
                if constexpr (BITS == 4) {  // the table is indexed by the normalised value
                    const float4_t s23i = s23 * inv, d23i = d23 * inv;
                    y[0][d0] = fma4(s01, inv, s23i);
                    y[1][d0] = fma4(d01, inv, d23i);
                    y[2][d0] = fma4(s01, inv, -s23i);
                    y[3][d0] = fma4(d01, inv, -d23i);
                } else {
                    y[0][d0] = s01 + s23;
                    y[1][d0] = d01 + d23;
                    y[2][d0] = s01 - s23;
                    y[3][d0] = d01 - d23;
                }
#endif
            }
            uint32_t n1[4] = {0, 0, 0, 0};  // 2-bit: per-token count of the level bit
            // groups in descending pair order: pair 4u + 2hf + i/2, high code (odd i) first
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                const int i = 3 - (g & 3), hf = g & 4 ? 0 : 1;
                const int j = grp_word(BITS, 4 * u);
                const float y0 = y[0 | (hf << 1)][0][i], y1 = y[0 | (hf << 1)][1][i];
                const float y2 = y[1 | (hf << 1)][0][i], y3 = y[1 | (hf << 1)][1][i];
#if TQ_KNOCKOUT & 1
                w[0][j] = (w[0][j] << 1) ^ __float_as_uint(y0); w[1][j] = (w[1][j] << 1) ^ __float_as_uint(y1);
                w[2][j] = (w[2][j] << 1) ^ __float_as_uint(y2); w[3][j] = (w[3][j] << 1) ^ __float_as_uint(y3);
                if constexpr (BITS == 99)
#endif
                if constexpr (BITS == 3) append_rows_b3(w[0][j], w[1][j], w[2][j], w[3][j], y0, y1, y2, y3, thr_tok[i]);
                else if constexpr (BITS == 2) append_rows_b2(w[0][j], w[1][j], w[2][j], w[3][j], n1[i], y0, y1, y2, y3, thr_tok[i]);
                else {
                    const char *ql = reinterpret_cast<const char *>(qlut);
                    append_rows_lut(w[0][j], w[1][j], w[2][j], w[3][j], y0, y1, y2, y3,
                                    *reinterpret_cast<const uint2 *>(ql + quant_lut_offset<DUP_LUT>(y0)),
                                    *reinterpret_cast<const uint2 *>(ql + quant_lut_offset<DUP_LUT>(y1)),
                                    *reinterpret_cast<const uint2 *>(ql + quant_lut_offset<DUP_LUT>(y2)),
                                    *reinterpret_cast<const uint2 *>(ql + quant_lut_offset<DUP_LUT>(y3)));
                }
            }
            // level counts of the four tokens, one byte per token, summed over the 16 columns
            uint32_t cnt[NT];
#if TQ_KNOCKOUT & 4
#pragma unroll
            for (int p = 0; p < NT; ++p) cnt[p] = 0x01010101u;
            if constexpr (BITS == 99)
#endif
            if constexpr (BITS == 4) {
                // dword u of every row is complete: vertical sums of the level-bit products over the rows
                constexpr uint32_t K0 = 0x11111111u;
                uint32_t sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int dd = 0; dd < 4; ++dd) {
                    const uint32_t ww = w[dd][u];
                    const uint32_t b0 = ww & K0, b1 = (ww >> 1) & K0, b2 = (ww >> 2) & K0, b01 = b0 & b1;
                    sum[1] += b0; sum[2] += b1; sum[3] += b01; sum[4] += b2;
                    sum[5] += b0 & b2; sum[6] += b1 & b2; sum[7] += b01 & b2;
                }
#pragma unroll
                for (int p = 1; p < 8; ++p) {
                    // token i sits at nibble i (hf 0) and nibble 4 + i (hf 1); bytes of cnt: tokens 0, 2, 1, 3
                    const uint32_t t = sum[p] + (sum[p] >> 16);
                    cnt[p] = (t & 0x0F0Fu) | ((t & 0xF0F0u) << 12);
                }
            } else if constexpr (BITS == 3) {
                // word u of every row (the tail word for u = 3) is complete: 3-bit fields 4hf + i hold token i's
                // code; field-wise sums of the level-bit products over the four rows stay below 8
                constexpr uint32_t K0 = 0x00249249u;
                uint32_t sum[4] = {0, 0, 0, 0};
#pragma unroll
                for (int dd = 0; dd < 4; ++dd) {
                    const uint32_t ww = w[dd][u];
                    const uint32_t b0 = ww & K0, b1 = (ww >> 1) & K0;
                    sum[1] += b0; sum[2] += b1; sum[3] += b0 & b1;
                }
#pragma unroll
                for (int p = 1; p < 4; ++p) {
                    // dim halves added in 6-bit lanes: e = tokens 0 and 2, o = tokens 1 and 3; then one byte per token
                    const uint32_t lo = sum[p] & 0xFFFu, hi = sum[p] >> 12;
                    const uint32_t e = (lo & 0x1C7u) + (hi & 0x1C7u), o = ((lo >> 3) & 0x1C7u) + ((hi >> 3) & 0x1C7u);
                    cnt[p] = (e & 0x3Fu) | ((o & 0x3Fu) << 8) | ((e & 0xFC0u) << 10) | ((o & 0xFC0u) << 18);
                }
            } else {
                cnt[1] = n1[0] | (n1[1] << 8) | (n1[2] << 16) | (n1[3] << 24);
            }
            float cs = 128.0f * coef[0];
            const int sh = BITS == 4 ? 8 * (((n16 & 1) << 1) | ((n16 >> 1) & 1)) : 8 * (n16 & 3);
#if TQ_KNOCKOUT & 4
            cs += (float)(cnt[NT - 1] >> sh);
#else
#pragma unroll
            for (int p = 1; p < NT; ++p) cs = fmaf(coef[p], (float)((row16_sum(cnt[p]) >> sh) & 0xFFu), cs);
#endif
            const int isel = n16 & 3;
            const float nsel = isel == 0 ? nrm[0] : isel == 1 ? nrm[1] : isel == 2 ? nrm[2] : nrm[3];
            const float gn = a.norm_correction ? nsel * __builtin_amdgcn_rsqf(cs) : nsel;
            if constexpr (DEFER) {
                park_norm = gn;
                if (completes(u)) {
                    // finish the dword this sub-tile completed: appended sign bit = "negative before s2", the xor makes it
                    // "positive after s2"; all-zero tokens (rare) get the sign field of an exact zero; then the fold
                    const int j = grp_word(BITS, 4 * u);
                    uint32_t zm = 0;
                    if (__builtin_amdgcn_ballot_w64(zbits != 0) != 0) {
#pragma unroll
                        for (int t = 0; t < 16; ++t)
                            zm |= (zbits >> t) & 1 ? (v_sign_mask(BITS, j, 0, 1u << t) | v_sign_mask(BITS, j, 1, 1u << t)) : 0u;
                    }
#pragma unroll
                    for (int dd = 0; dd < 4; ++dd) {
                        const uint32_t fm = (s2pos[dd][0] ? v_sign_mask(BITS, j, 0, 0xFFFFu) : 0u) | (s2pos[dd][1] ? v_sign_mask(BITS, j, 1, 0xFFFFu) : 0u);
                        uint32_t ww = w[dd][j] ^ fm;
                        ww = (ww & ~zm) | (zero_word & zm);
                        w[dd][j] = fold_codes<BITS>(ww);
                        if (storable(u) >= 0) {
                            park[dd] = w[dd][j];
                            if constexpr (BITS == 3) park[dd] = __builtin_amdgcn_perm(w[dd][3], w[dd][j], 0x04020100u + ((uint32_t)j << 24));
                        }
                    }
                }
            } else {
                if (n16 < 4) norms_out[4 * u + n16] = __float2half_rn(gn);
            }
        }
        if constexpr (DEFER) {
            pend_unit = unit;
            pending = true;
            unit = next;
            continue;
        }

        // sign fields: appended bit = "negative before s2"; xor makes it "positive after s2".  All-zero tokens
        // (rare: padding rows, empty vectors) get the sign field of an exact zero.
        const bool anyzero = __builtin_amdgcn_ballot_w64(zbits != 0) != 0;
#pragma unroll
        for (int j = 0; j < NW; ++j) {
            uint32_t zm = 0;
            if (anyzero) {
#pragma unroll
                for (int t = 0; t < 16; ++t)
                    zm |= (zbits >> t) & 1 ? (v_sign_mask(BITS, j, 0, 1u << t) | v_sign_mask(BITS, j, 1, 1u << t)) : 0u;
            }
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const uint32_t fm = (s2pos[dd][0] ? v_sign_mask(BITS, j, 0, 0xFFFFu) : 0u) | (s2pos[dd][1] ? v_sign_mask(BITS, j, 1, 0xFFFFu) : 0u);
                uint32_t ww = w[dd][j] ^ fm;
                ww = (ww & ~zm) | (zero_word & zm);
                w[dd][j] = fold_codes<BITS>(ww);
            }
        }
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) {
            const int row = half * 64 + 16 * dd + n16;
#pragma unroll
            for (int j = 0; j < BITS; ++j) {
                uint32_t g = w[dd][j];
                if constexpr (BITS == 3) g = __builtin_amdgcn_perm(w[dd][3], g, 0x04020100u + ((uint32_t)j << 24));
#if TQ_KNOCKOUT & 16
                if (g == 0x12345678u)   // keeps the codes alive; practically never taken
#endif
                stream_store<STREAM_STORE_CODES>(reinterpret_cast<uint32_t *>(block + j * 2048 + row * 16 + kq * 4), g);
            }
        }
        unit = next;
    }
    if constexpr (DEFER) {
        if (pending) flush_park(pend_unit, 0, 0, true);
    }
    TQ_TL(3);
    TQ_TL_VAL(6, (unsigned long long)tl_n);
}

__device__ __forceinline__ uint32_t wg_share(uint32_t n, uint32_t b, uint32_t g) { return (uint32_t)((uint64_t)n * b / g); }

// The +-1 operand fragments and sign tables are the same for every wavefront: a workgroup fetches them once
// into LDS (thousands of wavefronts asking the L2 for the same 8 KB delayed the start by several microseconds).

// single tensor: fixed strided share per wavefront (four workgroups of four wavefronts per CU for K, three for V)
template <int BITS, bool RAGGED, typename TI = __half>
__global__ __launch_bounds__(256, sizeof(TI) == 4 ? 3 : 4) void k_store_k(const TI *x, uint8_t *packed, StoreKArgs a) {
    // measured at 262 144 vectors: the LDS copy of the constants gains 1.6 us with 4-bit codes and 0.3 us with
    // 2-bit codes and loses 1.1 us with 3-bit codes, whose wavefronts then read them from memory themselves
    constexpr bool STAGED = BITS != 3;
    __shared__ uint32_t counter[4];
    __shared__ __attribute__((aligned(16))) uint2 qlut[BITS == 4 ? 4096 : 2];
    __shared__ __attribute__((aligned(16))) uint4 frag_s[STAGED ? 512 : 1];
    __shared__ uint32_t flip_s[16];
    const int t = threadIdx.x, wave = t >> 6;
    if ((t & 63) == 0) counter[wave] = K_UNITS_AHEAD;  // the first tickets are taken without asking
    if constexpr (STAGED) {
        const uint4 c0 = a.afrag[t], c1 = a.afrag[256 + t];
        const uint32_t c3 = a.s2flip[t & 15];
        if constexpr (BITS == 4) load_quant_lut<256>(qlut, a.quant_lut);
        auto stage = [&] {
            frag_s[t] = c0;
            frag_s[256 + t] = c1;
            if (t < 16) flip_s[t] = c3;
            __syncthreads();
        };
        store_k_units<BITS, RAGGED, false, false>(x, packed, a, blockIdx.x * 4 + wave, gridDim.x * 4, a.n_units, &counter[wave], qlut, frag_s,
                                    flip_s, 0u, stage);
    } else {
        store_k_units<BITS, RAGGED, false, false>(x, packed, a, blockIdx.x * 4 + wave, gridDim.x * 4, a.n_units, &counter[wave], qlut, a.afrag,
                                    a.s2flip, 0u, [] {});
    }
}

template <int BITS, bool RAGGED, typename TI = __half>
__global__ __launch_bounds__(256, 3) void k_store_v(const TI *x, uint8_t *packed, StoreVArgs a) {
    __shared__ uint32_t counter[4];
    __shared__ __attribute__((aligned(16))) uint2 qlut[BITS == 4 ? 4096 : 2];
    __shared__ __attribute__((aligned(16))) uint4 frag_s[512];
    __shared__ float s2_s[128];
    const int t = threadIdx.x, wave = t >> 6;
    const uint4 c0 = a.bfrag[t], c1 = a.bfrag[256 + t];
    const float c2 = a.s2[t & 127];
    if ((t & 63) == 0) counter[wave] = 1;  // ticket 0 is taken without asking
    if constexpr (BITS == 4) load_quant_lut<256>(qlut, a.quant_lut);
    auto stage = [&] {
        frag_s[t] = c0;
        frag_s[256 + t] = c1;
        if (t < 128) s2_s[t] = c2;
        __syncthreads();
    };
    store_v_units<BITS, RAGGED, false, false, false>(x, packed, a, blockIdx.x * 4 + wave, gridDim.x * 4, a.n_units, &counter[wave], qlut, frag_s, s2_s, 0u,
                                stage);
}

// K and V of one layer in one launch, one workgroup of 12 wavefronts per CU owning an equal
// contiguous share of both tensors: every wavefront takes V tiles until the workgroup's share
// is gone, then K units; the fine-grained K units level what the coarse V tiles leave uneven,
// and the launch and pipeline-fill time is paid once.
// The leading scalar parameters are what a wavefront needs for its first request; the two argument blocks follow.
// (Measured and not kept: the hardware's preloading of the leading arguments into scalar registers, 33.3 against 32.4 us
// for the 3-bit launch; reading one value of every cache line of the argument blocks in one batch at entry, 32.4 against
// 31.9 us; raised issue priority for wavefronts that hold a V tile, which shortens the V phase of the slowest wavefronts
// from 31 to 22 us and leaves the launch where it was.)
template <int KB, int VB, bool RAGGED, typename TI = __half>
__global__ __launch_bounds__(768) void k_store_kv(const TI *xv, const TI *xk, uint32_t v_units, uint32_t k_units, uint8_t *pv,
                                                  uint8_t *pk, StoreKArgs ka, StoreVArgs va) {
    // The +-1 operand fragments, sign masks, boundaries and c^2 coefficients are built from the argument block in
    // registers, so a wavefront's first memory request is its first input; only the 4-bit quantiser tables live in
    // LDS, and they are fetched behind the first input and waited for by the barrier that also publishes the
    // ticket counters.
    __shared__ uint32_t counter[2];
    __shared__ __attribute__((aligned(16))) uint2 qlut_k[KB == 4 ? 8192 : 2];  // every entry twice (load_quant_lut_dup)
    __shared__ __attribute__((aligned(16))) uint2 qlut_v[VB == 4 ? 8192 : 2];
    const int t = threadIdx.x;
    TQ_TL(0);
    if (t < 2) counter[t] = t == 0 ? 12u : 0u;  // V: the wavefronts' first tickets are their own numbers
    const bool share_lut = KB == 4 && VB == 4 && va.share_k_lut;  // equal tables: one copy serves both tensors
    auto stage = [&] {
        if constexpr (KB == 4) load_quant_lut_dup<768>(qlut_k, ka.quant_lut);
        if constexpr (VB == 4) {
            if (!share_lut) load_quant_lut_dup<768>(qlut_v, va.quant_lut);
        }
        __syncthreads();
    };
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane(t >> 6);
    store_v_units<VB, RAGGED, true, true, true>(xv, pv, va, wg_share(v_units, blockIdx.x, gridDim.x), 1,
                              wg_share(v_units, blockIdx.x + 1, gridDim.x), &counter[0], share_lut ? qlut_k : qlut_v, nullptr, nullptr,
                              wave, stage);
    store_k_units<KB, RAGGED, true, true>(xk, pk, ka, wg_share(k_units, blockIdx.x, gridDim.x), 1,
                              wg_share(k_units, blockIdx.x + 1, gridDim.x), &counter[1], qlut_k, nullptr, nullptr,
                              DRAW_TICKET, [] {});
}

// ---- K2: fused quantise + pack ---------------------------------------------------
// One vector on the 16 lanes of a DPP row, 8 values per lane: norm, s1, 128-point butterfly,
// s2/sqrt(128), normalise, compare-count against the boundaries, sum c^2.  Returns the
// lane's 8 codes as bytes and (valid on every lane of the row) the norm to store.
template <int BITS>
__device__ __forceinline__ float quantize_vec16(float (&xv)[8], int lane, const float (&bnd)[(1 << BITS) - 1], const float (&s1v)[8],
                                                const float (&s2v)[8], const float *csq_s, int norm_correction, uint2 &codes8) {
    constexpr int NB = (1 << BITS) - 1;
    float ss = 0.0f;
#pragma unroll
    for (int m = 0; m < 8; ++m) ss = fmaf(xv[m], xv[m], ss);
    ss = row16_sum(ss);
    const float norm = sqrtf(ss);
    const float inv = norm > 0.0f ? 1.0f / norm : 1.0f;
#pragma unroll
    for (int m = 0; m < 8; ++m) xv[m] *= s1v[m];
    wht128_row16(xv, lane);
    uint32_t w0 = 0, w1 = 0;
    float cs = 0.0f;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        const float yv = (xv[m] * s2v[m]) * inv;
        uint32_t c = 0;
#pragma unroll
        for (int k = 0; k < NB; ++k) c += (bnd[k] < yv) ? 1u : 0u;
        cs += csq_s[c];
        if (m < 4) w0 |= c << (8 * m);
        else w1 |= c << (8 * (m - 4));
    }
    cs = row16_sum(cs);
    codes8 = make_uint2(w0, w1);
    float g = norm;
    if (norm_correction) {
        const float cn = sqrtf(cs);
        g = norm / (cn > 1e-10f ? cn : 1.0f);
    }
    return g;
}

template <int BITS, typename TI>
__global__ __launch_bounds__(256) void k_store(const TI *x, uint8_t *packed, StoreArgs a) {
    constexpr int NB = (1 << BITS) - 1;
    __shared__ __attribute__((aligned(16))) uint8_t codes[TQ_ROWS_PER_BLOCK * CODE_STRIDE];
    __shared__ float norms_s[TQ_ROWS_PER_BLOCK];
    __shared__ float csq_s[1 << BITS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int li = lane & 15, grp = tid >> 4;
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / a.blocks_per_seq, bis = blk % a.blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;

    float bnd[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) bnd[k] = a.bounds[k];
    if (tid < (1 << BITS)) {
        const float c = a.cent[tid];
        csq_s[tid] = c * c;
    }
    float s1v[8], s2v[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        s1v[m] = a.s1[8 * li + m];
        s2v[m] = a.s2[8 * li + m] * RSQRT128;
    }
    __syncthreads();

#pragma unroll 1
    for (int it = 0; it < 8; ++it) {
        const int t = it * 16 + grp;
        const bool valid = tok0 + t < a.tokens;
        float xv[8];
        if (valid) {
            load8(x + ((seq * a.tokens + tok0 + t) * 128 + 8 * li), xv);
        } else {
#pragma unroll
            for (int m = 0; m < 8; ++m) xv[m] = 0.0f;
        }
        uint2 c8;
        const float g = quantize_vec16<BITS>(xv, lane, bnd, s1v, s2v, csq_s, a.norm_correction, c8);
        *reinterpret_cast<uint2 *>(&codes[t * CODE_STRIDE + 8 * li]) = c8;
        if (li == 0) norms_s[t] = g;
    }
    __syncthreads();
    pack_block<BITS, 256>(codes, norms_s, packed + blk * block_bytes(BITS), a.kind);
}

// ---- K2, streaming append -------------------------------------------------------------
// n_new tokens per sequence at positions pos .. pos+n_new-1 of a buffer laid out for
// blocks_per_seq blocks per sequence, one workgroup per touched block.  The new rows are quantised
// exactly as k_store does.  A block whose first token is among them is written whole: the rows
// past the new tokens get the code of 0.0 and norm 0 (what k_store writes past the end of a
// sequence).  A block that already holds tokens keeps them: K rows are tokens and are simply left
// alone, V rows get the new tokens' codes put into their packed words.  After any sequence of
// appends covering tokens 0 .. T-1 the touched blocks equal those of k_store on the first T tokens.
struct AppendArgs {
    const float *s1, *s2, *bounds, *cent;
    int kind, norm_correction, zero_code;
    int64_t pos, n_new, blocks_per_seq, first_block, n_touched;
    const int64_t *pos_dev;  // NULL, or where the position is read from when the launch runs (n_touched is then the
    int64_t capacity;        // largest number of blocks n_new tokens can touch, and some workgroups find nothing to do)
    uint32_t *overrun;       // NULL, or a sticky word that a refused position sets (TQ_OVERRUN_* bits)
};

// A position read from device memory that is negative or leaves no room for n_new tokens (n_new <= capacity is
// checked on the host, so the subtraction cannot wrap whatever the counter holds): nothing is written, and the
// launch's first workgroup records why in the caller's word, if there is one.
__device__ __forceinline__ bool append_position_ok(int64_t pos, int64_t n_new, int64_t capacity, uint32_t *overrun, bool reporter) {
    const uint32_t why = pos < 0 ? (uint32_t)TQ_OVERRUN_NEGATIVE : pos > capacity - n_new ? (uint32_t)TQ_OVERRUN_NO_ROOM : 0u;
    if (why && overrun && reporter && threadIdx.x == 0) atomicOr(overrun, why);
    return why == 0u;
}

// Position from device memory (a captured launch replayed while the cache grows): fills in pos and first_block and
// says whether workgroup `wg` has a block to rebuild.  Positions that do not fit the capacity write nothing.
__device__ __forceinline__ bool resolve_append(AppendArgs &a, int64_t wg) {
    if (!a.pos_dev) return true;
    const int64_t pos = *a.pos_dev;
    if (!append_position_ok(pos, a.n_new, a.capacity, a.overrun, wg == 0)) return false;
    a.pos = pos;
    a.first_block = pos / TQ_ROWS_PER_BLOCK;
    const int64_t touched = (pos + a.n_new - 1) / TQ_ROWS_PER_BLOCK - a.first_block + 1;
    return wg % a.n_touched < touched;
}

__device__ inline float block_norm(const uint8_t *block, int bits, int token);

// one workgroup rebuilds block `wg` (sequence wg / n_touched, touched block wg % n_touched)
template <int BITS, typename TI>
__device__ __forceinline__ void append_block(const TI *x, uint8_t *packed, const AppendArgs &a, const int64_t wg) {
    constexpr int NB = (1 << BITS) - 1;
    __shared__ __attribute__((aligned(16))) uint8_t codes[TQ_ROWS_PER_BLOCK * CODE_STRIDE];
    __shared__ float norms_s[TQ_ROWS_PER_BLOCK];
    __shared__ float csq_s[1 << BITS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int li = lane & 15, grp = tid >> 4;
    const int64_t seq = wg / a.n_touched, bis = a.first_block + wg % a.n_touched;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    uint8_t *block = packed + (seq * a.blocks_per_seq + bis) * block_bytes(BITS);

    float bnd[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) bnd[k] = a.bounds[k];
    if (tid < (1 << BITS)) {
        const float c = a.cent[tid];
        csq_s[tid] = c * c;
    }
    float s1v[8], s2v[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        s1v[m] = a.s1[8 * li + m];
        s2v[m] = a.s2[8 * li + m] * RSQRT128;
    }
    // rows already in the block: the block is copied into LDS with coalesced loads and unpacked from there
    const int n_old = (int)(a.pos - tok0 < 0 ? 0 : (a.pos - tok0 > TQ_ROWS_PER_BLOCK ? TQ_ROWS_PER_BLOCK : a.pos - tok0));
    const int n_end = (int)(a.pos + a.n_new - tok0 > TQ_ROWS_PER_BLOCK ? TQ_ROWS_PER_BLOCK : a.pos + a.n_new - tok0);  // first empty row
    __shared__ __attribute__((aligned(16))) uint8_t old_s[block_bytes(BITS)];
    // K rows are tokens: the rows already there stay untouched in memory and need not be unpacked
    const bool keep_rows = a.kind == TQ_KIND_K;
    if (n_old > 0 && !keep_rows) {
        // V rows of a block that already holds tokens: the new tokens' codes are put into the packed rows in
        // place (every row of the tile has one pair position per token), so nothing is unpacked or re-packed.
        // Rows past the new tokens keep the code of 0.0 that the block's first append gave them.
        constexpr int PIECES = block_bytes(BITS) / 16, NP = (PIECES + 255) / 256;
        constexpr uint32_t CM = (1u << BITS) - 1u;
        uint4 pre[NP];
#pragma unroll
        for (int i = 0; i < NP; ++i) pre[i] = reinterpret_cast<const uint4 *>(block)[min(tid + 256 * i, PIECES - 1)];
        __syncthreads();  // csq_s is ready
#pragma unroll 1
        for (int it = 0; it < 8; ++it) {
            const int t = it * 16 + grp;
            if (t < n_old || t >= n_end) continue;
            float xv[8];
            load8(x + ((seq * a.n_new + (tok0 + t - a.pos)) * 128 + 8 * li), xv);
            uint2 c8;
            const float g = quantize_vec16<BITS>(xv, lane, bnd, s1v, s2v, csq_s, a.norm_correction, c8);
            *reinterpret_cast<uint2 *>(&codes[t * CODE_STRIDE + 8 * li]) = c8;
            if (li == 0) norms_s[t] = g;
        }
#pragma unroll
        for (int i = 0; i < NP; ++i)
            if (tid + 256 * i < PIECES) reinterpret_cast<uint4 *>(old_s)[tid + 256 * i] = pre[i];
        __syncthreads();
        if (tid < TQ_ROWS_PER_BLOCK) {
            // new tokens take their codes; tokens from n_end to the end of their 16-token group take the code of 0.0
            // (as do the whole groups after it, below): what tq_store writes past the end of a sequence
            const int r = tid, rr = r & 63, t_lo = max(n_old, r & 64), t_end = (r & 64) + 64;
            const int t_hi = min(max((n_end + 15) & ~15, t_lo), t_end);
            for (int t = t_lo; t < t_hi; ++t) {
                const int tl = t & 63, g = tl >> 4, k0 = (tl & 12) | ((tl >> 1) & 1), hs = (tl & 1) * BITS;
                const bool fresh = t < n_end;
                const uint32_t c0 = fresh ? codes[t * CODE_STRIDE + rr] : (uint32_t)a.zero_code;
                const uint32_t c1 = fresh ? codes[t * CODE_STRIDE + 64 + rr] : (uint32_t)a.zero_code;
                uint8_t *rowp = old_s + r * 16 + g * 4;
                if (BITS == 3 && k0 >= 12) {
                    uint32_t *d0 = reinterpret_cast<uint32_t *>(rowp), *d1 = reinterpret_cast<uint32_t *>(rowp + 2048),
                             *d2 = reinterpret_cast<uint32_t *>(rowp + 4096);
                    uint32_t tail = (*d0 >> 24) | ((*d1 >> 24) << 8) | ((*d2 >> 24) << 16);
                    const int s0 = 6 * (k0 - 12) + hs, s1 = s0 + 12;
                    tail = (tail & ~((CM << s0) | (CM << s1))) | (c0 << s0) | (c1 << s1);
                    *d0 = (*d0 & 0x00FFFFFFu) | (tail << 24);
                    *d1 = (*d1 & 0x00FFFFFFu) | ((tail >> 8) << 24);
                    *d2 = (*d2 & 0x00FFFFFFu) | ((tail >> 16) << 24);
                } else {
                    uint32_t *d = reinterpret_cast<uint32_t *>(rowp + (k0 / tqd::pairs_per_dword(BITS)) * 2048);
                    const int s0 = 2 * BITS * (k0 % tqd::pairs_per_dword(BITS)) + hs, s1 = s0 + 4 * BITS;
                    *d = (*d & ~((CM << s0) | (CM << s1))) | (c0 << s0) | (c1 << s1);
                }
            }
            // whole 16-token groups past the new tokens: every field the code of 0.0
            uint32_t fill = 0;
#pragma unroll
            for (int f = 0; f < 32 / BITS; ++f) fill |= (uint32_t)a.zero_code << (f * BITS);
            for (int t = max(t_hi, t_lo); t < t_end; t += 16) {
                uint8_t *rowp = old_s + r * 16 + ((t & 63) >> 4) * 4;
#pragma unroll
                for (int j = 0; j < BITS; ++j) {
                    uint32_t w = fill;
                    if constexpr (BITS == 3) w = (fill & 0x00FFFFFFu) | (((fill & 0x00FFFFFFu) >> (8 * j)) << 24);
                    *reinterpret_cast<uint32_t *>(rowp + j * 2048) = w;
                }
            }
        }
        for (int t = n_old + tid; t < TQ_ROWS_PER_BLOCK; t += 256)
            reinterpret_cast<__half *>(old_s + block_code_bytes(BITS))[t] = __float2half_rn(t < n_end ? norms_s[t] : 0.0f);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NP; ++i)
            if (tid + 256 * i < PIECES) reinterpret_cast<uint4 *>(block)[tid + 256 * i] = reinterpret_cast<const uint4 *>(old_s)[tid + 256 * i];
        return;
    }
    // rows past the new tokens hold the code of 0.0 and norm 0 (what quantising a zero vector gives)
    for (int e = tid; e < (TQ_ROWS_PER_BLOCK - n_end) * 32; e += 256) {
        const int t = n_end + (e >> 5), q = e & 31;
        *reinterpret_cast<uint32_t *>(&codes[t * CODE_STRIDE + 4 * q]) = 0x01010101u * (uint32_t)a.zero_code;
    }
    for (int t = n_end + tid; t < TQ_ROWS_PER_BLOCK; t += 256) norms_s[t] = 0.0f;
    __syncthreads();

#pragma unroll 1
    for (int it = 0; it < 8; ++it) {
        const int t = it * 16 + grp;
        if (t < n_old || t >= n_end) continue;  // whole 16-lane rows skip together
        const int64_t rel = tok0 + t - a.pos;
        float xv[8];
        load8(x + ((seq * a.n_new + rel) * 128 + 8 * li), xv);
        uint2 c8;
        const float g = quantize_vec16<BITS>(xv, lane, bnd, s1v, s2v, csq_s, a.norm_correction, c8);
        *reinterpret_cast<uint2 *>(&codes[t * CODE_STRIDE + 8 * li]) = c8;
        if (li == 0) norms_s[t] = g;
    }
    __syncthreads();
    pack_block<BITS, 256>(codes, norms_s, block, a.kind, keep_rows ? n_old : 0);
}

template <int BITS, typename TI>
__global__ __launch_bounds__(256) void k_append(const TI *x, uint8_t *packed, AppendArgs a) {
    if (!resolve_append(a, blockIdx.x)) return;
    append_block<BITS, TI>(x, packed, a, blockIdx.x);
}

// K and V of a decode step in one launch: the first half of the grid rebuilds K blocks, the second half V blocks
template <int KB, int VB, typename TI>
__global__ __launch_bounds__(256) void k_append_kv(const TI *xk, uint8_t *pk, AppendArgs ka, const TI *xv, uint8_t *pv, AppendArgs va) {
    const unsigned half = gridDim.x >> 1;
    if (blockIdx.x < half) {
        if (resolve_append(ka, blockIdx.x)) append_block<KB, TI>(xk, pk, ka, blockIdx.x);
    } else {
        if (resolve_append(va, blockIdx.x - half)) append_block<VB, TI>(xv, pv, va, blockIdx.x - half);
    }
}

// ---- K2 + K4 in float64: codes, corrected norm, residual sign sketch ---------------
struct StoreQjlArgs {
    const double *s1, *s2, *bounds, *cent;
    const double *projrot_t;  // [128*128]: entry [k*128+j] = (S R^T)[j][k]
    const uint4 *frag;        // [3][4][8][64] B operands of the projection: 64 (S R^T) as three fp16 terms
    float tau;                // first pass: closer to zero than tau * |scaled residual| -> second pass
    double tau2;              // second pass: closer to zero than tau2 * |residual| -> third pass
    int norm_correction;
    int64_t tokens, blocks_per_seq;
};

// One workgroup of eight wavefronts per CU.  The wavefronts are independent after the constants are in place: each
// takes units of 16 tokens (a strided share), lane (token n16, quarter kq) holding the 32 dims d = 4 s + kq.  Norms
// and the first two butterfly stages (in the reference's stage order) exchange across the lane quarters, the other
// five stages are in-lane, all in float64, and so is the residual in the rotated domain, taken against the
// reconstruction the decoder will see (stored fp16 norm).
// Only the signs of the 128 projections (S R^T) r are stored, so the projection runs on the fp16 matrix cores with an
// error bound instead of on the float64 ones: the residual is scaled by a power of two to 512 <= |x| < 1024 and split
// into two fp16 terms, the matrix (times 64) was split into three when the handle was made (96 KB in LDS, laid out
// as B operands; the contraction runs over the dims in the order a lane holds them, so the A operands are the lane's
// own values), and hi*hi + hi*mid + lo*hi accumulate in fp32 on v_mfma_f32_16x16x32_f16: 96 instructions of 16
// clocks per unit instead of 256 float64 ones of 64 clocks.  A result at least tau |x| away from zero (the bound on
// this pass's error, worked out where the handle is made) has the exact projection's sign.  The others, about one
// per unit, get a second pass: the token's float64 residual goes through 1 KB of LDS, every lane multiplies two dims
// of it with hi + mid + lo read from the same operand table, and the wavefront adds the 64 partial products in float64
// (error 2^-31 relative; left to the four lanes that hold the token it took 0.7 us per value); the one in 10^8 of those that is still too close goes
// to the float64 matrix in memory.
// The sign bits of a token's 16 projections of one column block are one quarter of a ballot.  A wavefront packs its
// own 16 rows (rows of a K block are independent).  No barrier ties the wavefronts together, and the next unit's
// input is requested before the matrix phase starts.
typedef double double4_t __attribute__((ext_vector_type(4)));
template <int BITS, typename TI>
__global__ __launch_bounds__(512) void k_store_qjl_mfma(const TI *x, uint8_t *packed, uint8_t *sign_bits, __half *rnorms,
                                                       StoreQjlArgs a, int64_t n_blocks) {
    using namespace tq64;
    constexpr int NB = (1 << BITS) - 1;
    extern __shared__ uint4 frag_s[];  // [3 terms][4 steps][8 column blocks][64 lanes]: B operands of the projection
    __shared__ __attribute__((aligned(16))) uint8_t codes_s[8][16 * CODE_STRIDE];
    __shared__ double cent_s[1 << BITS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n16 = lane & 15, kq = lane >> 4;
    uint8_t *codes = codes_s[wave];
    double *stage = reinterpret_cast<double *>(frag_s + 3 * 4 * 8 * 64) + 128 * wave;  // second pass: one token's residual

    const int64_t n_units = n_blocks * 8;
    const int64_t unit_step = (int64_t)gridDim.x * 8;
    int64_t unit = (int64_t)blockIdx.x * 8 + wave;
    // this lane's 32 inputs of a unit, as stored (converted when the unit is processed)
    TI xin[32];
    bool xvalid = false;
    auto fetch = [&](int64_t un) {
        const int64_t blk = un >> 3;
        const int64_t seq = blk / a.blocks_per_seq, bis = blk % a.blocks_per_seq;
        const int64_t tok = bis * TQ_ROWS_PER_BLOCK + (un & 7) * 16 + n16;
        xvalid = un < n_units && tok < a.tokens;
        const TI *src = x + (seq * a.tokens + (xvalid ? tok : 0)) * 128 + kq;
        if (un >= n_units) src = x + kq;
#pragma unroll
        for (int s = 0; s < 32; ++s) xin[s] = src[4 * s];
    };
    fetch(unit);

    // the matrix operands are fetched once per workgroup, twelve 16-byte pieces per thread
    {
        uint4 piece[12];
#pragma unroll
        for (int i = 0; i < 12; ++i) piece[i] = a.frag[tid + 512 * i];
#pragma unroll
        for (int i = 0; i < 12; ++i) frag_s[tid + 512 * i] = piece[i];
    }
    if (tid < (1 << BITS)) cent_s[tid] = a.cent[tid];
    // the boundaries stay in registers (the byte stores of the code stage may alias anything as far as the compiler
    // knows, so boundaries kept in LDS were read again for every value)
    double bnd[NB];
#pragma unroll
    for (int k = 0; k < NB; ++k) bnd[k] = a.bounds[k];
    uint32_t neg1 = 0, neg2 = 0;  // bit s: s1 / s2 of dim 4 s + kq is -1
#pragma unroll
    for (int s = 0; s < 32; ++s) {
        neg1 |= (a.s1[4 * s + kq] < 0.0 ? 1u : 0u) << s;
        neg2 |= (a.s2[4 * s + kq] < 0.0 ? 1u : 0u) << s;
    }
    __syncthreads();
    // one reciprocal instead of 32 divisions per token, and 1 / sqrt(128) as a factor: at most one unit in the
    // last place away from the quotients, far inside the 1e-6 band the codes and signs are held to
    const double inv_rn = 1.0 / sqrt(128.0);
    auto quarter_sum = [&](double v) {
        v += xor_lane<16>(v);
        v += xor_lane<32>(v);
        return v;
    };

#pragma unroll 1
    for (; unit < n_units; unit += unit_step) {
        const int64_t blk = unit >> 3;
        const int u = (int)(unit & 7);
        const int64_t seq = blk / a.blocks_per_seq, bis = blk % a.blocks_per_seq;
        const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
        const int64_t row0 = seq * a.tokens;
        const int t = u * 16 + n16;
        const bool valid = xvalid;
        double e[32];
#pragma unroll
        for (int s = 0; s < 32; ++s) e[s] = valid ? ldd(xin, s) : 0.0;
        double ss = 0.0;
#pragma unroll
        for (int s = 0; s < 32; ++s) ss = fma(e[s], e[s], ss);
        const double nrm = sqrt(quarter_sum(ss));
        const double inv = nrm > 0.0 ? 1.0 / nrm : 1.0;
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            e[s] = e[s] * inv;
            if ((neg1 >> s) & 1u) e[s] = -e[s];
        }
        // butterfly, strides 1 and 2 across the lane quarters, then 4 .. 64 in the lane
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            const double p = xor_lane<16>(e[s]);
            e[s] = (kq & 1) ? p - e[s] : e[s] + p;
        }
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            const double p = xor_lane<32>(e[s]);
            e[s] = (kq & 2) ? p - e[s] : e[s] + p;
        }
#pragma unroll
        for (int hb = 1; hb < 32; hb <<= 1)
#pragma unroll
            for (int s = 0; s < 32; ++s)
                if (!(s & hb)) {
                    const double p = e[s], q = e[s + hb];
                    e[s] = p + q;
                    e[s + hb] = p - q;
                }
        uint32_t cw[4] = {0u, 0u, 0u, 0u};  // the 32 codes, 4 bits each
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            double yv = e[s] * inv_rn;
            if ((neg2 >> s) & 1u) yv = -yv;
            e[s] = yv;
            uint32_t c = 0;
#pragma unroll
            for (int k = 0; k < NB; ++k) c += (bnd[k] < yv) ? 1u : 0u;
            cw[s >> 3] |= c << (4 * (s & 7));
        }
        // the code stage takes the lane's codes as bytes (dim 4 s + kq of token n16)
#pragma unroll
        for (int s = 0; s < 32; ++s) codes[n16 * CODE_STRIDE + 4 * s + kq] = (uint8_t)((cw[s >> 3] >> (4 * (s & 7))) & 15u);
        double cv[32];
        double cs = 0.0;
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            cv[s] = cent_s[(cw[s >> 3] >> (4 * (s & 7))) & 15u];
            cs = fma(cv[s], cv[s], cs);
        }
        const double cn = sqrt(quarter_sum(cs));
        double g = nrm;
        if (a.norm_correction) g = nrm / (cn > 1e-10 ? cn : 1.0);
        const __half gh = double_to_half_rn(g);
        const double g16 = (double)__half2float(gh);
        uint8_t *block = packed + blk * block_bytes(BITS);
        if (kq == 0) reinterpret_cast<__half *>(block + block_code_bytes(BITS))[t] = gh;
        // residual in the rotated domain against the reconstruction the decoder will see
        double rs = 0.0;
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            e[s] = nrm * e[s] - g16 * cv[s];
            rs = fma(e[s], e[s], rs);
        }
        const double rnorm = sqrt(quarter_sum(rs));
        if (valid && kq == 0) rnorms[row0 + tok0 + t] = double_to_half_rn(rnorm);
        // the wavefront's 16 rows of the block: chunk c, row r = lane / 4, dword k = lane % 4 (pack_block's word)
        __builtin_amdgcn_wave_barrier();
        {
            constexpr int PER = pairs_per_dword(BITS);
            const int r = lane >> 2, k = lane & 3;
#pragma unroll
            for (int c = 0; c < BITS; ++c) {
                uint32_t word = 0;
#pragma unroll
                for (int i = 0; i < PER; ++i) word |= pair_from_stage<BITS>(codes, TQ_KIND_K, r, 16 * k + PER * c + i) << (2 * BITS * i);
                if constexpr (BITS == 3) {
                    uint32_t tail = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) tail |= pair_from_stage<3>(codes, TQ_KIND_K, r, 16 * k + 12 + i) << (6 * i);
                    word |= ((tail >> (8 * c)) & 0xFFu) << 24;
                }
                reinterpret_cast<uint32_t *>(block)[c * 512 + (u * 16 + r) * 4 + k] = word;
            }
        }
        __builtin_amdgcn_wave_barrier();
        // the next unit's input is under way while the matrix phase runs
        fetch(unit + unit_step);
        // the residual as fp16 pairs: x = e * 2^p with |x| < 1024 (p from the token's residual norm), x = hi + lo
        int ex;
        (void)frexp(rnorm, &ex);
        const double pw = ldexp(1.0, 10 - ex);
        half8_t xh[4], xl[4];
#pragma unroll
        for (int s = 0; s < 32; ++s) {
            const float xf = (float)(e[s] * pw);
            const _Float16 hi = (_Float16)xf;
            xh[s >> 3][s & 7] = hi;
            xl[s >> 3][s & 7] = (_Float16)(xf - (float)hi);
        }
        // first-pass threshold of this lane's token (0 for a token without a residual: nothing to recompute)
        const float tau_own = a.tau * (float)(rnorm * pw);
        // (S R^T) x for the 16 tokens: D[token][j] += X[token][k] M[k][j], 8 column blocks x 4 steps of 32 dims
        // (the two small terms have an accumulator of their own: the rounding of their 256 additions is then
        // relative to sums 2^-10 of the main term's and drops out of the error bound)
        float4_t acc[8], acc_s[8];
#pragma unroll
        for (int jb = 0; jb < 8; ++jb) acc[jb] = acc_s[jb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int jb = 0; jb < 8; ++jb) {
                const half8_t mh = __builtin_bit_cast(half8_t, frag_s[(c * 8 + jb) * 64 + lane]);
                const half8_t ml = __builtin_bit_cast(half8_t, frag_s[2048 + (c * 8 + jb) * 64 + lane]);
                acc_s[jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xl[c], mh, acc_s[jb], 0, 0, 0);
                acc_s[jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh[c], ml, acc_s[jb], 0, 0, 0);
                acc[jb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xh[c], mh, acc[jb], 0, 0, 0);
            }
        }
#pragma unroll
        for (int jb = 0; jb < 8; ++jb) acc[jb] += acc_s[jb];
        // lane (n16, kq) now holds the projections j = 16 jb + n16 of tokens 4 kq + i (register i of the result).
        // The sign bits of token 4 kq + i, column block jb, are a quarter of a ballot; lane (jb, kq) collects them for
        // its four tokens in `signs` (16 bits per i).  `doubt` marks this lane's results that are too close to zero
        // for the first pass to settle the sign (bit 31 - (8 i + jb)).
        uint32_t piece[4] = {0u, 0u, 0u, 0u};
        uint32_t doubt = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float tau_i = __shfl(tau_own, 4 * kq + i);  // of token 4 kq + i (held by lane quarter 0)
#pragma unroll
            for (int jb = 0; jb < 8; ++jb) {
                const uint64_t m = __builtin_amdgcn_ballot_w64(acc[jb][i] >= 0.0f);
                if (n16 == jb) piece[i] = (uint32_t)(m >> (16 * kq));
                doubt = (doubt << 1) | (fabsf(acc[jb][i]) < tau_i ? 1u : 0u);
            }
        }
        uint64_t signs = (uint64_t)((piece[0] & 0xFFFFu) | (piece[1] << 16)) | ((uint64_t)((piece[2] & 0xFFFFu) | (piece[3] << 16)) << 32);
        // The doubtful ones: one loop for all of them (wave-uniform control flow), each shared by the whole wavefront.
        uint64_t who = __builtin_amdgcn_ballot_w64(doubt != 0u);
#pragma unroll 1
        while (who) {
            const int l = __builtin_ctzll(who);
            who &= who - 1;
            uint32_t bits = (uint32_t)__builtin_amdgcn_readlane((int)doubt, l);
#pragma unroll 1
            while (bits) {
                const int idx = __builtin_clz(bits);  // 8 i + jb
                bits &= ~(0x80000000u >> idx);
                const int i = idx >> 3, jb = idx & 7;
                const int tokl = 4 * (l >> 4) + i, j = 16 * jb + (l & 15);
                // second pass: e . (hi + mid + lo) in float64.  The token's residual goes through LDS (stage[32 kq + s] =
                // dim 4 s + kq) so that the whole wavefront shares the product: lane (sp, kq') = (lane / 4, lane % 4)
                // takes dims 4 (2 sp) + kq' and 4 (2 sp + 1) + kq', two neighbouring halves of one fragment dword.
                if (n16 == tokl) {
#pragma unroll
                    for (int s2 = 0; s2 < 32; s2 += 2) *reinterpret_cast<double2 *>(stage + 32 * kq + s2) = make_double2(e[s2], e[s2 + 1]);
                }
                __builtin_amdgcn_wave_barrier();
                const int kqp = lane & 3, sp = lane >> 2;
                const double2 ev = *reinterpret_cast<const double2 *>(stage + 32 * kqp + 2 * sp);
                const uint32_t *fw = reinterpret_cast<const uint32_t *>(frag_s) + (((sp >> 2) * 8 + jb) * 64 + 16 * kqp + (l & 15)) * 4 + (sp & 3);
                const half2_t m1 = __builtin_bit_cast(half2_t, fw[0]);
                const half2_t m2 = __builtin_bit_cast(half2_t, fw[2048 * 4]);
                const half2_t m3 = __builtin_bit_cast(half2_t, fw[4096 * 4]);
                double part = ev.x * ((double)((float)m1[0] + (float)m2[0]) + (double)(float)m3[0]);
                part = fma(ev.y, (double)((float)m1[1] + (float)m2[1]) + (double)(float)m3[1], part);
                __builtin_amdgcn_wave_barrier();
                part = quarter_sum(row16_sum(part));
                double settled = part;  // every lane holds the sum
                const double rn_tok = __shfl(rnorm, tokl);
                if (fabs(settled) < a.tau2 * rn_tok) {  // third pass (wave-uniform: every lane holds the same values)
                    part = 0.0;
                    if (n16 == tokl) {
#pragma unroll
                        for (int s = 0; s < 32; ++s) part = fma(e[s], a.projrot_t[(4 * s + kq) * 128 + j], part);
                    }
                    part = quarter_sum(part);
                    settled = __shfl(part, tokl);
                }
                const int holder = 16 * (l >> 4) + jb, bit = 16 * i + (l & 15);  // where the first pass put the sign
                if (lane == holder && (((signs >> bit) & 1ull) != 0ull) != (settled >= 0.0)) signs ^= 1ull << bit;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t tk = tok0 + u * 16 + 4 * kq + i;
            if (n16 < 8 && tk < a.tokens)
                reinterpret_cast<uint16_t *>(sign_bits)[(row0 + tk) * 8 + n16] = (uint16_t)(signs >> (16 * i));
        }
    }
}

// ---- K3: packed block -> values ----------------------------------------------------
__device__ inline float block_norm(const uint8_t *block, int bits, int token) {
    const __half *nm = reinterpret_cast<const __half *>(block + block_code_bytes(bits));
    return __half2float(nm[token]);
}

struct LoadArgs {
    const float *s1, *s2, *cent;
    int bits, kind, domain;
    int64_t tokens, blocks_per_seq;
};

// The eight codes of dims 8li .. 8li+7 of token t, code m at bit m*BITS.  K rows: the lane's four pairs are
// one dword of a group (2-bit: half a dword; 3-bit: 24 bits of a dword, or the group's tail).  V rows: the same
// pair position of eight consecutive rows.
template <int BITS>
__device__ __forceinline__ uint32_t load_codes8(const uint8_t *block, int kind, int t, int li) {
    constexpr uint32_t CM = (1u << BITS) - 1u;
    if (kind == TQ_KIND_K) {
        const int g = li >> 2, q = li & 3;
        if constexpr (BITS == 4) return row_dword(block, t, 4 * q + g);
        if constexpr (BITS == 2) return (row_dword(block, t, 4 * (q >> 1) + g) >> (16 * (q & 1))) & 0xFFFFu;
        if constexpr (BITS == 3) {
            if (q < 3) return row_dword(block, t, 4 * q + g) & 0xFFFFFFu;
            return (row_dword(block, t, g) >> 24) | ((row_dword(block, t, 4 + g) >> 24) << 8) | ((row_dword(block, t, 8 + g) >> 24) << 16);
        }
    }
    const int r0 = (t & 64) | ((8 * li) & 63);
    const int p = ((t & 60) | ((li >> 3) << 1)) | ((t >> 1) & 1);
    const int g = p >> 4, k = p & 15;
    const int hs = (t & 1) * BITS;
    uint32_t w = 0;
    if (BITS == 3 && k >= 12) {
        const int sh = 6 * (k - 12) + hs;  // bit of the 24-bit tail; byte sh / 8 is the top byte of dword sh / 8
        // a 3-bit code at tail bit sh may straddle two bytes: assemble the tail from the three top bytes
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const uint32_t tail = (row_dword(block, r0 + m, g) >> 24) | ((row_dword(block, r0 + m, 4 + g) >> 24) << 8) |
                                  ((row_dword(block, r0 + m, 8 + g) >> 24) << 16);
            w |= ((tail >> sh) & CM) << (m * BITS);
        }
    } else {
        const int dw = 4 * (k / tqd::pairs_per_dword(BITS)) + g;
        const int sh = 2 * BITS * (k % tqd::pairs_per_dword(BITS)) + hs;
#pragma unroll
        for (int m = 0; m < 8; ++m) w |= ((row_dword(block, r0 + m, dw) >> sh) & CM) << (m * BITS);
    }
    return w;
}

template <typename TO, int BITS>
__global__ __launch_bounds__(256) void k_load(const uint8_t *packed, TO *out, LoadArgs a) {
    __shared__ float cent_s[16];
    const int tid = threadIdx.x, lane = tid & 63;
    const int li = lane & 15, grp = tid >> 4;
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / a.blocks_per_seq, bis = blk % a.blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    // the block is copied into LDS with coalesced 16-byte loads; codes are picked from there
    constexpr int block_size = TQ_ROWS_PER_BLOCK * (16 * BITS + 2);
    __shared__ __attribute__((aligned(16))) uint8_t block_s[block_size];
    {
        const uint4 *src = reinterpret_cast<const uint4 *>(packed + blk * (int64_t)block_size);
        for (int e = tid; e < block_size / 16; e += 256) reinterpret_cast<uint4 *>(block_s)[e] = src[e];
    }
    const uint8_t *block = block_s;
    if (tid < (1 << BITS)) cent_s[tid] = a.cent[tid];
    float s1v[8], s2v[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        s1v[m] = a.s1[8 * li + m] * RSQRT128;
        s2v[m] = a.s2[8 * li + m];
    }
    __syncthreads();
#pragma unroll 1
    for (int it = 0; it < 8; ++it) {
        const int t = it * 16 + grp;
        const bool valid = tok0 + t < a.tokens;
        const float g = block_norm(block, BITS, t);
        const uint32_t codes = load_codes8<BITS>(block, a.kind, t, li);
        float v[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) v[m] = cent_s[(codes >> (m * BITS)) & ((1u << BITS) - 1u)] * g;
        if (a.domain == TQ_DOMAIN_ORIGINAL) {
#pragma unroll
            for (int m = 0; m < 8; ++m) v[m] *= s2v[m];
            wht128_row16(v, lane);
#pragma unroll
            for (int m = 0; m < 8; ++m) v[m] *= s1v[m];
        }
        if (valid) store8(out + ((seq * a.tokens + tok0 + t) * 128 + 8 * li), v);
    }
}

// ---- tq_load, K rows, fp16 output, original domain: the transposed rotation on the matrix cores ----------
// The mirror image of store_k_units: a lane quarter's BITS dwords of a row are one pair group = 32 consecutive
// rotated-domain values of one token, which is the B operand of the factored transform (fragments with s2
// folded in); the 32 results of the lane are 32 consecutive output dims.  The centroids enter as fp16 (the pair
// table), which the fp16 output's tolerance covers; fp32 and fp64 outputs keep the fp32 butterfly of k_load.
struct LoadK16Args {
    const uint4 *afrag;        // tq_handle::rfrag16k_inv
    const float *s1;
    const uint32_t *pair_lut;  // half2 per pair code
    int64_t tokens;
    uint32_t blocks_per_seq, n_units;  // unit = 16 tokens
    FastDiv bps_div;                   // division by blocks_per_seq
};

// byte offset (pair code * 4) of pair k = 0..15 of a group, from the group's dwords (3-bit: and its 24-bit tail)
template <int BITS> __device__ __forceinline__ uint32_t group_pair_offset(const uint32_t (&cw)[BITS], uint32_t tail, int k) {
    if constexpr (BITS == 4) return tqd::field_offset<2>(cw[k >> 2], 8 * (k & 3), 8);
    else if constexpr (BITS == 2) return tqd::field_offset<2>(cw[k >> 3], 4 * (k & 7), 4);
    else return k < 12 ? tqd::field_offset<2>(cw[k >> 2], 6 * (k & 3), 6) : tqd::field_offset<2>(tail, 6 * (k - 12), 6);
}

// 32 rotated-domain fp16 values of one token per lane (xb[ks] = values 8ks .. 8ks+7 of the lane quarter's 32)
// -> the lane's 32 output dims as fp16 pairs: eight MFMAs, the butterfly over the slices, norm / sqrt(128), s1
__device__ __forceinline__ void unrotate_unit16(const half8_t (&af)[8], const uint4 (&xb)[4], float g, const uint32_t (&smask)[16],
                                                uint32_t (&o)[16]) {
    float4_t q[2][4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int f0 = 0; f0 < 2; ++f0)
            q[f0][ks] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[f0 * 4 + ks], __builtin_bit_cast(half8_t, xb[ks]),
                                                               float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    // fragment 2*fh + f0 holds dims 32kc + 8fh + 4f0 + i
    float4_t y[8];
#pragma unroll
    for (int f0 = 0; f0 < 2; ++f0) {
        const float4_t s01 = q[f0][0] + q[f0][1], d01 = q[f0][0] - q[f0][1];
        const float4_t s23 = q[f0][2] + q[f0][3], d23 = q[f0][2] - q[f0][3];
        y[0 + f0] = s01 + s23;
        y[2 + f0] = d01 + d23;
        y[4 + f0] = s01 - s23;
        y[6 + f0] = d01 - d23;
    }
    const float gs = g * RSQRT128;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        const int v = 2 * w;
        const uint32_t lo = __half_as_ushort(__float2half_rn(y[v >> 2][v & 3] * gs));
        const uint32_t hi = __half_as_ushort(__float2half_rn(y[(v + 1) >> 2][(v + 1) & 3] * gs));
        o[w] = (lo | (hi << 16)) ^ smask[w];
    }
}

constexpr int LOAD16_XROW = 256 + 16;  // bytes per token row of the transposition space (padding spreads the banks)
constexpr int LOAD16_XPOSE_BYTES = 4 * 16 * LOAD16_XROW;

// Workgroup `bid` of `nb` running the K-row loop; the LDS arrays belong to the calling kernel
// (lut_s: 1 << 2 BITS dwords, frag_s: 512 uint4, s1_s: 128 floats, xpose_s: LOAD16_XPOSE_BYTES).
template <int BITS>
__device__ __forceinline__ void load_k16_body(const uint8_t *packed, __half *out, const LoadK16Args &a, uint32_t bid, uint32_t nb,
                                              uint32_t *lut_s, uint4 *frag_s, float *s1_s, uint8_t *xpose_s) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n16 = lane & 15, kc = lane >> 4;
    for (int e = tid; e < (1 << (2 * BITS)); e += 256) lut_s[e] = a.pair_lut[e];
    constexpr int XROW = LOAD16_XROW;
    frag_s[tid] = a.afrag[tid];
    frag_s[256 + tid] = a.afrag[256 + tid];
    if (tid < 128) s1_s[tid] = a.s1[tid];
    __syncthreads();
    uint32_t smask[16];  // sign bits of s1 for the lane's 32 output dims, two fp16 per dword
#pragma unroll
    for (int w = 0; w < 16; ++w)
        smask[w] = (s1_s[32 * kc + 2 * w] < 0.0f ? 0x8000u : 0u) | (s1_s[32 * kc + 2 * w + 1] < 0.0f ? 0x80000000u : 0u);
    half8_t af[8];
#pragma unroll
    for (int f = 0; f < 8; ++f) af[f] = __builtin_bit_cast(half8_t, frag_s[f * 64 + lane]);
    const char *lut = reinterpret_cast<const char *>(lut_s);
    const uint32_t bps = a.blocks_per_seq;
    // the next unit's codes and norm are requested before the current one is worked on (the last fetch re-reads)
    auto fetch = [&](uint32_t u, uint32_t (&cw)[BITS], __half &gh) {
        u = u < a.n_units ? u : a.n_units - 1;
        const uint8_t *block = packed + (int64_t)(u >> 3) * block_bytes(BITS);
        const int row = (int)(u & 7) * 16 + n16;
#pragma unroll
        for (int j = 0; j < BITS; ++j) cw[j] = *reinterpret_cast<const uint32_t *>(block + j * 2048 + row * 16 + kc * 4);
        gh = reinterpret_cast<const __half *>(block + block_code_bytes(BITS))[row];
    };
    uint32_t cw_next[BITS];
    __half g_next;
    fetch(bid * 4 + wave, cw_next, g_next);
#pragma unroll 1
    for (uint32_t u = bid * 4 + wave; u < a.n_units; u += nb * 4) {
        const uint32_t blk = u >> 3, seq = a.bps_div.div(blk), bis = blk - seq * bps;
        uint32_t cw[BITS];
#pragma unroll
        for (int j = 0; j < BITS; ++j) cw[j] = cw_next[j];
        const float g = __half2float(g_next);
        fetch(u + nb * 4, cw_next, g_next);
        uint32_t tail = 0;
        if constexpr (BITS == 3) tail = (cw[0] >> 24) | ((cw[1] >> 24) << 8) | ((cw[2] >> 24) << 16);
        uint4 xb[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            xb[ks].x = *reinterpret_cast<const uint32_t *>(lut + group_pair_offset<BITS>(cw, tail, 4 * ks));
            xb[ks].y = *reinterpret_cast<const uint32_t *>(lut + group_pair_offset<BITS>(cw, tail, 4 * ks + 1));
            xb[ks].z = *reinterpret_cast<const uint32_t *>(lut + group_pair_offset<BITS>(cw, tail, 4 * ks + 2));
            xb[ks].w = *reinterpret_cast<const uint32_t *>(lut + group_pair_offset<BITS>(cw, tail, 4 * ks + 3));
        }
        uint32_t o[16];
        unrotate_unit16(af, xb, g, smask, o);
        // through this wavefront's 4.25 KB of LDS, so that a store instruction writes four whole token rows
        // (1 KB of contiguous memory) instead of sixty-four 16-byte pieces
        uint8_t *mine = xpose_s + wave * (16 * XROW);
#pragma unroll
        for (int c = 0; c < 4; ++c)
            *reinterpret_cast<uint4 *>(mine + n16 * XROW + kc * 64 + c * 16) = make_uint4(o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]);
        const int64_t tok_base = (int64_t)bis * TQ_ROWS_PER_BLOCK + (int)(u & 7) * 16;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int tr = 4 * c + (lane >> 4);  // token of the unit this lane stores a piece of
            const uint4 piece = *reinterpret_cast<const uint4 *>(mine + tr * XROW + (lane & 15) * 16);
            if (tok_base + tr < a.tokens)
                stream_store<STREAM_LOAD_OUT>(reinterpret_cast<uint4 *>(out + (((int64_t)seq * a.tokens + tok_base + tr) * 128 + 8 * (lane & 15))), piece);
        }
    }
}

template <int BITS>
__global__ __launch_bounds__(256) void k_load_k16(const uint8_t *packed, __half *out, LoadK16Args a) {
    __shared__ uint32_t lut_s[1 << (2 * BITS)];
    __shared__ __attribute__((aligned(16))) uint4 frag_s[512];
    __shared__ float s1_s[128];
    __shared__ __attribute__((aligned(16))) uint8_t xpose_s[LOAD16_XPOSE_BYTES];
    load_k16_body<BITS>(packed, out, a, blockIdx.x, gridDim.x, lut_s, frag_s, s1_s, xpose_s);
}

// The same for V rows (dim-major inside a 64-token tile): the tile's codes are staged in LDS and a lane gathers the
// 32 codes of its token from 32 rows (same pair position in each).  Wavefront w takes tokens 16a + 4w + i of the
// tile (a, i = 0..3), so that the dword a pair sits in - and for 3-bit codes whether it sits in the split tail -
// is the same for the whole wavefront.  a.n_units counts 64-token tiles here.
// (cent_s: 16 fp16 bit patterns, tile_s: (BITS * 64 + 8) * 16 bytes; the others as for K rows)
template <int BITS>
__device__ __forceinline__ void load_v16_body(const uint8_t *packed, __half *out, const LoadK16Args &a, uint32_t bid, uint32_t nb,
                                              uint16_t *cent_s, uint4 *frag_s, float *s1_s, uint8_t *xpose_s, uint8_t *tile_s) {
    constexpr int XROW = LOAD16_XROW;
    constexpr int PIECES = BITS * 64 + 8;  // 16-byte pieces of a tile: codes [BITS][64 rows][16 B], then 64 fp16 norms
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n16 = lane & 15, kc = lane >> 4;
    if (tid < (1 << BITS)) cent_s[tid] = (uint16_t)(a.pair_lut[tid] & 0xffffu);  // pair (lo = code, hi = 0): low half = c[code]
    frag_s[tid] = a.afrag[tid];
    frag_s[256 + tid] = a.afrag[256 + tid];
    if (tid < 128) s1_s[tid] = a.s1[tid];
    __syncthreads();
    uint32_t smask[16];
#pragma unroll
    for (int w = 0; w < 16; ++w)
        smask[w] = (s1_s[32 * kc + 2 * w] < 0.0f ? 0x8000u : 0u) | (s1_s[32 * kc + 2 * w + 1] < 0.0f ? 0x80000000u : 0u);
    half8_t af[8];
#pragma unroll
    for (int f = 0; f < 8; ++f) af[f] = __builtin_bit_cast(half8_t, frag_s[f * 64 + lane]);
    const uint32_t bps = a.blocks_per_seq;
    // this lane's token inside the tile and where its codes sit in a row
    const int tl = 16 * (n16 >> 2) + 4 * wave + (n16 & 3);
    const int hf = kc >> 1, r0 = 32 * (kc & 1);
    const int p = ((tl & 60) | (hf << 1)) | ((tl >> 1) & 1);
    const int grp = p >> 4, k = p & 15;  // k / pairs per dword depends on the wavefront only
    const int hs = (tl & 1) * BITS;
    constexpr uint32_t CM = (1u << BITS) - 1u;
    static_assert(PIECES <= 512, "two pieces per thread at most");
    uint4 pre0, pre1;  // pieces tid and tid + 256 of the next tile
    auto fetch_tile = [&](uint32_t tile) {
        tile = tile < a.n_units ? tile : a.n_units - 1;
        const uint8_t *block = packed + (int64_t)(tile >> 1) * block_bytes(BITS);
        const int half = (int)(tile & 1);
        auto piece = [&](int e) {
            e = min(e, PIECES - 1);
            const uint8_t *src = e < BITS * 64 ? block + (e >> 6) * 2048 + (64 * half + (e & 63)) * 16
                                               : block + block_code_bytes(BITS) + 128 * half + (e - BITS * 64) * 16;
            return *reinterpret_cast<const uint4 *>(src);
        };
        pre0 = piece(tid);
        if constexpr (PIECES > 256) pre1 = piece(tid + 256);
    };
    fetch_tile(bid);
#pragma unroll 1
    for (uint32_t tile = bid; tile < a.n_units; tile += nb) {
        const uint32_t blk = tile >> 1, half = tile & 1, seq = a.bps_div.div(blk), bis = blk - seq * bps;
        __syncthreads();  // the previous tile's codes are no longer needed
        if (tid < PIECES) reinterpret_cast<uint4 *>(tile_s)[tid] = pre0;
        if constexpr (PIECES > 256) {
            if (tid + 256 < PIECES) reinterpret_cast<uint4 *>(tile_s)[tid + 256] = pre1;
        }
        __syncthreads();
        fetch_tile(tile + nb);  // the next tile's pieces travel while this one is worked on
        const float g = __half2float(reinterpret_cast<const __half *>(tile_s + BITS * 1024)[tl]);
        uint32_t hv[32];  // fp16 bits of the lane's 32 values
        if (BITS == 3 && wave == 3) {
            const int sh = 6 * (k - 12) + hs;
#pragma unroll
            for (int v = 0; v < 32; ++v) {
                const uint8_t *rowp = tile_s + (r0 + v) * 16 + grp * 4;
                const uint32_t tail = (*reinterpret_cast<const uint32_t *>(rowp) >> 24) |
                                      ((*reinterpret_cast<const uint32_t *>(rowp + 1024) >> 24) << 8) |
                                      ((*reinterpret_cast<const uint32_t *>(rowp + 2048) >> 24) << 16);
                hv[v] = cent_s[(tail >> sh) & CM];
            }
        } else {
            const int dw = k / tqd::pairs_per_dword(BITS);
            const int sh = 2 * BITS * (k % tqd::pairs_per_dword(BITS)) + hs;
            const uint8_t *col = tile_s + dw * 1024 + grp * 4;
#pragma unroll
            for (int v = 0; v < 32; ++v) hv[v] = cent_s[(*reinterpret_cast<const uint32_t *>(col + (r0 + v) * 16) >> sh) & CM];
        }
        uint4 xb[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            xb[ks].x = hv[8 * ks] | (hv[8 * ks + 1] << 16);
            xb[ks].y = hv[8 * ks + 2] | (hv[8 * ks + 3] << 16);
            xb[ks].z = hv[8 * ks + 4] | (hv[8 * ks + 5] << 16);
            xb[ks].w = hv[8 * ks + 6] | (hv[8 * ks + 7] << 16);
        }
        uint32_t o[16];
        unrotate_unit16(af, xb, g, smask, o);
        uint8_t *mine = xpose_s + wave * (16 * XROW);
#pragma unroll
        for (int c = 0; c < 4; ++c)
            *reinterpret_cast<uint4 *>(mine + n16 * XROW + kc * 64 + c * 16) = make_uint4(o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]);
        const int64_t tok_base = (int64_t)bis * TQ_ROWS_PER_BLOCK + 64 * half;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            // row 4c + lane/16 of the wavefront's space is token 16c + 4 wave + lane/16 of the tile
            const int tr = 4 * c + (lane >> 4);
            const int64_t tok = tok_base + 16 * c + 4 * wave + (lane >> 4);
            const uint4 piece = *reinterpret_cast<const uint4 *>(mine + tr * XROW + (lane & 15) * 16);
            if (tok < a.tokens)
                stream_store<STREAM_LOAD_OUT>(reinterpret_cast<uint4 *>(out + (((int64_t)seq * a.tokens + tok) * 128 + 8 * (lane & 15))), piece);
        }
    }
}

template <int BITS>
__global__ __launch_bounds__(256) void k_load_v16(const uint8_t *packed, __half *out, LoadK16Args a) {
    __shared__ uint16_t cent_s[16];
    __shared__ __attribute__((aligned(16))) uint4 frag_s[512];
    __shared__ float s1_s[128];
    __shared__ __attribute__((aligned(16))) uint8_t xpose_s[LOAD16_XPOSE_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t tile_s[(BITS * 64 + 8) * 16];
    load_v16_body<BITS>(packed, out, a, blockIdx.x, gridDim.x, cent_s, frag_s, s1_s, xpose_s, tile_s);
}

// K and V of a layer in one launch.  The V tiles and the K turns (four 16-token units, one per wavefront) form one
// sequence of 64-token turns, V first, dealt round-robin to the workgroups: each runs the V-tile loop over its
// tiles and then the K-row loop from its first K turn on, reloading the tables in between (the handles may differ).
template <int KB, int VB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_load_kv16(const uint8_t *packed_k, __half *out_k, LoadK16Args ak, const uint8_t *packed_v,
                                                   __half *out_v, LoadK16Args av) {
    constexpr int TILE_V = (VB * 64 + 8) * 16, AUX_K = 4 << (2 * KB), AUX_V = TILE_V + 32;
    __shared__ __attribute__((aligned(16))) uint4 frag_s[512];
    __shared__ float s1_s[128];
    __shared__ __attribute__((aligned(16))) uint8_t xpose_s[LOAD16_XPOSE_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t aux_s[AUX_K > AUX_V ? AUX_K : AUX_V];
    const uint32_t bid = blockIdx.x, nb = gridDim.x, v_turns = av.n_units;
    if (bid < v_turns) load_v16_body<VB>(packed_v, out_v, av, bid, nb, reinterpret_cast<uint16_t *>(aux_s + TILE_V), frag_s, s1_s, xpose_s, aux_s);
    __syncthreads();  // every wavefront is done with the V tables and tiles
    const uint32_t first = bid >= v_turns ? bid : bid + (v_turns - bid + nb - 1) / nb * nb;  // this workgroup's first turn past V
    load_k16_body<KB>(packed_k, out_k, ak, first - v_turns, nb, reinterpret_cast<uint32_t *>(aux_s), frag_s, s1_s, xpose_s);
}

__global__ __launch_bounds__(256) void k_unpack_codes(const uint8_t *packed, uint8_t *idx, float *norms, int bits,
                                                      int kind, int64_t tokens, int64_t blocks_per_seq) {
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    const uint8_t *block = packed + blk * (int64_t)(TQ_ROWS_PER_BLOCK * (16 * bits + 2));
    for (int e = threadIdx.x; e < TQ_ROWS_PER_BLOCK * 128; e += 256) {
        const int t = e >> 7, dim = e & 127;
        if (tok0 + t >= tokens) continue;
        idx[(seq * tokens + tok0 + t) * 128 + dim] = (uint8_t)fetch_code(block, bits, kind, t, dim);
    }
    if (threadIdx.x < TQ_ROWS_PER_BLOCK && tok0 + threadIdx.x < tokens)
        norms[seq * tokens + tok0 + threadIdx.x] = block_norm(block, bits, threadIdx.x);
}

// ---- q8_0-style K blocks ------------------------------------------------------------
// Block of 128 tokens: [8 chunks][128 rows][16 B] int8 followed by [128][4] fp16 scales.
// One thread per 32-value group: scale = max|x| / 127, q = roundf(x / scale) (ggml).
template <typename TI>
__global__ __launch_bounds__(256) void k_q8_0_store(const TI *x, uint8_t *packed, int64_t tokens, int64_t blocks_per_seq) {
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    uint8_t *block = packed + blk * (int64_t)(TQ_ROWS_PER_BLOCK * 136);
    for (int u = threadIdx.x; u < TQ_ROWS_PER_BLOCK * 4; u += 256) {
        const int t = u >> 2, gq = u & 3;
        const bool valid = tok0 + t < tokens;
        float v[32];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            v[j] = valid ? ld1(x + (seq * tokens + tok0 + t) * 128 + gq * 32 + j) : 0.0f;
            amax = fmaxf(amax, fabsf(v[j]));
        }
        const float d = amax / 127.0f;
        const float id = d > 0.0f ? 1.0f / d : 0.0f;
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = 0;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const float tq = v[j] * id;
            const int qv = (int)roundf(tq);
            w[j >> 2] |= ((uint32_t)(qv & 0xFF)) << (8 * (j & 3));
        }
        // 32 values = two 16-byte chunks (2*gq, 2*gq+1) of row t
        *reinterpret_cast<uint4 *>(block + (2 * gq) * 2048 + t * 16) = make_uint4(w[0], w[1], w[2], w[3]);
        *reinterpret_cast<uint4 *>(block + (2 * gq + 1) * 2048 + t * 16) = make_uint4(w[4], w[5], w[6], w[7]);
        reinterpret_cast<__half *>(block + 8 * 2048)[t * 4 + gq] = __float2half_rn(d);
    }
}

// fp16 input: the block's 32 KB are read as 16-byte pieces that are contiguous across the lanes (four lanes
// per 32-value group, whose maximum takes two lane exchanges), the block image is put together in LDS and
// leaves as one contiguous copy.  Same arithmetic as k_q8_0_store: q = sign(t) floor(|t| + 0.5), t = x / scale.
constexpr int Q8_LDS_CHUNK = 2048 + 16;  // chunk stride of the LDS image (padding spreads the 8-byte writes over the banks)
__global__ __launch_bounds__(256) void k_q8_0_store_f16(const __half *x, uint8_t *packed, int64_t tokens, int64_t blocks_per_seq) {
    __shared__ __attribute__((aligned(16))) uint8_t img[8 * Q8_LDS_CHUNK + TQ_ROWS_PER_BLOCK * 8];
    const int tid = threadIdx.x;
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    const int rows_here = (int)min((int64_t)TQ_ROWS_PER_BLOCK, tokens - tok0);
    const uint4 *src = reinterpret_cast<const uint4 *>(x + (seq * tokens + tok0) * 128);
    uint4 v[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int i = tid + 256 * r;  // 16-byte piece of the block: row i / 16, values 8 (i % 16) .. + 7
        v[r] = (i >> 4) < rows_here ? src[i] : make_uint4(0, 0, 0, 0);
    }
    __half *scales = reinterpret_cast<__half *>(img + 8 * Q8_LDS_CHUNK);
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int i = tid + 256 * r, row = i >> 4, c8 = i & 15;
        const uint32_t u[4] = {v[r].x, v[r].y, v[r].z, v[r].w};
        float f[8];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = __half2float(__ushort_as_half((unsigned short)(u[j] & 0xffffu)));
            f[2 * j + 1] = __half2float(__ushort_as_half((unsigned short)(u[j] >> 16)));
            amax = fmaxf(amax, fmaxf(fabsf(f[2 * j]), fabsf(f[2 * j + 1])));
        }
        amax = fmaxf(amax, xor_lane<1>(amax));
        amax = fmaxf(amax, xor_lane<2>(amax));
        const float d = amax / 127.0f;
        const float id = d > 0.0f ? 1.0f / d : 0.0f;
        uint32_t w[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float t = f[j] * id;
            const int qv = (int)roundf(t);
            w[j >> 2] |= ((uint32_t)(qv & 0xFF)) << (8 * (j & 3));
        }
        *reinterpret_cast<uint2 *>(img + (c8 >> 1) * Q8_LDS_CHUNK + row * 16 + (c8 & 1) * 8) = make_uint2(w[0], w[1]);
        if ((c8 & 3) == 0) scales[row * 4 + (c8 >> 2)] = __float2half_rn(d);
    }
    __syncthreads();
    uint4 *dst = reinterpret_cast<uint4 *>(packed + blk * (int64_t)(TQ_ROWS_PER_BLOCK * 136));
    for (int i = tid; i < TQ_ROWS_PER_BLOCK * 136 / 16; i += 256) {
        const int c = i >> 7;  // chunks 0..7 of 128 pieces each, then the scales
        stream_store<STREAM_Q8>(dst + i, *reinterpret_cast<const uint4 *>(c < 8 ? img + c * Q8_LDS_CHUNK + (i & 127) * 16 : img + 8 * Q8_LDS_CHUNK + (i - 1024) * 16));
    }
}

// q8_0-style V blocks: the same 32-value groups and arithmetic, laid out as the decode kernel reads V rows.
// Byte of (token t of the block, dim): 16-byte chunk 4 * (dim / 64) + (t % 64) / 16 of row 64 * (t / 64) + dim % 64,
// byte t % 16; scale of (t, 32-dim group gq): fp16 [t / 64][gq][t % 64] behind the values.
__device__ __forceinline__ int q8v_byte(int t, int dim) {
    return (4 * (dim >> 6) + ((t & 63) >> 4)) * 2048 + (64 * (t >> 6) + (dim & 63)) * 16 + (t & 15);
}
__device__ __forceinline__ int q8v_scale(int t, int gq) { return ((t >> 6) * 4 + gq) * 64 + (t & 63); }

// One thread per 32-value group; the block image is put together in LDS and leaves as one contiguous copy, with
// zeros at the positions past the sequence's end.
template <typename TI>
__global__ __launch_bounds__(256) void k_q8_0_store_v(const TI *x, uint8_t *packed, int64_t tokens, int64_t blocks_per_seq) {
    __shared__ __attribute__((aligned(16))) uint8_t img[TQ_ROWS_PER_BLOCK * 136];
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    for (int u = threadIdx.x; u < TQ_ROWS_PER_BLOCK * 4; u += 256) {
        // consecutive threads take consecutive tokens of one group, so their bytes share LDS words rarely
        const int t = u & 127, gq = u >> 7;
        const bool valid = tok0 + t < tokens;
        float v[32];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            v[j] = valid ? ld1(x + (seq * tokens + tok0 + t) * 128 + gq * 32 + j) : 0.0f;
            amax = fmaxf(amax, fabsf(v[j]));
        }
        const float d = amax / 127.0f;
        const float id = d > 0.0f ? 1.0f / d : 0.0f;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const float tq = v[j] * id;
            const int qv = (int)roundf(tq);
            img[q8v_byte(t, gq * 32 + j)] = (uint8_t)(qv & 0xFF);
        }
        reinterpret_cast<__half *>(img + 8 * 2048)[q8v_scale(t, gq)] = __float2half_rn(d);
    }
    __syncthreads();
    uint4 *dst = reinterpret_cast<uint4 *>(packed + blk * (int64_t)(TQ_ROWS_PER_BLOCK * 136));
    for (int i = threadIdx.x; i < TQ_ROWS_PER_BLOCK * 136 / 16; i += 256) stream_store<STREAM_Q8>(dst + i, reinterpret_cast<const uint4 *>(img)[i]);
}

// fp16 input, 16-byte aligned: the block's 32 KB come in as 16-byte pieces that are contiguous across the lanes and
// are parked in LDS in token order; one thread per 32-value group finds the scale; then one thread per (dim, 16
// tokens) reads its column, quantises and stores one 16-byte chunk, so that 64 lanes write 1 KB in one piece.
// Same arithmetic as k_q8_0_store_v.
constexpr int Q8V_ROW = 256 + 16;  // LDS bytes per token: the padding spreads the 16-byte row reads over the banks
__global__ __launch_bounds__(256) void k_q8_0_store_v_f16(const __half *x, uint8_t *packed, int64_t tokens, int64_t blocks_per_seq) {
    __shared__ __attribute__((aligned(16))) uint8_t raw[TQ_ROWS_PER_BLOCK * Q8V_ROW];
    __shared__ float inv[TQ_ROWS_PER_BLOCK * 4];
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    uint8_t *block = packed + blk * (int64_t)(TQ_ROWS_PER_BLOCK * 136);
    const int n_valid = (int)min((int64_t)TQ_ROWS_PER_BLOCK, tokens - tok0);
    const uint4 *src = reinterpret_cast<const uint4 *>(x + (seq * tokens + tok0) * 128);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int i = threadIdx.x + 256 * k, t = i >> 4;
        const uint4 v = t < n_valid ? src[i] : make_uint4(0u, 0u, 0u, 0u);
        *reinterpret_cast<uint4 *>(raw + t * Q8V_ROW + (i & 15) * 16) = v;
    }
    __syncthreads();
    __half *scales = reinterpret_cast<__half *>(block + 8 * 2048);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int u = threadIdx.x + 256 * k, t = u >> 2, gq = u & 3;
        float amax = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint4 v = *reinterpret_cast<const uint4 *>(raw + t * Q8V_ROW + gq * 64 + c * 16);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                amax = fmaxf(amax, fabsf(__half2float(__ushort_as_half((unsigned short)(w[e] & 0xffff)))));
                amax = fmaxf(amax, fabsf(__half2float(__ushort_as_half((unsigned short)(w[e] >> 16)))));
            }
        }
        const float d = amax / 127.0f;
        inv[u] = d > 0.0f ? 1.0f / d : 0.0f;
        scales[q8v_scale(t, gq)] = __float2half_rn(d);
    }
    __syncthreads();
    // unit = (16-token group c16 of the block, dim): lanes along dim % 64, so a wavefront stores 64 consecutive rows
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int u = threadIdx.x + 256 * k;
        const int l = u & 63, hf = (u >> 6) & 1, c16 = u >> 7;  // c16 = 0..7: tile c16 / 4, tokens 16 * (c16 % 4) ..
        const int dim = 64 * hf + l, gq = dim >> 5;
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int t = 16 * c16 + e;
            const float v = __half2float(*reinterpret_cast<const __half *>(raw + t * Q8V_ROW + 2 * dim));
            const float tq = v * inv[t * 4 + gq];
            const int qv = (int)roundf(tq);
            w[e >> 2] |= ((uint32_t)(qv & 0xFF)) << (8 * (e & 3));
        }
        *reinterpret_cast<uint4 *>(block + (4 * hf + (c16 & 3)) * 2048 + (64 * (c16 >> 2) + l) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// Streaming append for both layouts: one workgroup per (sequence, touched block).  Tokens before `pos` stay, the
// n_new tokens from `pos` on are quantised from x [n_seqs, n_new, 128], and the rest of the last touched block
// becomes zeros (what the store kernels write past a sequence's end).  Bytes of neighbouring tokens share words in
// the V layout; byte stores keep them apart.
template <typename TI, int KIND>
__global__ __launch_bounds__(256) void k_q8_0_append(const TI *x, uint8_t *packed, int64_t pos, int64_t n_new,
                                                     int64_t blocks_per_seq, int64_t first_block, int64_t n_touched,
                                                     const int64_t *pos_dev, int64_t capacity, uint32_t *overrun) {
    if (pos_dev) {  // the position is read when the launch runs (see resolve_append)
        pos = *pos_dev;
        if (!append_position_ok(pos, n_new, capacity, overrun, blockIdx.x == 0)) return;
        first_block = pos / TQ_ROWS_PER_BLOCK;
        if ((int64_t)(blockIdx.x % n_touched) >= (pos + n_new - 1) / TQ_ROWS_PER_BLOCK - first_block + 1) return;
    }
    const int64_t seq = blockIdx.x / n_touched, bis = first_block + blockIdx.x % n_touched;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    uint8_t *block = packed + (seq * blocks_per_seq + bis) * (int64_t)(TQ_ROWS_PER_BLOCK * 136);
    __half *scales = reinterpret_cast<__half *>(block + 8 * 2048);
    for (int u = threadIdx.x; u < TQ_ROWS_PER_BLOCK * 4; u += 256) {
        const int t = KIND == TQ_KIND_V ? u & 127 : u >> 2, gq = KIND == TQ_KIND_V ? u >> 7 : u & 3;
        const int64_t tok = tok0 + t;
        if (tok < pos) continue;
        const bool valid = tok < pos + n_new;
        float v[32];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            v[j] = valid ? ld1(x + (seq * n_new + (tok - pos)) * 128 + gq * 32 + j) : 0.0f;
            amax = fmaxf(amax, fabsf(v[j]));
        }
        const float d = amax / 127.0f;
        const float id = d > 0.0f ? 1.0f / d : 0.0f;
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = 0;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const float tq = v[j] * id;
            const int qv = (int)roundf(tq);
            if constexpr (KIND == TQ_KIND_V) block[q8v_byte(t, gq * 32 + j)] = (uint8_t)(qv & 0xFF);
            else w[j >> 2] |= ((uint32_t)(qv & 0xFF)) << (8 * (j & 3));
        }
        if constexpr (KIND == TQ_KIND_V) {
            scales[q8v_scale(t, gq)] = __float2half_rn(d);
        } else {
            *reinterpret_cast<uint4 *>(block + (2 * gq) * 2048 + t * 16) = make_uint4(w[0], w[1], w[2], w[3]);
            *reinterpret_cast<uint4 *>(block + (2 * gq + 1) * 2048 + t * 16) = make_uint4(w[4], w[5], w[6], w[7]);
            scales[t * 4 + gq] = __float2half_rn(d);
        }
    }
}

__global__ __launch_bounds__(256) void k_q8_0_unpack(const uint8_t *packed, int8_t *q, float *scales, int64_t tokens,
                                                     int64_t blocks_per_seq, int kind) {
    const int64_t blk = blockIdx.x;
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    const uint8_t *block = packed + blk * (int64_t)(TQ_ROWS_PER_BLOCK * 136);
    for (int e = threadIdx.x; e < TQ_ROWS_PER_BLOCK * 128; e += 256) {
        const int t = e >> 7, dim = e & 127;
        if (tok0 + t >= tokens) continue;
        q[(seq * tokens + tok0 + t) * 128 + dim] =
            (int8_t)block[kind == TQ_KIND_V ? q8v_byte(t, dim) : (dim >> 4) * 2048 + t * 16 + (dim & 15)];
    }
    for (int e = threadIdx.x; e < TQ_ROWS_PER_BLOCK * 4; e += 256) {
        const int t = e >> 2;
        if (tok0 + t >= tokens) continue;
        scales[(seq * tokens + tok0 + t) * 4 + (e & 3)] =
            __half2float(reinterpret_cast<const __half *>(block + 8 * 2048)[kind == TQ_KIND_V ? q8v_scale(t, e & 3) : e]);
    }
}

#define DISPATCH_T(dt, NAME, F)                      \
    switch (dt) {                                    \
    case TQ_F16: { using NAME = __half; F; } break;  \
    case TQ_F32: { using NAME = float; F; } break;   \
    case TQ_F64: { using NAME = double; F; } break;  \
    default: tq_set_error("bad dtype %d", dt); return TQ_ERR_ARG; }

inline int64_t blocks_for(int64_t tokens) { return (tokens + TQ_ROWS_PER_BLOCK - 1) / TQ_ROWS_PER_BLOCK; }

template <typename TI>
int launch_wht128(const void *x, void *y, int64_t n, int out_dtype, const float *sa, const float *sb, hipStream_t s) {
    const unsigned grid = (unsigned)((n + 3) / 4 < 8192 ? (n + 3) / 4 : 8192);
    DISPATCH_T(out_dtype, TO, (k_wht128<TI, TO><<<grid, 256, 0, s>>>((const TI *)x, (TO *)y, n, sa, sb)));
    return tq_check_launch("wht128");
}

}  // namespace

int tqk_rotate128(const tq_handle *h, const void *x, void *y, int64_t n, int in_dtype, int out_dtype, int transpose,
                  hipStream_t s) {
    const float *sa = transpose ? h->s2_32 : h->s1_32;
    const float *sb = transpose ? h->s1_32 : h->s2_32;
    if (n == 0) return TQ_OK;
    DISPATCH_T(in_dtype, TI, return launch_wht128<TI>(x, y, n, out_dtype, sa, sb, s));
}

// fp16 input with a sign-symmetric codebook: rotation on the matrix cores, codes packed in
// registers.  The butterfly kernel serves every other case (fp32 / fp64 input, asymmetric codebooks).
static bool store_fast_ok(const tq_handle *h, int in_dtype, int64_t n_blocks) {
    return (in_dtype == TQ_F16 || in_dtype == TQ_F32) && h->symmetric && h->bits >= 2 && h->bits <= 4 &&
           (h->bits != 4 || h->quant_lut_ok) && n_blocks < (1ll << 28);
}

#ifdef TQ_TIMELINE
extern "C" int tq_dbg_read_timeline(void *host, long long bytes) { return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(g_tl), (size_t)bytes); }
#endif

static StoreKArgs make_k_args(const tq_handle *h, int64_t tokens, int64_t bps, int64_t n_blocks) {
    StoreKArgs ka;
    ka.afrag = (const uint4 *)h->rfrag16k; ka.s2flip = h->s2flip; ka.symthr = h->symthr32; ka.sqcoef = h->sqcoef32;
    ka.quant_lut = h->quant_lut;
    ka.norm_correction = h->norm_correction; ka.tokens = tokens;
    ka.blocks_per_seq = (uint32_t)bps; ka.bps_div = make_fast_div((uint32_t)bps); ka.n_units = (uint32_t)(n_blocks * 8);
    ka.out_blocks_per_seq = (uint32_t)bps;
    for (int i = 0; i < 4; ++i) ka.s1neg[i] = h->s1neg_host[i];
    for (int i = 0; i < 16; ++i) ka.flipw[i] = h->s2flip_host[i];
    for (int i = 0; i < 8; ++i) { ka.thr[i] = h->symthr_host[i]; ka.coef[i] = h->sqcoef_host[i]; }
    return ka;
}

static StoreVArgs make_v_args(const tq_handle *h, int64_t tokens, int64_t bps, int64_t n_blocks) {
    StoreVArgs va;
    va.bfrag = (const uint4 *)h->rfrag16v; va.s2 = h->s2_32; va.symthr = h->symthr32; va.sqcoef = h->sqcoef32;
    va.quant_lut = h->quant_lut;
    va.norm_correction = h->norm_correction; va.tokens = tokens; va.share_k_lut = 0;
    va.blocks_per_seq = (uint32_t)bps; va.bps_div = make_fast_div((uint32_t)bps); va.n_units = (uint32_t)(n_blocks * 2);
    va.out_blocks_per_seq = (uint32_t)bps;
    for (int i = 0; i < 4; ++i) { va.s1neg[i] = h->s1neg_host[i]; va.s2neg[i] = h->s2neg_host[i]; }
    for (int i = 0; i < 8; ++i) { va.thr[i] = h->symthr_host[i]; va.coef[i] = h->sqcoef_host[i]; }
    return va;
}

// Workgroups of `kernel` (256 threads, static LDS only) that fit on the device at once: the persistent loops
// below are launched with exactly that many, so that no workgroup waits for another one to finish.
template <typename K> static unsigned resident_workgroups(K kernel) {
    int per_cu = 0, dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || per_cu < 1)
        return 256u * 2u;
    return (unsigned)prop.multiProcessorCount * (unsigned)per_cu;
}

// single-tensor launches of the matrix-core store (fp16 or fp32 rows): as many workgroups of four wavefronts as are
// resident at once (registers and LDS decide: 2 to 4 per CU)
static int launch_store_k(const tq_handle *h, const void *x, int in_dtype, void *packed, const StoreKArgs &ka, bool ragged, hipStream_t s) {
    const unsigned kneed = (unsigned)((ka.n_units + 3) / 4);
#define TQ_STORE_K_T(B, T)                                                                              \
    {                                                                                                   \
        static const unsigned fit[2] = {resident_workgroups(k_store_k<B, false, T>), resident_workgroups(k_store_k<B, true, T>)}; \
        const unsigned kgrid = kneed < fit[ragged] ? kneed : fit[ragged];                               \
        if (ragged) k_store_k<B, true, T><<<kgrid, 256, 0, s>>>((const T *)x, (uint8_t *)packed, ka);     \
        else k_store_k<B, false, T><<<kgrid, 256, 0, s>>>((const T *)x, (uint8_t *)packed, ka);           \
    }
#define TQ_STORE_K(B)                                \
    if (in_dtype == TQ_F32) TQ_STORE_K_T(B, float)   \
    else TQ_STORE_K_T(B, __half)
    switch (h->bits) {
    case 2: TQ_STORE_K(2); break;
    case 3: TQ_STORE_K(3); break;
    default: TQ_STORE_K(4); break;
    }
#undef TQ_STORE_K
#undef TQ_STORE_K_T
    return tq_check_launch("store_k");
}

static int launch_store_v(const tq_handle *h, const void *x, int in_dtype, void *packed, const StoreVArgs &va, bool ragged, hipStream_t s) {
    const unsigned vneed = (unsigned)((va.n_units + 3) / 4);
#define TQ_STORE_V_T(B, T)                                                                              \
    {                                                                                                   \
        static const unsigned fit[2] = {resident_workgroups(k_store_v<B, false, T>), resident_workgroups(k_store_v<B, true, T>)}; \
        const unsigned vgrid = vneed < fit[ragged] ? vneed : fit[ragged];                               \
        if (ragged) k_store_v<B, true, T><<<vgrid, 256, 0, s>>>((const T *)x, (uint8_t *)packed, va);     \
        else k_store_v<B, false, T><<<vgrid, 256, 0, s>>>((const T *)x, (uint8_t *)packed, va);           \
    }
#define TQ_STORE_V(B)                                \
    if (in_dtype == TQ_F32) TQ_STORE_V_T(B, float)   \
    else TQ_STORE_V_T(B, __half)
    switch (h->bits) {
    case 2: TQ_STORE_V(2); break;
    case 3: TQ_STORE_V(3); break;
    default: TQ_STORE_V(4); break;
    }
#undef TQ_STORE_V
#undef TQ_STORE_V_T
    return tq_check_launch("store_v");
}

constexpr int64_t SINGLE_VIA_FUSED_BLOCKS = 512;  // 65 536 vectors
int tqk_store(const tq_handle *h, const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, int kind, void *packed,
              uint8_t *sign_bits, void *rnorms, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    if (sign_bits) {
        if (!h->has_proj || !h->projrot64_t || !h->qjl_frag) {
            tq_set_error("tq_store_qjl: handle has no projection");
            return TQ_ERR_ARG;
        }
        StoreQjlArgs a;
        a.s1 = h->s1_64; a.s2 = h->s2_64; a.bounds = h->bounds64; a.cent = h->centroids64;
        a.projrot_t = h->projrot64_t;
        a.frag = reinterpret_cast<const uint4 *>(h->qjl_frag);
        a.tau = h->qjl_tau;
        a.tau2 = h->qjl_tau2;
        a.norm_correction = h->norm_correction;
        a.tokens = tokens; a.blocks_per_seq = bps;
        constexpr int MAT_BYTES = 3 * 4 * 8 * 64 * 16 + 8 * 128 * 8;  // the operands and, per wavefront, one token's residual
        const unsigned qgrid = grid < 256u ? grid : 256u;  // one workgroup per CU (the matrix fills its LDS), looping over blocks
#define TQ_STOREQ_BITS(B)                                                                                          \
    DISPATCH_T(in_dtype, TI,                                                                                       \
               ((void)hipFuncSetAttribute((const void *)k_store_qjl_mfma<B, TI>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                          MAT_BYTES),                                                              \
                k_store_qjl_mfma<B, TI><<<qgrid, 512, MAT_BYTES, s>>>((const TI *)x, (uint8_t *)packed, sign_bits,  \
                                                                      (__half *)rnorms, a, (int64_t)grid)))
        switch (h->bits) {
        case 2: TQ_STOREQ_BITS(2); break;
        case 3: TQ_STOREQ_BITS(3); break;
        case 4: TQ_STOREQ_BITS(4); break;
        default: tq_set_error("tq_store_qjl: bits must be 2, 3 or 4 (got %d)", h->bits); return TQ_ERR_UNSUPPORTED;
        }
#undef TQ_STOREQ_BITS
        return tq_check_launch("store_qjl");
    }
    if (store_fast_ok(h, in_dtype, n_seqs * bps)) {
        const int64_t n_blocks = n_seqs * bps;
        const bool ragged = tokens != bps * TQ_ROWS_PER_BLOCK;
        if (kind == TQ_KIND_V && n_blocks >= SINGLE_VIA_FUSED_BLOCKS && in_dtype == TQ_F16) {
            // A large V tensor: the K+V kernel with an empty K share (one workgroup of twelve wavefronts per CU drawing
            // tiles from a queue) is faster than k_store_v - 262 144 vectors: 20.9 against 21.9 us (3-bit), 22.4
            // against 23.3 us (4-bit), 18.2 against 19.1 us (2-bit).  K tensors are slower that way (17.7 against
            // 16.6 us, 20.8 against 17.8 us with the 64 KB table) and keep k_store_k.
            StoreKArgs ka = make_k_args(h, tokens, bps, n_blocks);
            StoreVArgs va = make_v_args(h, tokens, bps, n_blocks);
            va.share_k_lut = 1;
            const uint32_t units12 = (va.n_units + 11) / 12;
            ka.n_units = 0;
            const unsigned grid = units12 < 256u ? units12 : 256u;
#define TQ_ONE(B)                                                                                                                  \
    if (ragged) k_store_kv<B, B, true><<<grid, 768, 0, s>>>((const __half *)x, (const __half *)x, va.n_units, ka.n_units, (uint8_t *)packed, (uint8_t *)packed, ka, va); \
    else k_store_kv<B, B, false><<<grid, 768, 0, s>>>((const __half *)x, (const __half *)x, va.n_units, ka.n_units, (uint8_t *)packed, (uint8_t *)packed, ka, va)
            switch (h->bits) {
            case 2: TQ_ONE(2); break;
            case 3: TQ_ONE(3); break;
            default: TQ_ONE(4); break;
            }
#undef TQ_ONE
            return tq_check_launch("store_v (through the K+V kernel)");
        }
        if (kind == TQ_KIND_K) return launch_store_k(h, x, in_dtype, packed, make_k_args(h, tokens, bps, n_blocks), ragged, s);
        return launch_store_v(h, x, in_dtype, packed, make_v_args(h, tokens, bps, n_blocks), ragged, s);
    }
    StoreArgs a;
    a.s1 = h->s1_32; a.s2 = h->s2_32; a.bounds = h->bounds32; a.cent = h->centroids32;
    a.kind = kind; a.norm_correction = h->norm_correction;
    a.tokens = tokens; a.blocks_per_seq = bps;
#define TQ_STORE_BITS(B) \
    DISPATCH_T(in_dtype, TI, (k_store<B, TI><<<grid, 256, 0, s>>>((const TI *)x, (uint8_t *)packed, a)))
    switch (h->bits) {
    case 2: TQ_STORE_BITS(2); break;
    case 3: TQ_STORE_BITS(3); break;
    case 4: TQ_STORE_BITS(4); break;
    default: tq_set_error("tq_store: bits must be 2, 3 or 4 (got %d)", h->bits); return TQ_ERR_UNSUPPORTED;
    }
#undef TQ_STORE_BITS
    return tq_check_launch("store");
}

// ---- temporal decay: re-quantise packed rows to a narrower codebook ------------------------
// Per row in the rotated domain: values = c_src[idx] * g, renormalise, nearest centroid of the
// destination codebook, corrected norm for the new codes.  K rows and V rows have a kernel each.
// ---- K rows: a lane owns a token -----------------------------------------------------------------
// A K row is one token's 128 codes, so one lane can requantise a row without exchanging anything.  The decision
// value of a code is c_src[k] / sqrt(S), S = sum of c_src[code]^2 over the row (the stored norm cancels), so the
// destination code depends on the source code and on S alone, and for S inside an interval around 1 that the host
// works out from the two codebooks (RequantKArgs::s_lo, s_hi) the map k -> code is one fixed table T0.  Such rows -
// all rows of a cache written by this library's store with its own codebooks - go through LDS tables indexed by
// four 3-bit codes (a quad: 12 contiguous bits of the row) or two 4-bit codes (a byte): the table entry carries the
// unit's share of S, its share of the destination's sum of squares, and the remapped codes.  A row whose S lies
// outside the interval (hand-made codebooks, constant rows) or whose norm is zero builds its own table in float64
// and remaps code by code.  Every source dword holds eight codes in both widths and its remapped codes are
// contiguous in the destination (16 bits of a 2-bit row, 24 bits of a 3-bit row), so packing is a few shifts.
struct RequantKArgs {
    const double *cent_src, *cent_dst, *bounds_dst;  // float64 tables in device memory
    unsigned long long t0;                          // 4 bits per source code: its destination code for S in (s_lo, s_hi)
    float s_lo, s_hi;
    uint32_t n_blocks;
    float src_sq[16], dst_sq[16];                   // c_src[k]^2, c_dst[k]^2: by value, so that no table build waits for memory
    uint32_t dst_fix[16];                           // c_dst[k]^2 / fix_unit, rounded: a row's 128 of them add up exactly in 32 bits
    float fix_unit;
    uint32_t src_fix[16];                           // the same for c_src[k]^2 / src_unit (V rows: sums across lanes in integers)
    float src_unit;
    int zero_dst;                                   // destination code of the value 0.0 (rows with norm 0)
};

// one workgroup per CU: the tables are built once for the CU's share of the rows
constexpr int RQK_THREADS = 1024, RQK_BLOCKS = RQK_THREADS / 128;
template <int SB, int DB>
__global__ __launch_bounds__(RQK_THREADS) void k_requantize_k(const uint8_t *src, uint8_t *dst, RequantKArgs a) {
    constexpr int U = SB == 3 ? 4 : 2;   // codes per table unit
    constexpr int NE = 1 << (SB * U);    // 4096 quads / 256 pairs
    constexpr int NS = 1 << SB, ND = 1 << DB;
    constexpr uint32_t SM = NS - 1;
    // per unit: .x = sum of c_src^2 (fp32 bits); .y = the unit's destination codes in the top byte over the unit's sum of
    // c_dst[T0]^2 in fixed point (24 bits, RequantKArgs::dst_fix per code, summed exactly in integers)
    __shared__ uint2 unit_s[NE];
    __shared__ uint2 pair_s[SB == 3 ? 64 : 1];
    __shared__ uint2 one_s[NS];          // .x = c_src[k]^2, .y = T0[k] << 24 | fixed-point c_dst[T0[k]]^2
    __shared__ float cdst2_s[ND];
    const int tid = threadIdx.x, row = tid & 127;
    // the first block's row is requested before the tables are built
    uint32_t w[4 * SB];
    float g = 0.0f;
    auto fetch = [&](uint32_t blk) {
        const uint8_t *sb = src + (int64_t)blk * block_bytes(SB);
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            const uint4 c = stream_load<STREAM_LOAD_OUT>(reinterpret_cast<const uint4 *>(sb + j * 2048 + row * 16));
            w[4 * j] = c.x; w[4 * j + 1] = c.y; w[4 * j + 2] = c.z; w[4 * j + 3] = c.w;
        }
        g = __half2float(reinterpret_cast<const __half *>(sb + block_code_bytes(SB))[row]);
    };
    uint32_t blk = RQK_BLOCKS * blockIdx.x + (tid >> 7);
    if (blk < a.n_blocks) fetch(blk);
    if (tid < 64) {   // the argument arrays are indexed with constants only (they live in scalar registers)
        float sq = 0.0f, dq = 0.0f;
        uint32_t fx = 0;
#pragma unroll
        for (int k = 0; k < NS; ++k) sq = tid == k ? a.src_sq[k] : sq;
#pragma unroll
        for (int k = 0; k < ND; ++k) dq = tid == k ? a.dst_sq[k] : dq;
        const uint32_t t = (uint32_t)((a.t0 >> (4 * (tid & 15))) & 15ull);
#pragma unroll
        for (int k = 0; k < ND; ++k) fx = t == (uint32_t)k ? a.dst_fix[k] : fx;
        if (tid < NS) one_s[tid] = make_uint2(__float_as_uint(sq), (t << 24) | fx);
        if (tid < ND) cdst2_s[tid] = dq;
    }
    __syncthreads();
    // two entries joined: squares and fixed-point sums add, the second entry's codes go above the first's
    auto join = [](uint2 e0, uint2 e1, int code_bits) {
        const uint32_t codes = (e0.y >> 24) | ((e1.y >> 24) << code_bits);
        return make_uint2(__float_as_uint(__uint_as_float(e0.x) + __uint_as_float(e1.x)),
                          (codes << 24) | ((e0.y & 0xFFFFFFu) + (e1.y & 0xFFFFFFu)));
    };
    if constexpr (SB == 3) {
        if (tid < 64) pair_s[tid] = join(one_s[tid & 7], one_s[tid >> 3], DB);
        __syncthreads();
        for (int e = tid; e < NE; e += RQK_THREADS) unit_s[e] = join(pair_s[e & 63], pair_s[e >> 6], 2 * DB);
    } else if (tid < NE) {
        unit_s[tid] = join(one_s[tid & 15], one_s[tid >> 4], DB);
    }
    __syncthreads();

#pragma unroll 1
    for (; blk < a.n_blocks;) {
        // source word j of group q: eight codes, SB bits each (3-bit rows: 24 bits of a dword, or the group's tail)
        auto src_word = [&](int q, int j) -> uint32_t {
            if constexpr (SB == 4) return w[4 * j + q];
            else return j < 3 ? (w[4 * j + q] & 0xFFFFFFu) : tail24(w, q);
        };
        uint32_t m[4][4];   // [group][source word]: the eight remapped codes, DB bits each
        float s1 = 0.0f;
        uint32_t fix = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t x = src_word(q, j);
                uint32_t acc = 0;
#pragma unroll
                for (int u = 0; u < 8 / U; ++u) {
                    const uint32_t e = (x >> (SB * U * u)) & (uint32_t)(NE - 1);
                    const uint2 en = unit_s[e];
                    s1 += __uint_as_float(en.x);
                    fix = __umul24(en.y, 1u) + fix;   // the low 24 bits
                    acc |= (en.y >> 24) << (DB * U * u);
                }
                m[q][j] = acc;
            }
        float recon = g * sqrtf(s1), s2 = (float)fix * a.fix_unit;
        const bool table_ok = s1 > a.s_lo && s1 < a.s_hi && recon > 1e-10f;
        if (__any(!table_ok)) {
            if (!table_ok) {
                // this row's own table, float64 as the reference's arithmetic: y = c_src[k] g / recon against the
                // destination's midpoints, a value on a midpoint taking the higher code
                const double rec = (double)g * sqrt((double)s1);
                const double inv = rec > 1e-10 ? 1.0 / rec : 1.0;
                recon = rec > 1e-10 ? (float)rec : 0.0f;
                unsigned long long t = 0;
                for (int k = 0; k < NS; ++k) {
                    const double y = a.cent_src[k] * (double)g * inv;
                    unsigned long long c = 0;
                    for (int b = 0; b < ND - 1; ++b) c += a.bounds_dst[b] <= y ? 1ull : 0ull;
                    t |= c << (4 * k);
                }
                s2 = 0.0f;
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t x = src_word(q, j);
                        uint32_t acc = 0;
#pragma unroll 1
                        for (int i = 0; i < 8; ++i) {
                            const uint32_t c = (uint32_t)(t >> (4 * ((x >> (SB * i)) & SM))) & 15u;
                            s2 += cdst2_s[c];
                            acc |= c << (DB * i);
                        }
                        m[q][j] = acc;
                    }
            }
        }
        const float cn = sqrtf(s2);
        const float gn = cn > 1e-10f ? recon / cn : recon;
        uint8_t *db = dst + (int64_t)blk * block_bytes(DB);
        blk += RQK_BLOCKS * gridDim.x;
        if (blk < a.n_blocks) fetch(blk);   // the codes of this row are in m[][] by now
        uint32_t d[4 * DB];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (DB == 2) {
                d[q] = m[q][0] | (m[q][1] << 16);
                d[4 + q] = m[q][2] | (m[q][3] << 16);
            } else {
#pragma unroll
                for (int j = 0; j < 3; ++j) d[4 * j + q] = m[q][j] | (((m[q][3] >> (8 * j)) & 0xFFu) << 24);
            }
        }
#pragma unroll
        for (int j = 0; j < DB; ++j)
            stream_store<STREAM_STORE_CODES>(reinterpret_cast<uint4 *>(db + j * 2048 + row * 16),
                                             make_uint4(d[4 * j], d[4 * j + 1], d[4 * j + 2], d[4 * j + 3]));
        reinterpret_cast<__half *>(db + block_code_bytes(DB))[row] = __float2half_rn(gn);
    }
}

// ---- V rows: a wavefront owns a 64-token tile ----------------------------------------------------
// Lane l holds packed row l of the tile: dims l and l + 64 of the tile's 64 tokens (word j of group q = tokens
// 16 q + 4 j .. + 3, first the four codes of dim l, then those of dim l + 64).  The codes are remapped through the
// same T0 table as K rows; a token's sums run over the 64 lanes, so every lane looks up the squares of its two codes
// per token (a table over pairs of codes: two tokens per read, fixed point, exact integer adds) and a six-stage
// exchange (lane ^ 1, 2, 4, 8 by DPP, 16 and 32 by the half-swap instructions) adds them up so that lane t ends
// with token t's two sums.  Tokens with norm 0 get the code of 0.0 and norm 0; a token whose S lies outside the
// plan's interval is redone on its own: its lane builds the token's table in float64, every lane re-maps its two
// codes of that token, and the token's destination sum is added up again.
template <int M> __device__ __forceinline__ uint32_t combine_lanes(uint32_t a, uint32_t b, int lane) {
    if constexpr (M == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
        return r[0] + r[1];
    } else if constexpr (M == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
        return r[0] + r[1];
    } else {
        const bool up = lane & M;
        const uint32_t give = up ? a : b;           // what the partner keeps
        return (up ? b : a) + xor_lane<M>(give);
    }
}

constexpr int RQV_THREADS = 1024;   // sixteen tiles (eight blocks) per workgroup and turn: the tables are built once per CU
template <int SB, int DB>
__global__ __launch_bounds__(RQV_THREADS) void k_requantize_v(const uint8_t *src, uint8_t *dst, RequantKArgs a) {
    constexpr int U = SB == 3 ? 4 : 2;   // codes per remap unit
    constexpr int NE = 1 << (SB * U);
    constexpr int NS = 1 << SB, ND = 1 << DB;
    constexpr int NPAIR = 1 << (2 * SB);
    constexpr uint32_t SM = NS - 1, DM = ND - 1;
    __shared__ uint8_t remap_s[NE];       // a unit's destination codes, DB bits each
    __shared__ uint8_t pair_remap_s[SB == 3 ? 64 : 1];
    __shared__ uint4 pairfix_s[NPAIR];    // codes (lo, hi): c_src^2 of lo, of hi, c_dst[T0]^2 of lo, of hi (fixed point)
    __shared__ uint32_t dstfix_s[ND];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t w[4 * SB];
    uint16_t gbits = 0;
    auto fetch = [&](uint32_t tile) {
        const uint8_t *sb = src + (int64_t)(tile >> 1) * block_bytes(SB);
        const int row = (int)(tile & 1) * 64 + lane;
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            const uint4 c = stream_load<STREAM_LOAD_OUT>(reinterpret_cast<const uint4 *>(sb + j * 2048 + row * 16));
            w[4 * j] = c.x; w[4 * j + 1] = c.y; w[4 * j + 2] = c.z; w[4 * j + 3] = c.w;
        }
        gbits = reinterpret_cast<const uint16_t *>(sb + block_code_bytes(SB))[row];   // lane <-> token for the norms
    };
    const uint32_t n_tiles = 2 * a.n_blocks;
    uint32_t tile = 16 * blockIdx.x + wave;
    if (tile < n_tiles) fetch(tile);
    // tables (argument arrays are indexed with constants only: they live in scalar registers)
    auto pick = [](const auto &arr, uint32_t k, int n) {
        auto v = arr[0];
#pragma unroll
        for (int i = 1; i < 16; ++i)
            if (i < n) v = k == (uint32_t)i ? arr[i] : v;
        return v;
    };
    if (tid < NPAIR) {
        const uint32_t k0 = tid & SM, k1 = (uint32_t)tid >> SB;
        const uint32_t t0 = (uint32_t)((a.t0 >> (4 * k0)) & 15ull), t1 = (uint32_t)((a.t0 >> (4 * k1)) & 15ull);
        pairfix_s[tid] = make_uint4(pick(a.src_fix, k0, NS), pick(a.src_fix, k1, NS), pick(a.dst_fix, t0, ND), pick(a.dst_fix, t1, ND));
        if constexpr (SB == 3) pair_remap_s[tid] = (uint8_t)(t0 | (t1 << DB));
        else remap_s[tid] = (uint8_t)(t0 | (t1 << DB));
    }
    if (tid < ND) dstfix_s[tid] = pick(a.dst_fix, (uint32_t)tid, ND);
    __syncthreads();
    if constexpr (SB == 3) {
        for (int e = tid; e < NE; e += RQV_THREADS) remap_s[e] = (uint8_t)(pair_remap_s[e & 63] | (pair_remap_s[e >> 6] << (2 * DB)));
        __syncthreads();
    }

#pragma unroll 1
    for (; tile < n_tiles;) {
        // source word j of group q: eight codes, SB bits each = tokens 16 q + 4 j .. + 3 of dim l, then of dim l + 64
        auto src_word = [&](int q, int j) -> uint32_t {
            if constexpr (SB == 4) return w[4 * j + q];
            else return j < 3 ? (w[4 * j + q] & 0xFFFFFFu) : tail24(w, q);
        };
        uint32_t m[4][4];
        // sums: the leaves are token pairs (t, t + 1), whose codes are one pair entry per dim half; lane ^ 1 joins them
        uint32_t f1_tree[7], f2_tree[7];   // results of finished subtrees by level (a binary counter over the 32 leaves)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t x = src_word(q, j);
                uint32_t acc = 0;
#pragma unroll
                for (int u = 0; u < 8 / U; ++u) acc |= (uint32_t)remap_s[(x >> (SB * U * u)) & (uint32_t)(NE - 1)] << (DB * U * u);
                m[q][j] = acc;
                // tokens 16 q + 4 j + (0, 1) and + (2, 3): pair i of the first dim half, pair 2 + i of the second
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const uint4 e0 = pairfix_s[(x >> (2 * SB * i)) & (uint32_t)(NPAIR - 1)];
                    const uint4 e1 = pairfix_s[(x >> (2 * SB * (2 + i))) & (uint32_t)(NPAIR - 1)];
                    uint32_t v1 = combine_lanes<1>(e0.x + e1.x, e0.y + e1.y, lane);
                    uint32_t v2 = combine_lanes<1>(e0.z + e1.z, e0.w + e1.w, lane);
                    // leaf number (token pair) 8 q + 2 j + i: carry it up the tree
                    const int leaf = 8 * q + 2 * j + i;
#pragma unroll
                    for (int lv = 1; lv < 6; ++lv) {
                        if (((leaf >> (lv - 1)) & 1) == 0) {
                            f1_tree[lv] = v1;
                            f2_tree[lv] = v2;
                            break;
                        }
                        if (lv == 1) { v1 = combine_lanes<2>(f1_tree[1], v1, lane); v2 = combine_lanes<2>(f2_tree[1], v2, lane); }
                        if (lv == 2) { v1 = combine_lanes<4>(f1_tree[2], v1, lane); v2 = combine_lanes<4>(f2_tree[2], v2, lane); }
                        if (lv == 3) { v1 = combine_lanes<8>(f1_tree[3], v1, lane); v2 = combine_lanes<8>(f2_tree[3], v2, lane); }
                        if (lv == 4) { v1 = combine_lanes<16>(f1_tree[4], v1, lane); v2 = combine_lanes<16>(f2_tree[4], v2, lane); }
                        if (lv == 5) {
                            f1_tree[6] = combine_lanes<32>(f1_tree[5], v1, lane);
                            f2_tree[6] = combine_lanes<32>(f2_tree[5], v2, lane);
                        }
                    }
                }
            }
        // lane t: token t of the tile
        const float g = __half2float(__ushort_as_half(gbits));
        const float s1 = (float)f1_tree[6] * a.src_unit;
        float s2 = (float)f2_tree[6] * a.fix_unit;
        float recon = g * sqrtf(s1);
        const bool zero_tok = !(recon > 1e-10f);
        const bool redo = !zero_tok && !(s1 > a.s_lo && s1 < a.s_hi);
        // tokens with norm 0: the code of 0.0 in every dim, norm 0
        const unsigned long long zmask = __builtin_amdgcn_ballot_w64(zero_tok);
        if (zmask) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t zb = (uint32_t)(zmask >> (16 * q + 4 * j)) & 15u;   // wave-uniform
                    if (zb) {
                        uint32_t fm = 0;
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if ((zb >> i) & 1u) fm |= (DM << (DB * i)) | (DM << (DB * (4 + i)));
                        uint32_t zz = 0;
#pragma unroll
                        for (int i = 0; i < 8; ++i) zz |= (uint32_t)a.zero_dst << (DB * i);
                        m[q][j] = (m[q][j] & ~fm) | (zz & fm);
                    }
                }
        }
        // tokens outside the interval, one at a time
        unsigned long long rmask = __builtin_amdgcn_ballot_w64(redo);
        while (rmask) {
            const int t = __builtin_ctzll(rmask);
            rmask &= rmask - 1;
            // token t's own table (its lane's values count; every lane runs the arithmetic)
            const double rec = (double)g * sqrt((double)s1);
            const double inv = rec > 1e-10 ? 1.0 / rec : 1.0;
            unsigned long long tab = 0;
            for (int k = 0; k < NS; ++k) {
                const double y = a.cent_src[k] * (double)g * inv;
                unsigned long long c = 0;
                for (int b = 0; b < ND - 1; ++b) c += a.bounds_dst[b] <= y ? 1ull : 0ull;
                tab |= c << (4 * k);
            }
            const uint32_t tab_lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)tab, t);
            const uint32_t tab_hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(tab >> 32), t);
            const unsigned long long tt = ((unsigned long long)tab_hi << 32) | tab_lo;
            // this lane's two codes of token t: word (t >> 4, (t >> 2) & 3), slots t & 3 and 4 + (t & 3)
            uint32_t x = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if ((t >> 4) == q && ((t >> 2) & 3) == j) x = src_word(q, j);
            const uint32_t c0 = (x >> (SB * (t & 3))) & SM, c1 = (x >> (SB * (4 + (t & 3)))) & SM;
            const uint32_t n0 = (uint32_t)(tt >> (4 * c0)) & 15u, n1 = (uint32_t)(tt >> (4 * c1)) & 15u;
            const uint32_t fm = (DM << (DB * (t & 3))) | (DM << (DB * (4 + (t & 3))));
            const uint32_t nv = (n0 << (DB * (t & 3))) | (n1 << (DB * (4 + (t & 3))));
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if ((t >> 4) == q && ((t >> 2) & 3) == j) m[q][j] = (m[q][j] & ~fm) | nv;
            // the token's destination sum, over all lanes
            uint32_t part = dstfix_s[n0] + dstfix_s[n1];
            part += xor_lane<1>(part);
            part += xor_lane<2>(part);
            part += xor_lane<4>(part);
            part += xor_lane<8>(part);
            part += xor_lane<16>(part);
            part += xor_lane<32>(part);
            if (lane == t) s2 = (float)part * a.fix_unit;
        }
        const float cn = sqrtf(s2);
        float gn = cn > 1e-10f ? recon / cn : recon;
        if (zero_tok) gn = 0.0f;
        const uint32_t out_tile = tile;
        tile += 16 * gridDim.x;
        // the source words are in m[][] by now
        const int row = (int)(out_tile & 1) * 64 + lane;
        uint8_t *db = dst + (int64_t)(out_tile >> 1) * block_bytes(DB);
        uint32_t d[4 * DB];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if constexpr (DB == 2) {
                d[q] = m[q][0] | (m[q][1] << 16);
                d[4 + q] = m[q][2] | (m[q][3] << 16);
            } else {
#pragma unroll
                for (int j = 0; j < 3; ++j) d[4 * j + q] = m[q][j] | (((m[q][3] >> (8 * j)) & 0xFFu) << 24);
            }
        }
        if (tile < n_tiles) fetch(tile);
#pragma unroll
        for (int j = 0; j < DB; ++j)
            stream_store<STREAM_STORE_CODES>(reinterpret_cast<uint4 *>(db + j * 2048 + row * 16),
                                             make_uint4(d[4 * j], d[4 * j + 1], d[4 * j + 2], d[4 * j + 3]));
        reinterpret_cast<__half *>(db + block_code_bytes(DB))[row] = __float2half_rn(gn);
    }
}

// T0 and the interval of S = sum of c_src[code]^2 for which every source code keeps its T0 destination: the decision
// value of code k is c_src[k] / r with r = sqrt(S), and it meets the midpoint b at r = c_src[k] / b.  The interval is
// what lies between the nearest such r below and above 1, shrunk by 1e-5 so that the fp32 sum decides safely.
static bool requant_plan(const tq_handle *hs, const tq_handle *hd, RequantKArgs *a) {
    const int ns = hs->n_centroids, nd = hd->n_centroids;
    if (ns > 16 || nd > 16) return false;
    double r_lo = 0.0, r_hi = 1e30;
    a->t0 = 0;
    for (int k = 0; k < ns; ++k) {
        const double c = hs->centroids_host[k];
        unsigned long long t = 0;
        for (int b = 0; b + 1 < nd; ++b) {
            const double bd = hd->bounds_host[b];
            t += bd <= c ? 1ull : 0ull;
            if (bd == 0.0 || c == 0.0 || (bd > 0.0) != (c > 0.0)) continue;
            const double r = c / bd;
            if (r <= 1.0 && r > r_lo) r_lo = r;
            if (r >= 1.0 && r < r_hi) r_hi = r;
        }
        a->t0 |= t << (4 * k);
    }
    a->s_lo = (float)(r_lo * r_lo * (1.0 + 1e-5));
    a->s_hi = (float)(r_hi * r_hi * (1.0 - 1e-5));
    a->cent_src = hs->centroids64; a->cent_dst = hd->centroids64; a->bounds_dst = hd->bounds64;
    for (int k = 0; k < 16; ++k) {
        a->src_sq[k] = k < ns ? (float)(hs->centroids_host[k] * hs->centroids_host[k]) : 0.0f;
        a->dst_sq[k] = k < nd ? (float)(hd->centroids_host[k] * hd->centroids_host[k]) : 0.0f;
    }
    // fixed point: the largest square just under 2^22, so that four of them fit the 24 bits of a table entry
    double top = 0.0;
    for (int k = 0; k < nd; ++k) top = fmax(top, hd->centroids_host[k] * hd->centroids_host[k]);
    const double unit = top > 0.0 ? top / 4194300.0 : 1.0;
    a->fix_unit = (float)unit;
    for (int k = 0; k < 16; ++k)
        a->dst_fix[k] = k < nd ? (uint32_t)llround(hd->centroids_host[k] * hd->centroids_host[k] / (double)a->fix_unit) : 0u;
    double stop = 0.0;
    for (int k = 0; k < ns; ++k) stop = fmax(stop, hs->centroids_host[k] * hs->centroids_host[k]);
    a->src_unit = (float)(stop > 0.0 ? stop / 4194300.0 : 1.0);
    for (int k = 0; k < 16; ++k)
        a->src_fix[k] = k < ns ? (uint32_t)llround(hs->centroids_host[k] * hs->centroids_host[k] / (double)a->src_unit) : 0u;
    a->zero_dst = 0;
    for (int b = 0; b + 1 < nd; ++b) a->zero_dst += hd->bounds_host[b] <= 0.0 ? 1 : 0;
    return true;
}

int tqk_requantize(const tq_handle *hs, const tq_handle *hd, const void *src, int64_t n_seqs, int64_t tokens, int kind, void *dst,
                   hipStream_t s) {
    const unsigned grid = (unsigned)(n_seqs * blocks_for(tokens));
    if (grid == 0) return TQ_OK;
    const int key = hs->bits * 10 + hd->bits;
    RequantKArgs ka;
    if ((key != 32 && key != 43 && key != 42) || !requant_plan(hs, hd, &ka)) {
        tq_set_error("tq_requantize: supported width pairs are 3->2, 4->3, 4->2 (got %d->%d)", hs->bits, hd->bits);
        return TQ_ERR_UNSUPPORTED;
    }
    ka.n_blocks = grid;
    if (kind == TQ_KIND_K) {
        const unsigned sets = (grid + RQK_BLOCKS - 1) / RQK_BLOCKS;
        const unsigned wgs = sets < 256u ? sets : 256u;
        switch (key) {
        case 32: k_requantize_k<3, 2><<<wgs, RQK_THREADS, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, ka); break;
        case 43: k_requantize_k<4, 3><<<wgs, RQK_THREADS, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, ka); break;
        default: k_requantize_k<4, 2><<<wgs, RQK_THREADS, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, ka); break;
        }
        return tq_check_launch("requantize (K rows)");
    }
    const unsigned sets = (grid + 7) / 8;
    const unsigned wgs = sets < 256u ? sets : 256u;
    switch (key) {
    case 32: k_requantize_v<3, 2><<<wgs, RQV_THREADS, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, ka); break;
    case 43: k_requantize_v<4, 3><<<wgs, RQV_THREADS, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, ka); break;
    default: k_requantize_v<4, 2><<<wgs, RQV_THREADS, 0, s>>>((const uint8_t *)src, (uint8_t *)dst, ka); break;
    }
    return tq_check_launch("requantize (V rows)");
}

// ---- interchange with the per-128 block layout of the llama.cpp fork --------------------------
// One block per vector, token order: norm fp16 | qs | signs (3-bit: two low bits of every index
// in qs, the third in signs; 2-bit: qs only) - 50 / 34 bytes; 4-bit: norm fp16 | rnorm fp16 | qs[64] nibbles -
// 68 bytes (4.25 bits per value).  rnorm is the residual-norm slot of the fork's earlier 3-bit + QJL turbo4,
// which its 4-bit PolarQuant block keeps and does not use: written as 0, ignored when read.
// The fork's earlier builds stored 2- and 3-bit rows in blocks of 32 values (QK_TURBO3 = QK_TURBO2 = 32; 64 was tried
// as well, docs/papers/block-size-experiment.md:27-39,270): a vector is then SUB = 4 or 2 blocks of norm | qs | signs
// over its own 32 or 64 values, one after the other, every block with the same (group) norm - 14 / 26 bytes per 3-bit
// block, 10 / 18 per 2-bit block.  The extraction formulas are those of the 128-value block applied inside a block.
// ForkRow gives the 16-bit positions of a vector's fields: a group g of 32 values has four pieces of qs (eight values
// each) and, for 3-bit rows, two pieces of signs (sixteen values each).
template <int BITS, int SUB> struct ForkRow {
    static constexpr int PER = 4 / SUB;                                       // groups of 32 values per storage block
    static constexpr int SH = 1 + 4 * PER + (BITS == 3 ? 2 * PER : 0);        // 16-bit pieces per storage block
    static constexpr int BYTES = BITS == 4 ? 68 : 2 * SUB * SH;               // one vector
    __host__ __device__ static constexpr int norm(int s) { return s * SH; }
    __host__ __device__ static constexpr int qs(int g, int j) { return (g / PER) * SH + 1 + 4 * (g % PER) + j; }
    __host__ __device__ static constexpr int sg(int g, int k) { return (g / PER) * SH + 1 + 4 * PER + 2 * (g % PER) + k; }
};
static_assert(ForkRow<3, 1>::BYTES == 50 && ForkRow<3, 2>::BYTES == 2 * 26 && ForkRow<3, 4>::BYTES == 4 * 14, "3-bit fork blocks");
static_assert(ForkRow<2, 1>::BYTES == 34 && ForkRow<2, 2>::BYTES == 2 * 18 && ForkRow<2, 4>::BYTES == 4 * 10, "2-bit fork blocks");
static_assert(ForkRow<3, 1>::qs(3, 3) == 16 && ForkRow<3, 1>::sg(0, 0) == 17 && ForkRow<3, 1>::sg(3, 1) == 24, "per-128 block");

// ---- K rows of the fork layout: a lane owns a token ------------------------------------------------
// The fork rows of one of this library's K blocks are 128 * FB contiguous bytes.  They move between memory and LDS
// as 16-byte pieces (the stage keeps the address's low four bits, so a piece is aligned on both sides; what comes
// before the first and after the last whole piece moves as 2-byte pieces, the alignment every fork buffer has), a
// lane takes its token's row from the stage as 2- or 4-byte pieces, and the packed block is read or written as
// 16-byte chunks contiguous over the lanes.  4- and 2-bit rows only change the order of their words; 3-bit rows
// interleave the fork's two-bit fields and sign bits through byte-indexed tables.
constexpr int FORK_K_THREADS = 256;   // two blocks per workgroup
template <int FB>
__device__ __forceinline__ void fork_stage_copy(uint8_t *stage, uint8_t *mem, int nbytes, bool to_mem, int t, int nt) {
    const int mis = (int)(reinterpret_cast<uintptr_t>(mem) & 15);
    uint8_t *lds = stage + mis;                              // same low address bits as the memory side
    const int head = mis ? (16 - mis < nbytes ? 16 - mis : nbytes) : 0;
    const int body = (nbytes - head) / 16, tail0 = head + 16 * body;
    for (int e = t; e < body; e += nt) {
        uint4 *m = reinterpret_cast<uint4 *>(mem + head) + e, *l = reinterpret_cast<uint4 *>(lds + head) + e;
        if (to_mem) *m = *l;
        else *l = *m;
    }
    const int edge = (head + (nbytes - tail0)) / 2;          // 2-byte pieces outside the whole 16-byte pieces
    for (int e = t; e < edge; e += nt) {
        const int off = 2 * e < head ? 2 * e : tail0 + (2 * e - head);
        uint16_t *m = reinterpret_cast<uint16_t *>(mem + off), *l = reinterpret_cast<uint16_t *>(lds + off);
        if (to_mem) *m = *l;
        else *l = *m;
    }
}

template <int BITS, bool TO_FORK, int SUB>
__global__ __launch_bounds__(FORK_K_THREADS) void k_fork_k(const uint8_t *packed_in, uint8_t *packed_out, const uint8_t *fork_in,
                                                            uint8_t *fork_out, int64_t tokens, int64_t blocks_per_seq,
                                                            uint32_t zero_code, uint32_t n_blocks) {
    using R = ForkRow<BITS, SUB>;
    constexpr int FB = R::BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t stage[2][TQ_ROWS_PER_BLOCK * FB + 16];
    __shared__ uint16_t spread2_s[BITS == 3 && !TO_FORK ? 256 : 1];   // byte of four 2-bit fields -> the fields at a stride of 3
    __shared__ uint32_t spread1_s[BITS == 3 && !TO_FORK ? 256 : 1];   // byte of eight sign bits -> bit 3m + 2
    __shared__ uint16_t gather_s[BITS == 3 && TO_FORK ? 4096 : 1];    // four 3-bit codes -> their low bits (8) | their top bits << 8
    const int tid = threadIdx.x, half = tid >> 7, row = tid & 127;
    const uint32_t blk = 2 * blockIdx.x + half;
    const bool live = blk < n_blocks;
    const int64_t seq = live ? blk / blocks_per_seq : 0, bis = live ? blk % blocks_per_seq : 0;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK;
    const int rows = !live ? 0 : tokens - tok0 < TQ_ROWS_PER_BLOCK ? (int)(tokens - tok0) : TQ_ROWS_PER_BLOCK;
    uint8_t *fork_rows = const_cast<uint8_t *>(TO_FORK ? fork_out : fork_in) + (seq * tokens + tok0) * FB;
    const int mis = (int)(reinterpret_cast<uintptr_t>(fork_rows) & 15);
    uint8_t *mine = stage[half] + mis + row * FB;            // this lane's row in the stage

    if constexpr (BITS == 3 && !TO_FORK) {
        uint32_t a = 0, b = 0;
#pragma unroll
        for (int m = 0; m < 4; ++m) a |= ((tid >> (2 * m)) & 3u) << (3 * m);
#pragma unroll
        for (int m = 0; m < 8; ++m) b |= ((tid >> m) & 1u) << (3 * m + 2);
        spread2_s[tid] = (uint16_t)a;
        spread1_s[tid] = b;
    }
    if constexpr (BITS == 3 && TO_FORK) {
        for (int e = tid; e < 4096; e += FORK_K_THREADS) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const uint32_t c = (e >> (3 * m)) & 7u;
                lo |= (c & 3u) << (2 * m);
                hi |= (c >> 2) << m;
            }
            gather_s[e] = (uint16_t)(lo | (hi << 8));
        }
    }
    uint32_t w[4 * BITS];
    uint16_t nrm = 0;
    if constexpr (TO_FORK) {
        if (live) {
            const uint8_t *sb = packed_in + (int64_t)blk * block_bytes(BITS);
#pragma unroll
            for (int j = 0; j < BITS; ++j) {
                const uint4 c = *reinterpret_cast<const uint4 *>(sb + j * 2048 + row * 16);
                w[4 * j] = c.x; w[4 * j + 1] = c.y; w[4 * j + 2] = c.z; w[4 * j + 3] = c.w;
            }
            nrm = reinterpret_cast<const uint16_t *>(sb + block_code_bytes(BITS))[row];
        }
        __syncthreads();   // the table
        if (row < rows) {
            if constexpr (BITS == 4) {
                uint32_t *d = reinterpret_cast<uint32_t *>(mine);   // 68-byte rows at a 4-byte aligned address
                d[0] = nrm;                                         // norm, and 0 in the unused rnorm slot
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) d[1 + 4 * g + j] = w[4 * j + g];
            } else if constexpr (BITS == 2) {
                uint16_t *h = reinterpret_cast<uint16_t *>(mine);
#pragma unroll
                for (int sb = 0; sb < SUB; ++sb) h[R::norm(sb)] = nrm;   // every storage block carries the group's norm
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        h[R::qs(g, 2 * j)] = (uint16_t)w[4 * j + g];
                        h[R::qs(g, 2 * j + 1)] = (uint16_t)(w[4 * j + g] >> 16);
                    }
            } else {
                uint16_t *h = reinterpret_cast<uint16_t *>(mine);
#pragma unroll
                for (int sb = 0; sb < SUB; ++sb) h[R::norm(sb)] = nrm;   // every storage block carries the group's norm
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint32_t sg = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t x = j < 3 ? (w[4 * j + g] & 0xFFFFFFu) : tail24(w, g);
                        const uint32_t e0 = gather_s[x & 0xFFFu], e1 = gather_s[x >> 12];
                        h[R::qs(g, j)] = (uint16_t)((e0 & 0xFFu) | ((e1 & 0xFFu) << 8));
                        sg |= ((e0 >> 8) | ((e1 >> 8) << 4)) << (8 * j);
                    }
                    h[R::sg(g, 0)] = (uint16_t)sg;
                    h[R::sg(g, 1)] = (uint16_t)(sg >> 16);
                }
            }
        }
        __syncthreads();
        fork_stage_copy<FB>(stage[half], fork_rows, rows * FB, true, row, 128);
    } else {
        fork_stage_copy<FB>(stage[half], fork_rows, rows * FB, false, row, 128);
        __syncthreads();
        if (!live) return;
        if (row < rows) {
            if constexpr (BITS == 4) {
                const uint32_t *d = reinterpret_cast<const uint32_t *>(mine);
                nrm = (uint16_t)d[0];
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) w[4 * j + g] = d[1 + 4 * g + j];
            } else if constexpr (BITS == 2) {
                const uint16_t *h = reinterpret_cast<const uint16_t *>(mine);
                nrm = h[0];
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 2; ++j) w[4 * j + g] = (uint32_t)h[R::qs(g, 2 * j)] | ((uint32_t)h[R::qs(g, 2 * j + 1)] << 16);
            } else {
                const uint16_t *h = reinterpret_cast<const uint16_t *>(mine);
                nrm = h[0];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t sg = (uint32_t)h[R::sg(g, 0)] | ((uint32_t)h[R::sg(g, 1)] << 16);
                    uint32_t x[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t q = h[R::qs(g, j)];
                        x[j] = (uint32_t)spread2_s[q & 0xFFu] | ((uint32_t)spread2_s[q >> 8] << 12) | spread1_s[(sg >> (8 * j)) & 0xFFu];
                    }
#pragma unroll
                    for (int j = 0; j < 3; ++j) w[4 * j + g] = x[j] | (((x[3] >> (8 * j)) & 0xFFu) << 24);
                }
            }
        } else {
            // rows past the sequence's end: the code of 0.0 and norm 0, as the store kernels write them
            const uint32_t pair = zero_code | (zero_code << BITS);
            const uint32_t fill = BITS == 4 ? pair * 0x01010101u : BITS == 2 ? pair * 0x11111111u : pair * 0x041041u;
#pragma unroll
            for (int q = 0; q < 4 * BITS; ++q) w[q] = BITS == 3 ? fill | (((fill >> (8 * (q >> 2))) & 0xFFu) << 24) : fill;
        }
        uint8_t *db = packed_out + (int64_t)blk * block_bytes(BITS);
#pragma unroll
        for (int j = 0; j < BITS; ++j)
            *reinterpret_cast<uint4 *>(db + j * 2048 + row * 16) = make_uint4(w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]);
        reinterpret_cast<uint16_t *>(db + block_code_bytes(BITS))[row] = nrm;
    }
}

// ---- V rows of the fork layout: a wavefront owns a 64-token tile ------------------------------------
// A V tile holds its 64 tokens dim-major (lane l of the wavefront = packed row l = dims l and l + 64), the fork's rows
// are token-major, so the tile is transposed on the way - in units of four codes (a 16-bit piece: four tokens of one
// dim on the V side, four dims of one token on the token side) through 32 LDS rows of 64 pieces: every lane writes
// its 32 pieces, one per row, then reads two rows' worth of 8-byte groups and keeps one code of each piece.  Rows
// are 136 bytes apart, so that lanes reading different rows hit different banks.  The token side then is what the
// K kernel has: a lane owns a token, takes or puts its fork row in the wavefront's stage, and the stage moves
// between LDS and memory in 16-byte pieces.
constexpr int FORK_V_WAVES = 8, FORK_X_ROW = 136;

// a row's sixteen words of eight codes (word j of group q) <-> its packed dwords
template <int BITS> __device__ __forceinline__ void words_from_packed(const uint32_t (&w)[4 * BITS], uint32_t (&cw)[4][4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (BITS == 4) cw[q][j] = w[4 * j + q];
            else if constexpr (BITS == 2) cw[q][j] = (w[4 * (j >> 1) + q] >> (16 * (j & 1))) & 0xFFFFu;
            else cw[q][j] = j < 3 ? (w[4 * j + q] & 0xFFFFFFu) : tail24(w, q);
        }
}
template <int BITS> __device__ __forceinline__ void packed_from_words(const uint32_t (&cw)[4][4], uint32_t (&w)[4 * BITS]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if constexpr (BITS == 4) {
#pragma unroll
            for (int j = 0; j < 4; ++j) w[4 * j + q] = cw[q][j];
        } else if constexpr (BITS == 2) {
            w[q] = cw[q][0] | (cw[q][1] << 16);
            w[4 + q] = cw[q][2] | (cw[q][3] << 16);
        } else {
#pragma unroll
            for (int j = 0; j < 3; ++j) w[4 * j + q] = cw[q][j] | (((cw[q][3] >> (8 * j)) & 0xFFu) << 24);
        }
    }
}
// code number `slot` of each of the four 16-bit pieces of an 8-byte group, as four codes side by side
template <int BITS> __device__ __forceinline__ uint32_t pick_codes(uint2 d, int off_lo, int off_hi) {
    const uint32_t a = __builtin_amdgcn_ubfe(d.x, off_lo, BITS) | (__builtin_amdgcn_ubfe(d.x, off_hi, BITS) << BITS);
    const uint32_t b = __builtin_amdgcn_ubfe(d.y, off_lo, BITS) | (__builtin_amdgcn_ubfe(d.y, off_hi, BITS) << BITS);
    return a | (b << (2 * BITS));
}

template <int BITS, bool TO_FORK, int SUB>
__global__ __launch_bounds__(64 * FORK_V_WAVES) void k_fork_v(const uint8_t *packed_in, uint8_t *packed_out, const uint8_t *fork_in,
                                                              uint8_t *fork_out, int64_t tokens, int64_t blocks_per_seq,
                                                              uint32_t zero_code, uint32_t n_blocks) {
    using R = ForkRow<BITS, SUB>;
    constexpr int FB = R::BYTES;
    constexpr uint32_t QM = (1u << (4 * BITS)) - 1u;   // four codes
    __shared__ __attribute__((aligned(16))) uint8_t stage_s[FORK_V_WAVES][64 * FB + 16];
    __shared__ __attribute__((aligned(8))) uint8_t xs_s[FORK_V_WAVES][32 * FORK_X_ROW];
    __shared__ uint16_t spread2_s[BITS == 3 && !TO_FORK ? 256 : 1];   // byte of four 2-bit fields -> the fields at a stride of 3
    __shared__ uint32_t spread1_s[BITS == 3 && !TO_FORK ? 256 : 1];   // byte of eight sign bits -> bit 3m + 2
    __shared__ uint16_t gather_s[BITS == 3 && TO_FORK ? 4096 : 1];    // four 3-bit codes -> their low bits (8) | their top bits << 8
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if constexpr (BITS == 3 && !TO_FORK) {
        if (tid < 256) {
            uint32_t a = 0, b = 0;
#pragma unroll
            for (int m = 0; m < 4; ++m) a |= ((tid >> (2 * m)) & 3u) << (3 * m);
#pragma unroll
            for (int m = 0; m < 8; ++m) b |= ((tid >> m) & 1u) << (3 * m + 2);
            spread2_s[tid] = (uint16_t)a;
            spread1_s[tid] = b;
        }
    }
    if constexpr (BITS == 3 && TO_FORK) {
        for (int e = tid; e < 4096; e += 64 * FORK_V_WAVES) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const uint32_t c = (e >> (3 * m)) & 7u;
                lo |= (c & 3u) << (2 * m);
                hi |= (c >> 2) << m;
            }
            gather_s[e] = (uint16_t)(lo | (hi << 8));
        }
    }
    const uint32_t tile = FORK_V_WAVES * blockIdx.x + wave;
    const bool live = tile < 2 * n_blocks;
    const uint32_t blk = live ? tile >> 1 : 0;
    const int half = (int)(tile & 1);
    const int64_t seq = blk / blocks_per_seq, bis = blk % blocks_per_seq;
    const int64_t tok0 = bis * TQ_ROWS_PER_BLOCK + half * 64;
    const int rows = !live || tokens <= tok0 ? 0 : tokens - tok0 < 64 ? (int)(tokens - tok0) : 64;
    uint8_t *fork_rows = const_cast<uint8_t *>(TO_FORK ? fork_out : fork_in) + (seq * tokens + tok0) * FB;
    const int mis = (int)(reinterpret_cast<uintptr_t>(fork_rows) & 15);
    uint8_t *stage = stage_s[wave], *xs = xs_s[wave];
    uint8_t *mine = stage + mis + lane * FB;       // this lane's token's row in the stage
    const int off_lo = BITS * (lane & 3), off_hi = 16 + off_lo;
    uint32_t vw[4][4], kw[4][4];                  // V row (lane = packed row) and token row (lane = token), as words of eight codes
    uint32_t w[4 * BITS];
    uint16_t nrm = 0;
    __syncthreads();   // the tables
    if (!live) return;

    if constexpr (TO_FORK) {
        const uint8_t *sb = packed_in + (int64_t)blk * block_bytes(BITS);
        const int prow = half * 64 + lane;
#pragma unroll
        for (int j = 0; j < BITS; ++j) {
            const uint4 c = *reinterpret_cast<const uint4 *>(sb + j * 2048 + prow * 16);
            w[4 * j] = c.x; w[4 * j + 1] = c.y; w[4 * j + 2] = c.z; w[4 * j + 3] = c.w;
        }
        nrm = reinterpret_cast<const uint16_t *>(sb + block_code_bytes(BITS))[prow];   // lane <-> token for the norms
        words_from_packed<BITS>(w, vw);
        // word (q, j): tokens 16 q + 4 j .. + 3 of dim l, then of dim l + 64 -> rows 2 (4 q + j) and + 1, column l
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                *reinterpret_cast<uint16_t *>(xs + (2 * (4 * q + j)) * FORK_X_ROW + 2 * lane) = (uint16_t)(vw[q][j] & QM);
                *reinterpret_cast<uint16_t *>(xs + (2 * (4 * q + j) + 1) * FORK_X_ROW + 2 * lane) = (uint16_t)(vw[q][j] >> (4 * BITS));
            }
        __builtin_amdgcn_wave_barrier();
        // token lane >> 2's group of four tokens, this token's place in it lane & 3: dims 32 q + 8 j .. + 7 sit in
        // row 2 T + (q >> 1), columns 32 (q & 1) + 8 j .. + 7
        const uint8_t *r0 = xs + (2 * (lane >> 2)) * FORK_X_ROW, *r1 = r0 + FORK_X_ROW;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint8_t *g = (q >> 1 ? r1 : r0) + 2 * (32 * (q & 1) + 8 * j);
                kw[q][j] = pick_codes<BITS>(*reinterpret_cast<const uint2 *>(g), off_lo, off_hi) |
                           (pick_codes<BITS>(*reinterpret_cast<const uint2 *>(g + 8), off_lo, off_hi) << (4 * BITS));
            }
        if (lane < rows) {
            if constexpr (BITS == 4) {
                uint32_t *d = reinterpret_cast<uint32_t *>(mine);   // 68-byte rows at a 4-byte aligned address
                d[0] = nrm;                                         // norm, and 0 in the unused rnorm slot
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) d[1 + 4 * g + j] = kw[g][j];
            } else if constexpr (BITS == 2) {
                uint16_t *h = reinterpret_cast<uint16_t *>(mine);
#pragma unroll
                for (int sb = 0; sb < SUB; ++sb) h[R::norm(sb)] = nrm;   // every storage block carries the group's norm
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) h[R::qs(g, j)] = (uint16_t)kw[g][j];
            } else {
                uint16_t *h = reinterpret_cast<uint16_t *>(mine);
#pragma unroll
                for (int sb = 0; sb < SUB; ++sb) h[R::norm(sb)] = nrm;   // every storage block carries the group's norm
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint32_t sg = 0;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t e0 = gather_s[kw[g][j] & 0xFFFu], e1 = gather_s[kw[g][j] >> 12];
                        h[R::qs(g, j)] = (uint16_t)((e0 & 0xFFu) | ((e1 & 0xFFu) << 8));
                        sg |= ((e0 >> 8) | ((e1 >> 8) << 4)) << (8 * j);
                    }
                    h[R::sg(g, 0)] = (uint16_t)sg;
                    h[R::sg(g, 1)] = (uint16_t)(sg >> 16);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        fork_stage_copy<FB>(stage, fork_rows, rows * FB, true, lane, 64);
    } else {
        fork_stage_copy<FB>(stage, fork_rows, rows * FB, false, lane, 64);
        __builtin_amdgcn_wave_barrier();
        if (lane < rows) {
            if constexpr (BITS == 4) {
                const uint32_t *d = reinterpret_cast<const uint32_t *>(mine);
                nrm = (uint16_t)d[0];
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) kw[g][j] = d[1 + 4 * g + j];
            } else if constexpr (BITS == 2) {
                const uint16_t *h = reinterpret_cast<const uint16_t *>(mine);
                nrm = h[0];
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j) kw[g][j] = h[R::qs(g, j)];
            } else {
                const uint16_t *h = reinterpret_cast<const uint16_t *>(mine);
                nrm = h[0];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t sg = (uint32_t)h[R::sg(g, 0)] | ((uint32_t)h[R::sg(g, 1)] << 16);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t q = h[R::qs(g, j)];
                        kw[g][j] = (uint32_t)spread2_s[q & 0xFFu] | ((uint32_t)spread2_s[q >> 8] << 12) | spread1_s[(sg >> (8 * j)) & 0xFFu];
                    }
                }
            }
        } else {
            // tokens past the sequence's end: the code of 0.0 and norm 0, as the store kernels write them
            uint32_t fill = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) fill |= zero_code << (BITS * i);
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int j = 0; j < 4; ++j) kw[g][j] = fill;
        }
        // word (q, j) of a token: dims 32 q + 8 j .. + 3 and .. + 4 .. + 7 -> rows 8 q + 2 j and + 1, column = token
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                *reinterpret_cast<uint16_t *>(xs + (8 * q + 2 * j) * FORK_X_ROW + 2 * lane) = (uint16_t)(kw[q][j] & QM);
                *reinterpret_cast<uint16_t *>(xs + (8 * q + 2 * j + 1) * FORK_X_ROW + 2 * lane) = (uint16_t)(kw[q][j] >> (4 * BITS));
            }
        __builtin_amdgcn_wave_barrier();
        // packed row l = dims l and l + 64: rows l >> 2 and 16 + (l >> 2), place l & 3 in a piece; word (q, j) = tokens 16 q + 4 j .. + 3
        const uint8_t *r0 = xs + (lane >> 2) * FORK_X_ROW, *r1 = r0 + 16 * FORK_X_ROW;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = 2 * (16 * q + 4 * j);
                vw[q][j] = pick_codes<BITS>(*reinterpret_cast<const uint2 *>(r0 + col), off_lo, off_hi) |
                           (pick_codes<BITS>(*reinterpret_cast<const uint2 *>(r1 + col), off_lo, off_hi) << (4 * BITS));
            }
        packed_from_words<BITS>(vw, w);
        uint8_t *db = packed_out + (int64_t)blk * block_bytes(BITS);
        const int prow = half * 64 + lane;
#pragma unroll
        for (int j = 0; j < BITS; ++j)
            *reinterpret_cast<uint4 *>(db + j * 2048 + prow * 16) = make_uint4(w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]);
        reinterpret_cast<uint16_t *>(db + block_code_bytes(BITS))[prow] = nrm;
    }
}

int tqk_fork_blocks(const tq_handle *h, int to_fork, const void *src, int64_t n_seqs, int64_t tokens, int kind, void *dst,
                    int block_values, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    // index of 0.0: number of boundaries below it (a zero vector stores this code in every dim)
    uint32_t zero_code = (uint32_t)(h->n_centroids / 2);
    if (h->zero_code >= 0) zero_code = (uint32_t)h->zero_code;
    const unsigned kgrid = (grid + 1) / 2, vgrid = (2 * grid + FORK_V_WAVES - 1) / FORK_V_WAVES;
#define TQ_FORK(B, SUB)                                                                                                   \
    if (kind == TQ_KIND_K && to_fork)                                                                                     \
        k_fork_k<B, true, SUB><<<kgrid, FORK_K_THREADS, 0, s>>>((const uint8_t *)src, nullptr, nullptr, (uint8_t *)dst, tokens, bps, zero_code, grid); \
    else if (kind == TQ_KIND_K)                                                                                           \
        k_fork_k<B, false, SUB><<<kgrid, FORK_K_THREADS, 0, s>>>(nullptr, (uint8_t *)dst, (const uint8_t *)src, nullptr, tokens, bps, zero_code, grid); \
    else if (to_fork)                                                                                                     \
        k_fork_v<B, true, SUB><<<vgrid, 64 * FORK_V_WAVES, 0, s>>>((const uint8_t *)src, nullptr, nullptr, (uint8_t *)dst, tokens, bps, zero_code, grid); \
    else                                                                                                                  \
        k_fork_v<B, false, SUB><<<vgrid, 64 * FORK_V_WAVES, 0, s>>>(nullptr, (uint8_t *)dst, (const uint8_t *)src, nullptr, tokens, bps, zero_code, grid)
    const int sub = block_values == 128 ? 1 : block_values == 64 ? 2 : block_values == 32 ? 4 : 0;
    switch (h->bits * 8 + sub) {
    case 2 * 8 + 1: TQ_FORK(2, 1); break;
    case 2 * 8 + 2: TQ_FORK(2, 2); break;
    case 2 * 8 + 4: TQ_FORK(2, 4); break;
    case 3 * 8 + 1: TQ_FORK(3, 1); break;
    case 3 * 8 + 2: TQ_FORK(3, 2); break;
    case 3 * 8 + 4: TQ_FORK(3, 4); break;
    case 4 * 8 + 1: TQ_FORK(4, 1); break;
    default:
        tq_set_error("fork blocks: %d-bit rows in storage blocks of %d values are not a layout of the fork (2- and 3-bit: "
                     "32, 64 or 128 values per block; 4-bit: 128)", h->bits, block_values);
        return TQ_ERR_UNSUPPORTED;
    }
#undef TQ_FORK
    return tq_check_launch("fork_blocks");
}

static AppendArgs make_append_args(const tq_handle *h, int64_t pos, const int64_t *pos_dev, int64_t n_new, int64_t capacity,
                                   int kind, uint32_t *overrun = nullptr) {
    AppendArgs a;
    a.s1 = h->s1_32; a.s2 = h->s2_32; a.bounds = h->bounds32; a.cent = h->centroids32;
    a.kind = kind; a.norm_correction = h->norm_correction; a.zero_code = h->zero_code;
    a.pos = pos; a.n_new = n_new; a.blocks_per_seq = blocks_for(capacity);
    a.pos_dev = pos_dev; a.capacity = capacity; a.overrun = pos_dev ? overrun : nullptr;
    a.first_block = pos / TQ_ROWS_PER_BLOCK;
    a.n_touched = pos_dev ? (n_new + TQ_ROWS_PER_BLOCK - 2) / TQ_ROWS_PER_BLOCK + 1  // at the worst alignment
                          : (pos + n_new - 1) / TQ_ROWS_PER_BLOCK - a.first_block + 1;
    return a;
}

int tqk_append_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t pos,
                  int64_t n_new, int64_t capacity, int in_dtype, void *packed_k, void *packed_v, hipStream_t s,
                  const int64_t *pos_dev, uint32_t *overrun) {
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    const AppendArgs ka = make_append_args(hk, pos, pos_dev, n_new, capacity, TQ_KIND_K, overrun);
    const AppendArgs va = make_append_args(hv, pos, pos_dev, n_new, capacity, TQ_KIND_V);  // the K half reports
    const unsigned grid = 2u * (unsigned)(n_seqs * ka.n_touched);
    const int kb = hk->bits, vb = hv->bits;
#define TQ_APPEND_KV(KB, VB)                                                                                                   \
    DISPATCH_T(in_dtype, TI, (k_append_kv<KB, VB, TI><<<grid, 256, 0, s>>>((const TI *)k, (uint8_t *)packed_k, ka, (const TI *)v, \
                                                                            (uint8_t *)packed_v, va)))
    if (kb == 3 && vb == 3) { TQ_APPEND_KV(3, 3); }
    else if (kb == 4 && vb == 4) { TQ_APPEND_KV(4, 4); }
    else if (kb == 2 && vb == 2) { TQ_APPEND_KV(2, 2); }
    else if (kb == 4 && vb == 2) { TQ_APPEND_KV(4, 2); }
    else if (kb == 3 && vb == 2) { TQ_APPEND_KV(3, 2); }
    else if (kb == 4 && vb == 3) { TQ_APPEND_KV(4, 3); }
    else {  // other pairs: two launches
        const int rc = tqk_append(hk, k, n_seqs, pos, n_new, capacity, in_dtype, TQ_KIND_K, packed_k, s, pos_dev, overrun);
        return rc ? rc : tqk_append(hv, v, n_seqs, pos, n_new, capacity, in_dtype, TQ_KIND_V, packed_v, s, pos_dev, overrun);
    }
#undef TQ_APPEND_KV
    return tq_check_launch("append_kv");
}

int tqk_append(const tq_handle *h, const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype,
               int kind, void *packed, hipStream_t s, const int64_t *pos_dev, uint32_t *overrun) {
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    const AppendArgs a = make_append_args(h, pos, pos_dev, n_new, capacity, kind, overrun);
    const unsigned grid = (unsigned)(n_seqs * a.n_touched);
#define TQ_APPEND_BITS(B) \
    DISPATCH_T(in_dtype, TI, (k_append<B, TI><<<grid, 256, 0, s>>>((const TI *)x, (uint8_t *)packed, a)))
    switch (h->bits) {
    case 2: TQ_APPEND_BITS(2); break;
    case 3: TQ_APPEND_BITS(3); break;
    case 4: TQ_APPEND_BITS(4); break;
    default: tq_set_error("tq_append: bits must be 2, 3 or 4 (got %d)", h->bits); return TQ_ERR_UNSUPPORTED;
    }
#undef TQ_APPEND_BITS
    return tq_check_launch("append");
}

// capacity > 0: the packed buffers are caches laid out for `capacity` tokens per sequence (tq_append's layout) and the
// `tokens` tokens of every sequence go to its first blocks; 0: sequences follow each other at blocks_for(tokens)
int tqk_store_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t tokens,
                 int64_t capacity, int in_dtype, void *packed_k, void *packed_v, hipStream_t s) {
    const int64_t bps = blocks_for(tokens), n_blocks = n_seqs * bps;
    const int64_t out_bps = capacity > 0 ? blocks_for(capacity) : bps;
    if (n_blocks == 0) return TQ_OK;
    if (!store_fast_ok(hk, in_dtype, n_blocks) || !store_fast_ok(hv, in_dtype, n_blocks) || out_bps * n_seqs >= (1ll << 28)) {
        if (out_bps != bps)  // the block-rebuilding append writes the same codes as the butterfly store
            return tqk_append_kv(hk, hv, k, v, n_seqs, 0, tokens, capacity, in_dtype, packed_k, packed_v, s);
        const int rc = tqk_store(hk, k, n_seqs, tokens, in_dtype, TQ_KIND_K, packed_k, nullptr, nullptr, s);
        return rc ? rc : tqk_store(hv, v, n_seqs, tokens, in_dtype, TQ_KIND_V, packed_v, nullptr, nullptr, s);
    }
    StoreKArgs ka = make_k_args(hk, tokens, bps, n_blocks);
    StoreVArgs va = make_v_args(hv, tokens, bps, n_blocks);
    ka.out_blocks_per_seq = va.out_blocks_per_seq = (uint32_t)out_bps;
    va.share_k_lut = hk->bits == 4 && hv->bits == 4 && hk->quant_lut_hash == hv->quant_lut_hash;
    const bool ragged = tokens != bps * TQ_ROWS_PER_BLOCK || out_bps != bps;
    // one workgroup of 12 wavefronts per CU
    const unsigned wg = 768;
    const unsigned grid = (unsigned)((va.n_units + 11) / 12 < 256 ? (va.n_units + 11) / 12 : 256);
    if (in_dtype != TQ_F16) {  // fp32 rows
        if (hk->bits == hv->bits) {
#define TQ_KV32(B)                                                                                                            \
    if (ragged) k_store_kv<B, B, true, float><<<grid, wg, 0, s>>>((const float *)v, (const float *)k, va.n_units, ka.n_units, \
                                                                   (uint8_t *)packed_v, (uint8_t *)packed_k, ka, va);           \
    else k_store_kv<B, B, false, float><<<grid, wg, 0, s>>>((const float *)v, (const float *)k, va.n_units, ka.n_units,       \
                                                             (uint8_t *)packed_v, (uint8_t *)packed_k, ka, va)
            switch (hk->bits) {
            case 2: TQ_KV32(2); break;
            case 3: TQ_KV32(3); break;
            default: TQ_KV32(4); break;
            }
#undef TQ_KV32
            return tq_check_launch("store_kv (fp32 rows)");
        }
        // K and V of different widths: the single-tensor kernels, one launch per tensor
        const int rc = launch_store_k(hk, k, in_dtype, packed_k, ka, ragged, s);
        return rc ? rc : launch_store_v(hv, v, in_dtype, packed_v, va, ragged, s);
    }
#define TQ_KV(KB, VB)                                                                                                       \
    if (ragged) k_store_kv<KB, VB, true><<<grid, wg, 0, s>>>((const __half *)v, (const __half *)k, va.n_units, ka.n_units,  \
                                                              (uint8_t *)packed_v, (uint8_t *)packed_k, ka, va);             \
    else k_store_kv<KB, VB, false><<<grid, wg, 0, s>>>((const __half *)v, (const __half *)k, va.n_units, ka.n_units,        \
                                                        (uint8_t *)packed_v, (uint8_t *)packed_k, ka, va)
#define TQ_KV_V(KB)                      \
    switch (hv->bits) {                  \
    case 2: TQ_KV(KB, 2); break;         \
    case 3: TQ_KV(KB, 3); break;         \
    default: TQ_KV(KB, 4); break;        \
    }
    switch (hk->bits) {
    case 2: TQ_KV_V(2); break;
    case 3: TQ_KV_V(3); break;
    default: TQ_KV_V(4); break;
    }
#undef TQ_KV_V
#undef TQ_KV
    return tq_check_launch("store_kv");
}

// K and V of a layer to fp16 in the original domain.  One launch when both handles hold the fragments of the
// inverse transform, else the two tq_load launches.
int tqk_load_kv(const tq_handle *hk, const tq_handle *hv, const void *packed_k, const void *packed_v, int64_t n_seqs,
                int64_t tokens, void *out_k, void *out_v, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    if (n_seqs * bps == 0) return TQ_OK;
    if (!hk->rfrag16k_inv || !hv->rfrag16k_inv) {
        const int rc = tqk_load(hk, packed_k, n_seqs, tokens, TQ_KIND_K, out_k, TQ_F16, TQ_DOMAIN_ORIGINAL, s);
        return rc ? rc : tqk_load(hv, packed_v, n_seqs, tokens, TQ_KIND_V, out_v, TQ_F16, TQ_DOMAIN_ORIGINAL, s);
    }
    LoadK16Args ak, av;
    ak.afrag = (const uint4 *)hk->rfrag16k_inv; ak.s1 = hk->s1_32; ak.pair_lut = (const uint32_t *)hk->pair_lut;
    ak.tokens = tokens; ak.blocks_per_seq = (uint32_t)bps; ak.bps_div = make_fast_div((uint32_t)bps); ak.n_units = (uint32_t)(n_seqs * bps * 8);
    av.afrag = (const uint4 *)hv->rfrag16k_inv; av.s1 = hv->s1_32; av.pair_lut = (const uint32_t *)hv->pair_lut;
    av.tokens = tokens; av.blocks_per_seq = (uint32_t)bps; av.bps_div = make_fast_div((uint32_t)bps); av.n_units = (uint32_t)(n_seqs * bps * 2);
    unsigned fit = 0;
#define TQ_LKV(KB, VB)                                                                                             \
    {                                                                                                              \
        static const unsigned f = resident_workgroups(k_load_kv16<KB, VB>);                                        \
        fit = f;                                                                                                   \
    }
#define TQ_LKV_V(KB, M)        \
    switch (hv->bits) {        \
    case 2: M(KB, 2); break;   \
    case 3: M(KB, 3); break;   \
    default: M(KB, 4); break;  \
    }
#define TQ_LKV_K(M)                  \
    switch (hk->bits) {              \
    case 2: TQ_LKV_V(2, M); break;   \
    case 3: TQ_LKV_V(3, M); break;   \
    default: TQ_LKV_V(4, M); break;  \
    }
    TQ_LKV_K(TQ_LKV)
    // a workgroup takes one V tile or four K units per turn: no more workgroups than turns
    const int64_t turns = ((int64_t)ak.n_units + 3) / 4 + av.n_units;
    const unsigned grid = (unsigned)std::min<int64_t>(fit, turns);
#define TQ_LKV_GO(KB, VB)                                                                                                \
    k_load_kv16<KB, VB><<<grid, 256, 0, s>>>((const uint8_t *)packed_k, (__half *)out_k, ak, (const uint8_t *)packed_v, \
                                              (__half *)out_v, av)
    TQ_LKV_K(TQ_LKV_GO)
#undef TQ_LKV_GO
#undef TQ_LKV_K
#undef TQ_LKV_V
#undef TQ_LKV
    return tq_check_launch("load_kv16");
}

int tqk_load(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, void *out,
             int out_dtype, int domain, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    if (out_dtype == TQ_F16 && kind == TQ_KIND_V && domain == TQ_DOMAIN_ORIGINAL && h->rfrag16k_inv) {
        LoadK16Args k;
        k.afrag = (const uint4 *)h->rfrag16k_inv; k.s1 = h->s1_32; k.pair_lut = (const uint32_t *)h->pair_lut;
        k.tokens = tokens; k.blocks_per_seq = (uint32_t)bps; k.bps_div = make_fast_div((uint32_t)bps); k.n_units = (uint32_t)(n_seqs * bps * 2);
        static const unsigned fit[3] = {resident_workgroups(k_load_v16<2>), resident_workgroups(k_load_v16<3>),
                                        resident_workgroups(k_load_v16<4>)};
        const unsigned g16 = (unsigned)std::min<int64_t>((int64_t)k.n_units, fit[h->bits - 2]);
        switch (h->bits) {
        case 2: k_load_v16<2><<<g16, 256, 0, s>>>((const uint8_t *)packed, (__half *)out, k); break;
        case 3: k_load_v16<3><<<g16, 256, 0, s>>>((const uint8_t *)packed, (__half *)out, k); break;
        default: k_load_v16<4><<<g16, 256, 0, s>>>((const uint8_t *)packed, (__half *)out, k); break;
        }
        return tq_check_launch("load_v16");
    }
    if (out_dtype == TQ_F16 && kind == TQ_KIND_K && domain == TQ_DOMAIN_ORIGINAL && h->rfrag16k_inv) {
        LoadK16Args k;
        k.afrag = (const uint4 *)h->rfrag16k_inv; k.s1 = h->s1_32; k.pair_lut = (const uint32_t *)h->pair_lut;
        k.tokens = tokens; k.blocks_per_seq = (uint32_t)bps; k.bps_div = make_fast_div((uint32_t)bps); k.n_units = (uint32_t)(n_seqs * bps * 8);
        static const unsigned fit[3] = {resident_workgroups(k_load_k16<2>), resident_workgroups(k_load_k16<3>),
                                        resident_workgroups(k_load_k16<4>)};
        const unsigned g16 = (unsigned)std::min<int64_t>(((int64_t)k.n_units + 3) / 4, fit[h->bits - 2]);
        switch (h->bits) {
        case 2: k_load_k16<2><<<g16, 256, 0, s>>>((const uint8_t *)packed, (__half *)out, k); break;
        case 3: k_load_k16<3><<<g16, 256, 0, s>>>((const uint8_t *)packed, (__half *)out, k); break;
        default: k_load_k16<4><<<g16, 256, 0, s>>>((const uint8_t *)packed, (__half *)out, k); break;
        }
        return tq_check_launch("load_k16");
    }
    LoadArgs a;
    a.s1 = h->s1_32; a.s2 = h->s2_32; a.cent = h->centroids32;
    a.bits = h->bits; a.kind = kind; a.domain = domain;
    a.tokens = tokens; a.blocks_per_seq = bps;
    switch (h->bits) {
    case 2: DISPATCH_T(out_dtype, TO, (k_load<TO, 2><<<grid, 256, 0, s>>>((const uint8_t *)packed, (TO *)out, a))); break;
    case 3: DISPATCH_T(out_dtype, TO, (k_load<TO, 3><<<grid, 256, 0, s>>>((const uint8_t *)packed, (TO *)out, a))); break;
    default: DISPATCH_T(out_dtype, TO, (k_load<TO, 4><<<grid, 256, 0, s>>>((const uint8_t *)packed, (TO *)out, a))); break;
    }
    return tq_check_launch("load");
}

int tqk_unpack_codes(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, uint8_t *idx,
                     float *norms, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    k_unpack_codes<<<grid, 256, 0, s>>>((const uint8_t *)packed, idx, norms, h->bits, kind, tokens, bps);
    return tq_check_launch("unpack_codes");
}

int tqk_q8_0_store(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    if (in_dtype == TQ_F16 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(packed)) & 15u) == 0) {
        k_q8_0_store_f16<<<grid, 256, 0, s>>>((const __half *)x, (uint8_t *)packed, tokens, bps);
        return tq_check_launch("q8_0_store");
    }
    DISPATCH_T(in_dtype, TI, (k_q8_0_store<TI><<<grid, 256, 0, s>>>((const TI *)x, (uint8_t *)packed, tokens, bps)));
    return tq_check_launch("q8_0_store");
}

int tqk_q8_0_store_v(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    if (in_dtype == TQ_F16 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(packed)) & 15u) == 0) {
        k_q8_0_store_v_f16<<<grid, 256, 0, s>>>((const __half *)x, (uint8_t *)packed, tokens, bps);
        return tq_check_launch("q8_0_store_v");
    }
    DISPATCH_T(in_dtype, TI, (k_q8_0_store_v<TI><<<grid, 256, 0, s>>>((const TI *)x, (uint8_t *)packed, tokens, bps)));
    return tq_check_launch("q8_0_store_v");
}

int tqk_q8_0_append(const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype, int kind,
                    void *packed, hipStream_t s, const int64_t *pos_dev, uint32_t *overrun) {
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    const int64_t bps = blocks_for(capacity);
    const int64_t first = pos / TQ_ROWS_PER_BLOCK;
    const int64_t n_touched = pos_dev ? (n_new + TQ_ROWS_PER_BLOCK - 2) / TQ_ROWS_PER_BLOCK + 1  // at the worst alignment
                                      : (pos + n_new - 1) / TQ_ROWS_PER_BLOCK - first + 1;
    const unsigned grid = (unsigned)(n_seqs * n_touched);
    if (kind == TQ_KIND_V) {
        DISPATCH_T(in_dtype, TI, (k_q8_0_append<TI, TQ_KIND_V><<<grid, 256, 0, s>>>((const TI *)x, (uint8_t *)packed, pos, n_new,
                                                                                   bps, first, n_touched, pos_dev, capacity, overrun)));
    } else {
        DISPATCH_T(in_dtype, TI, (k_q8_0_append<TI, TQ_KIND_K><<<grid, 256, 0, s>>>((const TI *)x, (uint8_t *)packed, pos, n_new,
                                                                                   bps, first, n_touched, pos_dev, capacity, overrun)));
    }
    return tq_check_launch("q8_0_append");
}

int tqk_q8_0_unpack(const void *packed, int64_t n_seqs, int64_t tokens, int8_t *q, float *scales, int kind, hipStream_t s) {
    const int64_t bps = blocks_for(tokens);
    const unsigned grid = (unsigned)(n_seqs * bps);
    if (grid == 0) return TQ_OK;
    k_q8_0_unpack<<<grid, 256, 0, s>>>((const uint8_t *)packed, q, scales, tokens, bps, kind);
    return tq_check_launch("q8_0_unpack");
}
