// Attention over packed KV and the prefill-shaped score tile.
//
// k_decode_attn: split-K decode attention for one GQA group of 4 query heads.
//   One 64-lane wavefront owns one context split and walks it in tiles of 64
//   tokens.  Lane l holds packed row l of the tile (K: token l; V: dims l and
//   64+l of all 64 tokens), loaded as 16-byte chunks that are contiguous across
//   lanes.  Codes are turned into fp16 values through a table in LDS: for 2- and
//   3-bit codes a quad table (8-byte entries indexed by the 4*BITS bits of two
//   adjacent pair codes, one ds_read_b64 per four values = one MFMA operand), for
//   4-bit codes a pair table (4-byte entries).  They feed the 4x4x4 fp16 MFMA with
//   16 independent blocks: block b multiplies the 4 tokens 4b..4b+3 by the 4
//   query heads, so all 64 lanes and all 16 blocks do useful work.
//   The MFMA's A-matrix broadcast (cbsz = 4, abid = source block) lets one block's
//   A operand serve all 16 blocks:
//     QK: A = q[4 heads][4 dims] read from block g%16 (each lane keeps only two
//         4-dim slices of q), B_b = K^T[4 dims][tokens 4b..4b+3] -> lane l gets the 4
//         heads' logits of token l; a 4x4 transpose inside each lane quad turns that
//         into head l%4, tokens 4b..4b+3 for the softmax.
//     PV: V rows are dim-major inside the tile (lane l holds dims l and 64+l of the
//         64 tokens), so block b covers dims 4b..4b+3: A = P[4 heads][tokens 4T..4T+3],
//         the fp16 weights held by block T and broadcast, B_b = V[tokens 4T..4T+3][dims
//         4b..4b+3] -> D_b = out[4 heads][4 dims].  16 token groups x 2 dim halves = 32
//         MFMAs per tile into 16 accumulator registers; no cross-lane reduction at the
//         end of the split and no LDS traffic besides the LUT reads.
//   q8_0-style V (VBITS = 8): the same dim-major rows hold int8 values, and the four fp16 scales of a token
//   (one per 32 dims) go into the weights: block b covers dims of one 32-dim block per dim half, so the A
//   operand is broadcast inside each half of the wavefront (cbsz = 3) from weights that were multiplied by that
//   half's scales.
//   Online softmax in base 2 (log2(e) folded into the query scale).  The wavefronts
//   of a workgroup (up to 16 splits) merge their results in LDS and write one partial.
//   The last workgroup of a group to finish merges the group's partials (log-sum-exp), applies the transpose
//   of the V rotation and writes the output rows (merge_group): a step is one launch.  Queries are rotated and
//   scaled inside the kernel.
// k_score_tile: TurboQuant inner-product estimate, 32x32x16 fp16 MFMA over a
//   K = 256 contraction ([R q | S q] against [g c[idx] | scale*rnorm*z]); key operands in registers, queries
//   through LDS, logit rows written 64 consecutive logits per store.
#include <atomic>
#include <mutex>
#include <cstring>
#include <type_traits>
#include <utility>

#include "tq_device.h"

namespace {

using namespace tqd;

constexpr float LOG2E = 1.4426950408889634f;
constexpr float RSQRT128 = 0.08838834764831845f;

template <typename T> __device__ inline float ldf(const T *p) { return (float)*p; }
template <> __device__ inline float ldf<__half>(const __half *p) { return __half2float(*p); }

template <int BITS> __device__ __forceinline__ uint32_t pair_off(const uint32_t (&w)[4 * BITS], int p) {
    return pair_lut_offset<BITS>(w, p);
}

// TQ_PAIRTAB3 (tq_measure.h; measurement builds only): 3-bit codes decode through a pair table with one copy
// per LDS bank (entry e of lane l at dword 64 e + l: no bank conflicts, two 4-byte reads per four values)
// instead of the 4096-entry quad table (one 8-byte read per four values, about 1.6 conflicts per read).
// bytes of the decode table of a codebook: quad entries for BITS <= 3, pair entries for 4
__host__ __device__ constexpr int lut_bytes(int bits) {
    if (TQ_PAIRTAB3 && bits == 3) return 64 * 64 * 4;
    return bits == 8 ? 0 : bits <= 3 ? 8 << (4 * bits) : 4 << (2 * bits);  // 8: int8 rows, no table
}

// the four values of quad Q (pairs 2Q, 2Q+1) of a row as an MFMA operand
template <int BITS> __device__ __forceinline__ half4_t quad_values(const uint32_t (&w)[4 * BITS], const char *lut, int Q) {
    if constexpr (TQ_PAIRTAB3 && BITS == 3) {
        // lut already points at this lane's bank (+ 4 * lane); a pair code selects the 256-byte row
        const uint32_t o0 = pair_lut_offset<BITS>(w, 2 * Q) << 6, o1 = pair_lut_offset<BITS>(w, 2 * Q + 1) << 6;
        const uint2 u = make_uint2(*reinterpret_cast<const uint32_t *>(lut + o0), *reinterpret_cast<const uint32_t *>(lut + o1));
        return __builtin_bit_cast(half4_t, u);
    } else if constexpr (BITS <= 3) {
        return __builtin_bit_cast(half4_t, *reinterpret_cast<const uint2 *>(lut + quad_lut_offset<BITS>(w, Q)));
    } else {
        const uint2 u = make_uint2(*reinterpret_cast<const uint32_t *>(lut + pair_lut_offset<BITS>(w, 2 * Q)),
                                   *reinterpret_cast<const uint32_t *>(lut + pair_lut_offset<BITS>(w, 2 * Q + 1)));
        return __builtin_bit_cast(half4_t, u);
    }
}

// build a codebook's decode table in LDS from its pair table (half2 per pair code) with n_waves wavefronts;
// `mine` is pair entry tid % 64, fetched by the caller ahead of time (used by the 3-bit table only)
template <int BITS>
__device__ __forceinline__ void build_lut(char *dst, const uint32_t *pair_lut, uint32_t mine, int tid, int n_waves) {
    constexpr int NP = 1 << (2 * BITS);
    if constexpr (TQ_PAIRTAB3 && BITS == 3) {
        uint32_t *t = reinterpret_cast<uint32_t *>(dst);
        const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        for (int e = wave; e < 64; e += n_waves) t[e * 64 + lane] = (uint32_t)__builtin_amdgcn_readlane((int)mine, e);
    } else if constexpr (BITS == 3) {
        // lane l holds pair entry l; wavefront w writes the rows hi = w, w + n_waves, ..
        uint2 *t = reinterpret_cast<uint2 *>(dst);
        const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        for (int hi = wave; hi < 64; hi += n_waves)
            t[hi * 64 + lane] = make_uint2(mine, (uint32_t)__builtin_amdgcn_readlane((int)mine, hi));
    } else if constexpr (BITS == 2) {
        for (int e = tid; e < 256; e += 64 * n_waves)
            reinterpret_cast<uint2 *>(dst)[e] = make_uint2(pair_lut[e & 15], pair_lut[e >> 4]);
    } else {
        static_assert(NP == 256, "pair table of 256 entries");
        for (int e = tid; e < 256; e += 64 * n_waves) reinterpret_cast<uint32_t *>(dst)[e] = pair_lut[e];
    }
}

// raise a progress mark in LDS to `mine` and return what it held before (one atomic per wavefront)
__device__ __forceinline__ uint32_t lead_progress(uint32_t *mark, uint32_t mine, int lane) {
    uint32_t t = 0;
    if (lane == 0) t = atomicMax(mark, mine);
    return __builtin_amdgcn_readfirstlane(t);
}

template <int BITS> __device__ __forceinline__ void load_row(const uint8_t *block, int row, uint32_t (&w)[4 * BITS]) {
#pragma unroll
    for (int c = 0; c < BITS; ++c) {
        const uint4 u = stream_load<STREAM_ATTN_ROWS>(reinterpret_cast<const uint4 *>(block + c * 2048 + row * 16));
        w[4 * c] = u.x; w[4 * c + 1] = u.y; w[4 * c + 2] = u.z; w[4 * c + 3] = u.w;
    }
}

__device__ __forceinline__ float4_t mfma4(half4_t a, half4_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 0, 0, 0);
}

// 4x4x4 MFMA whose A operand is taken from block ABID and broadcast to all 16 blocks
template <int ABID> __device__ __forceinline__ float4_t mfma4_bcast(half4_t a, half4_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 4, ABID, 0);
}

// the same with the A operand taken from block ABID of each group of 8 blocks (lanes 0..31 and 32..63 apart)
template <int ABID> __device__ __forceinline__ float4_t mfma4_bcast8(half4_t a, half4_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(a, b, c, 3, ABID, 0);
}

// four int8 of a dword as fp16, in the order 0, 2, 1, 3: 0x6400 | (x + 128) is the fp16 number 1024 + (x + 128),
// exactly, so a byte permute builds two of them at once and one packed fp16 subtraction of 1152 leaves (x0, x2)
// and (x1, x3)
__device__ __forceinline__ half4_t int8x4_to_half_0213(uint32_t w) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const uint32_t u = w ^ 0x80808080u;
    const half2_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    const half2_t h02 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u, 0x04020400u)) - bias;
    const half2_t h13 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, u, 0x04030401u)) - bias;
    half4_t kv;
    kv[0] = h02[0];
    kv[1] = h02[1];
    kv[2] = h13[0];
    kv[3] = h13[1];
    return kv;
}

// transpose the 4x4 matrix held by a quad of lanes (element [lane%4][register]), two exchange stages
__device__ __forceinline__ void quad_transpose(float (&r)[4], int lane) {
    const bool b0 = lane & 1, b1 = lane & 2;
#pragma unroll
    for (int p = 0; p < 4; p += 2) {  // swap (even lane, odd reg) <-> (odd lane, even reg)
        const float give = b0 ? r[p] : r[p + 1];
        const float got = xor_lane<1>(give);
        if (b0) r[p] = got;
        else r[p + 1] = got;
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {     // swap (lane bit1 clear, reg p+2) <-> (lane bit1 set, reg p)
        const float give = b1 ? r[p] : r[p + 2];
        const float got = xor_lane<2>(give);
        if (b1) r[p] = got;
        else r[p + 2] = got;
    }
}

// sum over the 16 lanes that share lane%4 (blocks b = 0..15)
__device__ __forceinline__ float sum_over_blocks(float v) {
    v += xor_lane<4>(v);
    v += xor_lane<8>(v);
    v += xor_lane<16>(v);
    v += xor_lane<32>(v);
    return v;
}
__device__ __forceinline__ float max_over_blocks(float v) {
    v = fmaxf(v, xor_lane<4>(v));
    v = fmaxf(v, xor_lane<8>(v));
    v = fmaxf(v, xor_lane<16>(v));
    v = fmaxf(v, xor_lane<32>(v));
    return v;
}

struct AttnArgs {
    const void *q;       // [groups*4][128] queries in the original domain, q_dtype
    int q_dtype;
    const float *ks1, *ks2;  // K rotation signs (NULL: K is not rotated, q is only scaled)
    float scale_log2e;       // logit scale * log2(e), folded into the fp16 query
    const uint8_t *k, *v;
    const uint32_t *klut, *vlut;  // pair tables (half2 per pair code)
    const float *bias;            // [groups*4][tokens] natural-log units, or NULL
    const int32_t *sbias_pos;     // sparse bias: [groups*q_group][sbias_n] positions, ascending within a head (entries that
    const float *sbias_val;       // do not exist: any position >= tokens), and their values (natural-log units)
    int sbias_n;                  // entries per head, 0 = no sparse bias
    float *part_o;                // [groups][workgroups per group][4][128]
    float *part_ml;               // [groups][workgroups per group][4][2]  (m in log2 units, l)
    unsigned long long *skip_slots;  // Sparse V: [workgroup] nonce tag | (query, position) pairs it skipped; 0 after the count
    // merge of the workgroups' partials by the last workgroup of a group to finish (see merge_group)
    float *out;                      // [groups * q_group][128]
    const float *vs1, *vs2;          // V rotation signs (NULL: V rows are stored unrotated)
    unsigned long long *flags;       // [group][workgroups per group]; word 0 of a group is its arrival counter (tag | count), 0 after the merge
    unsigned long long nonce;        // differs from call to call (and from whatever the workspace held before)
    int poll_slots;                       // Sparse V: the merging workgroups add the slots up themselves
    unsigned long long *pass_totals;      // Sparse V: [pass] skipped pairs of each four-head pass of this step
    unsigned long long *skip_count;       // caller's {skipped, total} or NULL
    unsigned long long total_pairs;
    int pass;                             // head_off / 4
    int64_t tokens, blocks_per_seq;
    const int64_t *tokens_dev;  // NULL, or where the step's context length is read from (<= tokens, which then is the maximum)
    int n_groups, n_splits, tiles_per_split, n_tiles;
    int q_group, head_off;  // query heads per KV head; first of the (up to) four heads this launch works on
    int d256;               // heads of 256 dims: a token is two 128-value rows (2 token + half) of the K and V caches
    int gpw;                // (batch, kv head) groups per workgroup: 1, or wavefronts per workgroup / n_splits when a group's
                            // splits are fewer than a workgroup's wavefronts (short contexts: the groups share the decode tables)
    int gw_shift;           // gpw > 1: log2(n_splits), a power of two then
    int wgs_per_group;      // gpw == 1: n_splits / wavefronts per workgroup
    float tau;
};

constexpr int KFMT_TURBO = 0, KFMT_Q8 = 1;
constexpr unsigned long long SKIP_COUNT_MASK = (1ull << 40) - 1ull;  // count bits of a Sparse-V slot; the rest is a nonce tag
constexpr int MERGE_FLOATS = 520;  // LDS floats per wavefront for the end-of-kernel merge: out[4][128], m[4], l[4]

// QK over the 32 dim groups: B = this lane's K row (4 dims per group), A = q from block G % 16
// (HG sets of four query heads share every dequantised operand: one table look-up, HG products)
template <int BITS, int HG, int... G>
__device__ __forceinline__ void qk_turbo(std::integer_sequence<int, G...>, const uint32_t (&kw)[4 * BITS],
                                         const char *lut, const half4_t (&qa)[HG][2], float4_t (&acc)[HG][4]) {
    (([&] {
         const half4_t kv = quad_values<BITS>(kw, lut, G);
#pragma unroll
         for (int hg = 0; hg < HG; ++hg) acc[hg][G & 3] = mfma4_bcast<(G & 15)>(qa[hg][G >> 4], kv, acc[hg][G & 3]);
     }()),
     ...);
}

// Heads of 256 dims: the lower half of the wavefront holds the rows of the tile's 32 tokens' first 128 dims, the
// upper half the rows of their second 128 dims, and each half takes its half of the query from its own blocks
// (A broadcast inside a half-wavefront, block G % 8; a lane keeps four dim groups)
template <int BITS, int... G>
__device__ __forceinline__ void qk_turbo_d256(std::integer_sequence<int, G...>, const uint32_t (&kw)[4 * BITS],
                                              const char *lut, const half4_t (&qa4)[4], float4_t (&acc)[4]) {
    (([&] {
         const half4_t kv = quad_values<BITS>(kw, lut, G);
         acc[G & 3] = mfma4_bcast8<(G & 7)>(qa4[G >> 3], kv, acc[G & 3]);
     }()),
     ...);
}

template <int... G>
__device__ __forceinline__ void qk_q8_d256(std::integer_sequence<int, G...>, const uint32_t (&kw)[32], const half4_t (&qa4)[4],
                                           float4_t (&acc)[4]) {
    (([&] {
         const half4_t kv = int8x4_to_half_0213(kw[G]);
         acc[G >> 3] = mfma4_bcast8<(G & 7)>(qa4[G >> 3], kv, acc[G >> 3]);
     }()),
     ...);
}

// ... and V rows whose 64 "tokens" are (token, half) pairs: quad T holds the rows of tokens 2T, 2T+1 in the order
// (2T, 0), (2T, 1), (2T+1, 0), (2T+1, 1).  The weights of tokens 4b..4b+3 sit in block b, so quad T takes them from
// block T / 2, with zeros in the places of the other half: one look-up feeds the output's two halves.
template <int BITS, int... T>
__device__ __forceinline__ void pv_all_d256(std::integer_sequence<int, T...>, const uint32_t (&vw)[4 * BITS], const char *lut,
                                            const half4_t (&pv_even)[2], const half4_t (&pv_odd)[2], float4_t (&acc_o)[2][2][2]) {
    (([&] {
         const half4_t v0 = quad_values<BITS>(vw, lut, 2 * T), v1 = quad_values<BITS>(vw, lut, 2 * T + 1);
#pragma unroll
         for (int dh = 0; dh < 2; ++dh) {
             const half4_t w = (T & 1) ? pv_odd[dh] : pv_even[dh];
             acc_o[dh][0][T & 1] = mfma4_bcast<(T >> 1)>(w, v0, acc_o[dh][0][T & 1]);
             acc_o[dh][1][T & 1] = mfma4_bcast<(T >> 1)>(w, v1, acc_o[dh][1][T & 1]);
         }
     }()),
     ...);
}

// q8_0-style K: one accumulator per 32-value block (dim groups 8*blk .. 8*blk+7), scaled afterwards
template <int HG, int... G>
__device__ __forceinline__ void qk_q8(std::integer_sequence<int, G...>, const uint32_t (&kw)[32],
                                      const half4_t (&qa)[HG][2], float4_t (&acc)[HG][4]) {
    // the values of a dim group come out in the order 0, 2, 1, 3; the kernel parks its queries in the same order
    (([&] {
         const half4_t kv = int8x4_to_half_0213(kw[G]);
#pragma unroll
         for (int hg = 0; hg < HG; ++hg) acc[hg][G >> 3] = mfma4_bcast<(G & 15)>(qa[hg][G >> 4], kv, acc[hg][G >> 3]);
     }()),
     ...);
}

// PV over the 16 token groups x 2 dim halves: A = weights of block T (broadcast), B = this lane's V row
template <int BITS, int HG, int... T>
__device__ __forceinline__ void pv_all(std::integer_sequence<int, T...>, const uint32_t (&vw)[4 * BITS],
                                       const char *lut, const half4_t (&pv)[HG], float4_t (&acc_o)[HG][2][2]) {
    // tokens 4T..4T+3 of dim half hf are quad 2T + hf of the row
    (([&] {
         const half4_t v0 = quad_values<BITS>(vw, lut, 2 * T), v1 = quad_values<BITS>(vw, lut, 2 * T + 1);
#pragma unroll
         for (int hg = 0; hg < HG; ++hg) {
             acc_o[hg][0][T & 1] = mfma4_bcast<T>(pv[hg], v0, acc_o[hg][0][T & 1]);
             acc_o[hg][1][T & 1] = mfma4_bcast<T>(pv[hg], v1, acc_o[hg][1][T & 1]);
         }
     }()),
     ...);
}

// q8_0-style V rows: dword 16*hf + T of the row = tokens 4T..4T+3 of dim half hf as int8.  a_lo / a_hi: the weights
// (times the scales of this half-wavefront's 32-dim block of dim half hf) that token groups T < 8 / T >= 8 take
// from block T % 8 of each half-wavefront.
template <int HG, int... T>
__device__ __forceinline__ void pv_all_q8(std::integer_sequence<int, T...>, const uint32_t (&vw)[32],
                                          const half4_t (&a_lo)[HG][2], const half4_t (&a_hi)[HG][2],
                                          float4_t (&acc_o)[HG][2][2]) {
    (([&] {
         const half4_t v0 = int8x4_to_half_0213(vw[T]), v1 = int8x4_to_half_0213(vw[16 + T]);
#pragma unroll
         for (int hg = 0; hg < HG; ++hg) {
             acc_o[hg][0][T & 1] = mfma4_bcast8<(T & 7)>(T < 8 ? a_lo[hg][0] : a_hi[hg][0], v0, acc_o[hg][0][T & 1]);
             acc_o[hg][1][T & 1] = mfma4_bcast8<(T & 7)>(T < 8 ? a_lo[hg][1] : a_hi[hg][1], v1, acc_o[hg][1][T & 1]);
         }
     }()),
     ...);
}

// q8_0-style V rows under heads of 256 dims: dword 16*hf + T = rows 4T..4T+3 = (token 2T, half 0), (2T, 1), (2T+1, 0),
// (2T+1, 1) of dim half hf, handed over in the order 0, 2, 1, 3.  a8[dh][hf][T & 1]: the weights of tokens 2T, 2T+1
// times the scales of their rows of half dh (for this half-wavefront's 32-dim block of dim half hf) in the places of
// that half's rows, zeros in the others; both half-wavefronts hold the same 32 tokens, so token pair T is served by
// block T / 2 of either half with its own scales.
template <int... T>
__device__ __forceinline__ void pv_all_q8_d256(std::integer_sequence<int, T...>, const uint32_t (&vw)[32],
                                               const half4_t (&a8)[2][2][2], float4_t (&acc_o)[2][2][2]) {
    (([&] {
         const half4_t v0 = int8x4_to_half_0213(vw[T]), v1 = int8x4_to_half_0213(vw[16 + T]);
#pragma unroll
         for (int dh = 0; dh < 2; ++dh) {
             acc_o[dh][0][T & 1] = mfma4_bcast8<(T >> 1)>(a8[dh][0][T & 1], v0, acc_o[dh][0][T & 1]);
             acc_o[dh][1][T & 1] = mfma4_bcast8<(T >> 1)>(a8[dh][1][T & 1], v1, acc_o[dh][1][T & 1]);
         }
     }()),
     ...);
}

// per-tile side data of the V rows: turbo = the fp16 norms of this lane's four tokens; q8_0-style = the fp16 scales
// [2 * dim half + swapped]: of this lane's four tokens (0) and of the four tokens of lane ^ 32 (1), for the 32-dim
// block that this lane's dims of that dim half lie in
// heads of 256 dims: the eight fp16 norms of the rows of this lane's four tokens (v[0], v[1]); q8_0-style: the eight
// scales of those rows for the 32-dim block of this lane's dims of dim half hf (v[2 hf], v[2 hf + 1])
template <int VBITS> struct VSide { uint2 v[VBITS == 8 ? 4 : 2]; };

constexpr unsigned long long ARRIVAL_COUNT_MASK = 0xFFFFFFull;  // workgroups of a group (the tag of the call sits above)
constexpr float Q8V_PRESCALE = 64.0f;  // keeps weight * scale products out of fp16's subnormals; 65504 / 64 > any scale

// ---- merging the workgroups' partials inside the launch -------------------------------------
// A group's partials are written by up to n_splits / wavefronts-per-workgroup workgroups that may run on
// different dies, whose L2 caches are not coherent with each other for ordinary accesses.  Everything the
// workgroups exchange therefore moves with device-scope atomic accesses (they go through to memory): a workgroup
// stores its partial, waits for the stores to complete, and then increments the group's arrival counter with one
// read-modify-write; the workgroup whose increment completes the count merges the group.  The counter carries a tag
// of the call, so what a fresh workspace happens to contain is not mistaken for arrivals, and the merging workgroup
// puts it back to zero, so a replay of a captured launch (same tag) starts clean.  No cache-wide write-back or
// invalidate is involved, which is what made a merge behind device-scope fences cost more than the second launch it
// saved.  (An earlier version raised a flag per workgroup and read the group's flags: two more trips to memory per
// workgroup, and "somebody sees every flag" needed a store-to-load ordering argument where the counter needs none.)
__device__ __forceinline__ void st_dev(float *p, float v) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev(unsigned long long *p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long ld_dev(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 ld_dev2(const float *p) {  // 8-byte aligned pair
    const unsigned long long u = ld_dev(reinterpret_cast<const unsigned long long *>(p));
    return make_float2(__uint_as_float((uint32_t)u), __uint_as_float((uint32_t)(u >> 32)));
}
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Log-sum-exp merge of a group's n_parts partials, transpose of the V rotation, output rows; one wavefront per
// query head (the partials come straight from memory: every load of a head is issued before the first is used
// when there are at most four).
// The partials [p_lo, p_hi) of one head of a group, merged by one wavefront: running maximum M (log2 units), weight
// sum L and this lane's two output dims, all relative to M.  Up to 16 partials have every load requested before the
// first is used, so the merge costs one trip to memory (in batches of four, sixteen partials took four trips at the
// very end of the launch).
struct MergedPart {
    float M, L, o0, o1;
};
__device__ __forceinline__ MergedPart merge_range(const float *ml0, const float *po0, int ML, int PO, int head, int p_lo, int p_hi,
                                                  int lane) {
    MergedPart r{-INFINITY, 0.0f, 0.0f, 0.0f};
    const int n = p_hi - p_lo;
    auto merge_few = [&](auto np_tag) {
        constexpr int NP = decltype(np_tag)::value;
        float2 ml[NP], v[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int pc = p_lo + (p < n ? p : 0);
            ml[p] = ld_dev2(ml0 + pc * ML + head * 2);
            v[p] = ld_dev2(po0 + (int64_t)pc * PO + head * 128 + 2 * lane);
            if (p >= n) ml[p].y = 0.0f;
        }
#pragma unroll
        for (int p = 0; p < NP; ++p)
            if (ml[p].y > 0.0f) r.M = fmaxf(r.M, ml[p].x);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const float w = ml[p].y > 0.0f ? exp2f(ml[p].x - r.M) : 0.0f;
            r.L = fmaf(ml[p].y, w, r.L);
            r.o0 = fmaf(v[p].x, w, r.o0);
            r.o1 = fmaf(v[p].y, w, r.o1);
        }
    };
    if (n <= 0) return r;
    if (n <= 4) {
        merge_few(std::integral_constant<int, 4>{});
    } else if (n <= 16) {
        merge_few(std::integral_constant<int, 16>{});
    } else {
        for (int p0 = p_lo; p0 < p_hi; p0 += 64) {  // lane <-> partial: maximum, then weights
            const int p = p0 + lane;
            float m = -INFINITY;
            if (p < p_hi) {
                const float2 e = ld_dev2(ml0 + p * ML + head * 2);
                if (e.y > 0.0f) m = e.x;
            }
            for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
            r.M = fmaxf(r.M, m);
        }
        for (int p0 = p_lo; p0 < p_hi; p0 += 64) {
            const int p = p0 + lane;
            float w = 0.0f, l = 0.0f;
            if (p < p_hi) {
                const float2 e = ld_dev2(ml0 + p * ML + head * 2);
                l = e.y;
                w = l > 0.0f ? exp2f(e.x - r.M) : 0.0f;
            }
            float lw = l * w;
            for (int o = 32; o > 0; o >>= 1) lw += __shfl_xor(lw, o);
            r.L += lw;
            const int cnt = min(64, p_hi - p0);
            // eight partials per trip to memory (a lane exchange cannot sit in a loop that the compiler unrolls with
            // a remainder, so the batches are written out: past the count the last partial is read again with weight 0)
            for (int t0 = 0; t0 < cnt; t0 += 8) {
                float2 v[8];
                float wt[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int t = min(t0 + k, cnt - 1);
                    v[k] = ld_dev2(po0 + (int64_t)(p0 + t) * PO + head * 128 + 2 * lane);
                    wt[k] = t0 + k < cnt ? __shfl(w, t) : 0.0f;
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    r.o0 = fmaf(v[k].x, wt[k], r.o0);
                    r.o1 = fmaf(v[k].y, wt[k], r.o1);
                }
            }
        }
    }
    return r;
}

// The group's partials -> output rows (log-sum-exp merge, then the V rotation's transpose).  A workgroup with at least
// twice as many wavefronts as the pass has heads gives every head several wavefronts, each merging a share of the
// partials, and joins their results through `lds` (free LDS of 132 floats per wavefront; unused otherwise): the merge
// runs at the very end of the launch, so its trips to memory are the launch's tail.
template <int HG>
__device__ __forceinline__ void merge_group(const AttnArgs &a, int group, int n_parts, int tid, int n_waves, float *lds) {
    constexpr int NH = 4 * HG, ML = 2 * NH, PO = 128 * NH;  // heads, (m, l) floats and output floats of one partial
    const int lane = tid & 63, wave = tid >> 6;
    const float *ml0 = a.part_ml + (int64_t)group * n_parts * ML;
    const float *po0 = a.part_o + (int64_t)group * n_parts * PO;
    auto finish = [&](int head, MergedPart r) {
        // heads of 256 dims (HG = 2): partial row 4 dh + i is dims 128 dh .. 128 dh + 127 of head i
        const int hq = a.d256 ? (head & 3) : head;
        const int64_t r_out = a.d256 ? 2 * ((int64_t)group * a.q_group + a.head_off + hq) + (head >> 2)
                                     : (int64_t)group * a.q_group + a.head_off + head;
        const float invL = r.L > 0.0f ? 1.0f / r.L : 0.0f;
        float o0 = r.o0, o1 = r.o1;
        float2 res;
        if (!a.vs1) {  // V rows were stored unrotated
            res = make_float2(o0 * invL, o1 * invL);
        } else {
            const float2 s1v = *reinterpret_cast<const float2 *>(a.vs1 + 2 * lane);
            const float2 s2v = *reinterpret_cast<const float2 *>(a.vs2 + 2 * lane);
            o0 *= invL * s2v.x;
            o1 *= invL * s2v.y;
            wht128_wave(o0, o1, lane);
            res = make_float2(o0 * (s1v.x * RSQRT128), o1 * (s1v.y * RSQRT128));
        }
        *reinterpret_cast<float2 *>(a.out + r_out * 128 + 2 * lane) = res;
    };
    // a repeated head of a group with fewer than four left is not written
    auto head_exists = [&](int head) { return a.head_off + (a.d256 ? (head & 3) : head) < a.q_group; };
    const int n_sub = lds && n_waves >= 2 * NH && n_parts > 4 ? n_waves / NH : 1;
    if (n_sub == 1) {
        for (int head = wave; head < NH; head += n_waves)
            if (head_exists(head)) finish(head, merge_range(ml0, po0, ML, PO, head, 0, n_parts, lane));
        return;
    }
    const int head = wave % NH, sub = wave / NH;
    const int per = (n_parts + n_sub - 1) / n_sub;
    const bool mine = sub < n_sub && head_exists(head);
    MergedPart r{-INFINITY, 0.0f, 0.0f, 0.0f};
    if (mine) r = merge_range(ml0, po0, ML, PO, head, min(sub * per, n_parts), min(sub * per + per, n_parts), lane);
    float *slot = lds + (head * n_sub + (sub < n_sub ? sub : 0)) * 132;
    if (mine) {
        *reinterpret_cast<float2 *>(slot + 2 * lane) = make_float2(r.o0, r.o1);
        if (lane == 0) {
            slot[128] = r.M;
            slot[129] = r.L;
        }
    }
    __syncthreads();
    if (mine && sub == 0) {
        const float *s0 = lds + head * n_sub * 132;
        float M = -INFINITY;
        for (int k = 0; k < n_sub; ++k)
            if (s0[k * 132 + 129] > 0.0f) M = fmaxf(M, s0[k * 132 + 128]);
        MergedPart t{M, 0.0f, 0.0f, 0.0f};
        for (int k = 0; k < n_sub; ++k) {
            const float l = s0[k * 132 + 129];
            const float w = l > 0.0f ? exp2f(s0[k * 132 + 128] - M) : 0.0f;
            const float2 o = *reinterpret_cast<const float2 *>(s0 + k * 132 + 2 * lane);
            t.L = fmaf(l, w, t.L);
            t.o0 = fmaf(o.x, w, t.o0);
            t.o1 = fmaf(o.y, w, t.o1);
        }
        finish(head, t);
    }
}


// sum over the workgroup of one 64-bit value per thread (every thread gets the total); red: one shared word
__device__ __forceinline__ unsigned long long block_sum(unsigned long long t, unsigned long long *red, int tid) {
    if (tid == 0) *red = 0ull;
    __syncthreads();
    for (int o = 32; o > 0; o >>= 1) t += __shfl_xor(t, o);
    if ((tid & 63) == 0 && t) atomicAdd(red, t);
    __syncthreads();
    return *red;
}

// SHARE: K and V decode through one table (same width, same centroids); table positions are
// compile-time constants so that they fold into the LDS instructions' offset fields.
//
// Work distribution: a workgroup of W wavefronts (W = blockDim / 64 divides n_splits) owns W
// consecutive splits of one group, one split per wavefront (a fixed share, so results do not
// depend on timing).  The hardware favours the oldest wavefronts of a SIMD, and left alone
// the youngest finish late and alone on a memory system that needs every wavefront's loads
// in flight to stay busy.  So the wavefronts of a workgroup publish their progress in LDS and
// each sets its own issue priority to how many tiles it is behind the leader (at most 3):
// they finish within a tile or two of each other.
// int8 V rows take 32 registers instead of 8 to 16: those variants run with at most 8 wavefronts per workgroup,
// which leaves each more than the 128 registers of a 16-wavefront workgroup.
// Two sets of four query heads per pass (HG = 2: GQA groups of more than four heads read K/V once per eight heads)
// double the accumulators and the softmax state and run with at most 8 wavefronts too.
// Wavefronts per workgroup that a variant is compiled for (its register budget follows: 16 -> 128, 12 -> 168, 8 -> 256).
// wide12: eight heads per pass on turbo K and V rows of 128-dim heads without a bias list - 145-165 registers, so twelve
// wavefronts (three per SIMD) fit where two workgroups of eight do not.
__host__ __device__ constexpr int max_waves_per_workgroup(int vbits, int hg, bool wide12 = false) {
    return vbits == 8 ? 8 : hg == 2 ? (wide12 ? 12 : 8) : 16;
}

// SBIAS: the call carries a sparse logit bias (a.sbias_n > 0).  A template parameter and not a branch: the cursor
// registers and the per-tile test cost the eight-head variant 4 us per step when they were compiled in unconditionally.
// D256: heads of 256 dims.  A token is rows 2 token and 2 token + 1 of caches that are
// otherwise those of 128-dim heads with twice the tokens; a 64-row tile is 32 tokens.  The two sets of HG = 2 are
// then the output's two halves of one set of four heads: one softmax, two accumulator sets.
template <int KFMT, int KBITS, int VBITS, bool SPARSE, bool SHARE, int HG, bool SBIAS, bool D256 = false>
__global__ __launch_bounds__(64 * max_waves_per_workgroup(VBITS, HG, KFMT == KFMT_TURBO && !D256 && !SBIAS),
                             D256 && KFMT == KFMT_TURBO && VBITS != 8 ? 4 : 1) void k_decode_attn(AttnArgs a) {
    // (256-dim heads on turbo K rows: four wavefronts per SIMD = two workgroups of eight per CU, i.e. at most 128 registers - the
    // variant sits at 119-136 without the bound, and one register over 128 halves its occupancy)
    static_assert(!D256 || HG == 2, "256-dim heads: two accumulator sets, the output's halves");
    constexpr int HQ = D256 ? 1 : HG;   // sets of four heads whose logits and softmax state the wavefront keeps
    constexpr int KROW_DW = KFMT == KFMT_TURBO ? 4 * KBITS : 32;
    constexpr int KBLOCK = KFMT == KFMT_TURBO ? TQ_ROWS_PER_BLOCK * (16 * KBITS + 2) : TQ_ROWS_PER_BLOCK * 136;
    constexpr int VBLOCK = VBITS == 8 ? TQ_ROWS_PER_BLOCK * 136 : TQ_ROWS_PER_BLOCK * (16 * VBITS + 2);
    constexpr int KLUT_BYTES = KFMT == KFMT_TURBO ? lut_bytes(KBITS) : 0;
    static_assert(!SHARE || (KFMT == KFMT_TURBO && KBITS == VBITS), "a shared table needs equal code widths");
    // static LDS (its address is a compile-time constant, so table positions fold into the LDS
    // instructions): [K table][V table unless shared with K], and 1 KB per set of four heads that stages the
    // group's rotated queries (a region of its own: the tables are built while the queries are still on their way)
    constexpr int LUT_TOTAL = KLUT_BYTES + (SHARE ? 0 : lut_bytes(VBITS));
    __shared__ __attribute__((aligned(16))) char smem[LUT_TOTAL > 16 ? LUT_TOTAL : 16];
    __shared__ uint32_t lead;  // tiles finished by the wavefront that is furthest ahead
    __shared__ uint32_t skipped;  // Sparse V: (query, position) pairs skipped by this workgroup
    char *klut_s = smem;
    char *vlut_s = SHARE ? klut_s : klut_s + KLUT_BYTES;

    const int tid = threadIdx.x, lane = tid & 63;
    // workgroup-uniform values in scalar registers: tile loop, block addresses and bounds become scalar work
    const int n_waves = (int)(blockDim.x >> 6), wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Wavefronts of this workgroup that work on one group: all of them, or - short contexts, a.gpw groups per
    // workgroup - as many as the group has splits; wave_g numbers them, tid_g their threads.
    // (shifts and masks prepared by the host: an integer division here is a few dozen instructions in front of the
    // first row request, which showed as half a microsecond per launch)
    const int gw = a.gpw > 1 ? a.n_splits : n_waves;
    const int wave_g = a.gpw > 1 ? (wave & (gw - 1)) : wave, wave0 = wave - wave_g;
    const int gidx = a.gpw > 1 ? (wave >> a.gw_shift) : 0;   // this wavefront's group among the workgroup's
    const int tid_g = tid - 64 * wave0;
    const int wgs_per_group = a.wgs_per_group;
    const int group = __builtin_amdgcn_readfirstlane(a.gpw > 1 ? (int)blockIdx.x * a.gpw + gidx : (int)(blockIdx.x / wgs_per_group));
    const int part = a.gpw > 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(blockIdx.x % wgs_per_group));
    const int split = part * n_waves + wave_g;  // index of this wavefront's partial
    // dynamic LDS: the wavefronts' merge space (end of the split), then 1 KB per group and set of four heads that
    // stages the rotated queries
    extern __shared__ float merge_s[];
    char *q_stage = reinterpret_cast<char *>(merge_s) + (n_waves > 1 ? (size_t)n_waves * HG * MERGE_FLOATS * sizeof(float) : 0) +
                    (size_t)gidx * (1024 * HG);
    // The context length: a kernel argument, or read from memory when the caller replays one captured launch at
    // changing lengths (the split geometry then follows the length; a.tokens stays the bias rows' stride).
    int tokens_now = (int)a.tokens, n_tiles = a.n_tiles, tiles_per_split = a.tiles_per_split;
    if (a.tokens_dev) {
        const int64_t t = *a.tokens_dev;
        tokens_now = __builtin_amdgcn_readfirstlane((int)(t < 0 ? 0 : (t < a.tokens ? t : a.tokens)));
        n_tiles = ((D256 ? 2 : 1) * tokens_now + 63) >> 6;
        tiles_per_split = (n_tiles + a.n_splits - 1) / a.n_splits;
    }
    const int rows_now = (D256 ? 2 : 1) * tokens_now;   // rows of the caches that hold the context
    const int t_begin = split * tiles_per_split;
    const int t_end = min(t_begin + tiles_per_split, n_tiles);
    const int b4 = lane & ~3;  // 4 * block index
    const int j = lane & 3;    // query head of the logits this lane holds; sub-row for V
    // K row of the tile that this lane owns, and the tile row of element i of its logits (e4 + es * i)
    const int krow = D256 ? 2 * (lane & 31) + (lane >> 5) : lane;
    const int e4 = D256 ? 2 * (b4 & 31) : b4, es = D256 ? 2 : 1;
    // tokens per tile, and the first of this lane's four tokens inside the tile
    constexpr int TT = D256 ? 32 : 64;
    const int t4 = D256 ? (b4 & 31) : b4;

    const uint8_t *kbase = a.k + (int64_t)group * a.blocks_per_seq * KBLOCK;
    const uint8_t *vbase = a.v + (int64_t)group * a.blocks_per_seq * VBLOCK;
    const char *klut_b = klut_s + (TQ_PAIRTAB3 && KFMT == KFMT_TURBO && KBITS == 3 ? 4 * lane : 0);
    const char *vlut_b = vlut_s + (TQ_PAIRTAB3 && VBITS == 3 ? 4 * lane : 0);

    // The first tile's rows are requested before anything else, so that the query rotation and
    // the table build overlap the first trip to memory.  Afterwards rows are fetched one tile
    // ahead into the same registers: the next K row right after QK has consumed the current
    // one, the next V row right after PV (with Sparse V only after a tile that used its V row).  After the split's last
    // tile the prefetch has every lane read row 0 of that tile's block (a handful of lines, never used): the rows are
    // read with the non-temporal hint, and a clamped re-read of the last tile's 64 rows went to memory again, one tile
    // in sixteen at 1024 tokens per split; a branch around the loads cost the eight-head variant 11 us.  The norms
    // travel with the rows, so no load is waited for in the tile that issued it.
    uint32_t kw[KROW_DW];
    uint32_t vw[4 * VBITS];
    // K: this lane's token's fp16 norm (turbo) or its four fp16 block scales (q8_0-style)
    auto load_knorm = [&](int tile) -> uint2 {
        const uint8_t *kb = kbase + (int64_t)(tile >> 1) * KBLOCK;
        const int r = (tile & 1) * 64 + krow;
        if constexpr (KFMT == KFMT_TURBO)
            return make_uint2(reinterpret_cast<const uint16_t *>(kb + TQ_ROWS_PER_BLOCK * 16 * KBITS)[r], 0u);
        else
            return *reinterpret_cast<const uint2 *>(kb + 8 * 2048 + 8 * r);
    };
    // V: fp16 norms of this lane's four tokens 4b..4b+3, or their q8_0-style scales ([tile][32-dim block][token])
    auto load_vnorm = [&](int tile) -> VSide<VBITS> {
        VSide<VBITS> r;
        const uint8_t *side = vbase + (int64_t)(tile >> 1) * VBLOCK + TQ_ROWS_PER_BLOCK * 16 * VBITS;
        if constexpr (VBITS == 8 && D256) {
            const int bh = lane >> 5;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {   // rows e4 .. e4 + 7 of the tile: this lane's four tokens, both halves
                const uint4 s8 = *reinterpret_cast<const uint4 *>(side + 2 * ((((tile & 1) * 4 + 2 * hf + bh) * 64) + e4));
                r.v[2 * hf] = make_uint2(s8.x, s8.y);
                r.v[2 * hf + 1] = make_uint2(s8.z, s8.w);
            }
        } else if constexpr (VBITS == 8) {
            const int bh = lane >> 5;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                r.v[e] = *reinterpret_cast<const uint2 *>(side + 2 * ((((tile & 1) * 4 + 2 * (e >> 1) + bh) * 64) +
                                                                      (e & 1 ? b4 ^ 32 : b4)));
        } else if constexpr (D256) {
            const uint4 n8 = *reinterpret_cast<const uint4 *>(side + 2 * ((tile & 1) * 64 + e4));
            r.v[0] = make_uint2(n8.x, n8.y);
            r.v[1] = make_uint2(n8.z, n8.w);
        } else {
            r.v[0] = *reinterpret_cast<const uint2 *>(side + 2 * ((tile & 1) * 64 + b4));
            r.v[1] = make_uint2(0u, 0u);
        }
        return r;
    };
    uint2 kn = make_uint2(0u, 0u);
    VSide<VBITS> gvu;
#pragma unroll
    for (auto &e : gvu.v) e = make_uint2(0u, 0u);
    int tile = t_begin;
    if (tile < t_end) {
        const int row0 = (tile & 1) * 64 + lane;
        const uint8_t *kb = kbase + (int64_t)(tile >> 1) * KBLOCK;
        if constexpr (KFMT == KFMT_TURBO) load_row<KBITS>(kb, (tile & 1) * 64 + krow, kw);
        else load_row<8>(kb, (tile & 1) * 64 + krow, kw);
        kn = load_knorm(tile);
        load_row<VBITS>(vbase + (int64_t)(tile >> 1) * VBLOCK, row0, vw);
        gvu = load_vnorm(tile);
    }
    if (tid == 0) {
        lead = 0;
        skipped = 0;
    }
    // pair-table entries for the table build below: requested now, needed after the query rotation
    uint32_t kpair = 0, vpair = 0;
    if constexpr (KFMT == KFMT_TURBO && KBITS == 3) kpair = a.klut[lane];
    if constexpr (!SHARE && VBITS == 3) vpair = a.vlut[lane];

    // one partial per workgroup: index (group, part), 4 HG heads each
    float *po = a.part_o + ((int64_t)group * wgs_per_group + part) * 4 * HG * 128;
    float *pml = a.part_ml + ((int64_t)group * wgs_per_group + part) * 4 * HG * 2;

    // A operand of QK, broadcast from one block per MFMA: lane (b, i) keeps q[head i] for the
    // dim groups g = b and g = b + 16 (4 dims each); MFMA g reads it from block g % 16.
    // The group's four queries are rotated by the first wavefronts (one 128-point butterfly per
    // head, two values per lane), scaled and parked as fp16 in 1 KB of LDS for everybody.
    auto load_q = [&](int h, float &x0, float &x1) {
        // heads past the group's last one repeat it (their results are not written)
        const int64_t e = D256 ? ((int64_t)group * a.q_group + min(a.head_off + (h & 3), a.q_group - 1)) * 256 + 128 * (h >> 2) + 2 * lane
                               : ((int64_t)group * a.q_group + min(a.head_off + h, a.q_group - 1)) * 128 + 2 * lane;
        if (a.q_dtype == TQ_F16) {
            const __half *qp = reinterpret_cast<const __half *>(a.q);
            x0 = __half2float(qp[e]);
            x1 = __half2float(qp[e + 1]);
        } else if (a.q_dtype == TQ_F32) {
            const float *qp = reinterpret_cast<const float *>(a.q);
            x0 = qp[e];
            x1 = qp[e + 1];
        } else {
            const double *qp = reinterpret_cast<const double *>(a.q);
            x0 = (float)qp[e];
            x1 = (float)qp[e + 1];
        }
    };
    // this wavefront's first head is requested now and rotated after the tables are built (the tables need only the
    // pair entries requested above, and nobody reads them before the barrier below)
    float xq0 = 0.0f, xq1 = 0.0f;
    if (wave_g < 4 * HG) load_q(wave_g, xq0, xq1);
    // (placed here, in front of the table build and the query rotation, so that its two dependent trips to memory - the
    // count of entries below the split, then the first window - pass while those run: behind them it delayed every
    // wavefront's first tile)
    // Sparse bias: a head's (position, value) list is walked as the tiles go by, sixteen entries at a time: lane (b, j)
    // holds entry sb_win + b of head j's list (b = lane / 4: the sixteen lanes that hold a head's logits hold a window
    // of its list), so a window is one load per lane, and a tile that has entries adds the window's sixteen to the
    // lanes that own their positions (an entry per dependent trip to memory made a list of 512 positions at the front
    // of the context double the step).  The window starts at the head's first entry inside this split: the number
    // of entries below the split's first token, counted with the whole wavefront (one entry per lane and round).
    int sb_win[HG], sb_pos[HG], sb_last[HG];   // sb_last: the window's last position (a cross-lane read per tile otherwise)
    float sb_val[HG];
#pragma unroll
    for (int hg = 0; hg < HG; ++hg) {
        sb_win[hg] = 0;
        sb_pos[hg] = sb_last[hg] = 0x7FFFFFFF;
        sb_val[hg] = 0.0f;
    }
    // entry e of the list of this lane's head in set hg (addresses are formed where they are needed: the path is rare)
    auto sb_entry = [&](int hg, int e) { return ((int64_t)group * a.q_group + min(a.head_off + 4 * hg + j, a.q_group - 1)) * a.sbias_n + e; };
    auto sb_load = [&](int hg) {   // this lane's entry of the window
        const int e = sb_win[hg] + (lane >> 2);
        const bool in = e < a.sbias_n;
        sb_pos[hg] = in ? a.sbias_pos[sb_entry(hg, in ? e : 0)] : 0x7FFFFFFF;
        sb_val[hg] = in ? a.sbias_val[sb_entry(hg, in ? e : 0)] : 0.0f;
        sb_last[hg] = __shfl(sb_pos[hg], 60 + j);   // the head's last lanes hold the window's last entry
    };
    if constexpr (SBIAS) {
        const int first_tok = t_begin * TT;
#pragma unroll
        for (int hg = 0; hg < HQ; ++hg) {
            int below[4];
#pragma unroll
            for (int h = 0; h < 4; ++h) {
                const int32_t *prow = a.sbias_pos + ((int64_t)group * a.q_group + min(a.head_off + 4 * hg + h, a.q_group - 1)) * a.sbias_n;
                int c = 0;
                for (int e0 = 0; e0 < a.sbias_n; e0 += 64) {
                    const int e = e0 + lane;
                    const int pe = e < a.sbias_n ? prow[e] : 0x7FFFFFFF;
                    c += __builtin_popcountll(__builtin_amdgcn_ballot_w64(pe < first_tok));
                }
                below[h] = c;
            }
            sb_win[hg] = j == 0 ? below[0] : j == 1 ? below[1] : j == 2 ? below[2] : below[3];
            sb_load(hg);
        }
    }
    if constexpr (KFMT == KFMT_TURBO) build_lut<KBITS>(klut_s, a.klut, kpair, tid, n_waves);
    if constexpr (!SHARE && VBITS != 8) build_lut<VBITS>(vlut_s, a.vlut, vpair, tid, n_waves);
    for (int h = wave_g; h < 4 * HG; h += gw) {
        _Float16 *qw = reinterpret_cast<_Float16 *>(q_stage) + h * 128;
        float x0 = xq0, x1 = xq1;
        if (h != wave_g) load_q(h, x0, x1);
        if (a.ks1) {
            x0 *= a.ks1[2 * lane];
            x1 *= a.ks1[2 * lane + 1];
            wht128_wave(x0, x1, lane);
            x0 *= a.ks2[2 * lane] * RSQRT128;
            x1 *= a.ks2[2 * lane + 1] * RSQRT128;
        }
        // q8_0-style K rows hand their four values of a dim group over in the order 0, 2, 1, 3 (qk_q8)
        const int d0 = 2 * lane, d1 = 2 * lane + 1;
        const int p0 = KFMT == KFMT_Q8 ? (d0 & ~3) | ((d0 & 1) << 1) | ((d0 >> 1) & 1) : d0;
        const int p1 = KFMT == KFMT_Q8 ? (d1 & ~3) | ((d1 & 1) << 1) | ((d1 >> 1) & 1) : d1;
        // turbo K: the rotated query is rounded to fp16 once, with the logit scale folded in.  q8_0-style K: an
        // fp16 query goes in as it is, so that its products with the int8 values are exact, and the logit scale
        // joins the rows' block scales in fp32 (rounding the scaled query would move logits of rows with large
        // channels by several 1e-3, which a peaked softmax over a long context turns into output error)
        const float qscale = KFMT == KFMT_Q8 ? 1.0f : a.scale_log2e;
        qw[p0] = (_Float16)(x0 * qscale);
        qw[p1] = (_Float16)(x1 * qscale);
    }
    __syncthreads();
    half4_t qa[HG][2];
    half4_t qa4[4];   // 256-dim heads: dim groups b, b + 8, b + 16, b + 24 of this half-wavefront's half of the query
#pragma unroll
    for (int hg = 0; hg < HG; ++hg) {
        const uint2 *qp = reinterpret_cast<const uint2 *>(reinterpret_cast<const _Float16 *>(q_stage) + (4 * hg + j) * 128);
        qa[hg][0] = __builtin_bit_cast(half4_t, qp[lane >> 2]);
        qa[hg][1] = __builtin_bit_cast(half4_t, qp[(lane >> 2) + 16]);
    }
    if constexpr (D256) {
        const uint2 *qp = reinterpret_cast<const uint2 *>(reinterpret_cast<const _Float16 *>(q_stage) + (4 * (lane >> 5) + j) * 128);
#pragma unroll
        for (int k = 0; k < 4; ++k) qa4[k] = __builtin_bit_cast(half4_t, qp[((lane >> 2) & 7) + 8 * k]);
    }
    // out[head i][dim 64*hf + lane] partial sums; two chains per dim half for MFMA issue overlap
    float4_t acc_o[HG][2][2];
    float m_run[HG], l_run[HG];
#pragma unroll
    for (int hg = 0; hg < HG; ++hg) {
#pragma unroll
        for (int c = 0; c < 4; ++c) acc_o[hg][c >> 1][c & 1] = float4_t{0.f, 0.f, 0.f, 0.f};
        m_run[hg] = -INFINITY;
        l_run[hg] = 0.0f;
    }
    // additive logit bias of this lane's head and four tokens (natural-log units), one 16-byte load when the row
    // allows it; positions past the context read as 0 (they are masked anyway)
    const bool bias_vec = a.bias && (a.tokens & 3) == 0 && (reinterpret_cast<uintptr_t>(a.bias) & 15u) == 0;
    auto load_bias = [&](int t, int hg, float (&bv)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bv[i] = 0.0f;
        if (!a.bias) return;
        const int tk = t * TT + t4;  // the launcher checks tokens < 2^31
        const float *row = a.bias + ((int64_t)group * a.q_group + min(a.head_off + 4 * hg + j, a.q_group - 1)) * a.tokens;
        if (bias_vec && tk + 3 < tokens_now) {
            const float4 v = *reinterpret_cast<const float4 *>(row + tk);
            bv[0] = v.x; bv[1] = v.y; bv[2] = v.z; bv[3] = v.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (tk + i < tokens_now) bv[i] = row[tk + i];
        }
    };
    float bias_next[HG][4];
#pragma unroll
    for (int hg = 0; hg < HQ; ++hg) load_bias(min(t_begin, max(t_end - 1, 0)), hg, bias_next[hg]);
    unsigned nskip = 0;  // Sparse V: skipped (query, position) pairs of this wavefront (wave-uniform: counted from lane masks)
    bool v_ahead = true;  // Sparse V: this tile's V row was requested while the previous tile was processed

    unsigned long long head_ok[HG];  // lanes whose head (lane % 4 of each set) exists in this pass
#pragma unroll
    for (int hg = 0; hg < HG; ++hg) head_ok[hg] = __builtin_amdgcn_ballot_w64(a.head_off + 4 * hg + j < a.q_group);
#pragma unroll 1
    while (tile < t_end) {
        const int64_t blk = tile >> 1;
        const int half = tile & 1;
        const int row = half * 64 + lane;
        const uint8_t *vb = vbase + blk * VBLOCK;

        {   // issue priority = tiles behind the leader (wave-uniform, so the branches are scalar)
            const uint32_t done = (uint32_t)(tile - t_begin);
            const uint32_t behind = max(lead_progress(&lead, done, lane), done) - done;
            if (behind == 0) __builtin_amdgcn_s_setprio(0);
            else if (behind == 1) __builtin_amdgcn_s_setprio(1);
            else if (behind == 2) __builtin_amdgcn_s_setprio(2);
            else __builtin_amdgcn_s_setprio(3);
        }
        const int tile_next = tile + 1;
        const int tile_n = min(tile_next, t_end - 1);
        const int row_n = tile_next < t_end ? (tile_n & 1) * 64 + lane : 0;  // past the split: every lane the same row
        const int krow_n = tile_next < t_end ? (tile_n & 1) * 64 + krow : 0;
        const VSide<VBITS> gvu_next = load_vnorm(tile_n);
        const int n_valid = rows_now - tile * 64;   // >= 64 except in the sequence's last tile
        // the bias of this tile was requested a tile ago, like the rows; now the next tile's
        float bias4[HG][4];
#pragma unroll
        for (int hg = 0; hg < HQ; ++hg) {
#pragma unroll
            for (int i = 0; i < 4; ++i) bias4[hg][i] = bias_next[hg][i] * LOG2E;
            load_bias(tile_n, hg, bias_next[hg]);
        }
        if constexpr (SBIAS) {
            // entries of this tile: positions ascend, so a window is done with once its last position lies below the
            // tile's end; a head then takes its next sixteen entries (wave-uniform loop, heads advance on their own)
            const int tile_lo = tile * TT, tile_hi = tile_lo + TT;
#pragma unroll
            for (int hg = 0; hg < HQ; ++hg) {
                bool fresh = true;   // this head's window has not been added to this tile yet
                while (true) {
                    const bool mine = fresh && sb_pos[hg] >= tile_lo && sb_pos[hg] < tile_hi;
                    // window slots (lane / 4) that hold an entry of this tile for any of the four heads
                    unsigned long long slots = __builtin_amdgcn_ballot_w64(mine);
                    slots = (slots | (slots >> 1) | (slots >> 2) | (slots >> 3)) & 0x1111111111111111ull;
                    auto add_slot = [&](int e4) {   // e4 = 4 * slot
                        const int pe = __shfl(sb_pos[hg], e4 + j);
                        const float ve = __shfl(sb_val[hg], e4 + j) * LOG2E;
                        const int d = pe - tile_lo - t4;   // positions outside this lane's four tokens (or this tile) match no i
                        if (fresh) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) bias4[hg][i] += d == i ? ve : 0.0f;
                        }
                    };
#pragma unroll 1
                    while (slots) {   // (unrolled over all sixteen slots this was faster for runs of positions and cost registers)
                        add_slot(__builtin_ctzll(slots));
                        slots &= slots - 1;
                    }
                    fresh = false;
                    const bool advance = sb_last[hg] < tile_hi;   // the whole window lies before the tile's end (padding never does)
                    if (__builtin_amdgcn_ballot_w64(advance) == 0ull) break;
                    if (advance) {
                        sb_win[hg] += 16;
                        fresh = true;
                    }
                    sb_load(hg);   // by every lane (the load ends in a cross-lane read); heads that stay reload what they hold
                }
            }
        }

        // ---- QK ------------------------------------------------------------------
        // D_b[head][token 4b + lane%4]: every lane gets the 4 heads' dot products of its own token
        float sc[HG][4];
        float4_t acc[HG][4];
#pragma unroll
        for (int hg = 0; hg < HG; ++hg)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[hg][c] = float4_t{0.f, 0.f, 0.f, 0.f};
        if constexpr (D256) {
            // each half-wavefront: its half of the query against its rows; a token's two halves meet across lane ^ 32
            float d[4];
            if constexpr (KFMT == KFMT_TURBO) {
                qk_turbo_d256<KBITS>(std::make_integer_sequence<int, 32>{}, kw, klut_b, qa4, acc[0]);
                d[0] = d[1] = d[2] = d[3] = __half2float(__ushort_as_half((unsigned short)kn.x));
            } else {
                qk_q8_d256(std::make_integer_sequence<int, 32>{}, kw, qa4, acc[0]);
                d[0] = __half2float(__ushort_as_half((unsigned short)(kn.x & 0xffff))) * a.scale_log2e;
                d[1] = __half2float(__ushort_as_half((unsigned short)(kn.x >> 16))) * a.scale_log2e;
                d[2] = __half2float(__ushort_as_half((unsigned short)(kn.y & 0xffff))) * a.scale_log2e;
                d[3] = __half2float(__ushort_as_half((unsigned short)(kn.y >> 16))) * a.scale_log2e;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float part = (acc[0][0][i] * d[0] + acc[0][1][i] * d[1]) + (acc[0][2][i] * d[2] + acc[0][3][i] * d[3]);
                sc[0][i] = part + xor_lane<32>(part);
            }
        } else if constexpr (KFMT == KFMT_TURBO) {
            qk_turbo<KBITS, HG>(std::make_integer_sequence<int, 32>{}, kw, klut_b, qa, acc);
            const float gk_own = __half2float(__ushort_as_half((unsigned short)kn.x));
#pragma unroll
            for (int hg = 0; hg < HG; ++hg)
#pragma unroll
                for (int i = 0; i < 4; ++i) sc[hg][i] = ((acc[hg][0][i] + acc[hg][1][i]) + (acc[hg][2][i] + acc[hg][3][i])) * gk_own;
        } else {
            qk_q8<HG>(std::make_integer_sequence<int, 32>{}, kw, qa, acc);
            const uint2 su = kn;
            const float d0 = __half2float(__ushort_as_half((unsigned short)(su.x & 0xffff))) * a.scale_log2e;
            const float d1 = __half2float(__ushort_as_half((unsigned short)(su.x >> 16))) * a.scale_log2e;
            const float d2 = __half2float(__ushort_as_half((unsigned short)(su.y & 0xffff))) * a.scale_log2e;
            const float d3 = __half2float(__ushort_as_half((unsigned short)(su.y >> 16))) * a.scale_log2e;
#pragma unroll
            for (int hg = 0; hg < HG; ++hg)
#pragma unroll
                for (int i = 0; i < 4; ++i) sc[hg][i] = (acc[hg][0][i] * d0 + acc[hg][1][i] * d1) + (acc[hg][2][i] * d2 + acc[hg][3][i] * d3);
        }
        {   // kw is dead now: fetch the next tile's K row into it
            const uint8_t *kbn = kbase + (int64_t)(tile_n >> 1) * KBLOCK;
            if constexpr (KFMT == KFMT_TURBO) load_row<KBITS>(kbn, krow_n, kw);
            else load_row<8>(kbn, krow_n, kw);
            kn = load_knorm(tile_n);
        }
        // -> lane (b, j): head j (of each set), tokens 4b..4b+3; then the online softmax in base 2
        float p[HG][4];
        // Sparse V bookkeeping on the scalar unit: a compare leaves a lane mask, and counting, the in-range test and
        // "does any lane keep anything" are mask arithmetic (the vector ALU only compares and zeroes the weight)
        unsigned long long any_keep = 0, token_ok[4] = {~0ull, ~0ull, ~0ull, ~0ull};
        if constexpr (SPARSE) {
            if (n_valid < 64) {
#pragma unroll
                for (int i = 0; i < 4; ++i) token_ok[i] = __builtin_amdgcn_ballot_w64(e4 + es * i < n_valid);
            }
        }
#pragma unroll
        for (int hg = 0; hg < HQ; ++hg) {
            quad_transpose(sc[hg], lane);
            float s[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) s[i] = sc[hg][i] + bias4[hg][i];
            if (n_valid < 64) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (e4 + es * i >= n_valid) s[i] = -INFINITY;
            }
            const float mx = max_over_blocks(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
            const float m_new = fmaxf(m_run[hg], mx);
            // After the first tiles the running maximum rarely moves, and a correction factor of exactly 1 changes
            // nothing: the rescaling is skipped when no lane's maximum moved (a wave-uniform branch; same results).
            if (__builtin_amdgcn_ballot_w64(m_new != m_run[hg]) != 0ull) {
                // 0 on the first tile, 1 when the maximum stays (also while every position so far is masked with -inf)
                const float corr = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run[hg] - m_new);
                l_run[hg] *= corr;
                // accumulator register i belongs to head i; the factor of head i lives in lanes with lane%4 == i
                const float c0 = dpp<0x00>(corr), c1 = dpp<0x55>(corr), c2 = dpp<0xAA>(corr), c3 = dpp<0xFF>(corr);
#pragma unroll
                for (int ho = 0; ho < HG; ++ho) {
                    if (!D256 && ho != hg) continue;   // 256-dim heads: both halves of the output share the softmax
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        acc_o[ho][c >> 1][c & 1][0] *= c0;
                        acc_o[ho][c >> 1][c & 1][1] *= c1;
                        acc_o[ho][c >> 1][c & 1][2] *= c2;
                        acc_o[ho][c >> 1][c & 1][3] *= c3;
                    }
                }
                m_run[hg] = m_new;
            }
            const float m_ref = m_run[hg] == -INFINITY ? 0.0f : m_run[hg];  // all masked so far: weights are exp2(-inf) = 0, not NaN
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p[hg][i] = __builtin_amdgcn_exp2f(s[i] - m_ref);  // results below 2^-126 flush to zero
                l_run[hg] += p[hg][i];
                if constexpr (SPARSE) {
                    const bool keep = p[hg][i] >= a.tau;
                    const unsigned long long keep_m = __builtin_amdgcn_ballot_w64(keep);
                    // 256-dim heads: both half-wavefronts hold the same 32 tokens; the lower one counts
                    const unsigned long long in_range = token_ok[i] & head_ok[hg] & (D256 ? 0xFFFFFFFFull : ~0ull);
                    nskip += (unsigned)__builtin_popcountll(in_range & ~keep_m);
                    if (!keep) p[hg][i] = 0.0f;
                    any_keep |= keep_m & in_range;
                }
            }
        }
        if constexpr (SPARSE) {
            // Every V row of the tile skipped: no dequant, and the next tile's V row is not requested in
            // advance (negligible weights come in runs); a tile that then does need its row fetches it here.
            if (any_keep == 0) {
                gvu = gvu_next;
                tile = tile_next;
                v_ahead = false;
                continue;
            }
            if (!v_ahead) load_row<VBITS>(vb, row, vw);
        }

        // ---- PV ------------------------------------------------------------------------
        // weights (times the stored V norm) as fp16: this lane is token group T = lane/4, head lane%4
        if constexpr (VBITS == 8 && D256) {
            half4_t a8[2][2][2];
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                // scales of rows 8b..8b+7 = (token 4b + i, half h) at 2 i + h
                const uint32_t sw[4] = {gvu.v[2 * hf].x, gvu.v[2 * hf].y, gvu.v[2 * hf + 1].x, gvu.v[2 * hf + 1].y};
#pragma unroll
                for (int dh = 0; dh < 2; ++dh) {
                    _Float16 w[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        w[i] = (_Float16)(p[0][i] * (__half2float(__ushort_as_half((unsigned short)(dh ? sw[i] >> 16 : sw[i] & 0xffff))) *
                                                     Q8V_PRESCALE));
                    const _Float16 z = (_Float16)0.0f;
                    a8[dh][hf][0] = dh ? half4_t{z, z, w[0], w[1]} : half4_t{w[0], w[1], z, z};
                    a8[dh][hf][1] = dh ? half4_t{z, z, w[2], w[3]} : half4_t{w[2], w[3], z, z};
                }
            }
            pv_all_q8_d256(std::make_integer_sequence<int, 16>{}, vw, a8, acc_o);
        } else if constexpr (VBITS == 8) {
            // The dims of block b lie in 32-dim block b / 8 (+ 2 for the upper dim half), so the weights carry that
            // block's scale and are broadcast inside each half of the wavefront: token group T is served by block
            // T % 8 of both halves, which therefore also needs the weights of the lane 32 away.
            auto weights = [&](const float (&w)[4], uint2 sc) {
                const float s0 = __half2float(__ushort_as_half((unsigned short)(sc.x & 0xffff))) * Q8V_PRESCALE;
                const float s1 = __half2float(__ushort_as_half((unsigned short)(sc.x >> 16))) * Q8V_PRESCALE;
                const float s2 = __half2float(__ushort_as_half((unsigned short)(sc.y & 0xffff))) * Q8V_PRESCALE;
                const float s3 = __half2float(__ushort_as_half((unsigned short)(sc.y >> 16))) * Q8V_PRESCALE;
                half4_t r;  // token order 0, 2, 1, 3, as int8x4_to_half_0213 hands the values over
                r[0] = (_Float16)(w[0] * s0);
                r[1] = (_Float16)(w[2] * s2);
                r[2] = (_Float16)(w[1] * s1);
                r[3] = (_Float16)(w[3] * s3);
                return r;
            };
            const bool upper = lane >= 32;
            half4_t a_lo[HG][2], a_hi[HG][2];
#pragma unroll
            for (int hg = 0; hg < HG; ++hg) {
                float ps[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) ps[i] = __shfl_xor(p[hg][i], 32);
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const half4_t own = weights(p[hg], gvu.v[2 * hf]), swp = weights(ps, gvu.v[2 * hf + 1]);
                    a_lo[hg][hf] = upper ? swp : own;
                    a_hi[hg][hf] = upper ? own : swp;
                }
            }
            pv_all_q8<HG>(std::make_integer_sequence<int, 16>{}, vw, a_lo, a_hi, acc_o);
        } else if constexpr (D256) {
            // norms of rows 8b..8b+7 = (token 4b + i, half h) at 2 i + h
            const uint32_t nw[4] = {gvu.v[0].x, gvu.v[0].y, gvu.v[1].x, gvu.v[1].y};
            half4_t pv_even[2], pv_odd[2];
#pragma unroll
            for (int dh = 0; dh < 2; ++dh) {
                float g[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) g[i] = __half2float(__ushort_as_half((unsigned short)(dh ? nw[i] >> 16 : nw[i] & 0xffff)));
                const _Float16 z = (_Float16)0.0f;
                const _Float16 w0 = (_Float16)(p[0][0] * g[0]), w1 = (_Float16)(p[0][1] * g[1]);
                const _Float16 w2 = (_Float16)(p[0][2] * g[2]), w3 = (_Float16)(p[0][3] * g[3]);
                pv_even[dh] = dh ? half4_t{z, w0, z, w1} : half4_t{w0, z, w1, z};
                pv_odd[dh] = dh ? half4_t{z, w2, z, w3} : half4_t{w2, z, w3, z};
            }
            pv_all_d256<VBITS>(std::make_integer_sequence<int, 16>{}, vw, vlut_b, pv_even, pv_odd, acc_o);
        } else {
            const float g0 = __half2float(__ushort_as_half((unsigned short)(gvu.v[0].x & 0xffff)));
            const float g1 = __half2float(__ushort_as_half((unsigned short)(gvu.v[0].x >> 16)));
            const float g2 = __half2float(__ushort_as_half((unsigned short)(gvu.v[0].y & 0xffff)));
            const float g3 = __half2float(__ushort_as_half((unsigned short)(gvu.v[0].y >> 16)));
            half4_t pv[HG];
#pragma unroll
            for (int hg = 0; hg < HG; ++hg) {
                pv[hg][0] = (_Float16)(p[hg][0] * g0);
                pv[hg][1] = (_Float16)(p[hg][1] * g1);
                pv[hg][2] = (_Float16)(p[hg][2] * g2);
                pv[hg][3] = (_Float16)(p[hg][3] * g3);
            }
            // V row of this lane: dims lane and 64+lane for the tile's 64 tokens; quad 2T + hf =
            // tokens 4T..4T+3 of dim half hf.  Block b = lane/4 of the MFMA covers dims 4b..4b+3 (+64*hf); the
            // weights of token group T sit in block T and are broadcast to every block.
            pv_all<VBITS, HG>(std::make_integer_sequence<int, 16>{}, vw, vlut_b, pv, acc_o);
        }
        load_row<VBITS>(vbase + (int64_t)(tile_n >> 1) * VBLOCK, row_n, vw);
        v_ahead = true;
        gvu = gvu_next;
        tile = tile_next;
    }

    // ---- end of split: the workgroup's wavefronts merge their partials in LDS and write one ------
    if constexpr (VBITS == 8) {
#pragma unroll
        for (int hg = 0; hg < HG; ++hg)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc_o[hg][c >> 1][c & 1] *= 1.0f / Q8V_PRESCALE;
    }
    float l_tot[HG];
#pragma unroll
    for (int hg = 0; hg < HG; ++hg) l_tot[hg] = sum_over_blocks(l_run[hg]);
    if constexpr (D256) {
        // both half-wavefronts added the same 32 weights; the second accumulator set shares the softmax state
        l_tot[0] *= 0.5f;
        l_tot[1] = l_tot[0];
        m_run[1] = m_run[0];
    }
    if (gw == 1) {
#pragma unroll
        for (int hg = 0; hg < HG; ++hg) {
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    st_dev(po + (4 * hg + i) * 128 + 64 * hf + lane, acc_o[hg][hf][0][i] + acc_o[hg][hf][1][i]);
            if (lane < 4) {
                st_dev(pml + 2 * (4 * hg + j), m_run[hg]);
                st_dev(pml + 2 * (4 * hg + j) + 1, l_tot[hg]);
            }
        }
    } else {
        // per wavefront and set of four heads: out[4][128], then m[4], l[4]; a group's wavefronts are wave0 .. wave0 + gw - 1
        constexpr int MS = MERGE_FLOATS * HG;
        float *mine = merge_s + wave * MS;
#pragma unroll
        for (int hg = 0; hg < HG; ++hg)
            if (lane < 4) {
                mine[hg * MERGE_FLOATS + 512 + j] = m_run[hg];
                mine[hg * MERGE_FLOATS + 516 + j] = l_tot[hg];
            }
        __syncthreads();
        float M[HG];
#pragma unroll
        for (int hg = 0; hg < HG; ++hg) {
            // head j's maximum over the wavefronts that saw an unmasked position
            M[hg] = -INFINITY;
            const float *ml_g = merge_s + wave0 * MS + hg * MERGE_FLOATS;   // the group's first wavefront
#pragma unroll 8
            for (int w = 0; w < gw; ++w)
                if (ml_g[w * MS + 516 + j] > 0.0f) M[hg] = fmaxf(M[hg], ml_g[w * MS + 512 + j]);
            const float f = l_tot[hg] > 0.0f ? __builtin_amdgcn_exp2f(m_run[hg] - M[hg]) : 0.0f;
            const float f4[4] = {dpp<0x00>(f), dpp<0x55>(f), dpp<0xAA>(f), dpp<0xFF>(f)};
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    mine[hg * MERGE_FLOATS + i * 128 + 64 * hf + lane] = (acc_o[hg][hf][0][i] + acc_o[hg][hf][1][i]) * f4[i];
        }
        __syncthreads();
        for (int e = tid_g; e < 512 * HG; e += 64 * gw) {
            const int src = (e >> 9) * MERGE_FLOATS + (e & 511);  // partial element e = head e / 128, dim e % 128
            float sum = 0.0f;
            const float *col = merge_s + wave0 * MS + src;
#pragma unroll 8
            for (int w = 0; w < gw; ++w) sum += col[w * MS];
            st_dev(po + e, sum);
        }
        if (tid_g < 4) {  // lanes 0..3 of the group's first wavefront hold heads 0..3 of each set
#pragma unroll
            for (int hg = 0; hg < HG; ++hg) {
                float L = 0.0f;
                const float *ml_g = merge_s + wave0 * MS + hg * MERGE_FLOATS;
#pragma unroll 8
                for (int w = 0; w < gw; ++w) {
                    const float lw = ml_g[w * MS + 516 + j];
                    if (lw > 0.0f) L = fmaf(lw, __builtin_amdgcn_exp2f(ml_g[w * MS + 512 + j] - M[hg]), L);
                }
                st_dev(pml + 2 * (4 * hg + j), M[hg]);
                st_dev(pml + 2 * (4 * hg + j) + 1, L);
            }
        }
    }
    if constexpr (SPARSE) {
        // one slot per workgroup, added up by the merge kernel: thousands of wavefronts finishing together
        // on one atomic would queue for longer than the kernel's own tail, and nothing needs clearing
        if (lane == 0 && nskip) atomicAdd(&skipped, nskip);
        __syncthreads();
        if (tid == 0) st_dev(a.skip_slots + blockIdx.x, (a.nonce & ~SKIP_COUNT_MASK) | (unsigned long long)skipped);
    }

    // ---- the group's last workgroup merges the partials and writes the output rows -----------------
    const int n_parts = wgs_per_group;
    wait_stores();  // this lane's part of the partial (and the skip slot) is in memory
    __syncthreads();
    if (n_parts > 1) {
        // Arrival counter of the group: the call's tag in the upper 40 bits, the number of workgroups whose partial is
        // in memory in the lower 24.  One read-modify-write per workgroup; a word that does not carry the tag (whatever a
        // fresh workspace held, or the zero a finished call leaves) counts as zero arrivals.  Read-modify-writes on one
        // word happen one after the other, so exactly one workgroup brings the count to n_parts: it merges, and every
        // other partial was complete in memory before its owner's increment, hence before this one's.
        __shared__ int i_am_last;
        if (tid == 0) {
            unsigned long long *ctr = a.flags + (int64_t)group * n_parts;
            const unsigned long long tag = a.nonce & ~ARRIVAL_COUNT_MASK;
            unsigned long long seen = ld_dev(ctr), count;
            for (;;) {
                if ((seen & ~ARRIVAL_COUNT_MASK) == tag) {
                    // the word is this call's (it stays so until the merge): a plain increment, no retry however many
                    // workgroups arrive together
                    count = (__hip_atomic_fetch_add(ctr, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & ARRIVAL_COUNT_MASK) + 1ull;
                    break;
                }
                // first arrival of the call: install the tag with a count of one, unless somebody else just did
                if (__hip_atomic_compare_exchange_strong(ctr, &seen, tag | 1ull, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                    count = 1ull;
                    break;
                }
            }
            i_am_last = (int)count == n_parts;
        }
        __syncthreads();
        if (!i_am_last) return;
    }
    // Sparse V: every workgroup's slot carries its count (40 bits: at most 4 heads x 2^31 positions) under 24 bits
    // of the nonce.  A merging workgroup reads all slots of the launch now, so that the trip to memory overlaps
    // the merge; the one that finds them all tagged (the merging workgroup of the group that finishes last does)
    // writes the step's total.  Launches with more workgroups than one can poll are added up by a launch of their
    // own (poll_slots == 0).
    int all_in = 1;
    unsigned long long counted = 0ull;
    if constexpr (SPARSE) {
        if (a.poll_slots) {
            const unsigned long long tag = a.nonce & ~SKIP_COUNT_MASK;
            for (int g = tid; g < (int)gridDim.x; g += (int)blockDim.x) {
                const unsigned long long word = ld_dev(a.skip_slots + g);
                all_in &= (word & ~SKIP_COUNT_MASK) == tag;
                counted += word & SKIP_COUNT_MASK;
            }
        }
    }
    // the wavefronts' merge space is free again (every partial of this workgroup is in memory); with several groups
    // per workgroup every group's wavefronts finish their own group (one partial: no exchange between them)
    merge_group<HG>(a, group, n_parts, tid_g, gw, n_waves > 1 && a.gpw <= 1 ? merge_s : nullptr);
    if (n_parts > 1 && tid == 0) st_dev(a.flags + (int64_t)group * n_parts, 0ull);  // a replay of a captured launch (same tag) starts from zero
    if constexpr (SPARSE) {
        if (a.poll_slots) {
            if (!__syncthreads_and(all_in)) return;
            __shared__ unsigned long long red;
            const unsigned long long pass_total = block_sum(counted, &red, tid);
            for (int g = tid; g < (int)gridDim.x; g += (int)blockDim.x) st_dev(a.skip_slots + g, 0ull);
            if (tid == 0) {
                // this pass's total is kept apart so that writing the step's total twice (two groups finishing
                // together) gives the same value both times
                st_dev(a.pass_totals + a.pass, pass_total);
                unsigned long long sum = pass_total;
                for (int k = 0; k < a.pass; ++k) sum += ld_dev(a.pass_totals + k);
                a.skip_count[0] = sum;
                a.skip_count[1] = a.total_pairs;
            }
        }
    }
}

// Sparse-V bookkeeping for launches with more groups than one workgroup polls (and for a caller that asks for the
// counts of a dense step): skip[0] = the sum of the decode workgroups' slots (plus the earlier passes'), skip[1] =
// all (query, position) pairs.  One workgroup.
__global__ __launch_bounds__(1024) void k_skip_sum(const unsigned long long *slots, int n_slots, unsigned long long *skip,
                                                   unsigned long long total_pairs, int accumulate) {
    __shared__ unsigned long long red;
    unsigned long long t = 0ull;
    for (int i = (int)threadIdx.x; i < n_slots; i += (int)blockDim.x) t += slots[i] & SKIP_COUNT_MASK;
    const unsigned long long sum = block_sum(t, &red, (int)threadIdx.x);
    if (threadIdx.x == 0) {
        skip[0] = (accumulate ? skip[0] : 0ull) + sum;
        skip[1] = total_pairs;
    }
}

constexpr int MAX_POLLED_SLOTS = 4096;  // workgroups of a launch whose Sparse-V slots the merging workgroups add up themselves
constexpr int MAX_PASSES = 64;           // four-head passes of one step (query heads per KV head <= 256)

inline int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

// a value that no earlier call of this process used and that leftovers in a fresh workspace are unlikely to
// equal (splitmix64 of a process-wide counter; never 0, which is what a lowered flag holds)
std::atomic<unsigned long long> g_attn_seq{0};
unsigned long long next_nonce() {
    unsigned long long z = (g_attn_seq.fetch_add(1, std::memory_order_relaxed) + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (z >> 40) ? z : z | (1ull << 63);  // the upper 24 bits tag the Sparse-V words and must not be zero
}

struct WsLayout {
    int64_t part_o, part_ml, skip_slots, flags, pass_totals, total;
};
// How a parameter set is run: sets of four query heads per pass (2 when a KV head serves more than four query
// heads), wavefronts per workgroup (the largest power of two up to the variant's limit that divides the split
// count) and workgroups = partials per group.
struct AttnPlan {
    int hg, wpw, n_parts, gpw;
};
AttnPlan attn_plan(const tq_attn_params *p, bool bias_list) {
    AttnPlan pl;
    // 256-dim heads run as two accumulator sets (the output's halves) of one set of four heads
    pl.hg = p->head_dim == 256 || p->n_q_heads / p->n_kv_heads > 4 ? 2 : 1;
    const bool turbo_k = p->k_format == TQ_KFMT_TURBO, turbo_v = p->v_format == TQ_KFMT_TURBO;
    const bool wide12 = turbo_k && p->head_dim != 256 && !bias_list;
    pl.wpw = max_waves_per_workgroup(turbo_v ? 0 : 8, pl.hg, wide12);
    if (pl.wpw == 12 && p->n_splits % 12 != 0) pl.wpw = 8;
    while (p->n_splits % pl.wpw) pl.wpw >>= 1;
    // few groups (small batches): smaller workgroups, so that every CU gets one (a tile costs a wavefront the same
    // issue time however many share the SIMD)
    const int64_t groups = (int64_t)p->batch * p->n_kv_heads;
    // short contexts: a group has fewer splits than a workgroup has room for wavefronts.  Several groups then share a
    // workgroup (and its decode tables), provided that still makes a workgroup per CU
    const int wmax = max_waves_per_workgroup(turbo_v ? 0 : 8, pl.hg);   // groups share a workgroup in powers of two
    pl.gpw = 1;
    if (p->n_splits < wmax && wmax % p->n_splits == 0) {
        int g = wmax / p->n_splits;
        while (g > 1 && (groups % g != 0 || groups / g < 256)) g >>= 1;
        if (g > 1) {
            pl.gpw = g;
            pl.wpw = g * p->n_splits;
            pl.n_parts = 1;
            return pl;
        }
    }
    while (pl.wpw > 4 && pl.wpw % 2 == 0 && groups * (p->n_splits / pl.wpw) < 256) pl.wpw >>= 1;
    pl.n_parts = p->n_splits / pl.wpw;
    return pl;
}
WsLayout ws_layout(const tq_attn_params *p) {
    const int64_t groups = (int64_t)p->batch * p->n_kv_heads;
    // a call with a bias list may run smaller workgroups (more partials per group) than one without: room for either
    const AttnPlan pl = attn_plan(p, false), pl_list = attn_plan(p, true);
    const int64_t parts = groups * (pl.n_parts > pl_list.n_parts ? pl.n_parts : pl_list.n_parts);
    WsLayout w;
    w.part_o = 0;
    w.part_ml = w.part_o + align256(parts * 4 * pl.hg * 128 * 4);
    w.skip_slots = w.part_ml + align256(parts * 4 * pl.hg * 2 * 4);
    w.flags = w.skip_slots + align256(parts * 8);
    w.pass_totals = w.flags + align256(parts * 8);
    w.total = w.pass_totals + align256(MAX_PASSES * 8);
    return w;
}

}  // namespace

int64_t tqk_attn_workspace_bytes(const tq_attn_params *p) { return ws_layout(p).total; }

int tqk_decode_attention(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q, int q_dtype,
                         const void *k, const void *k_aux, const void *v, const float *bias, float *out,
                         unsigned long long *skip_count, void *ws, int64_t ws_bytes, hipStream_t s) {
    (void)k_aux;
    const WsLayout w = ws_layout(p);
    if (ws_bytes < w.total) {
        tq_set_error("tq_decode_attention: workspace %lld < %lld bytes", (long long)ws_bytes, (long long)w.total);
        return TQ_ERR_ARG;
    }
    const int64_t rows = (int64_t)p->batch * p->n_q_heads;
    const int groups = p->batch * p->n_kv_heads;
    const bool d256 = p->head_dim == 256;
    if (p->head_dim != 0 && p->head_dim != 128 && p->head_dim != 256) {
        tq_set_error("tq_decode_attention: head_dim %d (128 or 256)", (int)p->head_dim);
        return TQ_ERR_UNSUPPORTED;
    }
    const int64_t cache_rows = (d256 ? 2 : 1) * p->tokens;   // a 256-dim token is two rows of the caches
    float *part_o = reinterpret_cast<float *>((char *)ws + w.part_o);
    float *part_ml = reinterpret_cast<float *>((char *)ws + w.part_ml);
    const bool turbo_k = p->k_format == TQ_KFMT_TURBO;
    const float sc = p->scale * LOG2E;
    const unsigned long long total_pairs = (unsigned long long)rows * (unsigned long long)p->tokens;
    int rc = TQ_OK;
    if (q_dtype != TQ_F16 && q_dtype != TQ_F32 && q_dtype != TQ_F64) {
        tq_set_error("bad q dtype %d", q_dtype);
        return TQ_ERR_ARG;
    }

    AttnArgs a;
    a.q = q;
    a.q_dtype = q_dtype;
    a.ks1 = turbo_k ? hk->s1_32 : nullptr;
    a.ks2 = turbo_k ? hk->s2_32 : nullptr;
    a.scale_log2e = sc;
    a.k = (const uint8_t *)k;
    a.v = (const uint8_t *)v;
    a.klut = turbo_k ? (const uint32_t *)hk->pair_lut : nullptr;
    const bool turbo_v = p->v_format == TQ_KFMT_TURBO;
    a.vlut = turbo_v ? (const uint32_t *)hv->pair_lut : nullptr;
    const float *vs1 = turbo_v ? hv->s1_32 : nullptr, *vs2 = turbo_v ? hv->s2_32 : nullptr;
    const bool share = turbo_k && turbo_v && hk->bits == hv->bits &&
                       std::memcmp(hk->pair_lut_host, hv->pair_lut_host, sizeof(hk->pair_lut_host)) == 0;
    a.bias = bias;
    a.sbias_n = p->bias_entries;
    a.sbias_pos = p->bias_pos;
    a.sbias_val = p->bias_val;
    if (p->bias_entries < 0 || (p->bias_entries > 0 && (!p->bias_pos || !p->bias_val))) {
        tq_set_error("tq_decode_attention: bias_entries %d needs bias_pos and bias_val", (int)p->bias_entries);
        return TQ_ERR_ARG;
    }
    a.part_o = part_o;
    a.part_ml = part_ml;
    a.skip_slots = reinterpret_cast<unsigned long long *>((char *)ws + w.skip_slots);
    if (cache_rows >= ((int64_t)1 << 31)) {
        tq_set_error("tq_decode_attention: tokens %lld beyond 2^31 - 1", (long long)p->tokens);
        return TQ_ERR_UNSUPPORTED;
    }
    a.tokens = p->tokens;
    a.tokens_dev = p->tokens_dev;
    if (p->tokens_dev && skip_count) {
        tq_set_error("tq_decode_attention: the Sparse-V count is not kept for a context length read from memory (tokens_dev)");
        return TQ_ERR_UNSUPPORTED;
    }
    a.blocks_per_seq = ((d256 ? 2 : 1) * (p->capacity > 0 ? p->capacity : p->tokens) + TQ_ROWS_PER_BLOCK - 1) / TQ_ROWS_PER_BLOCK;
    a.n_groups = groups;
    a.n_splits = p->n_splits;
    a.n_tiles = (int)((cache_rows + 63) / 64);
    a.d256 = d256 ? 1 : 0;
    a.tiles_per_split = (a.n_tiles + p->n_splits - 1) / p->n_splits;
    a.tau = p->sparse_v_tau;
    const bool sparse = p->sparse_v_tau > 0.0f;
    if (sparse && !skip_count) {
        tq_set_error("tq_decode_attention: sparse_v_tau > 0 needs skip_count");
        return TQ_ERR_ARG;
    }
    // wavefronts per workgroup: the largest power of two up to 16 (8 for int8 V rows and for eight heads per pass)
    // that divides the split count
    const AttnPlan pl = attn_plan(p, p->bias_entries > 0);
    const int wpw = pl.wpw, hg = pl.hg;
    const unsigned grid = (unsigned)((int64_t)groups * pl.n_parts / pl.gpw);
    const unsigned wg = 64u * (unsigned)wpw;
    const int n_parts = pl.n_parts;  // partials per group: the wavefronts of a workgroup merge theirs in LDS
    // dynamic LDS: the wavefronts' merge space, then the staged queries of the workgroup's groups
    const size_t merge_bytes = (wpw > 1 ? (size_t)wpw * hg * MERGE_FLOATS * sizeof(float) : 0) + (size_t)pl.gpw * 1024 * hg;
    a.gpw = pl.gpw;
    a.gw_shift = 0;
    while ((1 << a.gw_shift) < p->n_splits) ++a.gw_shift;
    a.wgs_per_group = pl.gpw > 1 ? 1 : p->n_splits / wpw;
    const int vb = turbo_v ? hv->bits : 8;
    const int kb = turbo_k ? hk->bits : 8;
    // The kernels work on four query heads of a KV head at a time (the 4-row MFMA block), or on eight (two sets
    // against the same dequantised rows) when a KV head serves more than four: a group of G heads takes
    // ceil(G / 8) passes over the same K/V; a last pass with fewer heads than it has rows repeats the group's
    // last head and does not write the repeats.
    a.q_group = p->n_q_heads / p->n_kv_heads;
    const int heads_per_pass = d256 ? 4 : 4 * hg;
    if ((a.q_group + heads_per_pass - 1) / heads_per_pass > MAX_PASSES) {
        tq_set_error("tq_decode_attention: %d query heads per KV head (at most %d)", a.q_group, 4 * MAX_PASSES);
        return TQ_ERR_UNSUPPORTED;
    }
    a.out = out;
    a.vs1 = vs1;
    a.vs2 = vs2;
    a.flags = reinterpret_cast<unsigned long long *>((char *)ws + w.flags);
    a.poll_slots = sparse && grid <= (unsigned)MAX_POLLED_SLOTS;
    a.pass_totals = reinterpret_cast<unsigned long long *>((char *)ws + w.pass_totals);
    a.skip_count = skip_count;
    a.total_pairs = total_pairs;
    (void)n_parts;
    (void)kb;
    for (a.head_off = 0; a.head_off < a.q_group; a.head_off += heads_per_pass) {
        a.pass = a.head_off / heads_per_pass;
        a.nonce = next_nonce();
        if (d256) {
#define TQ_ATTN_256_ONE(KF, KB, VB, SH)                                                                              \
    {                                                                                                                 \
        if (sparse && a.sbias_n) k_decode_attn<KF, KB, VB, true, SH, 2, true, true><<<grid, wg, merge_bytes, s>>>(a);  \
        else if (sparse) k_decode_attn<KF, KB, VB, true, SH, 2, false, true><<<grid, wg, merge_bytes, s>>>(a);         \
        else if (a.sbias_n) k_decode_attn<KF, KB, VB, false, SH, 2, true, true><<<grid, wg, merge_bytes, s>>>(a);      \
        else k_decode_attn<KF, KB, VB, false, SH, 2, false, true><<<grid, wg, merge_bytes, s>>>(a);                   \
    }
#define TQ_ATTN_256(B)                                   \
    if (share) TQ_ATTN_256_ONE(KFMT_TURBO, B, B, true)   \
    else TQ_ATTN_256_ONE(KFMT_TURBO, B, B, false)
#define TQ_ATTN_256X(KF, KB, VB) TQ_ATTN_256_ONE(KF, KB, VB, false)
            if (turbo_k && kb == vb && kb == 3) { TQ_ATTN_256(3); }
            else if (turbo_k && kb == vb && kb == 4) { TQ_ATTN_256(4); }
            else if (turbo_k && kb == vb && kb == 2) { TQ_ATTN_256(2); }
            else if (turbo_k && kb == 4 && vb == 2) { TQ_ATTN_256X(KFMT_TURBO, 4, 2); }
            else if (turbo_k && kb == 3 && vb == 2) { TQ_ATTN_256X(KFMT_TURBO, 3, 2); }
            else if (turbo_k && kb == 4 && vb == 3) { TQ_ATTN_256X(KFMT_TURBO, 4, 3); }
            else if (!turbo_k && vb == 2) { TQ_ATTN_256X(KFMT_Q8, 3, 2); }
            else if (!turbo_k && vb == 3) { TQ_ATTN_256X(KFMT_Q8, 3, 3); }
            else if (!turbo_k && vb == 4) { TQ_ATTN_256X(KFMT_Q8, 3, 4); }
            else if (!turbo_k && vb == 8) { TQ_ATTN_256X(KFMT_Q8, 3, 8); }
            else if (turbo_k && kb == 2 && vb == 8) { TQ_ATTN_256X(KFMT_TURBO, 2, 8); }
            else if (turbo_k && kb == 3 && vb == 8) { TQ_ATTN_256X(KFMT_TURBO, 3, 8); }
            else if (turbo_k && kb == 4 && vb == 8) { TQ_ATTN_256X(KFMT_TURBO, 4, 8); }
            else {
                tq_set_error("tq_decode_attention: head_dim 256 with K %d bits, V %d bits is not built", kb, vb);
                return TQ_ERR_UNSUPPORTED;
            }
#undef TQ_ATTN_256
#undef TQ_ATTN_256X
#undef TQ_ATTN_256_ONE
        } else {
#define TQ_ATTN_ONE(KF, KB, VB, SP, SH)                                            \
    {                                                                             \
        if (hg == 2 && a.sbias_n) k_decode_attn<KF, KB, VB, SP, SH, 2, true><<<grid, wg, merge_bytes, s>>>(a);   \
        else if (hg == 2) k_decode_attn<KF, KB, VB, SP, SH, 2, false><<<grid, wg, merge_bytes, s>>>(a);        \
        else if (a.sbias_n) k_decode_attn<KF, KB, VB, SP, SH, 1, true><<<grid, wg, merge_bytes, s>>>(a);        \
        else k_decode_attn<KF, KB, VB, SP, SH, 1, false><<<grid, wg, merge_bytes, s>>>(a);                      \
    }
#define TQ_ATTN(KF, KB, VB)                         \
    if (sparse) TQ_ATTN_ONE(KF, KB, VB, true, false)  \
    else TQ_ATTN_ONE(KF, KB, VB, false, false)
    // same width and same centroids: one table
#define TQ_ATTN_SAME(B)                                         \
    if (share && sparse) TQ_ATTN_ONE(KFMT_TURBO, B, B, true, true)    \
    else if (share) TQ_ATTN_ONE(KFMT_TURBO, B, B, false, true)        \
    else if (sparse) TQ_ATTN_ONE(KFMT_TURBO, B, B, true, false)       \
    else TQ_ATTN_ONE(KFMT_TURBO, B, B, false, false)
    if (turbo_k && kb == 3 && vb == 3) { TQ_ATTN_SAME(3); }
    else if (turbo_k && kb == 4 && vb == 4) { TQ_ATTN_SAME(4); }
    else if (turbo_k && kb == 2 && vb == 2) { TQ_ATTN_SAME(2); }
    else if (turbo_k && kb == 4 && vb == 2) { TQ_ATTN(KFMT_TURBO, 4, 2); }
    else if (turbo_k && kb == 3 && vb == 2) { TQ_ATTN(KFMT_TURBO, 3, 2); }
    else if (turbo_k && kb == 3 && vb == 4) { TQ_ATTN(KFMT_TURBO, 3, 4); }
    else if (turbo_k && kb == 4 && vb == 3) { TQ_ATTN(KFMT_TURBO, 4, 3); }
    else if (turbo_k && kb == 2 && vb == 3) { TQ_ATTN(KFMT_TURBO, 2, 3); }
    else if (turbo_k && kb == 2 && vb == 4) { TQ_ATTN(KFMT_TURBO, 2, 4); }
    else if (turbo_k && kb == 2 && vb == 8) { TQ_ATTN(KFMT_TURBO, 2, 8); }
    else if (!turbo_k && vb == 2) { TQ_ATTN(KFMT_Q8, 3, 2); }
    else if (!turbo_k && vb == 3) { TQ_ATTN(KFMT_Q8, 3, 3); }
    else if (!turbo_k && vb == 4) { TQ_ATTN(KFMT_Q8, 3, 4); }
    else if (!turbo_k && vb == 8) { TQ_ATTN(KFMT_Q8, 3, 8); }
    else if (turbo_k && kb == 3 && vb == 8) { TQ_ATTN(KFMT_TURBO, 3, 8); }
    else if (turbo_k && kb == 4 && vb == 8) { TQ_ATTN(KFMT_TURBO, 4, 8); }
    else {
        tq_set_error("tq_decode_attention: unsupported K/V format pair (k bits %d, v bits %d)", kb, vb);
        return TQ_ERR_UNSUPPORTED;
    }
        }
#undef TQ_ATTN
#undef TQ_ATTN_SAME
#undef TQ_ATTN_ONE
    rc = tq_check_launch("decode_attn");
    if (rc) return rc;
    if (skip_count && !a.poll_slots) {
        // more groups than the finishing workgroups poll (or a dense step whose caller wants the counts)
        k_skip_sum<<<1, 1024, 0, s>>>(a.skip_slots, sparse ? (int)grid : 0, skip_count, total_pairs, a.head_off > 0);
        rc = tq_check_launch("skip_sum");
        if (rc) return rc;
    }
    }
    return TQ_OK;
}

// ---- decode attention for callers that cannot allocate -----------------------------------
// The split partials live in a file-scope device array instead of a caller's workspace.  Every
// GPU the library runs on holds its own copy of the array, at its own address, until the process
// ends; the address is looked up once per device (with that device current) and kept.  In host
// code the array's name is only a handle for that lookup, never a device address.
namespace {
constexpr int64_t STATIC_WS_BYTES = TQ_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_WS_BYTES];
constexpr int MAX_DEVICES = 64;
void *g_scratch_ptr[MAX_DEVICES];  // per device: device address of that GPU's copy of `scratch`
std::mutex g_scratch_mutex;
}  // namespace

// Device address of the current device's scratch array (looked up on the first call per device).
int tqk_static_scratch(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        tq_set_error("static workspace: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
        return TQ_ERR_HIP;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            tq_set_error("static workspace: hipGetSymbolAddress: %s", hipGetErrorString(e));
            return TQ_ERR_HIP;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return TQ_OK;
}

int tqk_decode_attention_static(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q,
                                int q_dtype, const void *k, const void *v, const float *bias, float *out,
                                unsigned long long *skip_count, hipStream_t s) {
    const int64_t need = ws_layout(p).total;
    if (need > STATIC_WS_BYTES) {
        tq_set_error("tq_decode_attention_static: batch * n_kv_heads * n_splits = %lld needs %lld bytes of split "
                     "partials, the built-in workspace holds %lld; lower n_splits or use tq_decode_attention",
                     (long long)p->batch * p->n_kv_heads * p->n_splits, (long long)need, (long long)STATIC_WS_BYTES);
        return TQ_ERR_UNSUPPORTED;
    }
    void *ptr = nullptr;
    const int rc = tqk_static_scratch(&ptr);
    if (rc) return rc;
    // every partial and every skip slot that the merge kernel reads is written by this call's main kernel first,
    // so nothing of the previous call's contents needs clearing
    return tqk_decode_attention(hk, hv, p, q, q_dtype, k, nullptr, v, bias, out, skip_count, ptr, STATIC_WS_BYTES, s);
}

// ---- prefill-shaped TurboQuant inner-product estimator --------------------------------
namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
constexpr int KT_STRIDE = 264;  // halves per staged key row (256 + 8: 16-byte reads of 16 rows hit 64 distinct banks)

// [R q | S q] as fp16 on the matrix cores: a workgroup of four wavefronts takes 32 queries, wavefront w the output
// rows 32w .. 32w+31 of the rotation and of the projection, as (W Q^T) with W's fragments prepared with the handle
// (rotation: +-1 entries, exact; projection: two fp16 terms) and the queries as the column side.  Queries that are
// not fp16 are split into two fp16 terms as well, so that every product is exact and the sums carry fp32 rounding
// only (as the scalar loop did).  Lane l ends up with query l % 32 and four consecutive outputs per register
// group: an 8-byte store, 512 contiguous bytes per wavefront.
template <typename TI>
__global__ __launch_bounds__(256) void k_prep_score_q(const TI *q, __half *qa, int64_t nq, const uint4 *wfrag) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int r = lane & 31, kb = lane >> 5;
    const int64_t blk = blockIdx.x;
    const int64_t v = min(blk * 32 + r, nq - 1);  // rows past the last query repeat it (their block is allocated)
    constexpr bool SPLIT = !std::is_same<TI, __half>::value;
    half8_t xh[8], xl[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const TI *src = q + v * 128 + 16 * t + 8 * kb;
        if constexpr (!SPLIT) {
            xh[t] = *reinterpret_cast<const half8_t *>(src);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float x = ldf(src + e);
                const _Float16 hi = (_Float16)x;
                xh[t][e] = hi;
                xl[t][e] = (_Float16)(x - (float)hi);
            }
        }
    }
    constexpr int SET = 4 * 8 * 64;  // fragments (16 bytes) per set
    const uint4 *fr = wfrag + (w * 8) * 64 + lane;
    float16_t rot, prj;
#pragma unroll
    for (int e = 0; e < 16; ++e) rot[e] = prj[e] = 0.0f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const half8_t wr = __builtin_bit_cast(half8_t, fr[t * 64]);
        const half8_t wh = __builtin_bit_cast(half8_t, fr[SET + t * 64]);
        const half8_t wl = __builtin_bit_cast(half8_t, fr[2 * SET + t * 64]);
        rot = __builtin_amdgcn_mfma_f32_32x32x16_f16(wr, xh[t], rot, 0, 0, 0);
        prj = __builtin_amdgcn_mfma_f32_32x32x16_f16(wl, xh[t], prj, 0, 0, 0);
        if constexpr (SPLIT) {
            rot = __builtin_amdgcn_mfma_f32_32x32x16_f16(wr, xl[t], rot, 0, 0, 0);
            prj = __builtin_amdgcn_mfma_f32_32x32x16_f16(wh, xl[t], prj, 0, 0, 0);
        }
        prj = __builtin_amdgcn_mfma_f32_32x32x16_f16(wh, xh[t], prj, 0, 0, 0);
    }
    // operand-major layout: the 16-byte chunk (row r of query block v / 32, K values 16t + 8kb .. + 7) that
    // lane r + 32kb of the score tile's MFMA reads in K step t sits at chunk index (block * 16 + t) * 64 + r + 32kb,
    // so one wave-wide operand load is 1 KB of contiguous memory.  Register group j of this lane holds outputs
    // 32w + 8j + 4kb + i, i = 0..3: elements 4kb .. 4kb+3 of the chunk of step (32w + 8j) / 16, half (j & 1).
#pragma unroll
    for (int part = 0; part < 2; ++part)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int o = 128 * part + 32 * w + 8 * j;  // first K value of the chunk
            const int t = o >> 4, half_sel = (o >> 3) & 1;
            const float sc = part == 0 ? RSQRT128 : 1.0f;
            const float16_t &a = part == 0 ? rot : prj;
            const __half2 lo2 = __halves2half2(__float2half_rn(a[4 * j] * sc), __float2half_rn(a[4 * j + 1] * sc));
            const __half2 hi2 = __halves2half2(__float2half_rn(a[4 * j + 2] * sc), __float2half_rn(a[4 * j + 3] * sc));
            uint2 u;
            u.x = *reinterpret_cast<const uint32_t *>(&lo2);
            u.y = *reinterpret_cast<const uint32_t *>(&hi2);
            *reinterpret_cast<uint2 *>(qa + (((blk * 16 + t) * 64 + r + 32 * half_sel) * 8 + 4 * kb)) = u;
        }
}

// One workgroup of eight wavefronts per 256 keys.  The keys are dequantised once into LDS as fp16
// [g*c[idx] | scale*rnorm*z]; every wavefront then takes the operands of its 64 keys into registers (128 of
// them) and the same LDS carries the queries instead, 128 at a time, double-buffered, brought in by loads that
// write LDS directly.  Matrix tiles are 32 x 32 x 16 with the queries on the M side and the keys on the N side.
// Wavefront w works on key group w % 4 (64 keys) and on the query half w / 4 of a tile, 32 queries at a time:
// per K step one query operand from LDS feeds two matrix instructions (the two 32-key halves of the group).
// The four wavefronts of a query half finish the same 32 logit rows at about the same time, each its own 64
// logits of them, so a row leaves the workgroup as 256 consecutive logits (1 KB in fp32) within a short time,
// not as 128-byte pieces spread over a sweep: the memory side takes that order markedly faster.
constexpr int SCORE_KEYS = 256;  // keys per workgroup (two 128-row blocks)
constexpr int SCORE_QT = 128;  // queries per LDS tile: four operand blocks of 16 KB
template <int BITS, typename TO, bool DRAIN>
__global__ __launch_bounds__(512, 1) void k_score_tile(const __half *qa, const uint8_t *packed, const uint8_t *sign_bits,
                                                      const __half *rnorms, int64_t nq, int64_t nk, TO *logits,
                                                      const uint32_t *pair_lut, float proj_scale) {
    extern __shared__ __attribute__((aligned(16))) _Float16 kt[];  // keys [SCORE_KEYS][KT_STRIDE], then two query tiles
    __shared__ uint32_t ptab[1 << (2 * BITS)];                     // pair code -> (c[lo], c[hi]) as two halves
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int64_t key0 = (int64_t)blockIdx.x * SCORE_KEYS;
    const int n_blocks = (int)((nq + 31) / 32);  // operand blocks the preparation wrote
    const int n_tiles = (int)((nq + SCORE_QT - 1) / SCORE_QT);
    typedef uint32_t chunk_t __attribute__((ext_vector_type(4)));   // 16 bytes: what a lane feeds to one matrix instruction
    const chunk_t *qchunks = reinterpret_cast<const chunk_t *>(qa);  // [block][K step][lane]
    // chunk group g (0..7) of a tile: lanes tid + 512 g of its 4096 chunks, i.e. half g % 2 of operand block g / 2
    auto tile_chunk = [&](int tile, int g) __attribute__((always_inline)) {
        const int blk = min(tile * (SCORE_QT / 32) + (g >> 1), n_blocks - 1);  // past the end: the last block again
        return qchunks + (int64_t)blk * 1024 + (g & 1) * 512 + tid;
    };
    // the first tile is requested before anything else and waits in registers until the keys have left LDS
    chunk_t first_tile[8];
#pragma unroll
    for (int g = 0; g < 8; ++g) first_tile[g] = *tile_chunk(0, g);
    if (tid < (1 << (2 * BITS))) ptab[tid] = pair_lut[tid];
    __syncthreads();
    {
        // threads 0..255 dequantise the codes of one key each, threads 256..511 its sign bits; eight halves
        // (16 bytes) per LDS write
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        const int key = tid & (SCORE_KEYS - 1), part = tid >> 8;
        uint4 *row = reinterpret_cast<uint4 *>(kt + key * KT_STRIDE) + part * 16;
        const bool valid = key0 + key < nk;
        if (part == 0) {
            if (valid) {
                const uint8_t *block = packed + (key0 + key) / TQ_ROWS_PER_BLOCK * (TQ_ROWS_PER_BLOCK * (16 * BITS + 2));
                uint32_t wv[4 * BITS];
                load_row<BITS>(block, key & (TQ_ROWS_PER_BLOCK - 1), wv);
                const _Float16 g = __builtin_bit_cast(
                    _Float16, reinterpret_cast<const unsigned short *>(block + TQ_ROWS_PER_BLOCK * 16 * BITS)[key & (TQ_ROWS_PER_BLOCK - 1)]);
                const half2_t g2 = {g, g};
#pragma unroll
                for (int c = 0; c < 16; ++c) {
                    uint32_t u[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t e = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const char *>(ptab) +
                                                                               pair_off<BITS>(wv, 4 * c + i));
                        u[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, e) * g2);
                    }
                    row[c] = make_uint4(u[0], u[1], u[2], u[3]);
                }
            } else {
#pragma unroll
                for (int c = 0; c < 16; ++c) row[c] = make_uint4(0, 0, 0, 0);
            }
        } else {
            float rs = 0.f;
            uint4 sb = make_uint4(0, 0, 0, 0);
            if (valid) {
                rs = proj_scale * __half2float(rnorms[key0 + key]);
                sb = *reinterpret_cast<const uint4 *>(sign_bits + (key0 + key) * 16);
            }
            const uint32_t sw[4] = {sb.x, sb.y, sb.z, sb.w};
            // +rs where the bit is set, -rs where it is clear: two halves per word, the sign bits from the inverted bits
            const uint32_t mag = (uint32_t)__half_as_ushort(__float2half_rn(rs)) * 0x00010001u;
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                uint32_t u[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int jj = 8 * c + 2 * i;  // sign bits jj, jj + 1
                    const uint32_t nb = ~sw[jj >> 5] >> (jj & 31);
                    u[i] = mag ^ (((nb & 1u) << 15) | ((nb & 2u) << 30));
                }
                row[c] = make_uint4(u[0], u[1], u[2], u[3]);
            }
        }
    }
    __syncthreads();

    // lane l of a 32 x 32 result tile holds key column l % 32 for the query rows 8j + 4(l/32) + i
    const int kg = __builtin_amdgcn_readfirstlane(w & 3), qh = __builtin_amdgcn_readfirstlane(w >> 2);
    const int c32 = lane & 31, kb = lane >> 5;
    half8_t kf[2][16];  // [32-key half of the group][K step of 16]
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
        for (int t = 0; t < 16; ++t)
            kf[kh][t] = *reinterpret_cast<const half8_t *>(kt + (kg * 64 + kh * 32 + c32) * KT_STRIDE + t * 16 + 8 * kb);
    __syncthreads();  // every wavefront has its keys: the memory now holds query tiles
    chunk_t *qtile = reinterpret_cast<chunk_t *>(kt);  // [2][4096] chunks
#pragma unroll
    for (int g = 0; g < 8; ++g) qtile[g * 512 + tid] = first_tile[g];
    // (LDS only: a __syncthreads would also wait for the logit stores in flight)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // A finished (32 queries, 64 keys) block is written while the next one is being multiplied: one store
    // instruction after each matrix instruction, from a second set of accumulators.  One v_permlane32_swap per
    // accumulator pair puts the row 8j + i of both key halves into one register (lanes 0..31 the first half's 32
    // keys, lanes 32..63 the second's) and the row 8j + 4 + i into the other, so a store writes 64 consecutive
    // logits of one row.  The stores are buffer stores whose resource is that row's piece (scalar arithmetic): its
    // size is 0 for a row past the last query and ends at the last key, so the hardware drops what does not exist
    // and no store needs an address register or a branch.
    constexpr int NT_AUX = (TQ_STREAM_SITES & STREAM_LOGITS) ? 2 : 0;  // the non-temporal bit of a buffer instruction
    const int64_t key0w = key0 + kg * 64;
    const uint32_t piece_bytes = (uint32_t)max((int64_t)0, min((int64_t)64, nk - key0w)) * (uint32_t)sizeof(TO);
    const int lane_off = lane * (int)sizeof(TO);
    struct Pending {
        TO *base;  // first logit of the block's first row in this wavefront's key group
        int rows;  // rows of the block that exist (0: nothing is pending)
    };
    auto pend = [&](int row0) __attribute__((always_inline)) {
        Pending pb;
        pb.rows = __builtin_amdgcn_readfirstlane(max(0, min(32, (int)nq - row0)));
        const uint64_t b = reinterpret_cast<uint64_t>(logits + (int64_t)row0 * nk + key0w);
        // wave-uniform by construction; said explicitly so that the resources are built by scalar instructions
        pb.base = reinterpret_cast<TO *>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b >> 32)) << 32) |
                                         (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b));
        return pb;
    };
    auto store_row = [&](const Pending &pb, const uint32_t bits, const int row) __attribute__((always_inline)) {
        const uint32_t size = row < pb.rows ? piece_bytes : 0u;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(pb.base + (int64_t)row * nk, 0, (int)size, 0x00020000);
        if constexpr (sizeof(TO) == 4) {
            __builtin_amdgcn_raw_buffer_store_b32(bits, rs, lane_off, 0, NT_AUX);
        } else {
            __builtin_amdgcn_raw_buffer_store_b16(__half_as_ushort(__float2half_rn(__uint_as_float(bits))), rs, lane_off, 0, NT_AUX);
        }
    };

    float keep = 0.0f;  // measurement mode (no logits): the products stay live through a store that never happens
    // one block of 32 queries (operand block `b` of the tile in `cur`) against the 64 resident keys into acc, while
    // the pending block leaves from pacc; the first block of a tile also asks for the next tile (eight loads that
    // write LDS directly, one per step: no registers, no LDS write instructions, and a lead of at least 20 steps).
    // Query operands come from LDS AHEAD steps ahead, across blocks too: `pre` holds the first AHEAD operands of this
    // block on entry and those of the block that follows (operand block `b_after` of the buffer `after`) on exit.  The
    // second block of a tile therefore carries the tile's barrier, at the step in which its own last operand read has
    // been issued: behind it no wavefront reads `cur` any more, so the next tile may start filling it, and `next` is
    // complete.  Vector memory operations complete in issue order and 21 steps of two stores each lie between a
    // tile's last load and that step, so "at most 32 outstanding" covers the loads with a margin and leaves the
    // youngest logit stores in flight (a __syncthreads would wait for all of them).
    constexpr int AHEAD = 3;
    auto block = [&](const chunk_t *cur, chunk_t *next, const int b, const chunk_t *after, const int b_after, auto half,
                     const int tile_next, half8_t (&pre)[AHEAD], float16_t (&acc)[2], const float16_t (&pacc)[2],
                     const Pending &pb) __attribute__((always_inline)) {
        constexpr int HALF = decltype(half)::value;
        const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const chunk_t *arow = cur + b * 1024 + lane;
        const chunk_t *arow_after = after + b_after * 1024 + lane;
        // the scheduling fence after every step keeps the compiler from hoisting all sixteen steps' reads to the top
        half8_t af[AHEAD + 1];
#pragma unroll
        for (int t = 0; t < AHEAD; ++t) af[t] = pre[t];
        uint32_t swapped = 0u;
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            if (t + AHEAD < 16) af[(t + AHEAD) & AHEAD] = __builtin_bit_cast(half8_t, arow[(t + AHEAD) * 64]);
            if (HALF == 1 && t + AHEAD == 16) {
                if constexpr (DRAIN) asm volatile("s_waitcnt vmcnt(32) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
            if (t + AHEAD >= 16) pre[t + AHEAD - 16] = __builtin_bit_cast(half8_t, arow_after[(t + AHEAD - 16) * 64]);
            if (HALF == 0 && t < 8) {
                // lane l of the wavefront brings chunk l of the wavefront's 1 KB piece of chunk group g
                const int g = t;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(tile_chunk(tile_next, g)),
                                                 (__attribute__((address_space(3))) void *)(next + g * 512 + w * 64), 16, 0, 0);
            }
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                acc[kh] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[t & AHEAD], kf[kh][t], t == 0 ? zero : acc[kh], 0, 0, 0);
                if constexpr (DRAIN) {
                    // accumulator element t = 4j + i: rows 8j + i (kh = 0 here) and 8j + 4 + i (kh = 1)
                    const int row = 8 * (t >> 2) + (t & 3);
                    if (kh == 0) {
                        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(pacc[0][t]), __float_as_uint(pacc[1][t]), false, false);
                        swapped = r[1];
                        store_row(pb, r[0], row);
                    } else {
                        store_row(pb, swapped, row + 4);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (!DRAIN) {
#pragma unroll
            for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                for (int e = 0; e < 16; ++e) keep += acc[kh][e];
        }
    };
    float16_t acc_a[2], acc_b[2];
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc_b[kh][e] = 0.0f;
    Pending pb = pend(0);
    pb.rows = 0;  // nothing is pending before the first block
    half8_t pre[AHEAD];
#pragma unroll
    for (int t = 0; t < AHEAD; ++t) pre[t] = __builtin_bit_cast(half8_t, qtile[(2 * qh) * 1024 + t * 64 + lane]);
#pragma unroll 1
    for (int tile = 0; tile < n_tiles; ++tile) {
        const chunk_t *cur = qtile + (tile & 1) * 4096;
        chunk_t *next = qtile + ((tile + 1) & 1) * 4096;
        const int row0 = tile * SCORE_QT + qh * 64;
        const int tile_next = min(tile + 1, n_tiles - 1);  // the last tile re-reads itself
        block(cur, next, 2 * qh, cur, 2 * qh + 1, std::integral_constant<int, 0>{}, tile_next, pre, acc_a, acc_b, pb);
        pb = pend(row0);
        block(cur, next, 2 * qh + 1, next, 2 * qh, std::integral_constant<int, 1>{}, tile_next, pre, acc_b, acc_a, pb);
        pb = pend(row0 + 32);
    }
    if constexpr (DRAIN) {  // the last block (in acc_b)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc_b[0][e]), __float_as_uint(acc_b[1][e]), false, false);
            const int row = 8 * (e >> 2) + (e & 3);
            store_row(pb, r[0], row);
            store_row(pb, r[1], row + 4);
        }
    } else {
        if (keep == 1.25e38f) reinterpret_cast<float *>(const_cast<__half *>(qa))[0] = keep;
    }
}

}  // namespace

int tqk_score_tile(const tq_handle *h, const void *q, int q_dtype, int64_t nq, const void *packed,
                   const uint8_t *sign_bits, const void *rnorms, int64_t nk, void *logits, int out_dtype, void *ws,
                   int64_t ws_bytes, hipStream_t s) {
    (void)ws_bytes;
    if (nq >= ((int64_t)1 << 31) / 128) {
        tq_set_error("tq_score_tile: %lld queries beyond 2^24 - 1", (long long)nq);
        return TQ_ERR_UNSUPPORTED;
    }
    __half *qa = reinterpret_cast<__half *>(ws);
    const unsigned qgrid = (unsigned)((nq + 31) / 32);
    const uint4 *wfrag = reinterpret_cast<const uint4 *>(h->score_wfrag);
    switch (q_dtype) {
    case TQ_F16: k_prep_score_q<__half><<<qgrid, 256, 0, s>>>((const __half *)q, qa, nq, wfrag); break;
    case TQ_F32: k_prep_score_q<float><<<qgrid, 256, 0, s>>>((const float *)q, qa, nq, wfrag); break;
    case TQ_F64: k_prep_score_q<double><<<qgrid, 256, 0, s>>>((const double *)q, qa, nq, wfrag); break;
    default: tq_set_error("bad q dtype %d", q_dtype); return TQ_ERR_ARG;
    }
    int rc = tq_check_launch("prep_score_q");
    if (rc) return rc;
    const unsigned grid = (unsigned)((nk + SCORE_KEYS - 1) / SCORE_KEYS);
    const size_t lds = (size_t)SCORE_KEYS * KT_STRIDE * sizeof(_Float16);
#define TQ_SCORE(B, T, DR)                                                                                             \
    {                                                                                                                  \
        (void)hipFuncSetAttribute((const void *)k_score_tile<B, T, DR>, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                  (int)lds);                                                                           \
        k_score_tile<B, T, DR><<<grid, 512, lds, s>>>(qa, (const uint8_t *)packed, sign_bits, (const __half *)rnorms, \
                                                      nq, nk, (T *)logits, (const uint32_t *)h->pair_lut, (float)h->proj_scale); \
    }
#define TQ_SCORE_BITS(T, DR)                                                                              \
    if (h->bits == 2) TQ_SCORE(2, T, DR) else if (h->bits == 3) TQ_SCORE(3, T, DR) else TQ_SCORE(4, T, DR)
    if (!logits) {
        TQ_SCORE_BITS(float, false)  // measurement mode: everything but the stores
    } else if (out_dtype == TQ_F32) {
        TQ_SCORE_BITS(float, true)
    } else {
        TQ_SCORE_BITS(__half, true)
    }
#undef TQ_SCORE_BITS
#undef TQ_SCORE
    return tq_check_launch("score_tile");
}
