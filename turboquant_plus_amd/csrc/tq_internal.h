// Internal declarations shared by the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include "tq.h"

#define TQ_MAX_D 4096
#define TQ_ROWS_PER_BLOCK 128

// Device-resident constant tables of a quantiser.  Everything the kernels read
// through this struct is written once in tq_create.
struct tq_handle {
    int d, pd, bits, n_centroids, rotation, norm_correction;
    int device;
    // float64 tables (reference-API kernels)
    double *centroids64;   // [n_centroids]
    double *bounds64;      // [n_centroids-1] midpoints
    double *s1_64, *s2_64; // [pd] (WHT)
    double *rot64;         // [d*d]  Pi,   row-major          (dense)
    double *rot64_t;       // [d*d]  Pi^T, row-major          (dense)
    double *proj64;        // [d*d]  S
    double *proj64_t;      // [d*d]  S^T
    double proj_scale;
    int has_proj;
    // float32 tables (production kernels, d == 128, WHT)
    float *centroids32;    // [n_centroids]
    float *bounds32;       // [n_centroids-1]
    float *s1_32, *s2_32;  // [128]
    double *projrot64_t;   // [128*128] entry [k*128+j] = (S R^T)[j][k]   (d == 128, WHT, projection)
    void *pair_lut;        // [4^bits] half2: (c[lo], c[hi]) for a pair code (bits <= 3), or [256] for 4
    uint32_t pair_lut_host[256];  // host copy of pair_lut (two handles with equal tables can share one LDS copy)
    uint16_t *qjl_frag;    // [3][4][8][64][8] fp16: 64 (S R^T) split into three fp16 terms, as B operands of 16x16x32 matrix instructions (QJL store)
    float qjl_tau;         // first pass (fp16 matrix cores): |value| below qjl_tau * |scaled residual| goes to the second pass
    double qjl_tau2;       // second pass (float64 against the three terms): |value| below qjl_tau2 * |residual| goes to the float64 matrix
    uint16_t *score_wfrag; // [3][4][8][64][8] fp16: operand fragments of [D2 H D1 ; S hi ; S lo] (query preparation, score tile)
    void *rfrag16k;        // [8][64][8] fp16 +-1: fragment f0*4+ks, lane l, element e = s1[k] H[m][k] with
                           // m = 32(l%16/4) + 4 f0 + l%4, k = 32(l/16) + 8 ks + e (factored transform, K rows)
    void *rfrag16k_inv;    // rfrag16k with s2 in place of s1: the transposed rotation of K-row-shaped data (tq_load)
    void *rfrag16v;        // [8][64][8] fp16 +-1: fragment d0*4+ks, lane l, element e = s1[k] H[16 d0 + l%16][k],
                           // k = 32 ks + 8(l/16) + e (factored transform, V rows: B operand)
    uint32_t *s2flip;      // [4][4]: per lane quarter and output dword, sign-field positions of dims with s2 = +1
    float *symthr32;       // [2^(bits-1)]: middle boundary, then the positive boundaries
    float *sqcoef32;       // [2^(bits-1)]: c[mid+1+m]^2 = sum over subsets S of the set bits of m of sqcoef32[S]
    uint2 *quant_lut;      // [4096] indexed by the top 12 bits (sign, exponent, 3 mantissa bits) of a normalised
                           // rotated value: .x = sign << (bits-1) | number of positive boundaries below the bin,
                           // .y = fp32 bits of the one boundary inside the bin (+inf when there is none)
    int quant_lut_ok;      // every bin holds at most one boundary (else the table cannot decide a level)
    uint64_t quant_lut_hash;  // hash of the table's contents
    // host copies of the small constants, passed to the fused K+V store by value (kernel arguments), so that its
    // wavefronts need nothing from memory before their first input
    uint32_t s1neg_host[4], s2neg_host[4];  // bit k of word k / 32: s1[k] < 0, s2[k] < 0
    uint32_t s2flip_host[16];               // host copy of s2flip
    float symthr_host[8], sqcoef_host[8];   // host copies of symthr32, sqcoef32 (2^(bits-1) entries used)
    double centroids_host[16], bounds_host[15];  // host copies of the codebook and its midpoints (n_centroids <= 16)
    int zero_code;         // codebook index of the value 0.0 (#boundaries below 0)
    int symmetric;         // boundaries are sign-symmetric in fp32 (fast quantiser usable)
};

static inline int tq_padded_dim(int d) {
    int p = 1;
    while (p < d) p <<= 1;
    return p;
}

// ---- launchers implemented in the kernel files -------------------------------
int tqk_fwht(const void *x, void *y, int64_t n, int len, int in_dtype, int out_dtype, hipStream_t s);
int tqk_rotate64(const tq_handle *h, const void *x, void *y, int64_t n, int in_dtype, int out_dtype, int transpose,
                 hipStream_t s);
int tqk_nearest(const double *values, int64_t n, const double *bounds_host, int nb, int32_t *idx, hipStream_t s);
int tqk_quantize_indices(const tq_handle *h, const void *x, int64_t n, int in_dtype, uint8_t *idx, double *norms,
                         double *rotated, hipStream_t s);
int tqk_dequantize_indices(const tq_handle *h, const uint8_t *idx, const double *norms, int64_t n, double *out,
                           const void *x, int x_dtype, double *residual, hipStream_t s);
int tqk_qjl_quantize(const tq_handle *h, const void *r, int64_t n, int in_dtype, int8_t *signs, double *norms,
                     hipStream_t s);
int tqk_qjl_dequantize(const tq_handle *h, const int8_t *signs, const double *norms, double shrinkage, int64_t n,
                       double *out, hipStream_t s);
int tqk_pack_bits(const int8_t *signs, int64_t n, int d, uint8_t *packed, hipStream_t s);
int tqk_unpack_bits(const uint8_t *packed, int64_t n, int d, int8_t *signs, hipStream_t s);
int tqk_pack_indices(const uint8_t *idx, int64_t count, int bits, uint8_t *packed, hipStream_t s);

int tqk_rotate128(const tq_handle *h, const void *x, void *y, int64_t n, int in_dtype, int out_dtype, int transpose,
                  hipStream_t s);
int tqk_store(const tq_handle *h, const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, int kind, void *packed,
              uint8_t *sign_bits, void *rnorms, hipStream_t s);
int tqk_append(const tq_handle *h, const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype,
               int kind, void *packed, hipStream_t s, const int64_t *pos_dev = nullptr, uint32_t *overrun = nullptr);
int tqk_append_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t pos,
                  int64_t n_new, int64_t capacity, int in_dtype, void *packed_k, void *packed_v, hipStream_t s,
                  const int64_t *pos_dev = nullptr, uint32_t *overrun = nullptr);
int tqk_requantize(const tq_handle *hs, const tq_handle *hd, const void *src, int64_t n_seqs, int64_t tokens, int kind, void *dst,
                   hipStream_t s);
int tqk_fork_blocks(const tq_handle *h, int to_fork, const void *src, int64_t n_seqs, int64_t tokens, int kind, void *dst,
                    int block_values, hipStream_t s);
int tqk_store_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t tokens,
                 int64_t capacity, int in_dtype, void *packed_k, void *packed_v, hipStream_t s);
int tqk_load(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, void *out,
             int out_dtype, int domain, hipStream_t s);
int tqk_load_kv(const tq_handle *hk, const tq_handle *hv, const void *packed_k, const void *packed_v, int64_t n_seqs,
                int64_t tokens, void *out_k, void *out_v, hipStream_t s);
int tqk_unpack_codes(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, uint8_t *idx,
                     float *norms, hipStream_t s);
int tqk_q8_0_store(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, hipStream_t s);
int tqk_q8_0_append(const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype, int kind,
                    void *packed, hipStream_t s, const int64_t *pos_dev = nullptr, uint32_t *overrun = nullptr);
int tqk_q8_0_store_v(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, hipStream_t s);
int tqk_q8_0_unpack(const void *packed, int64_t n_seqs, int64_t tokens, int8_t *q, float *scales, int kind, hipStream_t s);

int64_t tqk_attn_workspace_bytes(const tq_attn_params *p);
int tqk_decode_attention(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q, int q_dtype,
                         const void *k, const void *k_aux, const void *v, const float *bias, float *out,
                         unsigned long long *skip_count, void *ws, int64_t ws_bytes, hipStream_t s);
int tqk_static_scratch(void **out);
int tqk_decode_attention_static(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q,
                                int q_dtype, const void *k, const void *v, const float *bias, float *out,
                                unsigned long long *skip_count, hipStream_t s);
int tqk_score_tile(const tq_handle *h, const void *q, int q_dtype, int64_t nq, const void *packed,
                   const uint8_t *sign_bits, const void *rnorms, int64_t nk, void *logits, int out_dtype, void *ws,
                   int64_t ws_bytes, hipStream_t s);

void tq_set_error(const char *fmt, ...);
int tq_check_launch(const char *what);
