/*
 * tq.h - C ABI of the MI355X (gfx950) TurboQuant+ KV-codec library.
 *
 * The reference (TheTom/turboquant_plus) has no FFI for this path: it is plain
 * Python over NumPy.  Each entry point below names the reference function whose
 * per-vector arithmetic it replaces (file:line in the reference tree); the
 * Python classes of the same names call these through ctypes.
 *
 * Conventions
 *   - every data pointer is DEVICE memory unless the comment says "host";
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - all entry points enqueue work and return without synchronising;
 *   - return value 0 = TQ_OK, negative = error (tq_last_error() has the text);
 *   - a handle is immutable after tq_create and may be shared across threads;
 *   - the library allocates device memory only in tq_create (small constant
 *     tables) and frees it in tq_destroy.
 */
#ifndef TQ_H
#define TQ_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TQ_OK 0
#define TQ_ERR_ARG (-1)         /* null pointer, negative size, bad enum          */
#define TQ_ERR_UNSUPPORTED (-2) /* shape / mode the kernels do not cover           */
#define TQ_ERR_ALIGN (-3)       /* pointer not aligned as the entry point requires */
#define TQ_ERR_HIP (-4)         /* HIP runtime error (no device, launch failure)   */

enum { TQ_F16 = 0, TQ_F32 = 1, TQ_F64 = 2 };
enum { TQ_ROT_DENSE = 0, TQ_ROT_WHT = 1 };
enum { TQ_KIND_K = 0, TQ_KIND_V = 1 };
enum { TQ_DOMAIN_ROTATED = 0, TQ_DOMAIN_ORIGINAL = 1 };
enum { TQ_KFMT_TURBO = 0, TQ_KFMT_Q8_0 = 1 };

typedef struct tq_handle tq_handle;

/* All pointers in tq_config are HOST pointers, copied at tq_create. */
typedef struct tq_config {
    int32_t d;                /* vector dimension (1..4096; fused kernels need 128)   */
    int32_t bits;             /* codebook bits, 1..8                                  */
    int32_t rotation;         /* TQ_ROT_DENSE | TQ_ROT_WHT                            */
    int32_t norm_correction;  /* polar_quant.py:109-112                               */
    const double *centroids;  /* [1<<bits], sorted (codebook.py:29-49)                */
    const double *signs1;     /* [padded_d], WHT mode (rotation.py:94)                */
    const double *signs2;     /* [padded_d], WHT mode (rotation.py:95)                */
    const double *rotation_matrix; /* [d*d] row-major, dense mode (rotation.py:25-50) */
    const double *projection; /* [d*d] row-major QJL matrix S or NULL (qjl.py:57-62)  */
    double projection_scale;  /* sqrt(pi/2)/sqrt(d) (qjl.py:131) or sqrt(pi/2)/d      */
} tq_config;

int tq_version(void);
const char *tq_last_error(void);           /* thread-local text of the last failure  */
int tq_device_count(void);                 /* 0 when no GPU is visible               */

int tq_create(tq_handle **out, const tq_config *cfg);
void tq_destroy(tq_handle *h);

/* ---- reference-API kernels: float64 arithmetic, any d <= 4096 ---------------- */

/* rotation.py:99-121 fast_walsh_hadamard_transform on each of n rows of length
 * len (power of two <= 4096); normalised by 1/sqrt(len). */
int tq_fwht(const void *x, void *y, int64_t n, int32_t len, int in_dtype, int out_dtype, void *stream);

/* The handle's rotation applied to n rows of length d: dense Pi x (polar_quant.py:78)
 * or D2 H D1 x with zero padding (rotation.py:124-185); transpose != 0 applies the
 * transpose (polar_quant.py:114, rotation.py:148-160).  With d == 128, WHT mode and
 * no float64 on either side the one-wavefront-per-vector fp32 butterfly runs. */
int tq_rotate(const tq_handle *h, const void *x, void *y, int64_t n, int in_dtype, int out_dtype,
              int transpose, void *stream);

/* codebook.py:121-134 nearest_centroid_indices: idx = #{midpoints < value}.
 * centroids: host pointer, n_centroids <= 256. */
int tq_nearest_centroid(const double *values, int64_t n, const double *centroids_host, int32_t n_centroids,
                        int32_t *idx, void *stream);

/* polar_quant.py:56-85 PolarQuant.quantize: idx [n,d] uint8, norms [n] float64.
 * rotated (optional, may be NULL) receives the rotated unit vectors [n,d] float64. */
int tq_quantize_indices(const tq_handle *h, const void *x, int64_t n, int in_dtype, uint8_t *idx, double *norms,
                        double *rotated, void *stream);

/* polar_quant.py:87-119 PolarQuant.dequantize -> out [n,d] float64.  When x is not
 * NULL also writes residual = x - out (polar_quant.py:121-132). */
int tq_dequantize_indices(const tq_handle *h, const uint8_t *idx, const double *norms, int64_t n, double *out,
                          const void *x, int x_dtype, double *residual, void *stream);

/* qjl.py:72-94 QJL.quantize: signs [n,d] int8 in {+1,-1} (0 -> +1), norms [n] float64. */
int tq_qjl_quantize(const tq_handle *h, const void *r, int64_t n, int in_dtype, int8_t *signs, double *norms,
                    void *stream);

/* qjl.py:96-134 QJL.dequantize: out = S^T z * (projection_scale * norm * shrinkage). */
int tq_qjl_dequantize(const tq_handle *h, const int8_t *signs, const double *norms, double shrinkage, int64_t n,
                      double *out, void *stream);

/* utils.py:20-49 pack_bits / utils.py:52-68 unpack_bits on [n,d] int8 signs. */
int tq_pack_bits(const int8_t *signs, int64_t n, int32_t d, uint8_t *packed, void *stream);
int tq_unpack_bits(const uint8_t *packed, int64_t n, int32_t d, int8_t *signs, void *stream);

/* utils.py:71-98 pack_indices: one MSB-first bit stream over count indices (bits 1..4);
 * packed must hold ceil(count*bits/8) bytes. */
int tq_pack_indices(const uint8_t *idx, int64_t count, int32_t bits, uint8_t *packed, void *stream);

/* ---- production format ("turbo2/3/4"): d = 128, WHT rotation, fp32 arithmetic,
 *      corrected fp16 norm, 128-token blocks ----------------------------------- */

/* Bytes of the packed buffer for n_seqs sequences of `tokens` tokens each
 * (blocks never straddle sequences): n_seqs * ceil(tokens/128) * 128*(16*bits+2). */
int64_t tq_packed_bytes(int32_t bits, int64_t n_seqs, int64_t tokens);

/* Norm -> normalise -> D2 H D1 -> nearest centroid -> corrected fp16 norm -> pack.
 * Replaces the per-vector work of KVCacheCompressor.compress (kv_cache.py:98-141)
 * for the MSE-only ("turboN") format; arithmetic of polar_quant.py:56-85 with the
 * rotation of rotation.py:163-185 and the write-side norm correction of
 * benchmarks/temporal_decay_prototype.py:58-90.  x is [n_seqs, tokens, 128];
 * x and packed must be 16-byte aligned. */
int tq_store(const tq_handle *h, const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, int kind,
             void *packed, void *stream);

/* K and V of one layer in one launch: the two tensors that KVCacheCompressor.compress
 * (kv_cache.py:98-141) takes together.  Same results as tq_store(hk, k, .., TQ_KIND_K, ..)
 * followed by tq_store(hv, v, .., TQ_KIND_V, ..); k and v are [n_seqs, tokens, 128] of the
 * same dtype.  With fp16 input the two run as one kernel whose wavefronts are given equal
 * shares of the combined work, so launch and pipeline-fill time is paid once. */
int tq_store_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs,
                int64_t tokens, int in_dtype, void *packed_k, void *packed_v, void *stream);

/* Prefill of a growing cache: tq_store_kv of the `tokens` tokens of every sequence into buffers laid out
 * for `capacity` tokens per sequence (tq_packed_bytes(bits, n_seqs, capacity), the layout tq_append_kv and
 * tq_decode_attention use), written from position 0.  Sequence i's first ceil(tokens/128) blocks hold the
 * same bytes that tq_store_kv writes for it (positions past `tokens` in the last of them hold the code of
 * a zero vector, as after tq_append_kv); the other blocks are not touched.  Same kernels and speed as
 * tq_store_kv for fp16 input; where that call falls back to the butterfly kernels this one runs
 * tq_append_kv from position 0.  No counterpart in the reference, whose cache (kv_cache.py:41-66) is
 * rebuilt from whole tensors. */
int tq_store_kv_cache(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs,
                      int64_t tokens, int64_t capacity, int in_dtype, void *packed_k, void *packed_v, void *stream);


/* Streaming append: n_new tokens per sequence at token positions pos .. pos+n_new-1 of a
 * packed buffer laid out for `capacity` tokens per sequence (tq_packed_bytes(bits, n_seqs,
 * capacity)); x is [n_seqs, n_new, 128].  The per-token compress step that kv_cache.py:65-66
 * names ("compress_token") and PLAN.md:119-122 plans; the reference does not implement it.
 * Same arithmetic as tq_store on fp32/fp64 input.  In the touched 128-token blocks the tokens
 * before pos are kept and the tokens from pos+n_new to the end of the last touched block get the
 * code of 0.0 and norm 0 (what tq_store writes past the end of a sequence), so an append below
 * the tokens already written truncates.  After appends covering tokens 0 .. T-1 in any chunking
 * the touched blocks equal tq_store's of the first T tokens.  Appends to one buffer must be
 * ordered (same stream). */
int tq_append(const tq_handle *h, const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity,
              int in_dtype, int kind, void *packed, void *stream);

/* tq_append of the K and the V tokens of one decode step (same n_seqs, pos, n_new, capacity, dtype) in one
 * launch: what a serving loop runs between two attention steps.  Same results as two tq_append calls. */
int tq_append_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t pos,
                 int64_t n_new, int64_t capacity, int in_dtype, void *packed_k, void *packed_v, void *stream);

/* tq_append_kv with the position read from device memory when the launch runs (*pos_dev, an int64): a decode
 * step captured once (HIP graph) can be replayed while the cache grows; the caller advances the counter
 * between replays (any kernel on the same stream).  A position that is negative or does not leave room for
 * n_new tokens writes nothing to the cache; when overrun_dev is not NULL (a 4-byte aligned uint32 in device
 * memory that the caller zeroes once) such a launch ORs TQ_OVERRUN_NEGATIVE or TQ_OVERRUN_NO_ROOM into it, and the
 * word keeps the bits until the caller clears it: a serving loop reads it once after its graph replays instead
 * of trusting TQ_OK, which only says that the launch was issued.  Together with tq_attn_params.tokens_dev.  No
 * counterpart in the reference; for the callers that replay captured launches. */
#define TQ_OVERRUN_NEGATIVE 1u /* *pos_dev < 0                      */
#define TQ_OVERRUN_NO_ROOM 2u  /* *pos_dev + n_new > capacity       */
int tq_append_kv_at(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs,
                    const int64_t *pos_dev, int64_t n_new, int64_t capacity, int in_dtype, void *packed_k,
                    void *packed_v, uint32_t *overrun_dev, void *stream);
/* The same for one tensor (tq_append) and for q8_0-style buffers (tq_q8_0_append). */
int tq_append_at(const tq_handle *h, const void *x, int64_t n_seqs, const int64_t *pos_dev, int64_t n_new,
                 int64_t capacity, int in_dtype, int kind, void *packed, uint32_t *overrun_dev, void *stream);
int tq_q8_0_append_at(const void *x, int64_t n_seqs, const int64_t *pos_dev, int64_t n_new, int64_t capacity,
                      int in_dtype, int kind, void *packed, uint32_t *overrun_dev, void *stream);


/* Temporal decay: re-quantise a packed buffer to a narrower width without going back to the
 * original vectors (`requantize_3to2`, benchmarks/temporal_decay_prototype.py:93-125): per row
 * decode with the stored norm, renormalise, nearest centroid of `dst`'s codebook (a value equal
 * to a midpoint takes the higher index, as np.digitize does there), corrected fp16 norm for the
 * new codes.  src holds tq_packed_bytes(src bits, ..) bytes, dst tq_packed_bytes(dst bits, ..);
 * width pairs 3->2, 4->3, 4->2; both handles must describe the same rotation. */
int tq_requantize(const tq_handle *src_h, const tq_handle *dst_h, const void *packed_src, int64_t n_seqs,
                  int64_t tokens, int kind, void *packed_dst, void *stream);

/* Interchange with the llama.cpp fork's per-128 block layout, one block per vector in token
 * order: norm fp16 | qs[32] | signs[16] (turbo3, 50 B: idx = low2 | hi1 << 2, low2 =
 * (qs[j/4] >> ((j%4)*2)) & 3, hi1 = (signs[j/8] >> (j%8)) & 1; docs/papers/block-size-experiment.md:33-39,
 * docs/papers/turbo4-resurrection.md:130-134), norm fp16 | rnorm fp16 | qs[64] nibbles (turbo4, 68 B = 4.25 bits
 * per value: docs/papers/turbo4-resurrection.md:169,208, README.md:43; rnorm is the residual-norm slot that
 * the fork's struct keeps from its 3-bit + QJL days, docs/turbo4-investigation.md:42-49: exported as 0, ignored
 * on import; that it sits right after norm is this library's reading of the documents, which print the size and
 * the nibble formula but not the field order), norm | qs[32] (turbo2, 34 B).  The norm is the corrected group
 * norm in both formats, so codes and norms move unchanged; blocks is [n_seqs, tokens, tq_fork_block_bytes(bits)]
 * bytes, 2-byte aligned (4-byte aligned for turbo4, whose rows move as 4-byte words; TQ_ERR_ALIGN otherwise).  Import fills the rows
 * past `tokens` of the last block like tq_store does.  The layout is known from the fork's
 * documents only (the reference tree holds no code for it). */
int64_t tq_fork_block_bytes(int32_t bits);
int tq_export_fork_blocks(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind,
                          void *blocks, void *stream);
int tq_import_fork_blocks(const tq_handle *h, const void *blocks, int64_t n_seqs, int64_t tokens, int kind,
                          void *packed, void *stream);

/* The same interchange for caches written by the fork's earlier builds, whose 2- and 3-bit storage blocks hold
 * block_values = 32 values (QK_TURBO3 = QK_TURBO2 = 32; 64 was measured too), docs/papers/block-size-experiment.md:27-39,270:
 * a vector is 128 / block_values blocks of norm fp16 | qs | signs over its own values, one after the other, the
 * extraction formulas above applied inside a block - 14 B (3.5 bits per value) and 26 B (3.25) per 3-bit block,
 * 10 B and 18 B per 2-bit block.  Rotation and norm correction work on the 128-value group whatever the block
 * size, so every block of a vector carries the same norm: export writes it into each, import reads the first.
 * tq_fork_row_bytes: bytes of one vector, (128 / block_values) * (2 + block_values * bits / 8); -1 for a pair the fork
 * does not have (4-bit rows exist with 128 values per block only).  block_values = 128 is the layout of the entry
 * points above.  blocks is [n_seqs, tokens, tq_fork_row_bytes(bits, block_values)] bytes, 2-byte aligned. */
int64_t tq_fork_row_bytes(int32_t bits, int32_t block_values);
int tq_export_fork_blocks_sized(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind,
                                int32_t block_values, void *blocks, void *stream);
int tq_import_fork_blocks_sized(const tq_handle *h, const void *blocks, int64_t n_seqs, int64_t tokens, int kind,
                                int32_t block_values, void *packed, void *stream);

/* Inverse of tq_store (KVCacheCompressor.decompress, kv_cache.py:143-165, MSE-only
 * format): out [n_seqs, tokens, 128] in the rotated domain (norm * centroid) or the
 * original domain (transpose rotation applied). */
int tq_load(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, void *out,
            int out_dtype, int domain, void *stream);

/* K and V of one layer back to fp16 in the original domain, the two tensors that
 * KVCacheCompressor.decompress (kv_cache.py:143-165) returns together.  Same results as
 * tq_load(hk, packed_k, .., TQ_KIND_K, out_k, TQ_F16, TQ_DOMAIN_ORIGINAL, ..) followed by
 * tq_load(hv, packed_v, .., TQ_KIND_V, out_v, ..); out_k and out_v are [n_seqs, tokens, 128]
 * fp16.  The two run as one kernel whose workgroups are divided between the tensors, so launch
 * and pipeline-fill time is paid once. */
int tq_load_kv(const tq_handle *hk, const tq_handle *hv, const void *packed_k, const void *packed_v,
               int64_t n_seqs, int64_t tokens, void *out_k, void *out_v, void *stream);

/* Codebook indices [n_seqs, tokens, 128] uint8 and stored norms [n_seqs, tokens]
 * float32 of a packed buffer (test and interop aid; no reference counterpart). */
int tq_unpack_codes(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind,
                    uint8_t *idx, float *norms, void *stream);

/* tq_store (kind K) plus the QJL sketch of the residual against the stored
 * reconstruction: TurboQuant.quantize (turboquant.py:79-100) in device format.
 * sign_bits [n,16] uint8: bit j%8 of byte j/8 is set when (S r)_j >= 0 (zero maps
 * to +1 as in qjl.py:89-90); rnorms [n] fp16 = ||residual||.  The handle needs a
 * projection.  n = n_seqs*tokens rows; sign_bits / rnorms are in token order.
 * Codes, norms and the residual are computed in float64; a sign bit is the sign of
 * the float64 projection (taken from an fp16 matrix-core pass where that pass's error
 * bound settles it, recomputed in float64 where it does not).
 * The k argument of TQ_KFMT_Q8_0 attention is a tq_q8_0_store buffer. */
int tq_store_qjl(const tq_handle *h, const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed,
                 uint8_t *sign_bits, void *rnorms_f16, void *stream);

/* q8_0-style K rows (textbook ggml block_q8_0 arithmetic: per 32 values
 * scale = max|x|/127 as fp16, q = roundf(x/scale); the reference tree has no
 * code for it).  x [n_seqs, tokens, 128] -> 128-token blocks of
 * [8 chunks][128 rows][16 B] int8 followed by [128][4] fp16 scales
 * (136 bytes per token); tq_q8_0_bytes gives the buffer size.  x and packed must be
 * 16-byte aligned (also for tq_q8_0_store_v). */
int64_t tq_q8_0_bytes(int64_t n_seqs, int64_t tokens);
int tq_q8_0_store(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, void *stream);
/* q [n_seqs, tokens, 128] int8 and scales [n_seqs, tokens, 4] fp32 of such a buffer. */
int tq_q8_0_unpack(const void *packed, int64_t n_seqs, int64_t tokens, int8_t *q, float *scales, void *stream);
/* The same arithmetic for V rows (the boundary layers of the fork's Boundary V policy keep V as q8_0,
 * docs/papers/layer-aware-v-compression.md:83-87; no reference code): blocks of the same size, values
 * dim-major inside 64-token tiles as the decode kernel reads V (row 64*tile + dim % 64 of a block holds
 * dims dim and dim + 64 of the tile's 64 tokens), then [2 tiles][4][64 tokens] fp16 scales.  Positions
 * past `tokens` in the last block hold zeros.  tq_q8_0_unpack_v gives q and scales in token order as
 * tq_q8_0_unpack does. */
int tq_q8_0_store_v(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, void *stream);
int tq_q8_0_unpack_v(const void *packed, int64_t n_seqs, int64_t tokens, int8_t *q, float *scales, void *stream);
/* tq_append for q8_0-style buffers of either kind (laid out for `capacity` tokens per sequence,
 * tq_q8_0_bytes(n_seqs, capacity)): same positions, truncation and ordering rules; after appends
 * covering tokens 0 .. T-1 the touched blocks equal tq_q8_0_store's / tq_q8_0_store_v's of the
 * first T tokens.  The buffer must start out zeroed: blocks that no append has touched are read by
 * the attention kernel's last tile and must hold finite scales. */
int tq_q8_0_append(const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype, int kind,
                   void *packed, void *stream);

/* ---- attention over packed KV ------------------------------------------------ */

typedef struct tq_attn_params {
    int32_t batch, n_q_heads, n_kv_heads;  /* GQA group = n_q_heads / n_kv_heads; the kernels take */
                                           /* four heads of a group per pass over K/V, eight when  */
                                           /* the group has more than four                          */
    int64_t tokens;                        /* context length per sequence                    */
    int64_t capacity;                      /* tokens per sequence the K/V buffers are laid   */
                                           /* out for (tq_append caches); 0 = tokens         */
    int32_t n_splits;                      /* context splits per (batch, kv head), >= 1; a   */
                                           /* multiple of 16 lets 16 splits share a workgroup */
    int32_t k_format;                      /* TQ_KFMT_TURBO | TQ_KFMT_Q8_0                   */
    int32_t v_format;                      /* the same for V: TQ_KFMT_TURBO (0) | TQ_KFMT_Q8_0 */
    float scale;                           /* logit scale, e.g. 1/sqrt(128)                  */
    float sparse_v_tau;                    /* 0 = dense; skip V rows with weight < tau       */
    const int64_t *tokens_dev;             /* NULL, or device memory the step's context      */
                                           /* length is read from when the launch runs       */
                                           /* (clamped to 0 .. tokens; `tokens` then is the  */
                                           /* maximum, sizes the workspace and is the stride */
                                           /* of the bias rows): one captured launch replays */
                                           /* at a growing length.  skip_count must be NULL. */
    int32_t bias_entries;                  /* sparse additive logit bias: entries per query   */
                                           /* head, 0 = none (a bias that is zero but for a   */
                                           /* few positions costs its list, not a dense row   */
                                           /* per head); added to the dense bias if both come */
    const int32_t *bias_pos;               /* [batch, n_q_heads, bias_entries] positions in   */
                                           /* device memory, ascending within a head and each */
                                           /* position at most once; a list shorter than      */
                                           /* bias_entries is filled up with positions >=     */
                                           /* tokens (INT32_MAX)                              */
    const float *bias_val;                 /* [batch, n_q_heads, bias_entries] values, fp32,  */
                                           /* natural-log units like the dense bias           */
    int32_t head_dim;                      /* 0 or 128: heads of 128 dims.  256: a head's     */
                                           /* vector is two 128-value groups, each rotated,   */
                                           /* quantised and normed by itself (the fork's      */
                                           /* 128-value blocks, docs/getting-started.md:68):  */
                                           /* K and V caches are those of 128-dim heads with  */
                                           /* 2 * tokens rows, row 2 * token + half, written  */
                                           /* by tq_store(_kv) / tq_append(_kv) from the      */
                                           /* [tokens, 256] tensor taken as [2 * tokens, 128];*/
                                           /* q and out are [batch, n_q_heads, 256].  K and V */
                                           /* turbo of one width or of 4|2, 3|2, 4|3 bits, or */
                                           /* q8_0-style rows on either side (written the     */
                                           /* same way by tq_q8_0_store / tq_q8_0_store_v);   */
                                           /* Sparse V tests tiles of 32 tokens; bias rows    */
                                           /* and lists count tokens                          */
} tq_attn_params;

/* Bytes of workspace tq_decode_attention needs: one partial (2 KB; 4 KB when a KV head serves more than four
 * query heads) per workgroup, plus flags and Sparse-V slots; it does not depend on bias_entries / bias_pos /
 * bias_val, which may change from call to call (a call with a bias list may run smaller workgroups: the size covers
 * either).  The workspace may hold anything on entry; calls that share one workspace must not overlap in time.
 * n_splits: any count >= 1; workgroups take the largest power of two up to 16 that divides it (8 for q8_0-style V
 * rows, for 256-dim heads and for more than four query heads per KV head - there 12 when 12 divides it and K and V
 * are turbo rows, which is the best shape for large steps: 256 workgroups of twelve). */
int64_t tq_attn_workspace_bytes(const tq_attn_params *p);

/* softmax(scale * q k^T) v over packed K/V (tests/test_kv_cache.py:73-89,128-131
 * evaluated on stored codes; no reference kernel exists).
 *   q      [batch, n_q_heads, 128] q_dtype, in the ORIGINAL domain; the kernel
 *          rotates it with the K handle's rotation (or leaves it for q8_0 K);
 *   k/v    packed buffers of [batch*n_kv_heads] sequences: tq_store (kind K / V) buffers for
 *          TQ_KFMT_TURBO, tq_q8_0_store / tq_q8_0_store_v buffers for TQ_KFMT_Q8_0 (then the
 *          handle of that side may be NULL; a q8_0 V is not rotated); k_aux is unused;
 *   bias   optional additive logit bias [batch, n_q_heads, tokens] fp32 or NULL;
 *   out    [batch, n_q_heads, 128] fp32, original domain;
 *   skip_count optional uint64[2]: {skipped (query, position) pairs, total pairs}. */
int tq_decode_attention(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q,
                        int q_dtype, const void *k, const void *k_aux, const void *v, const float *bias,
                        float *out, unsigned long long *skip_count, void *workspace, int64_t workspace_bytes,
                        void *stream);

/* tq_decode_attention for callers that cannot allocate device memory or pass a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, kernels and results as tq_decode_attention; the split partials go to a workspace of
 * TQ_STATIC_WORKSPACE_BYTES that is built into the library's device code (every GPU the library runs on
 * holds one copy until the process ends), so the call allocates nothing.  Parameter sets whose
 * tq_attn_workspace_bytes() exceeds that size (about 8000 workgroups: batch * n_kv_heads * n_splits / 16 of them
 * when n_splits is a multiple of 16) are rejected with TQ_ERR_UNSUPPORTED.  All calls on one GPU share the one workspace: calls that overlap in time on the same
 * GPU (different streams or threads) race; order them.  The workspace's address is looked up once per
 * device, in tq_create or in the first call on that device. */
#define TQ_STATIC_WORKSPACE_BYTES (16 * 1024 * 1024)
int tq_decode_attention_static(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q,
                               int q_dtype, const void *k, const void *v, const float *bias, float *out,
                               unsigned long long *skip_count, void *stream);

/* TurboQuant inner-product estimate for nq queries x nk keys (turboquant.py:102-124
 * moved to the rotated/projected domain): logits[i,j] = <R q_i, g_j c[idx_j]> +
 * projection_scale * rnorm_j * <S q_i, z_j>.  q [nq,128] q_dtype, packed/sign_bits/
 * rnorms from tq_store_qjl with n_seqs = 1, logits [nq, nk] fp32 (or fp16 when
 * out_dtype == TQ_F16).  workspace: 512 bytes per query, query count rounded up to a
 * multiple of 32.  logits == NULL runs the whole computation and stores nothing (for
 * measuring the contraction without the logit stores).  Limit: nq < 2^24 (TQ_ERR_UNSUPPORTED
 * beyond: score the queries in slices); any nk.  logits needs only the alignment of its
 * element type. */
int tq_score_tile(const tq_handle *h, const void *q, int q_dtype, int64_t nq, const void *packed,
                  const uint8_t *sign_bits, const void *rnorms_f16, int64_t nk, void *logits, int out_dtype,
                  void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TQ_H */
