// Reference-API kernels: float64 arithmetic, any dimension up to 4096.
//
// These back the Python classes that keep the reference's signatures
// (PolarQuant, QJL, the rotation and codebook free functions, pack helpers).
// One workgroup of 128 threads handles VB = 8 vectors (4 or 2 for dimensions above 1024 / 2048) staged in LDS; the
// rotation is either a dense d x d product read from L2 (matrix stored so
// that consecutive threads read consecutive addresses) or the sign-diagonal
// Walsh-Hadamard butterfly done in LDS with the reference's stage order, which
// makes the float64 WHT results bit-identical to NumPy's.
#include "tq_internal.h"
#include "tq_device64.h"

namespace {

using namespace tq64;

template <int VB, typename TI, typename TO>
__global__ __launch_bounds__(NT) void k_rotate64(const TI *x, TO *y, int64_t n, RotArgs r) {
    extern __shared__ double sm[];
    double *xs = sm, *ys = sm + VB * r.pd;
    const int64_t v0 = (int64_t)blockIdx.x * VB;
    load_block<VB>(x, n, v0, r.d, r.pd, xs);
    rotate_block<VB>(r, xs, ys);
    for (int i = threadIdx.x; i < VB * r.d; i += NT) {
        const int v = i / r.d, j = i % r.d;
        if (v0 + v < n) std_(y, (v0 + v) * r.d + j, ys[v * r.pd + j]);
    }
}

template <int VB, typename T>
__global__ __launch_bounds__(NT) void k_quantize64(const T *x, int64_t n, RotArgs r, const double *bounds, int nb,
                                                  uint8_t *idx, double *norms, double *rotated) {
    extern __shared__ double sm[];
    __shared__ double nrm[VB];
    double *xs = sm, *ys = sm + VB * r.pd;
    const int64_t v0 = (int64_t)blockIdx.x * VB;
    load_block<VB>(x, n, v0, r.d, r.pd, xs);
    norms_block<VB>(xs, r.d, r.pd, nrm);
    for (int i = threadIdx.x; i < VB * r.pd; i += NT) {
        const double nv = nrm[i / r.pd];
        xs[i] = xs[i] / (nv > 0.0 ? nv : 1.0);
    }
    __syncthreads();
    rotate_block<VB>(r, xs, ys);
    for (int i = threadIdx.x; i < VB * r.d; i += NT) {
        const int v = i / r.d, j = i % r.d;
        if (v0 + v >= n) continue;
        const double yv = ys[v * r.pd + j];
        int c = 0;
        for (int k = 0; k < nb; ++k) c += (bounds[k] < yv) ? 1 : 0;
        idx[(v0 + v) * r.d + j] = (uint8_t)c;
        if (rotated) rotated[(v0 + v) * r.d + j] = yv;
    }
    if (threadIdx.x < VB && v0 + threadIdx.x < n) norms[v0 + threadIdx.x] = nrm[threadIdx.x];
}

template <int VB, typename T>
__global__ __launch_bounds__(NT) void k_dequantize64(const uint8_t *idx, const double *norms, int64_t n, RotArgs r,
                                                    const double *centroids, int norm_correction, double *out,
                                                    const T *x, double *residual) {
    extern __shared__ double sm[];
    __shared__ double nrm[VB];
    double *xs = sm, *ys = sm + VB * r.pd;
    const int64_t v0 = (int64_t)blockIdx.x * VB;
    for (int i = threadIdx.x; i < VB * r.pd; i += NT) {
        const int v = i / r.pd, j = i % r.pd;
        xs[i] = (v0 + v < n && j < r.d) ? centroids[idx[(v0 + v) * r.d + j]] : 0.0;
    }
    __syncthreads();
    if (norm_correction) {
        norms_block<VB>(xs, r.d, r.pd, nrm);
        for (int i = threadIdx.x; i < VB * r.pd; i += NT) {
            const double nv = nrm[i / r.pd];
            xs[i] = xs[i] / (nv > 1e-10 ? nv : 1.0);
        }
        __syncthreads();
    }
    rotate_block<VB>(r, xs, ys);
    for (int i = threadIdx.x; i < VB * r.d; i += NT) {
        const int v = i / r.d, j = i % r.d;
        if (v0 + v >= n) continue;
        const double o = ys[v * r.pd + j] * norms[v0 + v];
        out[(v0 + v) * r.d + j] = o;
        if (residual) residual[(v0 + v) * r.d + j] = ldd(x, (v0 + v) * r.d + j) - o;
    }
}

template <int VB, typename T>
__global__ __launch_bounds__(NT) void k_qjl_quantize64(const T *x, int64_t n, RotArgs r, int8_t *signs, double *norms) {
    extern __shared__ double sm[];
    __shared__ double nrm[VB];
    double *xs = sm, *ys = sm + VB * r.pd;
    const int64_t v0 = (int64_t)blockIdx.x * VB;
    load_block<VB>(x, n, v0, r.d, r.pd, xs);
    norms_block<VB>(xs, r.d, r.pd, nrm);
    rotate_block<VB>(r, xs, ys);
    for (int i = threadIdx.x; i < VB * r.d; i += NT) {
        const int v = i / r.d, j = i % r.d;
        if (v0 + v < n) signs[(v0 + v) * r.d + j] = ys[v * r.pd + j] < 0.0 ? (int8_t)-1 : (int8_t)1;
    }
    if (threadIdx.x < VB && v0 + threadIdx.x < n) norms[v0 + threadIdx.x] = nrm[threadIdx.x];
}

template <int VB>
__global__ __launch_bounds__(NT) void k_qjl_dequantize64(const int8_t *signs, const double *norms, int64_t n, RotArgs r,
                                                        double proj_scale, double shrinkage, double *out) {
    extern __shared__ double sm[];
    double *xs = sm, *ys = sm + VB * r.pd;
    const int64_t v0 = (int64_t)blockIdx.x * VB;
    load_block<VB>(signs, n, v0, r.d, r.pd, xs);
    rotate_block<VB>(r, xs, ys);
    for (int i = threadIdx.x; i < VB * r.d; i += NT) {
        const int v = i / r.d, j = i % r.d;
        if (v0 + v >= n) continue;
        const double sc = (proj_scale * norms[v0 + v]) * shrinkage;
        out[(v0 + v) * r.d + j] = ys[v * r.pd + j] * sc;
    }
}

struct Bounds {
    double b[255];
};

__global__ void k_nearest(const double *values, int64_t n, Bounds bd, int nb, int32_t *idx) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const double v = values[i];
    int c = 0;
    for (int k = 0; k < nb; ++k) c += (bd.b[k] < v) ? 1 : 0;
    idx[i] = c;
}

// signs [n,d] int8 -> packed [n, ceil(d/8)], first element in the MSB.
__global__ void k_pack_bits(const int8_t *signs, int64_t n, int d, uint8_t *packed) {
    const int nbytes = (d + 7) / 8;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n * nbytes) return;
    const int64_t row = i / nbytes;
    const int byte = (int)(i % nbytes);
    unsigned v = 0;
    for (int b = 0; b < 8; ++b) {
        const int j = byte * 8 + b;
        if (j < d && signs[row * d + j] > 0) v |= 0x80u >> b;
    }
    packed[i] = (uint8_t)v;
}

__global__ void k_unpack_bits(const uint8_t *packed, int64_t n, int d, int8_t *signs) {
    const int nbytes = (d + 7) / 8;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n * d) return;
    const int64_t row = i / d;
    const int j = (int)(i % d);
    const unsigned bit = (packed[row * nbytes + j / 8] >> (7 - (j % 8))) & 1u;
    signs[i] = bit ? (int8_t)1 : (int8_t)-1;
}

// One MSB-first bit stream: bit t of the stream is bit (bits-1 - t%bits) of idx[t/bits].
__global__ void k_pack_indices(const uint8_t *idx, int64_t count, int bits, uint8_t *packed) {
    const int64_t nbytes = (count * bits + 7) / 8;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nbytes) return;
    unsigned v = 0;
    for (int b = 0; b < 8; ++b) {
        const int64_t t = i * 8 + b;
        const int64_t e = t / bits;
        if (e < count && ((idx[e] >> (bits - 1 - (int)(t % bits))) & 1u)) v |= 0x80u >> b;
    }
    packed[i] = (uint8_t)v;
}

inline size_t lds_bytes(int pd) { return (size_t)2 * vectors_per_workgroup(pd) * pd * sizeof(double); }

// Workgroups that stage more than 48 KB need the limit raised per kernel.
template <typename K> inline void allow_lds(K kernel, size_t bytes) {
    if (bytes > 48 * 1024)
        (void)hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}
inline unsigned nblocks(int64_t n, int pd) {
    const int vb = vectors_per_workgroup(pd);
    return (unsigned)((n + vb - 1) / vb);
}
// F uses VB as a compile-time constant
#define DISPATCH_VB(pd, F)                                         \
    switch (vectors_per_workgroup(pd)) {                           \
    case 8: { constexpr int VB = 8; F; } break;                    \
    case 4: { constexpr int VB = 4; F; } break;                    \
    default: { constexpr int VB = 2; F; } break; }

RotArgs rot_args(const tq_handle *h, int transpose) {
    RotArgs r;
    r.d = h->d;
    r.pd = h->rotation == TQ_ROT_WHT ? h->pd : h->d;
    r.mode = h->rotation;
    // forward dense: out[j] = sum_k Pi[j][k] in[k]  -> M[k*d+j] = Pi^T row-major
    r.mat = transpose ? h->rot64 : h->rot64_t;
    r.sa = transpose ? h->s2_64 : h->s1_64;
    r.sb = transpose ? h->s1_64 : h->s2_64;
    return r;
}

#define DISPATCH_IN(dt, F)          \
    switch (dt) {                   \
    case TQ_F16: { using TI = __half; F; } break; \
    case TQ_F32: { using TI = float; F; } break;  \
    case TQ_F64: { using TI = double; F; } break; \
    default: tq_set_error("bad dtype %d", dt); return TQ_ERR_ARG; }

template <typename TI, typename TO>
int launch_rotate_to(const void *x, void *y, int64_t n, const RotArgs &r, hipStream_t s) {
    const size_t lds = lds_bytes(r.pd);
    DISPATCH_VB(r.pd, (allow_lds(k_rotate64<VB, TI, TO>, lds),
                       k_rotate64<VB, TI, TO><<<nblocks(n, r.pd), NT, lds, s>>>((const TI *)x, (TO *)y, n, r)));
    return tq_check_launch("rotate64");
}

template <typename TI>
int launch_rotate(const void *x, void *y, int64_t n, int out_dtype, const RotArgs &r, hipStream_t s) {
    switch (out_dtype) {
    case TQ_F16: return launch_rotate_to<TI, __half>(x, y, n, r, s);
    case TQ_F32: return launch_rotate_to<TI, float>(x, y, n, r, s);
    case TQ_F64: return launch_rotate_to<TI, double>(x, y, n, r, s);
    default: tq_set_error("bad dtype %d", out_dtype); return TQ_ERR_ARG;
    }
}

}  // namespace

int tqk_fwht(const void *x, void *y, int64_t n, int len, int in_dtype, int out_dtype, hipStream_t s) {
    RotArgs r;
    r.d = r.pd = len;
    r.mode = TQ_ROT_WHT;
    r.mat = nullptr;
    r.sa = r.sb = nullptr;
    DISPATCH_IN(in_dtype, return launch_rotate<TI>(x, y, n, out_dtype, r, s));
}

int tqk_rotate64(const tq_handle *h, const void *x, void *y, int64_t n, int in_dtype, int out_dtype, int transpose,
                 hipStream_t s) {
    const RotArgs r = rot_args(h, transpose);
    DISPATCH_IN(in_dtype, return launch_rotate<TI>(x, y, n, out_dtype, r, s));
}

int tqk_nearest(const double *values, int64_t n, const double *bounds_host, int nb, int32_t *idx, hipStream_t s) {
    Bounds bd;
    for (int k = 0; k < nb; ++k) bd.b[k] = bounds_host[k];
    k_nearest<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(values, n, bd, nb, idx);
    return tq_check_launch("nearest");
}

int tqk_quantize_indices(const tq_handle *h, const void *x, int64_t n, int in_dtype, uint8_t *idx, double *norms,
                         double *rotated, hipStream_t s) {
    const RotArgs r = rot_args(h, 0);
    DISPATCH_IN(in_dtype, DISPATCH_VB(r.pd, (allow_lds(k_quantize64<VB, TI>, lds_bytes(r.pd)),
                                             k_quantize64<VB, TI><<<nblocks(n, r.pd), NT, lds_bytes(r.pd), s>>>(
                                                 (const TI *)x, n, r, h->bounds64, h->n_centroids - 1, idx, norms, rotated))));
    return tq_check_launch("quantize64");
}

int tqk_dequantize_indices(const tq_handle *h, const uint8_t *idx, const double *norms, int64_t n, double *out,
                           const void *x, int x_dtype, double *residual, hipStream_t s) {
    const RotArgs r = rot_args(h, 1);
    if (!residual) x_dtype = TQ_F64;
    DISPATCH_IN(x_dtype, DISPATCH_VB(r.pd, (allow_lds(k_dequantize64<VB, TI>, lds_bytes(r.pd)),
                                            k_dequantize64<VB, TI><<<nblocks(n, r.pd), NT, lds_bytes(r.pd), s>>>(
                                                idx, norms, n, r, h->centroids64, h->norm_correction, out, (const TI *)x, residual))));
    return tq_check_launch("dequantize64");
}

int tqk_qjl_quantize(const tq_handle *h, const void *rr, int64_t n, int in_dtype, int8_t *signs, double *norms,
                     hipStream_t s) {
    RotArgs r;
    r.d = r.pd = h->d;
    r.mode = TQ_ROT_DENSE;
    r.mat = h->proj64_t;  // out[j] = sum_k S[j][k] in[k]
    r.sa = r.sb = nullptr;
    DISPATCH_IN(in_dtype, DISPATCH_VB(r.pd, (allow_lds(k_qjl_quantize64<VB, TI>, lds_bytes(r.pd)),
                                             k_qjl_quantize64<VB, TI><<<nblocks(n, r.pd), NT, lds_bytes(r.pd), s>>>(
                                                 (const TI *)rr, n, r, signs, norms))));
    return tq_check_launch("qjl_quantize64");
}

int tqk_qjl_dequantize(const tq_handle *h, const int8_t *signs, const double *norms, double shrinkage, int64_t n,
                       double *out, hipStream_t s) {
    RotArgs r;
    r.d = r.pd = h->d;
    r.mode = TQ_ROT_DENSE;
    r.mat = h->proj64;  // out[j] = sum_k S[k][j] z[k]
    r.sa = r.sb = nullptr;
    DISPATCH_VB(r.pd, (allow_lds(k_qjl_dequantize64<VB>, lds_bytes(r.pd)),
                       k_qjl_dequantize64<VB><<<nblocks(n, r.pd), NT, lds_bytes(r.pd), s>>>(signs, norms, n, r, h->proj_scale,
                                                                                          shrinkage, out)));
    return tq_check_launch("qjl_dequantize64");
}

int tqk_pack_bits(const int8_t *signs, int64_t n, int d, uint8_t *packed, hipStream_t s) {
    const int64_t total = n * ((d + 7) / 8);
    k_pack_bits<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(signs, n, d, packed);
    return tq_check_launch("pack_bits");
}

int tqk_unpack_bits(const uint8_t *packed, int64_t n, int d, int8_t *signs, hipStream_t s) {
    const int64_t total = n * d;
    k_unpack_bits<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(packed, n, d, signs);
    return tq_check_launch("unpack_bits");
}

int tqk_pack_indices(const uint8_t *idx, int64_t count, int bits, uint8_t *packed, hipStream_t s) {
    const int64_t nbytes = (count * bits + 7) / 8;
    k_pack_indices<<<(unsigned)((nbytes + 255) / 256), 256, 0, s>>>(idx, count, bits, packed);
    return tq_check_launch("pack_indices");
}
