// float64 block helpers shared by the reference-API kernels and the QJL store
// kernel: VB vectors staged in LDS, rotated by a dense matrix read from L2 or
// by the sign-diagonal Walsh-Hadamard butterfly in the reference's stage order.
#pragma once
#include "tq_internal.h"

namespace tq64 {

constexpr int NT = 128;  // threads per workgroup
// vectors per workgroup (template parameter VB): two staging arrays of VB * pd doubles must fit in LDS,
// so wide vectors get fewer per workgroup
constexpr int vectors_per_workgroup(int pd) { return pd <= 1024 ? 8 : pd <= 2048 ? 4 : 2; }

template <typename T> __device__ inline double ldd(const T *p, int64_t i) { return (double)p[i]; }
template <> __device__ inline double ldd<__half>(const __half *p, int64_t i) { return (double)__half2float(p[i]); }
template <typename T> __device__ inline void std_(T *p, int64_t i, double v) { p[i] = (T)v; }
template <> __device__ inline void std_<__half>(__half *p, int64_t i, double v) { p[i] = __float2half_rn((float)v); }

struct RotArgs {
    int d, pd, mode;        // mode: TQ_ROT_DENSE / TQ_ROT_WHT
    const double *mat;      // dense: matrix M with out[j] = sum_k M[k*d+j] * in[k]
    const double *sa, *sb;  // wht: signs applied before / after the butterfly (NULL = ones)
};

// in: xs[VB][pd] (entries >= d zero in WHT mode); out: ys[VB][pd].  All threads call.
template <int VB>
__device__ void rotate_block(const RotArgs &r, double *xs, double *ys) {
    const int tid = threadIdx.x;
    const int d = r.d, pd = r.pd;
    if (r.mode == TQ_ROT_DENSE) {
        for (int j = tid; j < d; j += NT) {
            double acc[VB];
#pragma unroll
            for (int v = 0; v < VB; ++v) acc[v] = 0.0;
            for (int k = 0; k < d; ++k) {
                const double m = r.mat[(int64_t)k * d + j];
#pragma unroll
                for (int v = 0; v < VB; ++v) acc[v] = fma(m, xs[v * pd + k], acc[v]);
            }
#pragma unroll
            for (int v = 0; v < VB; ++v) ys[v * pd + j] = acc[v];
        }
        __syncthreads();
        return;
    }
    if (r.sa) {
        for (int i = tid; i < VB * pd; i += NT) xs[i] *= r.sa[i % pd];
        __syncthreads();
    }
    const int half = pd >> 1;
    for (int h = 1; h < pd; h <<= 1) {
        for (int p = tid; p < VB * half; p += NT) {
            const int v = p / half, q = p % half;
            const int i = v * pd + (q / h) * 2 * h + (q % h);
            const double a = xs[i], b = xs[i + h];
            xs[i] = a + b;
            xs[i + h] = a - b;
        }
        __syncthreads();
    }
    const double rn = sqrt((double)pd);
    for (int i = tid; i < VB * pd; i += NT) {
        double v = xs[i] / rn;
        if (r.sb) v *= r.sb[i % pd];
        ys[i] = v;
    }
    __syncthreads();
}

template <int VB, typename T>
__device__ void load_block(const T *x, int64_t n, int64_t v0, int d, int pd, double *xs) {
    for (int i = threadIdx.x; i < VB * pd; i += NT) {
        const int v = i / pd, j = i % pd;
        xs[i] = (v0 + v < n && j < d) ? ldd(x, (v0 + v) * d + j) : 0.0;
    }
    __syncthreads();
}

// L2 norms of the VB staged vectors -> nrm[VB] (shared).
template <int VB>
__device__ void norms_block(const double *xs, int d, int pd, double *nrm) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int v = wave; v < VB; v += NT / 64) {
        double s = 0.0;
        for (int j = lane; j < d; j += 64) s = fma(xs[v * pd + j], xs[v * pd + j], s);
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
        if (lane == 0) nrm[v] = sqrt(s);
    }
    __syncthreads();
}


// float64 -> fp16 with a single round-to-nearest-even (no double rounding
// through float): choose among the float-rounded candidate and its neighbours.
__device__ inline __half double_to_half_rn(double v) {
    const __half h0 = __float2half_rn((float)v);
    unsigned short b0 = __half_as_ushort(h0);
    if ((b0 & 0x7C00u) == 0x7C00u) return h0;  // inf / nan
    __half best = h0;
    double berr = fabs((double)__half2float(h0) - v);
    const unsigned short cand[2] = {(unsigned short)(b0 + 1), (unsigned short)(b0 - 1)};
    for (int i = 0; i < 2; ++i) {
        if ((b0 & 0x7FFFu) == 0 && i == 1) continue;  // do not step below +-0
        const __half h = __ushort_as_half(cand[i]);
        if ((cand[i] & 0x7C00u) == 0x7C00u) continue;
        const double err = fabs((double)__half2float(h) - v);
        if (err < berr || (err == berr && (cand[i] & 1u) == 0 && (__half_as_ushort(best) & 1u) != 0)) {
            best = h;
            berr = err;
        }
    }
    return best;
}

}  // namespace tq64
