// extern "C" surface of the library: argument checks, handle lifetime, dispatch.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "tq_internal.h"

namespace {

thread_local char g_err[512] = "";

// float64 -> fp16 bit pattern, one round-to-nearest-even
uint16_t f64_to_f16_bits(double v) {
    if (std::isnan(v)) return 0x7e00;
    const uint16_t sign = std::signbit(v) ? 0x8000 : 0;
    double a = std::fabs(v);
    if (a >= 65520.0) return sign | 0x7c00;
    if (a < 5.9604644775390625e-08 * 0.5) return sign;  // below half the smallest subnormal
    int e;
    double m = std::frexp(a, &e);  // a = m * 2^e, m in [0.5, 1)
    int exp = e - 1;               // a = (2m) * 2^exp, 2m in [1, 2)
    if (exp < -14) {               // subnormal: units of 2^-24
        const double q = a / 5.9604644775390625e-08;
        double r = std::nearbyint(q);
        return sign | (uint16_t)r;
    }
    const double frac = (2.0 * m - 1.0) * 1024.0;
    double r = std::nearbyint(frac);  // default rounding mode: nearest-even
    uint32_t bits = ((uint32_t)(exp + 15) << 10) + (uint32_t)r;  // mantissa overflow carries into the exponent
    return sign | (uint16_t)bits;
}

double f16_bits_to_f64(uint16_t b) {
    const double sign = (b & 0x8000) ? -1.0 : 1.0;
    const int e = (b >> 10) & 31, m = b & 1023;
    if (e == 0) return sign * std::ldexp((double)m, -24);
    if (e == 31) return m ? NAN : sign * INFINITY;
    return sign * std::ldexp(1.0 + m / 1024.0, e - 15);
}

template <typename T> int upload(T **dst, const std::vector<T> &src) {
    *dst = nullptr;
    if (src.empty()) return TQ_OK;
    hipError_t e = hipMalloc((void **)dst, src.size() * sizeof(T));
    if (e != hipSuccess) {
        tq_set_error("hipMalloc(%zu): %s", src.size() * sizeof(T), hipGetErrorString(e));
        return TQ_ERR_HIP;
    }
    e = hipMemcpy(*dst, src.data(), src.size() * sizeof(T), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        tq_set_error("hipMemcpy: %s", hipGetErrorString(e));
        return TQ_ERR_HIP;
    }
    return TQ_OK;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

bool fast_ok(const tq_handle *h) { return h->d == 128 && h->rotation == TQ_ROT_WHT && h->s1_32; }

}  // namespace

void tq_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int tq_check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        tq_set_error("%s: %s", what, hipGetErrorString(e));
        return TQ_ERR_HIP;
    }
    return TQ_OK;
}

extern "C" {

int tq_version(void) { return 101; }

const char *tq_last_error(void) { return g_err; }

int tq_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int tq_create(tq_handle **out, const tq_config *cfg) {
    if (!out || !cfg || !cfg->centroids) {
        tq_set_error("tq_create: null argument");
        return TQ_ERR_ARG;
    }
    *out = nullptr;
#ifdef TQ_MEASUREMENT_BUILD
    // a library with a measurement switch compiled in computes wrong results on purpose: it serves nobody who did not ask
    {
        const char *ok = std::getenv("TQ_ALLOW_MEASUREMENT_BUILD");
        if (!ok || std::strcmp(ok, "1") != 0) {
            tq_set_error("tq_create: this library is a measurement build (TQ_MEASUREMENT_BUILD); set TQ_ALLOW_MEASUREMENT_BUILD=1 to use it");
            return TQ_ERR_UNSUPPORTED;
        }
    }
#endif
    if (cfg->d < 1 || cfg->d > TQ_MAX_D) {
        tq_set_error("tq_create: d must be in 1..%d (got %d)", TQ_MAX_D, cfg->d);
        return TQ_ERR_UNSUPPORTED;
    }
    if (cfg->bits < 1 || cfg->bits > 8) {
        tq_set_error("tq_create: bits must be in 1..8 (got %d)", cfg->bits);
        return TQ_ERR_ARG;
    }
    if (cfg->rotation == TQ_ROT_DENSE ? !cfg->rotation_matrix : (cfg->rotation != TQ_ROT_WHT || !cfg->signs1 || !cfg->signs2)) {
        tq_set_error("tq_create: rotation tables missing for mode %d", cfg->rotation);
        return TQ_ERR_ARG;
    }
    if (tq_device_count() < 1) {
        tq_set_error("tq_create: no HIP device visible");
        return TQ_ERR_HIP;
    }
    tq_handle *h = new tq_handle();
    memset(h, 0, sizeof(*h));
    h->d = cfg->d;
    h->pd = tq_padded_dim(cfg->d);
    h->bits = cfg->bits;
    h->n_centroids = 1 << cfg->bits;
    h->rotation = cfg->rotation;
    h->norm_correction = cfg->norm_correction;
    h->proj_scale = cfg->projection_scale;
    h->has_proj = cfg->projection != nullptr;
    (void)hipGetDevice(&h->device);
    {   // look up this device's built-in attention workspace now, where set-up work is expected
        void *ws = nullptr;
        const int rcw = tqk_static_scratch(&ws);
        if (rcw) {
            delete h;
            return rcw;
        }
    }

    const int d = h->d, pd = h->pd, nc = h->n_centroids;
    int rc = TQ_OK;
    std::vector<double> cent(cfg->centroids, cfg->centroids + nc), bounds(nc - 1);
    for (int k = 0; k + 1 < nc; ++k) bounds[k] = (cent[k] + cent[k + 1]) / 2.0;
    h->zero_code = 0;
    for (int k = 0; k + 1 < nc; ++k) h->zero_code += bounds[k] < 0.0 ? 1 : 0;
    for (int k = 0; k < nc && k < 16; ++k) h->centroids_host[k] = cent[k];
    for (int k = 0; k + 1 < nc && k < 15; ++k) h->bounds_host[k] = bounds[k];
    rc = rc ? rc : upload(&h->centroids64, cent);
    rc = rc ? rc : upload(&h->bounds64, bounds);
    std::vector<double> s1, s2;
    if (cfg->rotation == TQ_ROT_WHT) {
        s1.assign(cfg->signs1, cfg->signs1 + pd);
        s2.assign(cfg->signs2, cfg->signs2 + pd);
        rc = rc ? rc : upload(&h->s1_64, s1);
        rc = rc ? rc : upload(&h->s2_64, s2);
    } else {
        std::vector<double> m(cfg->rotation_matrix, cfg->rotation_matrix + (size_t)d * d), mt((size_t)d * d);
        for (int i = 0; i < d; ++i)
            for (int j = 0; j < d; ++j) mt[(size_t)j * d + i] = m[(size_t)i * d + j];
        rc = rc ? rc : upload(&h->rot64, m);
        rc = rc ? rc : upload(&h->rot64_t, mt);
    }
    std::vector<double> S;
    if (cfg->projection) {
        S.assign(cfg->projection, cfg->projection + (size_t)d * d);
        std::vector<double> st((size_t)d * d);
        for (int i = 0; i < d; ++i)
            for (int j = 0; j < d; ++j) st[(size_t)j * d + i] = S[(size_t)i * d + j];
        rc = rc ? rc : upload(&h->proj64, S);
        rc = rc ? rc : upload(&h->proj64_t, st);
    }
    if (d == 128 && cfg->rotation == TQ_ROT_WHT && cfg->bits <= 4) {
        std::vector<float> c32(cent.begin(), cent.end()), b32(bounds.begin(), bounds.end());
        std::vector<float> s1f(s1.begin(), s1.end()), s2f(s2.begin(), s2.end());
        rc = rc ? rc : upload(&h->centroids32, c32);
        rc = rc ? rc : upload(&h->bounds32, b32);
        rc = rc ? rc : upload(&h->s1_32, s1f);
        rc = rc ? rc : upload(&h->s2_32, s2f);
        // pair LUT: entry (hi << bits | lo) = half2(c[lo], c[hi])
        const int b = cfg->bits;
        std::vector<uint32_t> lut((size_t)1 << (2 * b));
        for (int hi = 0; hi < nc; ++hi)
            for (int lo = 0; lo < nc; ++lo)
                lut[(size_t)(hi << b) | lo] = (uint32_t)f64_to_f16_bits(cent[lo]) | ((uint32_t)f64_to_f16_bits(cent[hi]) << 16);
        uint32_t *dl = nullptr;
        rc = rc ? rc : upload(&dl, lut);
        h->pair_lut = dl;
        std::memset(h->pair_lut_host, 0, sizeof(h->pair_lut_host));
        std::memcpy(h->pair_lut_host, lut.data(), lut.size() * sizeof(uint32_t));
        // factored transform for K rows: fragment f0*4+ks, row 4c+i, column 8kb+e
        {
            std::vector<uint16_t> rk((size_t)8 * 64 * 8);
            for (int f = 0; f < 8; ++f)
                for (int l = 0; l < 64; ++l)
                    for (int e = 0; e < 8; ++e) {
                        const int r = l & 15, f0 = f >> 2, ks = f & 3;
                        const int m = 32 * (r >> 2) + 4 * f0 + (r & 3), k = 32 * (l >> 4) + 8 * ks + e;
                        const double v = s1[k] * ((__builtin_popcount(m & k) & 1) ? -1.0 : 1.0);
                        rk[((size_t)f * 64 + l) * 8 + e] = v < 0 ? 0xBC00 : 0x3C00;
                    }
            uint16_t *drk = nullptr;
            rc = rc ? rc : upload(&drk, rk);
            h->rfrag16k = drk;
            // the same fragments for the way back (x = D1 H D2 y / sqrt(128)): the input-side signs are s2
            for (int f = 0; f < 8; ++f)
                for (int l = 0; l < 64; ++l)
                    for (int e = 0; e < 8; ++e) {
                        const int r = l & 15, f0 = f >> 2, ks = f & 3;
                        const int m = 32 * (r >> 2) + 4 * f0 + (r & 3), k = 32 * (l >> 4) + 8 * ks + e;
                        const double v = s2[k] * ((__builtin_popcount(m & k) & 1) ? -1.0 : 1.0);
                        rk[((size_t)f * 64 + l) * 8 + e] = v < 0 ? 0xBC00 : 0x3C00;
                    }
            uint16_t *dri = nullptr;
            rc = rc ? rc : upload(&dri, rk);
            h->rfrag16k_inv = dri;
            for (int f = 0; f < 8; ++f)
                for (int l = 0; l < 64; ++l)
                    for (int e = 0; e < 8; ++e) {
                        const int m = 16 * (f >> 2) + (l & 15), k = 32 * (f & 3) + 8 * (l >> 4) + e;
                        const double v = s1[k] * ((__builtin_popcount(m & k) & 1) ? -1.0 : 1.0);
                        rk[((size_t)f * 64 + l) * 8 + e] = v < 0 ? 0xBC00 : 0x3C00;
                    }
            uint16_t *drv = nullptr;
            rc = rc ? rc : upload(&drv, rk);
            h->rfrag16v = drv;
            // sign-field positions of the values with s2 = +1 inside a lane quarter's unfolded dwords: the
            // kernel appends the sign bit of s2 * y' (1 = negative) and xors with this to get "positive"
            std::vector<uint32_t> fl(16, 0u);
            for (int c = 0; c < 4; ++c)
                for (int v = 0; v < 32; ++v) {
                    if (s2[32 * c + v] < 0) continue;
                    if (b == 4) fl[c * 4 + v / 8] |= 1u << (4 * (v % 8) + 3);
                    else if (b == 2) fl[c * 4 + v / 16] |= 1u << (2 * (v % 16) + 1);
                    else if (b == 3) fl[c * 4 + v / 8] |= 1u << (3 * (v % 8) + 2);  // entry 3: the tail word
                }
            rc = rc ? rc : upload(&h->s2flip, fl);
            for (int i = 0; i < 16; ++i) h->s2flip_host[i] = fl[i];
            for (int w = 0; w < 4; ++w) h->s1neg_host[w] = h->s2neg_host[w] = 0u;
            for (int k = 0; k < 128; ++k) {
                if (s1[k] < 0) h->s1neg_host[k >> 5] |= 1u << (k & 31);
                if (s2[k] < 0) h->s2neg_host[k >> 5] |= 1u << (k & 31);
            }
        }
        // sign-symmetric boundaries (in fp32) allow the thermometer quantiser
        const int nb = nc - 1, mid = nb / 2;
        h->symmetric = 1;
        for (int j = 1; j <= mid; ++j)
            if (b32[mid + j] != -b32[mid - j] || !(b32[mid + j] > 0.0f)) h->symmetric = 0;
        if (std::fabs(b32[mid]) > 1e-12f) h->symmetric = 0;
        for (int m = 0; m <= mid; ++m)
            if (std::fabs(cent[mid + 1 + m] + cent[mid - m]) > 1e-9 * std::fabs(cent[mid + 1 + m])) h->symmetric = 0;
        std::vector<float> st((size_t)mid + 1);
        st[0] = b32[mid];
        for (int j = 1; j <= mid; ++j) st[j] = b32[mid + j];
        rc = rc ? rc : upload(&h->symthr32, st);
        for (int j = 0; j < 8; ++j) h->symthr_host[j] = j <= mid ? st[j] : 0.0f;
        // magnitude level by table: a bin of the value's top 12 bits holds at most one boundary, so
        // level = (boundaries below the bin) + (|value| > the bin's boundary)
        {
            std::vector<uint2> ql(4096);
            h->quant_lut_ok = 1;
            for (uint32_t idx = 0; idx < 4096; ++idx) {
                const uint32_t s = idx >> 11, e3 = idx & 2047u;
                const uint32_t lo_bits = e3 << 20, hi_bits = (e3 + 1u) << 20;
                float lo, hi;
                std::memcpy(&lo, &lo_bits, 4);
                std::memcpy(&hi, &hi_bits, 4);
                const bool top = e3 >= 2040u;  // infinities and NaNs: the highest level
                uint32_t below = 0, inside = 0, tbits = 0x7f800000u;
                for (int j = 1; j <= mid; ++j) {
                    if (top || st[j] < lo) ++below;
                    else if (st[j] < hi) {
                        ++inside;
                        std::memcpy(&tbits, &st[j], 4);
                    }
                }
                if (inside > 1) h->quant_lut_ok = 0;
                ql[idx] = make_uint2((s << (b - 1)) | below, tbits);
            }
            rc = rc ? rc : upload(&h->quant_lut, ql);
            // two handles whose tables hash alike (FNV-1a over the bytes; the tables are a function of `bits` and the
            // fp32 boundaries) can share one LDS copy in the fused K+V store
            uint64_t hash = 1469598103934665603ull;
            const unsigned char *bytes = reinterpret_cast<const unsigned char *>(ql.data());
            for (size_t i = 0; i < ql.size() * sizeof(uint2); ++i) hash = (hash ^ bytes[i]) * 1099511628211ull;
            h->quant_lut_hash = hash;
        }
        // squared centroid of magnitude level m as a multilinear form in the bits of m
        // (Moebius transform over subsets), for counting-based sums of c^2
        {
            const int nl = mid + 1;  // levels 0..mid, a power of two
            std::vector<double> f((size_t)nl);
            for (int m = 0; m < nl; ++m) f[m] = cent[mid + 1 + m] * cent[mid + 1 + m];
            for (int bit = 1; bit < nl; bit <<= 1)
                for (int m = 0; m < nl; ++m)
                    if (m & bit) f[m] -= f[m ^ bit];
            std::vector<float> cf(f.begin(), f.end());
            rc = rc ? rc : upload(&h->sqcoef32, cf);
            for (int j = 0; j < 8; ++j) h->sqcoef_host[j] = j < nl ? cf[j] : 0.0f;
        }
        if (cfg->projection) {
            // M = S R^T with R[k][m] = s2[k] H[k][m] s1[m] / sqrt(128); stored as [k*128+j] = M[j][k]
            std::vector<double> mt((size_t)128 * 128);
            const double rs = 1.0 / std::sqrt(128.0);
            for (int j = 0; j < 128; ++j)
                for (int k = 0; k < 128; ++k) {
                    double acc = 0.0;
                    for (int m = 0; m < 128; ++m) {
                        const double hkm = (__builtin_popcount(k & m) & 1) ? -1.0 : 1.0;
                        acc += S[(size_t)j * 128 + m] * (s2[k] * hkm * s1[m]);
                    }
                    mt[(size_t)k * 128 + j] = acc * rs;
                }
            rc = rc ? rc : upload(&h->projrot64_t, mt);
            // The QJL store's projection: 64 M split into three fp16 terms (hi + mid to 2^-22 of the entry, all three to
            // 2^-31; the factor keeps the middle terms out of fp16's subnormals), laid out as B operands of
            // v_mfma_f32_16x16x32_f16.  Fragment (step c, column block jb), lane l, element e =
            // 64 M[j = 16 jb + l % 16][k = 4 (8 c + e) + l / 16]: the contraction runs over the dims in the order in
            // which a lane of the store kernel holds them.
            // First pass, matrix cores: the kernel scales a token's residual r by a power of two to x with
            // 512 <= |x| < 1024, splits x into two fp16 terms and accumulates hi*hi in one fp32 accumulator and
            // hi*mid + lo*hi in another.  Against the exact sum the result is off by at most
            //   (128 * 2^-23 [main term: one fp32 rounding per product, taken as truncation, partial sums bounded by
            //   sum |x_k| |64 M_jk|] + 3 * 2^-22 [both splits and the dropped lo*mid] + 2^-23 [the small terms'
            //   roundings and the final addition]) * |x| |64 M_j| + 6.8e-4 (|x| + |64 M_j|) [fp16 subnormals of the
            //   low terms, should the matrix cores flush them]
            //   <=  (1.61e-5 max_j |64 M_j| + 6.8e-4 (1 + max_j |64 M_j| / 512)) |x|,
            // so a projection whose fast value is at least qjl_tau |x| (that bound with 2.0e-5 for 1.61e-5) away from
            // zero has the sign of the exact one.  Second pass, for the few that are closer (about one in 3000): the
            // float64 residual against hi + mid + lo in float64, off by at most 2^-31 |r| |64 M_j|; qjl_tau2 |r| (twice
            // that) settles all but one in 10^8 of those, which a third pass takes from the float64 matrix in memory.
            {
                std::vector<uint16_t> qf((size_t)3 * 4 * 8 * 64 * 8);
                const size_t set = (size_t)4 * 8 * 64 * 8;
                double maxrow = 0.0;
                for (int j = 0; j < 128; ++j) {
                    double ss = 0.0;
                    for (int k = 0; k < 128; ++k) ss += mt[(size_t)k * 128 + j] * mt[(size_t)k * 128 + j];
                    maxrow = std::max(maxrow, 64.0 * std::sqrt(ss));
                }
                for (int c = 0; c < 4; ++c)
                    for (int jb = 0; jb < 8; ++jb)
                        for (int l = 0; l < 64; ++l)
                            for (int e = 0; e < 8; ++e) {
                                const int j = 16 * jb + (l & 15), k = 4 * (8 * c + e) + (l >> 4);
                                const double mv = 64.0 * mt[(size_t)k * 128 + j];
                                const size_t at = ((((size_t)c * 8 + jb) * 64) + l) * 8 + e;
                                const uint16_t hi = f64_to_f16_bits(mv);
                                const double r1 = mv - f16_bits_to_f64(hi);
                                const uint16_t mid = f64_to_f16_bits(r1);
                                qf[at] = hi;
                                qf[set + at] = mid;
                                qf[2 * set + at] = f64_to_f16_bits(r1 - f16_bits_to_f64(mid));
                            }
                rc = rc ? rc : upload(&h->qjl_frag, qf);
                h->qjl_tau = (float)(2.0e-5 * maxrow + 6.8e-4 * (1.0 + maxrow / 512.0));
                h->qjl_tau2 = 2.0 * std::ldexp(1.0, -31) * maxrow;
            }
            // Operand fragments of the query preparation (score tile): W = [D2 H D1 ; S] as the row side of
            // 32 x 32 x 16 matrix instructions.  Set 0: the rotation's +-1 entries (its 1/sqrt(128) is applied to the
            // sums), sets 1 and 2: S split into two fp16 terms (S = hi + lo to 2^-22).  Fragment (row block cb, step
            // t), lane l, element e = W[32 cb + l % 32][16 t + 8 (l / 32) + e].
            std::vector<uint16_t> wf((size_t)3 * 4 * 8 * 64 * 8);
            for (int cb = 0; cb < 4; ++cb)
                for (int t = 0; t < 8; ++t)
                    for (int l = 0; l < 64; ++l)
                        for (int e = 0; e < 8; ++e) {
                            const int j = 32 * cb + (l & 31), k = 16 * t + 8 * (l >> 5) + e;
                            const size_t at = ((((size_t)cb * 8 + t) * 64) + l) * 8 + e, set = (size_t)4 * 8 * 64 * 8;
                            const double r = s2[j] * ((__builtin_popcount(j & k) & 1) ? -1.0 : 1.0) * s1[k];
                            wf[at] = r < 0 ? 0xBC00 : 0x3C00;
                            const double sv = S[(size_t)j * 128 + k];
                            const uint16_t hi = f64_to_f16_bits(sv);
                            wf[set + at] = hi;
                            wf[2 * set + at] = f64_to_f16_bits(sv - f16_bits_to_f64(hi));
                        }
            rc = rc ? rc : upload(&h->score_wfrag, wf);
        }
    }
    if (rc) {
        tq_destroy(h);
        return rc;
    }
    *out = h;
    return TQ_OK;
}

void tq_destroy(tq_handle *h) {
    if (!h) return;
    void *ptrs[] = {h->centroids64, h->bounds64, h->s1_64,  h->s2_64,       h->rot64, h->rot64_t,  h->proj64, h->proj64_t,
                    h->centroids32, h->bounds32, h->s1_32,  h->s2_32,       h->projrot64_t, h->pair_lut, h->score_wfrag, h->qjl_frag,
                    h->symthr32,    h->rfrag16k,    h->sqcoef32, h->s2flip,      h->rfrag16v, h->quant_lut,
                    h->rfrag16k_inv};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    delete h;
}

#define REQUIRE(cond, code, ...)      \
    do {                              \
        if (!(cond)) {                \
            tq_set_error(__VA_ARGS__); \
            return code;              \
        }                             \
    } while (0)

int tq_fwht(const void *x, void *y, int64_t n, int32_t len, int in_dtype, int out_dtype, void *stream) {
    REQUIRE(n >= 0 && (n == 0 || (x && y)), TQ_ERR_ARG, "tq_fwht: bad argument");
    REQUIRE(len >= 1 && (len & (len - 1)) == 0, TQ_ERR_ARG, "Input length must be a positive power of 2, got %d", len);
    REQUIRE(len <= TQ_MAX_D, TQ_ERR_UNSUPPORTED, "tq_fwht: length %d > %d", len, TQ_MAX_D);
    if (n == 0) return TQ_OK;
    return tqk_fwht(x, y, n, len, in_dtype, out_dtype, (hipStream_t)stream);
}

int tq_rotate(const tq_handle *h, const void *x, void *y, int64_t n, int in_dtype, int out_dtype, int transpose,
              void *stream) {
    REQUIRE(h && n >= 0 && (n == 0 || (x && y)), TQ_ERR_ARG, "tq_rotate: bad argument");
    if (n == 0) return TQ_OK;
    if (fast_ok(h) && in_dtype != TQ_F64 && out_dtype != TQ_F64)
        return tqk_rotate128(h, x, y, n, in_dtype, out_dtype, transpose, (hipStream_t)stream);
    return tqk_rotate64(h, x, y, n, in_dtype, out_dtype, transpose, (hipStream_t)stream);
}

int tq_nearest_centroid(const double *values, int64_t n, const double *centroids_host, int32_t n_centroids,
                        int32_t *idx, void *stream) {
    REQUIRE(values && centroids_host && idx && n >= 0, TQ_ERR_ARG, "tq_nearest_centroid: bad argument");
    REQUIRE(n_centroids >= 1 && n_centroids <= 256, TQ_ERR_UNSUPPORTED, "tq_nearest_centroid: %d centroids (max 256)",
            n_centroids);
    if (n == 0) return TQ_OK;
    double bounds[255];
    for (int k = 0; k + 1 < n_centroids; ++k) bounds[k] = (centroids_host[k] + centroids_host[k + 1]) / 2.0;
    return tqk_nearest(values, n, bounds, n_centroids - 1, idx, (hipStream_t)stream);
}

int tq_quantize_indices(const tq_handle *h, const void *x, int64_t n, int in_dtype, uint8_t *idx, double *norms,
                        double *rotated, void *stream) {
    REQUIRE(h && x && idx && norms && n >= 0, TQ_ERR_ARG, "tq_quantize_indices: bad argument");
    if (n == 0) return TQ_OK;
    return tqk_quantize_indices(h, x, n, in_dtype, idx, norms, rotated, (hipStream_t)stream);
}

int tq_dequantize_indices(const tq_handle *h, const uint8_t *idx, const double *norms, int64_t n, double *out,
                          const void *x, int x_dtype, double *residual, void *stream) {
    REQUIRE(h && idx && norms && out && n >= 0, TQ_ERR_ARG, "tq_dequantize_indices: bad argument");
    REQUIRE(!residual || x, TQ_ERR_ARG, "tq_dequantize_indices: residual needs x");
    if (n == 0) return TQ_OK;
    return tqk_dequantize_indices(h, idx, norms, n, out, x, x_dtype, residual, (hipStream_t)stream);
}

int tq_qjl_quantize(const tq_handle *h, const void *r, int64_t n, int in_dtype, int8_t *signs, double *norms,
                    void *stream) {
    REQUIRE(h && r && signs && norms && n >= 0, TQ_ERR_ARG, "tq_qjl_quantize: bad argument");
    REQUIRE(h->has_proj, TQ_ERR_ARG, "tq_qjl_quantize: handle has no projection");
    if (n == 0) return TQ_OK;
    return tqk_qjl_quantize(h, r, n, in_dtype, signs, norms, (hipStream_t)stream);
}

int tq_qjl_dequantize(const tq_handle *h, const int8_t *signs, const double *norms, double shrinkage, int64_t n,
                      double *out, void *stream) {
    REQUIRE(h && signs && norms && out && n >= 0, TQ_ERR_ARG, "tq_qjl_dequantize: bad argument");
    REQUIRE(h->has_proj, TQ_ERR_ARG, "tq_qjl_dequantize: handle has no projection");
    if (n == 0) return TQ_OK;
    return tqk_qjl_dequantize(h, signs, norms, shrinkage, n, out, (hipStream_t)stream);
}

int tq_pack_bits(const int8_t *signs, int64_t n, int32_t d, uint8_t *packed, void *stream) {
    REQUIRE(signs && packed && n >= 0 && d >= 1, TQ_ERR_ARG, "tq_pack_bits: bad argument");
    if (n == 0) return TQ_OK;
    return tqk_pack_bits(signs, n, d, packed, (hipStream_t)stream);
}

int tq_unpack_bits(const uint8_t *packed, int64_t n, int32_t d, int8_t *signs, void *stream) {
    REQUIRE(signs && packed && n >= 0 && d >= 1, TQ_ERR_ARG, "tq_unpack_bits: bad argument");
    if (n == 0) return TQ_OK;
    return tqk_unpack_bits(packed, n, d, signs, (hipStream_t)stream);
}

int tq_pack_indices(const uint8_t *idx, int64_t count, int32_t bits, uint8_t *packed, void *stream) {
    REQUIRE(bits >= 1 && bits <= 8, TQ_ERR_ARG, "bit_width must be 1-8, got %d", bits);
    REQUIRE(idx && packed && count >= 0, TQ_ERR_ARG, "tq_pack_indices: bad argument");
    if (count == 0) return TQ_OK;
    return tqk_pack_indices(idx, count, bits, packed, (hipStream_t)stream);
}

int64_t tq_packed_bytes(int32_t bits, int64_t n_seqs, int64_t tokens) {
    if (bits < 2 || bits > 4 || n_seqs < 0 || tokens < 0) return -1;
    return n_seqs * ((tokens + TQ_ROWS_PER_BLOCK - 1) / TQ_ROWS_PER_BLOCK) * (int64_t)(TQ_ROWS_PER_BLOCK * (16 * bits + 2));
}

int64_t tq_q8_0_bytes(int64_t n_seqs, int64_t tokens) {
    if (n_seqs < 0 || tokens < 0) return -1;
    return n_seqs * ((tokens + TQ_ROWS_PER_BLOCK - 1) / TQ_ROWS_PER_BLOCK) * (int64_t)(TQ_ROWS_PER_BLOCK * 136);
}

static int check_fast(const tq_handle *h, const char *who) {
    REQUIRE(h, TQ_ERR_ARG, "%s: null handle", who);
    REQUIRE(fast_ok(h), TQ_ERR_UNSUPPORTED, "%s: needs d == 128 and WHT rotation (handle has d=%d, rotation=%d)", who,
            h->d, h->rotation);
    REQUIRE(h->bits >= 2 && h->bits <= 4, TQ_ERR_UNSUPPORTED, "%s: bits must be 2, 3 or 4 (got %d)", who, h->bits);
    return TQ_OK;
}

int tq_store(const tq_handle *h, const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, int kind, void *packed,
             void *stream) {
    int rc = check_fast(h, "tq_store");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_store: bad argument");
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(x && packed, TQ_ERR_ARG, "tq_store: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_store: bad kind %d", kind);
    REQUIRE(aligned16(x) && aligned16(packed), TQ_ERR_ALIGN, "tq_store: x and packed must be 16-byte aligned");
    return tqk_store(h, x, n_seqs, tokens, in_dtype, kind, packed, nullptr, nullptr, (hipStream_t)stream);
}

int tq_append(const tq_handle *h, const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype,
              int kind, void *packed, void *stream) {
    int rc = check_fast(h, "tq_append");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && pos >= 0 && n_new >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_append: bad argument");
    REQUIRE(pos + n_new <= capacity, TQ_ERR_ARG, "tq_append: tokens %lld..%lld do not fit a capacity of %lld", (long long)pos,
            (long long)(pos + n_new), (long long)capacity);
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    REQUIRE(x && packed, TQ_ERR_ARG, "tq_append: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_append: bad kind %d", kind);
    REQUIRE(aligned16(x) && aligned16(packed), TQ_ERR_ALIGN, "tq_append: x and packed must be 16-byte aligned");
    return tqk_append(h, x, n_seqs, pos, n_new, capacity, in_dtype, kind, packed, (hipStream_t)stream);
}

int tq_append_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t pos,
                 int64_t n_new, int64_t capacity, int in_dtype, void *packed_k, void *packed_v, void *stream) {
    int rc = check_fast(hk, "tq_append_kv");
    rc = rc ? rc : check_fast(hv, "tq_append_kv");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && pos >= 0 && n_new >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_append_kv: bad argument");
    REQUIRE(pos + n_new <= capacity, TQ_ERR_ARG, "tq_append_kv: tokens %lld..%lld do not fit a capacity of %lld", (long long)pos,
            (long long)(pos + n_new), (long long)capacity);
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    REQUIRE(k && v && packed_k && packed_v, TQ_ERR_ARG, "tq_append_kv: null pointer");
    REQUIRE(aligned16(k) && aligned16(v) && aligned16(packed_k) && aligned16(packed_v), TQ_ERR_ALIGN,
            "tq_append_kv: inputs and packed buffers must be 16-byte aligned");
    return tqk_append_kv(hk, hv, k, v, n_seqs, pos, n_new, capacity, in_dtype, packed_k, packed_v, (hipStream_t)stream);
}

int tq_append_at(const tq_handle *h, const void *x, int64_t n_seqs, const int64_t *pos_dev, int64_t n_new, int64_t capacity,
                 int in_dtype, int kind, void *packed, uint32_t *overrun_dev, void *stream) {
    int rc = check_fast(h, "tq_append_at");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && n_new >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_append_at: bad argument");
    REQUIRE(n_new <= capacity, TQ_ERR_ARG, "tq_append_at: %lld tokens do not fit a capacity of %lld", (long long)n_new,
            (long long)capacity);
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    REQUIRE(x && packed && pos_dev, TQ_ERR_ARG, "tq_append_at: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_append_at: bad kind %d", kind);
    REQUIRE(aligned16(x) && aligned16(packed), TQ_ERR_ALIGN, "tq_append_at: x and packed must be 16-byte aligned");
    REQUIRE((reinterpret_cast<uintptr_t>(pos_dev) & 7u) == 0, TQ_ERR_ALIGN, "tq_append_at: pos_dev must be 8-byte aligned");
    REQUIRE((reinterpret_cast<uintptr_t>(overrun_dev) & 3u) == 0, TQ_ERR_ALIGN, "tq_append_at: overrun_dev must be 4-byte aligned");
    return tqk_append(h, x, n_seqs, 0, n_new, capacity, in_dtype, kind, packed, (hipStream_t)stream, pos_dev, overrun_dev);
}

int tq_q8_0_append_at(const void *x, int64_t n_seqs, const int64_t *pos_dev, int64_t n_new, int64_t capacity, int in_dtype,
                      int kind, void *packed, uint32_t *overrun_dev, void *stream) {
    REQUIRE(n_seqs >= 0 && n_new >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_q8_0_append_at: bad argument");
    REQUIRE(n_new <= capacity, TQ_ERR_ARG, "tq_q8_0_append_at: %lld tokens do not fit a capacity of %lld", (long long)n_new,
            (long long)capacity);
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    REQUIRE(x && packed && pos_dev, TQ_ERR_ARG, "tq_q8_0_append_at: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_q8_0_append_at: bad kind %d", kind);
    REQUIRE(aligned16(packed), TQ_ERR_ALIGN, "tq_q8_0_append_at: packed must be 16-byte aligned");
    REQUIRE((reinterpret_cast<uintptr_t>(pos_dev) & 7u) == 0, TQ_ERR_ALIGN, "tq_q8_0_append_at: pos_dev must be 8-byte aligned");
    REQUIRE((reinterpret_cast<uintptr_t>(overrun_dev) & 3u) == 0, TQ_ERR_ALIGN, "tq_q8_0_append_at: overrun_dev must be 4-byte aligned");
    return tqk_q8_0_append(x, n_seqs, 0, n_new, capacity, in_dtype, kind, packed, (hipStream_t)stream, pos_dev, overrun_dev);
}

int tq_append_kv_at(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs,
                    const int64_t *pos_dev, int64_t n_new, int64_t capacity, int in_dtype, void *packed_k, void *packed_v,
                    uint32_t *overrun_dev, void *stream) {
    int rc = check_fast(hk, "tq_append_kv_at");
    rc = rc ? rc : check_fast(hv, "tq_append_kv_at");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && n_new >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_append_kv_at: bad argument");
    REQUIRE(n_new <= capacity, TQ_ERR_ARG, "tq_append_kv_at: %lld tokens do not fit a capacity of %lld", (long long)n_new,
            (long long)capacity);
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    REQUIRE(k && v && packed_k && packed_v && pos_dev, TQ_ERR_ARG, "tq_append_kv_at: null pointer");
    REQUIRE(aligned16(k) && aligned16(v) && aligned16(packed_k) && aligned16(packed_v), TQ_ERR_ALIGN,
            "tq_append_kv_at: inputs and packed buffers must be 16-byte aligned");
    REQUIRE((reinterpret_cast<uintptr_t>(pos_dev) & 7u) == 0, TQ_ERR_ALIGN, "tq_append_kv_at: pos_dev must be 8-byte aligned");
    REQUIRE((reinterpret_cast<uintptr_t>(overrun_dev) & 3u) == 0, TQ_ERR_ALIGN, "tq_append_kv_at: overrun_dev must be 4-byte aligned");
    return tqk_append_kv(hk, hv, k, v, n_seqs, 0, n_new, capacity, in_dtype, packed_k, packed_v, (hipStream_t)stream, pos_dev,
                         overrun_dev);
}

int tq_requantize(const tq_handle *src_h, const tq_handle *dst_h, const void *packed_src, int64_t n_seqs, int64_t tokens,
                  int kind, void *packed_dst, void *stream) {
    int rc = check_fast(src_h, "tq_requantize");
    rc = rc ? rc : check_fast(dst_h, "tq_requantize");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_requantize: bad argument");
    REQUIRE(dst_h->bits < src_h->bits, TQ_ERR_UNSUPPORTED, "tq_requantize: destination must be narrower (%d -> %d bits)",
            src_h->bits, dst_h->bits);
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(packed_src && packed_dst, TQ_ERR_ARG, "tq_requantize: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_requantize: bad kind %d", kind);
    REQUIRE(aligned16(packed_src) && aligned16(packed_dst), TQ_ERR_ALIGN, "tq_requantize: buffers must be 16-byte aligned");
    return tqk_requantize(src_h, dst_h, packed_src, n_seqs, tokens, kind, packed_dst, (hipStream_t)stream);
}

// bytes of one 128-value vector in the fork's layout: 128 / block_values storage blocks of norm | qs | signs
int64_t tq_fork_row_bytes(int32_t bits, int32_t block_values) {
    if (bits == 4) return block_values == 128 ? 68 : -1;
    if ((bits != 2 && bits != 3) || (block_values != 32 && block_values != 64 && block_values != 128)) return -1;
    return (128 / block_values) * (2 + block_values * bits / 8);
}

int64_t tq_fork_block_bytes(int32_t bits) { return tq_fork_row_bytes(bits, 128); }

static int fork_blocks(const tq_handle *h, int to_fork, const void *src, int64_t n_seqs, int64_t tokens, int kind, void *dst,
                       int block_values, void *stream, const char *who) {
    int rc = check_fast(h, who);
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "%s: bad argument", who);
    REQUIRE(tq_fork_row_bytes(h->bits, block_values) > 0, TQ_ERR_UNSUPPORTED,
            "%s: %d-bit rows in storage blocks of %d values are not a layout of the fork (2- and 3-bit: 32, 64 or 128 values "
            "per block; 4-bit: 128)", who, h->bits, block_values);
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(src && dst, TQ_ERR_ARG, "%s: null pointer", who);
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "%s: bad kind %d", who, kind);
    REQUIRE(aligned16(to_fork ? src : dst), TQ_ERR_ALIGN, "%s: the packed buffer must be 16-byte aligned", who);
    // 4-bit blocks are 68 bytes (norm, rnorm, 16 code words): their rows are read and written as 4-byte words
    const uintptr_t fork_align = h->bits == 4 ? 4u : 2u;
    REQUIRE(((uintptr_t)(to_fork ? dst : src) & (fork_align - 1u)) == 0, TQ_ERR_ALIGN,
            "%s: the blocks must be %d-byte aligned (a block starts with an fp16 norm%s)", who, (int)fork_align,
            h->bits == 4 ? " and its 68-byte rows move as 4-byte words" : "");
    return tqk_fork_blocks(h, to_fork, src, n_seqs, tokens, kind, dst, block_values, (hipStream_t)stream);
}

int tq_export_fork_blocks(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, void *blocks,
                          void *stream) {
    return fork_blocks(h, 1, packed, n_seqs, tokens, kind, blocks, 128, stream, "tq_export_fork_blocks");
}

int tq_import_fork_blocks(const tq_handle *h, const void *blocks, int64_t n_seqs, int64_t tokens, int kind, void *packed,
                          void *stream) {
    return fork_blocks(h, 0, blocks, n_seqs, tokens, kind, packed, 128, stream, "tq_import_fork_blocks");
}

int tq_export_fork_blocks_sized(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind,
                                int32_t block_values, void *blocks, void *stream) {
    return fork_blocks(h, 1, packed, n_seqs, tokens, kind, blocks, block_values, stream, "tq_export_fork_blocks_sized");
}

int tq_import_fork_blocks_sized(const tq_handle *h, const void *blocks, int64_t n_seqs, int64_t tokens, int kind,
                                int32_t block_values, void *packed, void *stream) {
    return fork_blocks(h, 0, blocks, n_seqs, tokens, kind, packed, block_values, stream, "tq_import_fork_blocks_sized");
}

int tq_store_kv(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t tokens,
                int in_dtype, void *packed_k, void *packed_v, void *stream) {
    int rc = check_fast(hk, "tq_store_kv");
    rc = rc ? rc : check_fast(hv, "tq_store_kv");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_store_kv: bad argument");
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(k && v && packed_k && packed_v, TQ_ERR_ARG, "tq_store_kv: null pointer");
    REQUIRE(aligned16(k) && aligned16(v) && aligned16(packed_k) && aligned16(packed_v), TQ_ERR_ALIGN,
            "tq_store_kv: inputs and outputs must be 16-byte aligned");
    return tqk_store_kv(hk, hv, k, v, n_seqs, tokens, 0, in_dtype, packed_k, packed_v, (hipStream_t)stream);
}

int tq_store_kv_cache(const tq_handle *hk, const tq_handle *hv, const void *k, const void *v, int64_t n_seqs, int64_t tokens,
                      int64_t capacity, int in_dtype, void *packed_k, void *packed_v, void *stream) {
    int rc = check_fast(hk, "tq_store_kv_cache");
    rc = rc ? rc : check_fast(hv, "tq_store_kv_cache");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_store_kv_cache: bad argument");
    REQUIRE(tokens <= capacity, TQ_ERR_ARG, "tq_store_kv_cache: %lld tokens do not fit a capacity of %lld", (long long)tokens,
            (long long)capacity);
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(k && v && packed_k && packed_v, TQ_ERR_ARG, "tq_store_kv_cache: null pointer");
    REQUIRE(aligned16(k) && aligned16(v) && aligned16(packed_k) && aligned16(packed_v), TQ_ERR_ALIGN,
            "tq_store_kv_cache: inputs and outputs must be 16-byte aligned");
    return tqk_store_kv(hk, hv, k, v, n_seqs, tokens, capacity, in_dtype, packed_k, packed_v, (hipStream_t)stream);
}

int tq_store_qjl(const tq_handle *h, const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed,
                 uint8_t *sign_bits, void *rnorms_f16, void *stream) {
    int rc = check_fast(h, "tq_store_qjl");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_store_qjl: bad argument");
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(x && packed && sign_bits && rnorms_f16, TQ_ERR_ARG, "tq_store_qjl: null pointer");
    REQUIRE(h->has_proj, TQ_ERR_ARG, "tq_store_qjl: handle has no projection");
    REQUIRE(aligned16(packed), TQ_ERR_ALIGN, "tq_store_qjl: packed must be 16-byte aligned");
    return tqk_store(h, x, n_seqs, tokens, in_dtype, TQ_KIND_K, packed, sign_bits, rnorms_f16, (hipStream_t)stream);
}

int tq_load(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, void *out, int out_dtype,
            int domain, void *stream) {
    int rc = check_fast(h, "tq_load");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_load: bad argument");
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(out && packed, TQ_ERR_ARG, "tq_load: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_load: bad kind %d", kind);
    REQUIRE(domain == TQ_DOMAIN_ROTATED || domain == TQ_DOMAIN_ORIGINAL, TQ_ERR_ARG, "tq_load: bad domain %d", domain);
    REQUIRE(aligned16(out) && aligned16(packed), TQ_ERR_ALIGN, "tq_load: out and packed must be 16-byte aligned");
    return tqk_load(h, packed, n_seqs, tokens, kind, out, out_dtype, domain, (hipStream_t)stream);
}

int tq_load_kv(const tq_handle *hk, const tq_handle *hv, const void *packed_k, const void *packed_v, int64_t n_seqs,
               int64_t tokens, void *out_k, void *out_v, void *stream) {
    int rc = check_fast(hk, "tq_load_kv");
    rc = rc ? rc : check_fast(hv, "tq_load_kv");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_load_kv: bad argument");
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(packed_k && packed_v && out_k && out_v, TQ_ERR_ARG, "tq_load_kv: null pointer");
    REQUIRE(aligned16(packed_k) && aligned16(packed_v) && aligned16(out_k) && aligned16(out_v), TQ_ERR_ALIGN,
            "tq_load_kv: inputs and outputs must be 16-byte aligned");
    return tqk_load_kv(hk, hv, packed_k, packed_v, n_seqs, tokens, out_k, out_v, (hipStream_t)stream);
}

int tq_unpack_codes(const tq_handle *h, const void *packed, int64_t n_seqs, int64_t tokens, int kind, uint8_t *idx,
                    float *norms, void *stream) {
    int rc = check_fast(h, "tq_unpack_codes");
    if (rc) return rc;
    REQUIRE(n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_unpack_codes: bad argument");
    if (n_seqs == 0 || tokens == 0) return TQ_OK;
    REQUIRE(idx && norms && packed, TQ_ERR_ARG, "tq_unpack_codes: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_unpack_codes: bad kind %d", kind);
    return tqk_unpack_codes(h, packed, n_seqs, tokens, kind, idx, norms, (hipStream_t)stream);
}

int tq_q8_0_store(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, void *stream) {
    REQUIRE(x && packed && n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_q8_0_store: bad argument");
    REQUIRE(aligned16(packed) && aligned16(x), TQ_ERR_ALIGN, "tq_q8_0_store: x and packed must be 16-byte aligned");
    return tqk_q8_0_store(x, n_seqs, tokens, in_dtype, packed, (hipStream_t)stream);
}

int tq_q8_0_unpack(const void *packed, int64_t n_seqs, int64_t tokens, int8_t *q, float *scales, void *stream) {
    REQUIRE(q && scales && packed && n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_q8_0_unpack: bad argument");
    return tqk_q8_0_unpack(packed, n_seqs, tokens, q, scales, TQ_KIND_K, (hipStream_t)stream);
}

int tq_q8_0_store_v(const void *x, int64_t n_seqs, int64_t tokens, int in_dtype, void *packed, void *stream) {
    REQUIRE(x && packed && n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_q8_0_store_v: bad argument");
    REQUIRE(aligned16(packed) && aligned16(x), TQ_ERR_ALIGN, "tq_q8_0_store_v: x and packed must be 16-byte aligned");
    return tqk_q8_0_store_v(x, n_seqs, tokens, in_dtype, packed, (hipStream_t)stream);
}

int tq_q8_0_append(const void *x, int64_t n_seqs, int64_t pos, int64_t n_new, int64_t capacity, int in_dtype, int kind,
                   void *packed, void *stream) {
    REQUIRE(n_seqs >= 0 && pos >= 0 && n_new >= 0 && capacity >= 0, TQ_ERR_ARG, "tq_q8_0_append: bad argument");
    REQUIRE(pos + n_new <= capacity, TQ_ERR_ARG, "tq_q8_0_append: tokens %lld..%lld do not fit a capacity of %lld",
            (long long)pos, (long long)(pos + n_new), (long long)capacity);
    if (n_seqs == 0 || n_new == 0) return TQ_OK;
    REQUIRE(x && packed, TQ_ERR_ARG, "tq_q8_0_append: null pointer");
    REQUIRE(kind == TQ_KIND_K || kind == TQ_KIND_V, TQ_ERR_ARG, "tq_q8_0_append: bad kind %d", kind);
    REQUIRE(aligned16(packed), TQ_ERR_ALIGN, "tq_q8_0_append: packed must be 16-byte aligned");
    return tqk_q8_0_append(x, n_seqs, pos, n_new, capacity, in_dtype, kind, packed, (hipStream_t)stream);
}

int tq_q8_0_unpack_v(const void *packed, int64_t n_seqs, int64_t tokens, int8_t *q, float *scales, void *stream) {
    REQUIRE(q && scales && packed && n_seqs >= 0 && tokens >= 0, TQ_ERR_ARG, "tq_q8_0_unpack_v: bad argument");
    return tqk_q8_0_unpack(packed, n_seqs, tokens, q, scales, TQ_KIND_V, (hipStream_t)stream);
}

static int check_attn(const tq_attn_params *p) {
    REQUIRE(p, TQ_ERR_ARG, "attention: null params");
    REQUIRE(p->batch >= 1 && p->n_q_heads >= 1 && p->n_kv_heads >= 1 && p->tokens >= 1 && p->n_splits >= 1, TQ_ERR_ARG,
            "attention: sizes must be positive");
    REQUIRE(p->n_q_heads % p->n_kv_heads == 0, TQ_ERR_ARG,
            "attention: the query head count must be a multiple of the KV head count (got %d / %d)", p->n_q_heads, p->n_kv_heads);
    REQUIRE(p->k_format == TQ_KFMT_TURBO || p->k_format == TQ_KFMT_Q8_0, TQ_ERR_ARG, "attention: bad k_format %d",
            p->k_format);
    REQUIRE(p->v_format == TQ_KFMT_TURBO || p->v_format == TQ_KFMT_Q8_0, TQ_ERR_ARG, "attention: bad v_format %d",
            p->v_format);
    REQUIRE(p->tokens < ((int64_t)1 << 36), TQ_ERR_UNSUPPORTED, "attention: context too long");
    REQUIRE(p->capacity == 0 || p->capacity >= p->tokens, TQ_ERR_ARG, "attention: capacity %lld < tokens %lld",
            (long long)p->capacity, (long long)p->tokens);
    REQUIRE(p->sparse_v_tau >= 0.0f, TQ_ERR_ARG, "attention: sparse_v_tau must be >= 0");
    return TQ_OK;
}

int64_t tq_attn_workspace_bytes(const tq_attn_params *p) {
    if (check_attn(p)) return -1;
    return tqk_attn_workspace_bytes(p);
}

int tq_decode_attention(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q, int q_dtype,
                        const void *k, const void *k_aux, const void *v, const float *bias, float *out,
                        unsigned long long *skip_count, void *workspace, int64_t workspace_bytes, void *stream) {
    int rc = check_attn(p);
    if (rc) return rc;
    if (p->v_format == TQ_KFMT_TURBO) {
        rc = check_fast(hv, "tq_decode_attention (V)");
        if (rc) return rc;
    }
    if (p->k_format == TQ_KFMT_TURBO) {
        rc = check_fast(hk, "tq_decode_attention (K)");
        if (rc) return rc;
    }
    REQUIRE(q && k && v && out && workspace, TQ_ERR_ARG, "tq_decode_attention: null pointer");
    REQUIRE(aligned16(k) && aligned16(v) && aligned16(workspace), TQ_ERR_ALIGN,
            "tq_decode_attention: k, v and workspace must be 16-byte aligned");
    return tqk_decode_attention(hk, hv, p, q, q_dtype, k, k_aux, v, bias, out, skip_count, workspace, workspace_bytes,
                                (hipStream_t)stream);
}

int tq_decode_attention_static(const tq_handle *hk, const tq_handle *hv, const tq_attn_params *p, const void *q,
                               int q_dtype, const void *k, const void *v, const float *bias, float *out,
                               unsigned long long *skip_count, void *stream) {
    int rc = check_attn(p);
    if (rc) return rc;
    if (p->v_format == TQ_KFMT_TURBO) {
        rc = check_fast(hv, "tq_decode_attention_static (V)");
        if (rc) return rc;
    }
    if (p->k_format == TQ_KFMT_TURBO) {
        rc = check_fast(hk, "tq_decode_attention_static (K)");
        if (rc) return rc;
    }
    REQUIRE(q && k && v && out, TQ_ERR_ARG, "tq_decode_attention_static: null pointer");
    REQUIRE(aligned16(k) && aligned16(v), TQ_ERR_ALIGN, "tq_decode_attention_static: k and v must be 16-byte aligned");
    return tqk_decode_attention_static(hk, hv, p, q, q_dtype, k, v, bias, out, skip_count, (hipStream_t)stream);
}

int tq_score_tile(const tq_handle *h, const void *q, int q_dtype, int64_t nq, const void *packed,
                  const uint8_t *sign_bits, const void *rnorms_f16, int64_t nk, void *logits, int out_dtype,
                  void *workspace, int64_t workspace_bytes, void *stream) {
    int rc = check_fast(h, "tq_score_tile");
    if (rc) return rc;
    REQUIRE(q && packed && sign_bits && rnorms_f16 && workspace && nq >= 0 && nk >= 0, TQ_ERR_ARG,
            "tq_score_tile: bad argument");
    REQUIRE(h->has_proj, TQ_ERR_ARG, "tq_score_tile: handle has no projection");
    REQUIRE(out_dtype == TQ_F32 || out_dtype == TQ_F16, TQ_ERR_ARG, "tq_score_tile: logits must be fp32 or fp16");
    REQUIRE(workspace_bytes >= (nq + 31) / 32 * 32 * 256 * 2, TQ_ERR_ARG, "tq_score_tile: workspace %lld < %lld bytes",
            (long long)workspace_bytes, (long long)(nq * 256 * 2));
    REQUIRE(aligned16(packed) && aligned16(workspace), TQ_ERR_ALIGN, "tq_score_tile: packed and workspace must be 16-byte aligned");
    // the logits leave as single-element buffer stores: a row slice of a larger matrix is fine
    REQUIRE((reinterpret_cast<uintptr_t>(logits) & (out_dtype == TQ_F32 ? 3u : 1u)) == 0, TQ_ERR_ALIGN,
            "tq_score_tile: logits must be aligned to their element type");
    if (nq == 0 || nk == 0) return TQ_OK;
    return tqk_score_tile(h, q, q_dtype, nq, packed, sign_bits, rnorms_f16, nk, logits, out_dtype, workspace,
                          workspace_bytes, (hipStream_t)stream);
}

}  // extern "C"
