/*
 * miw_oracle.c -- CPU restatement of the WMMA fragment semantics and of the
 * GEMM D = alpha*A*B + beta*C built on them.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared
 * against; nothing shipped may call it.  Only tests, the smoke check and the
 * CPU-baseline leg of the benchmark load this library.
 *
 * The reference (CUDAnative.jl v3.1.0) holds no arithmetic for this path: its
 * WMMA module only names NVVM intrinsics (src/device/cuda/wmma.jl:124,177,234)
 * and the tensor cores do the math.  What the reference fixes is the contract
 *   load_{a,b,c}(addr, stride, layout, config)   src/device/cuda/wmma.jl:507-530
 *   mma(a, b, c, config)  D = A*B + C            src/device/cuda/wmma.jl:558-583
 *   store_d(addr, d, stride, layout, config)     src/device/cuda/wmma.jl:613-632
 *   fill_c(value, config)                        src/device/cuda/wmma.jl:654-667
 *   f.(fragment, scalar) broadcasting            src/device/cuda/wmma.jl:678-716
 * and the checks in test/device/wmma.jl (constant-42 tiles :28-57,:71-98;
 * a*b+c within rtol sqrt(eps(Float16)) :146-149, :237-245).
 * This file restates that contract on whole 16x16 tiles (the per-lane register
 * order is documented as unspecified, docs/src/device/wmma.md:49) with every
 * product and sum carried in double, so it is at least as accurate as any
 * conforming implementation.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   half<->float conversion : exhaustive over all 65536 half patterns vs numpy
 *   tile load/store          : constant-42 known answers of the reference, the
 *                              identity/transposition invariants, distinct-valued tiles
 *   mma / gemm (f32 acc)     : brute-force triple loop, numpy float64 matmul, exact
 *                              integer and identity special cases, linearity
 *   gemm (f16 acc, chunked)  : exact on small-integer inputs (where every partial
 *                              sum is representable), equals the f32 result rounded
 *                              once when one chunk spans K, hand-built case that
 *                              shows the intermediate rounding
 *   Bit-level rounding of the tensor-core instruction itself is parity-unpinned:
 *   the reference asserts tolerances only.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>
#include <stdlib.h>

#define MIWO_ROW 0
#define MIWO_COL 1
#define MIWO_F16 0
#define MIWO_F32 1

/* ---------------------------------------------------------------- half ---- */

/* IEEE binary16 -> binary32, exact. */
float miwo_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int e = -1;
            do { e++; man <<= 1; } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even, overflow to inf, subnormals kept. */
uint16_t miwo_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u) /* <= 2^-25 rounds to zero (tie goes to even = 0) */
        return (uint16_t)sign;
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7fffffu) | 0x800000u;
    uint32_t shift, half_exp;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(e + 15);
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    /* q carries the implicit bit for normals; adding it to the exponent field
       also handles the carry out of the mantissa. */
    uint32_t out;
    if (half_exp == 0) out = q;
    else out = ((half_exp - 1) << 10) + q;
    return (uint16_t)(sign | out);
}

/* double -> binary16 through one rounding only (no double rounding through float). */
uint16_t miwo_double_to_half(double d)
{
    /* Round d to a float with round-to-odd on the discarded bits so that the
       following float->half rounding sees a sticky bit; float has 13 more
       mantissa bits than half, which is enough for this to be exact. */
    float f = (float)d;
    if (isnan(d) || isinf(f)) return miwo_float_to_half(f);
    if ((double)f != d) {
        uint32_t x;
        memcpy(&x, &f, 4);
        if ((x & 1u) == 0) {
            /* make it odd in the direction of d */
            double fd = (double)f;
            int away = (fabs(d) > fabs(fd));
            if (away) x += 1u; else x -= 1u;
            memcpy(&f, &x, 4);
        }
    }
    return miwo_float_to_half(f);
}

void miwo_half_to_float_n(const uint16_t *h, float *f, size_t n)
{
    for (size_t i = 0; i < n; i++) f[i] = miwo_half_to_float(h[i]);
}

void miwo_float_to_half_n(const float *f, uint16_t *h, size_t n)
{
    for (size_t i = 0; i < n; i++) h[i] = miwo_float_to_half(f[i]);
}

/* ---------------------------------------------------------------- PRNG ---- */
/* Counter-based SplitMix64: element i of stream `seed` depends on (seed, i)
   only, so C, numpy and Julia produce identical inputs.  The reference draws
   unseeded rand() (test/device/wmma.jl:121-125); seeded inputs are this
   build's own. */
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t i)
{
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

uint64_t miwo_splitmix64_at(uint64_t seed, uint64_t i) { return splitmix64_at(seed, i); }

/* u in [0,1) with 24 random bits, exactly representable in float. */
static inline float unit24(uint64_t r) { return (float)(r >> 40) * (1.0f / 16777216.0f); }

/* out[i] = lo + (hi-lo)*u_i in float, i = 0..n-1 */
void miwo_fill_uniform_f32(float *out, size_t n, uint64_t seed, float lo, float hi)
{
    for (size_t i = 0; i < n; i++) out[i] = lo + (hi - lo) * unit24(splitmix64_at(seed, i));
}

void miwo_fill_uniform_f16(uint16_t *out, size_t n, uint64_t seed, float lo, float hi)
{
    for (size_t i = 0; i < n; i++)
        out[i] = miwo_float_to_half(lo + (hi - lo) * unit24(splitmix64_at(seed, i)));
}

/* Box-Muller on two consecutive counters; value i uses counters 2i, 2i+1. */
void miwo_fill_normal_f32(float *out, size_t n, uint64_t seed, float sigma)
{
    for (size_t i = 0; i < n; i++) {
        double u1 = ((double)(splitmix64_at(seed, 2 * i) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        double u2 = (double)(splitmix64_at(seed, 2 * i + 1) >> 11) * (1.0 / 9007199254740992.0);
        out[i] = (float)((double)sigma * sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2));
    }
}

void miwo_fill_normal_f16(uint16_t *out, size_t n, uint64_t seed, float sigma)
{
    for (size_t i = 0; i < n; i++) {
        float v;
        double u1 = ((double)(splitmix64_at(seed, 2 * i) >> 11) + 1.0) * (1.0 / 9007199254740992.0);
        double u2 = (double)(splitmix64_at(seed, 2 * i + 1) >> 11) * (1.0 / 9007199254740992.0);
        v = (float)((double)sigma * sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2));
        out[i] = miwo_float_to_half(v);
    }
}

/* -------------------------------------------------------- element access -- */

static inline size_t idx2(int layout, size_t i, size_t j, size_t ld)
{
    return layout == MIWO_COL ? i + j * ld : i * ld + j;
}

static inline double get_elem(const void *p, int dtype, size_t k)
{
    if (dtype == MIWO_F16) return (double)miwo_half_to_float(((const uint16_t *)p)[k]);
    return (double)((const float *)p)[k];
}

static inline void put_elem(void *p, int dtype, size_t k, double v)
{
    if (dtype == MIWO_F16) ((uint16_t *)p)[k] = miwo_double_to_half(v);
    else ((float *)p)[k] = (float)v;
}

/* ----------------------------------------------------- fragment contract -- */
/* A "tile" here is the whole 16x16 matrix a warp/wavefront holds collectively,
   kept as tile[i*16 + j] = element (row i, column j) in double. */

/* load_a / load_b / load_c  (src/device/cuda/wmma.jl:507-530): read a 16x16
   tile at addr whose leading dimension is `stride` elements in `layout`. */
void miwo_load_tile(double *tile, const void *addr, int dtype, int stride, int layout)
{
    for (int i = 0; i < 16; i++)
        for (int j = 0; j < 16; j++)
            tile[i * 16 + j] = get_elem(addr, dtype, idx2(layout, (size_t)i, (size_t)j, (size_t)stride));
}

/* store_d  (src/device/cuda/wmma.jl:613-632) */
void miwo_store_tile(void *addr, const double *tile, int dtype, int stride, int layout)
{
    for (int i = 0; i < 16; i++)
        for (int j = 0; j < 16; j++)
            put_elem(addr, dtype, idx2(layout, (size_t)i, (size_t)j, (size_t)stride), tile[i * 16 + j]);
}

/* fill_c  (src/device/cuda/wmma.jl:654-667) */
void miwo_fill_tile(double *tile, double value)
{
    for (int i = 0; i < 256; i++) tile[i] = value;
}

/* f.(frag, s): elementwise scale/shift in the fragment's element type
   (src/device/cuda/wmma.jl:703-716; test/device/wmma.jl:182-183). op 0: s*x, 1: s+x */
void miwo_map_tile(double *out, const double *in, int dtype, int op, double s)
{
    for (int i = 0; i < 256; i++) {
        double v = op == 0 ? s * in[i] : s + in[i];
        if (dtype == MIWO_F16) v = (double)miwo_half_to_float(miwo_double_to_half(v));
        else v = (double)(float)v;
        out[i] = v;
    }
}

/* mma  (src/device/cuda/wmma.jl:558-583): D = A*B + C on one 16x16x16 tile,
   exact sum, then one rounding to d_type. */
void miwo_mma_tile(double *d, const double *a, const double *b, const double *c, int d_type)
{
    for (int i = 0; i < 16; i++)
        for (int j = 0; j < 16; j++) {
            double s = 0.0;
            for (int k = 0; k < 16; k++) s += a[i * 16 + k] * b[k * 16 + j];
            s += c[i * 16 + j];
            if (d_type == MIWO_F16) s = (double)miwo_half_to_float(miwo_double_to_half(s));
            else s = (double)(float)s;
            d[i * 16 + j] = s;
        }
}

/* ----------------------------------------------------------------- GEMM --- */

typedef struct {
    int64_t M, N, K;
    int64_t lda, ldb, ldc, ldd;
    int a_layout, b_layout, c_layout, d_layout; /* MIWO_ROW / MIWO_COL */
    int c_type, d_type;                         /* MIWO_F16 / MIWO_F32 */
    double alpha, beta;
    int use_c;                                  /* 0: C is not read (fill_c(0)) */
    int64_t batch, stride_a, stride_b, stride_c, stride_d; /* in elements */
} miwo_gemm_desc;

/* Gather op(A) (M x K) and op(B) (K x N) into row-major-of-A / column-major-of-B
   double panels so the inner product runs over contiguous memory. */
static double *pack_a(const miwo_gemm_desc *g, const uint16_t *A)
{
    double *p = (double *)malloc(sizeof(double) * (size_t)g->M * (size_t)g->K);
    if (!p) return NULL;
    for (int64_t i = 0; i < g->M; i++)
        for (int64_t k = 0; k < g->K; k++)
            p[i * g->K + k] = (double)miwo_half_to_float(A[idx2(g->a_layout, (size_t)i, (size_t)k, (size_t)g->lda)]);
    return p;
}

static double *pack_b(const miwo_gemm_desc *g, const uint16_t *B)
{
    double *p = (double *)malloc(sizeof(double) * (size_t)g->N * (size_t)g->K);
    if (!p) return NULL;
    for (int64_t j = 0; j < g->N; j++)
        for (int64_t k = 0; k < g->K; k++)
            p[j * g->K + k] = (double)miwo_half_to_float(B[idx2(g->b_layout, (size_t)k, (size_t)j, (size_t)g->ldb)]);
    return p;
}

/* Exact-as-double reference: dref[i + j*M] (column-major, ld = M, per batch
   M*N) = alpha * sum_k A[i,k]*B[k,j] + beta*C[i,j], all in double, no rounding
   to d_type.  This is the D_ref of the normalized-error metric. */
int miwo_gemm_f64(const miwo_gemm_desc *g, const uint16_t *A, const uint16_t *B, const void *C, double *dref)
{
    for (int64_t bt = 0; bt < (g->batch > 0 ? g->batch : 1); bt++) {
        const uint16_t *Ab = A + bt * g->stride_a;
        const uint16_t *Bb = B + bt * g->stride_b;
        const char *Cb = (const char *)C + (size_t)(bt * g->stride_c) * (g->c_type == MIWO_F16 ? 2 : 4);
        double *Db = dref + bt * g->M * g->N;
        double *pa = pack_a(g, Ab), *pb = pack_b(g, Bb);
        if (!pa || !pb) { free(pa); free(pb); return -1; }
#pragma omp parallel for schedule(static)
        for (int64_t j = 0; j < g->N; j++) {
            const double *bj = pb + j * g->K;
            for (int64_t i = 0; i < g->M; i++) {
                const double *ai = pa + i * g->K;
                double s = 0.0;
                for (int64_t k = 0; k < g->K; k++) s += ai[k] * bj[k];
                s *= g->alpha;
                if (g->use_c && C)
                    s += g->beta * get_elem(Cb, g->c_type, idx2(g->c_layout, (size_t)i, (size_t)j, (size_t)g->ldc));
                Db[i + j * g->M] = s;
            }
        }
        free(pa);
        free(pb);
    }
    return 0;
}

/* Same product, rounded once to d_type and written to D with its layout/ld:
   what an fp32-accumulating implementation should produce up to summation
   order. */
int miwo_gemm(const miwo_gemm_desc *g, const uint16_t *A, const uint16_t *B, const void *C, void *D)
{
    size_t per = (size_t)g->M * (size_t)g->N;
    int64_t nb = g->batch > 0 ? g->batch : 1;
    double *dref = (double *)malloc(sizeof(double) * per * (size_t)nb);
    if (!dref) return -1;
    int rc = miwo_gemm_f64(g, A, B, C, dref);
    if (rc == 0) {
        for (int64_t bt = 0; bt < nb; bt++) {
            char *Db = (char *)D + (size_t)(bt * g->stride_d) * (g->d_type == MIWO_F16 ? 2 : 4);
            for (int64_t j = 0; j < g->N; j++)
                for (int64_t i = 0; i < g->M; i++)
                    put_elem(Db, g->d_type, idx2(g->d_layout, (size_t)i, (size_t)j, (size_t)g->ldd),
                             dref[(size_t)bt * per + (size_t)(i + j * g->M)]);
        }
    }
    free(dref);
    return rc;
}

/* fp16-accumulate model: the running sum lives in binary16 between K-chunks
   of `kc` elements.  This is the chain "use D of one mma as C of the next"
   (docs/src/device/wmma.md:51-52) with Float16 accumulator fragments, where
   each link is one mma over kc k-values (kc = 16 for the reference's tile):
       acc = half(beta*C)                          (or 0 when use_c == 0)
       for each chunk:  acc = half( acc + alpha * sum_{k in chunk} a*b )  [sum exact]
       D   = acc
   The fragment API scales A by alpha in Float16 before the mma
   (test/device/wmma.jl:223); scaling the chunk sum instead is the same value
   without that extra rounding of A. */
int miwo_gemm_f16acc(const miwo_gemm_desc *g, int64_t kc, const uint16_t *A, const uint16_t *B,
                     const void *C, uint16_t *D)
{
    if (kc <= 0) kc = g->K;
    for (int64_t bt = 0; bt < (g->batch > 0 ? g->batch : 1); bt++) {
        const uint16_t *Ab = A + bt * g->stride_a;
        const uint16_t *Bb = B + bt * g->stride_b;
        const char *Cb = (const char *)C + (size_t)(bt * g->stride_c) * (g->c_type == MIWO_F16 ? 2 : 4);
        uint16_t *Db = D + bt * g->stride_d;
        double *pa = pack_a(g, Ab), *pb = pack_b(g, Bb);
        if (!pa || !pb) { free(pa); free(pb); return -1; }
#pragma omp parallel for schedule(static)
        for (int64_t j = 0; j < g->N; j++) {
            const double *bj = pb + j * g->K;
            for (int64_t i = 0; i < g->M; i++) {
                const double *ai = pa + i * g->K;
                double acc = 0.0;
                if (g->use_c && C) {
                    double c = get_elem(Cb, g->c_type, idx2(g->c_layout, (size_t)i, (size_t)j, (size_t)g->ldc));
                    acc = (double)miwo_half_to_float(miwo_double_to_half(g->beta * c));
                }
                for (int64_t k0 = 0; k0 < g->K; k0 += kc) {
                    int64_t k1 = k0 + kc < g->K ? k0 + kc : g->K;
                    double s = 0.0;
                    for (int64_t k = k0; k < k1; k++) s += ai[k] * bj[k];
                    acc = (double)miwo_half_to_float(miwo_double_to_half(acc + g->alpha * s));
                }
                Db[idx2(g->d_layout, (size_t)i, (size_t)j, (size_t)g->ldd)] = miwo_double_to_half(acc);
            }
        }
        free(pa);
        free(pb);
    }
    return 0;
}

/* max_ij |D - Dref| / max_ij |Dref| over one batch-stacked result.
   D is given in its own dtype/layout, dref column-major ld=M as written by
   miwo_gemm_f64. */
double miwo_normalized_error(const miwo_gemm_desc *g, const void *D, const double *dref)
{
    double maxdiff = 0.0, maxref = 0.0;
    int saw_nan = 0;
    size_t per = (size_t)g->M * (size_t)g->N;
    for (int64_t bt = 0; bt < (g->batch > 0 ? g->batch : 1); bt++) {
        const char *Db = (const char *)D + (size_t)(bt * g->stride_d) * (g->d_type == MIWO_F16 ? 2 : 4);
        for (int64_t j = 0; j < g->N; j++)
            for (int64_t i = 0; i < g->M; i++) {
                double r = dref[(size_t)bt * per + (size_t)(i + j * g->M)];
                double v = get_elem(Db, g->d_type, idx2(g->d_layout, (size_t)i, (size_t)j, (size_t)g->ldd));
                double df = fabs(v - r);
                if (df != df) saw_nan = 1;
                else if (df > maxdiff) maxdiff = df;
                if (fabs(r) > maxref) maxref = fabs(r);
            }
    }
    if (saw_nan) return NAN;
    return maxref > 0.0 ? maxdiff / maxref : maxdiff;
}
