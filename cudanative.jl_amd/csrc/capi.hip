// C ABI of libmiwmma.so (declared in include/miwmma.h): argument validation,
// error reporting, memory / stream / event plumbing and kernel dispatch.
// Nothing here falls back to the CPU: without a usable HIP device every entry
// that needs one returns the HIP error.
#include "../../include/miwmma.h"
#include "kernels.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <ctime>
#include <string>
#include <vector>

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char *what)
{
    // Clear the sticky "last error" so that it is not reported by a later call.
    (void)hipGetLastError();
    return fail((int)e, "%s: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

// Set by miw_init.  Entries that touch the device check it after their arguments: an invalid call
// is reported as such with or without a device, a valid one needs the gfx950 check of miw_init.
std::atomic<bool> g_initialized{false};
#define REQUIRE_INIT(what)                                                                              \
    do {                                                                                                \
        if (!g_initialized.load(std::memory_order_acquire))                                             \
            return fail(MIW_ERR_NOT_INITIALIZED, "%s: miw_init has not been called (it selects the device and " \
                        "checks that it is a gfx950 part)", what);                                      \
    } while (0)

bool valid_layout(int l) { return l == MIW_ROW_MAJOR || l == MIW_COL_MAJOR; }
bool valid_dtype(int t) { return t == MIW_F16 || t == MIW_F32; }
bool valid_as(int a) { return a == MIW_AS_GENERIC || a == MIW_AS_GLOBAL || a == MIW_AS_SHARED; }
size_t dtype_size(int t) { return t == MIW_F16 ? 2 : 4; }

int check_shape(int m, int n, int k)
{
    if (m != 16 || n != 16 || k != 16)
        return fail(MIW_ERR_INVALID_SHAPE, "Invalid shape for WMMA: (M, N, K) = (%d, %d, %d)", m, n, k);
    return 0;
}

hipStream_t as_stream(void *s) { return (hipStream_t)s; }

struct named_kernel {
    std::string name;
    const void *fn;
    int launchable;  // 0: lookup and attribute queries only
};

std::vector<named_kernel> &registry()
{
    static std::vector<named_kernel> r = [] {
        std::vector<named_kernel> v;
        for (int i = 0; i < miw::frag_kernel_count(); i++) {
            const char *n = miw::frag_kernel_name(i);
            v.push_back({n, miw::frag_kernel_symbol(n), 1});
        }
        for (int i = 0; i < miw::tiled_variant_count(); i++)
            v.push_back({std::string("gemm_") + miw::tiled_variant_at(i).name, miw::tiled_kernel_symbol(i), 0});
        return v;
    }();
    return r;
}

// Fill defaults and validate a GEMM descriptor; on success writes kernel params.
int resolve_gemm(const miw_gemm_desc *d, const void *A, const void *B, const void *C, void *D, miw::gemm_params *out,
                 bool *f16acc)
{
    if (!d) return fail(MIW_ERR_NULL_POINTER, "gemm: null descriptor");
    if (!valid_layout(d->a_layout) || !valid_layout(d->b_layout) || !valid_layout(d->c_layout) ||
        !valid_layout(d->d_layout))
        return fail(MIW_ERR_INVALID_LAYOUT, "Invalid layout for WMMA: a=%d b=%d c=%d d=%d", d->a_layout, d->b_layout,
                    d->c_layout, d->d_layout);
    if (!valid_dtype(d->c_type) || !valid_dtype(d->d_type) || !valid_dtype(d->acc_type))
        return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: c=%d d=%d acc=%d", d->c_type, d->d_type,
                    d->acc_type);
    if (d->m <= 0 || d->n <= 0 || d->k <= 0 || d->m % 16 || d->n % 16 || d->k % 16)
        return fail(MIW_ERR_INVALID_SHAPE, "gemm: M, N, K must be positive multiples of 16, got (%lld, %lld, %lld)",
                    (long long)d->m, (long long)d->n, (long long)d->k);
    if (d->m > (1ll << 30) || d->n > (1ll << 30) || d->k > (1ll << 30))
        return fail(MIW_ERR_INVALID_SHAPE, "gemm: dimension too large");
    if (d->batch < 1 || d->batch > 65535)
        return fail(MIW_ERR_INVALID_VALUE, "gemm: batch must be in 1..65535, got %lld", (long long)d->batch);
    *f16acc = d->acc_type == MIW_F16;
    if (*f16acc && (d->c_type != MIW_F16 || d->d_type != MIW_F16))
        return fail(MIW_ERR_INVALID_TYPE, "gemm: Float16 accumulation needs Float16 C and D");
    if (!A || !B || !D || (d->use_c && !C)) return fail(MIW_ERR_NULL_POINTER, "gemm: null operand pointer");

    miw::gemm_params p{};
    p.A = (const _Float16 *)A;
    p.B = (const _Float16 *)B;
    p.C = C;
    p.D = D;
    p.M = d->m; p.N = d->n; p.K = d->k;
    p.a_row = d->a_layout == MIW_ROW_MAJOR;
    p.b_row = d->b_layout == MIW_ROW_MAJOR;
    p.c_row = d->c_layout == MIW_ROW_MAJOR;
    p.d_row = d->d_layout == MIW_ROW_MAJOR;
    const long mina = p.a_row ? p.K : p.M, minb = p.b_row ? p.N : p.K;
    const long minc = p.c_row ? p.N : p.M, mind = p.d_row ? p.N : p.M;
    p.lda = d->lda ? d->lda : mina;
    p.ldb = d->ldb ? d->ldb : minb;
    p.ldc = d->ldc ? d->ldc : minc;
    p.ldd = d->ldd ? d->ldd : mind;
    if (p.lda < mina || p.ldb < minb || p.ldd < mind || (d->use_c && p.ldc < minc))
        return fail(MIW_ERR_INVALID_VALUE, "gemm: leading dimension smaller than the matrix extent");
    p.sa = d->stride_a ? d->stride_a : p.lda * (p.a_row ? p.M : p.K);
    p.sb = d->stride_b ? d->stride_b : p.ldb * (p.b_row ? p.K : p.N);
    p.sc = d->stride_c ? d->stride_c : p.ldc * (p.c_row ? p.M : p.N);
    p.sd = d->stride_d ? d->stride_d : p.ldd * (p.d_row ? p.M : p.N);
    p.batch = d->batch;
    p.use_c = d->use_c != 0;
    p.alpha = d->alpha;
    p.beta = d->beta;
    if (((uintptr_t)A & 1) || ((uintptr_t)B & 1) || ((uintptr_t)D & (dtype_size(d->d_type) - 1)) ||
        (p.use_c && ((uintptr_t)C & (dtype_size(d->c_type) - 1))))
        return fail(MIW_ERR_MISALIGNED, "gemm: operand pointer not aligned to its element type");
    *out = p;
    return 0;
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// Can tiled variant i (0-based) run this problem?
// Where the tile does not divide M or N the edge tiles overlap their neighbours (both compute the
// overlap), which C and D sharing memory (in_place) forbids.
bool tiled_fits(int i, const miw::gemm_params &p, int c_type, int d_type, bool f16acc, int acc_chunk, bool in_place)
{
    const miw::tiled_variant &v = miw::tiled_variant_at(i);
    // In canonical terms bm tiles the contiguous dimension of D.
    const long I = p.d_row ? p.N : p.M, J = p.d_row ? p.M : p.N;
    if (I < v.bm || J < v.bn || p.K < v.bk) return false;  // (K is a multiple of 16: a last slot that 64 does not divide is shifted back and masked)
    if (v.kind == miw::KIND_WAVE128 && p.K < 2 * v.bk) return false;  // (its loop is peeled over the last two slots)
    if ((I % v.bm || J % v.bn) && in_place) return false;
    if (!miw::tiled_supports_layout(i, p) || !miw::tiled_grid_fits(i, p)) return false;
    if (!aligned16(p.A) || !aligned16(p.B) || !aligned16(p.D) || (p.use_c && !aligned16(p.C))) return false;
    if (p.lda % 8 || p.ldb % 8 || p.sa % 8 || p.sb % 8) return false;
    const long cper = 16 / (long)dtype_size(c_type), dper = 16 / (long)dtype_size(d_type);
    if (p.ldd % dper || p.sd % dper) return false;
    if (p.use_c && (p.ldc % cper || p.sc % cper)) return false;
    // 32-bit offsets inside one operand tile
    if (p.lda * 256 >= (1l << 31) || p.ldb * 256 >= (1l << 31)) return false;
    // fp16 accumulation: the pipelined kernels round their MFMA accumulators in place, which needs
    // alpha == 1; the 64-k ping-pong kernels keep the running sum apart and take any alpha
    if (f16acc && (!miw::tiled_supports_f16acc(i) || (p.alpha != 1.0f && v.kind != miw::KIND_PINGPONG64) ||
                   (acc_chunk != 0 && acc_chunk != miw::tiled_f16acc_chunk())))
        return false;
    return true;
}

int g_cu_count = 0;

// Kernels of code objects the caller loaded (miw_module_load): handle -> module it belongs to.
// miw_launch and the attribute queries tell them from the library's own kernels by this table.
std::mutex g_module_mu;
std::unordered_map<void *, void *> g_module_kernels;
std::unordered_map<void *, int> g_modules;

// Do the headers of a code object image stay inside its buffer?  ELF64: the section header table and
// every section with file contents; clang offload bundle: every entry's offset + size, and each
// entry that is an ELF by the same rule.
bool elf_fits(const unsigned char *img, size_t bytes)
{
    if (bytes < 64 || memcmp(img, "\177ELF", 4) != 0 || img[4] != 2 /* ELFCLASS64 */) return false;
    uint64_t shoff;
    uint16_t shentsize, shnum;
    memcpy(&shoff, img + 0x28, 8);
    memcpy(&shentsize, img + 0x3a, 2);
    memcpy(&shnum, img + 0x3c, 2);
    if (shnum == 0) return true;
    if (shentsize < 64 || shoff > bytes || (uint64_t)shnum * shentsize > bytes - shoff) return false;
    for (unsigned i = 0; i < shnum; i++) {
        const unsigned char *sh = img + shoff + (uint64_t)i * shentsize;
        uint32_t type;
        uint64_t off, size;
        memcpy(&type, sh + 4, 4);
        memcpy(&off, sh + 0x18, 8);
        memcpy(&size, sh + 0x20, 8);
        if (type == 8 /* SHT_NOBITS */) continue;
        if (off > bytes || size > bytes - off) return false;
    }
    return true;
}

bool image_fits(const void *image, size_t bytes)
{
    const unsigned char *img = (const unsigned char *)image;
    if (bytes >= 4 && memcmp(img, "\177ELF", 4) == 0) return elf_fits(img, bytes);
    // __CLANG_OFFLOAD_BUNDLE__ (24 bytes), u64 entry count, then per entry: u64 offset, u64 size, u64 id length, id
    if (bytes < 32) return false;
    uint64_t n;
    memcpy(&n, img + 24, 8);
    size_t at = 32;
    for (uint64_t i = 0; i < n; i++) {
        if (at > bytes || bytes - at < 24) return false;
        uint64_t off, size, idlen;
        memcpy(&off, img + at, 8);
        memcpy(&size, img + at + 8, 8);
        memcpy(&idlen, img + at + 16, 8);
        at += 24;
        if (idlen > bytes - at) return false;
        at += idlen;
        if (off > bytes || size > bytes - off) return false;
        if (size >= 4 && memcmp(img + off, "\177ELF", 4) == 0 && !elf_fits(img + off, size)) return false;
    }
    return true;
}

bool is_module_kernel(void *kernel)
{
    std::lock_guard<std::mutex> lock(g_module_mu);
    return g_module_kernels.count(kernel) != 0;
}
int splitk_scratch(void **out);  // address of the current device's static split-K workspace (below)

// Estimated duration of one launch of tiled variant i, in microseconds: a fixed cost per round of
// workgroups, the C and D traffic at what the fabric sustains beside a running K loop, and the K
// loop at the variant's measured pace (a CU that holds a queue of workgroups works through it at
// the queued pace; below that, one workgroup cannot go faster than when it is alone on its CU).
double estimate_us(int i, const miw::gemm_params &p, int c_type, int d_type)
{
    const miw::tiled_variant &v = miw::tiled_variant_at(i);
    const int cus = g_cu_count > 0 ? g_cu_count : 256;
    const long I = p.d_row ? p.N : p.M, J = p.d_row ? p.M : p.N;
    const long tiles = ((I + v.bm - 1) / v.bm) * ((J + v.bn - 1) / v.bn) * p.batch;  // edge tiles overlap their neighbours
    const long per_cu = (tiles + cus - 1) / cus;
    const long rounds = (per_cu + v.occupancy - 1) / v.occupancy;
    const double per_pair = std::max((double)v.us_pair_alone, (double)per_cu * v.us_pair_queued);
    const double cd_bytes = (double)I * (double)J * (double)p.batch * (double)(dtype_size(d_type) + (p.use_c ? dtype_size(c_type) : 0));
    return 4.5 * (double)rounds + cd_bytes / 5.5e6 + (double)((p.K + v.bk - 1) / v.bk) * per_pair;
}

// The one-wavefront-per-SIMD kernel reads C in its epilogue (its accumulators live in AGPRs, out of the
// VALU's reach, so C is not folded into the K loop), and a CU never overlaps one workgroup's epilogue
// with another's loop: measured against the ping-pong kernel of the same tile it is 1 to 5 % ahead on a
// problem without a C operand whose tiles the CUs take in one round, level on longer ones, and 4 to 24 %
// behind whenever C is read.
bool wave128_pays(int i, const miw::gemm_params &p)
{
    const miw::tiled_variant &v = miw::tiled_variant_at(i);
    const int cus = g_cu_count > 0 ? g_cu_count : 256;
    const long I = p.d_row ? p.N : p.M, J = p.d_row ? p.M : p.N;
    const long tiles = ((I + v.bm - 1) / v.bm) * ((J + v.bn - 1) / v.bn) * p.batch;
    return !p.use_c && tiles <= cus;
}

// Tiled variants from large tiles to small, of two kernels for one tile the ping-pong form first.
const std::vector<int> &variant_order()
{
    static const std::vector<int> order = [] {
        std::vector<int> o;
        for (int i = 0; i < miw::tiled_variant_count(); i++) o.push_back(i);
        std::stable_sort(o.begin(), o.end(), [](int a, int b) {
            const miw::tiled_variant &va = miw::tiled_variant_at(a), &vb = miw::tiled_variant_at(b);
            if (va.bm * va.bn != vb.bm * vb.bn) return va.bm * va.bn > vb.bm * vb.bn;
            return va.kind > vb.kind;
        });
        return o;
    }();
    return order;
}

int pick_variant(const miw::gemm_params &p, int c_type, int d_type, bool f16acc, int acc_chunk, bool in_place)
{
    // Candidates in the order of variant_order(); a later candidate replaces an earlier one only when it is estimated 3 % faster.
    const std::vector<int> &order = variant_order();
    int best = -1;
    double best_us = 0.0;
    for (int i : order) {
        if (!tiled_fits(i, p, c_type, d_type, f16acc, acc_chunk, in_place)) continue;
        if (miw::tiled_variant_at(i).kind == miw::KIND_WAVE128 && !wave128_pays(i, p)) continue;
        const double us = estimate_us(i, p, c_type, d_type);
        if (best < 0 || us < 0.97 * best_us) { best = i; best_us = us; }
    }
    if (best >= 0) return best + 1;
    return miw::tiled_variant_count() + 1;  // fragment-op kernel
}

// Resolve the variant (0 = pick) and check that it can run this problem; touches no device.
int check_gemm(const miw_gemm_desc *d, const miw::gemm_params &p, bool f16acc, bool in_place, int *variant_out)
{
    const int nt = miw::tiled_variant_count();
    int variant = d->variant;
    if (variant < 0 || variant > nt + 1) return fail(MIW_ERR_INVALID_VALUE, "gemm: unknown variant %d", variant);
    if (variant == 0) variant = pick_variant(p, d->c_type, d->d_type, f16acc, d->acc_chunk, in_place);
    if (variant == nt + 1) {
        if (f16acc && d->acc_chunk != 0 && d->acc_chunk != 16)
            return fail(MIW_ERR_UNSUPPORTED, "gemm: the fragment-op kernel rounds every 16 k-values (acc_chunk %d asked)",
                        d->acc_chunk);
        if ((p.M / 16) * (p.N / 16) / 4 >= (1l << 31))
            return fail(MIW_ERR_UNSUPPORTED, "gemm: %lld x %lld tiles of 16 x 16 do not fit the launch grid",
                        (long long)(p.M / 16), (long long)(p.N / 16));
    } else if (!tiled_fits(variant - 1, p, d->c_type, d->d_type, f16acc, d->acc_chunk, in_place)) {
        return fail(MIW_ERR_UNSUPPORTED,
                    "gemm: variant %d (%s) needs M and N of at least one tile (whole tiles when C and D share memory), "
                    "K of at least 64, 16-byte aligned operands and leading "
                    "dimensions, and a tile count that fits the launch grid%s",
                    variant, miw::tiled_variant_at(variant - 1).name,
                    f16acc ? ", alpha == 1 (the 64-k ping-pong kernels take any alpha), its own acc_chunk, and accumulators that fit in VGPRs" : "");
    }
    *variant_out = variant;
    return 0;
}

int launch_gemm(int variant, const miw::gemm_params &p, int c_type, int d_type, bool f16acc, hipStream_t s)
{
    if (variant == miw::tiled_variant_count() + 1) HIP_TRY(miw::launch_gemm_fragops(p, c_type, d_type, f16acc, s));
    else HIP_TRY(miw::launch_gemm_tiled(variant - 1, p, c_type, d_type, f16acc, s));
    return 0;
}

// ---- ragged problems ----
// The tiled kernels take any M and N of at least one tile: where the tile does not divide an
// extent the last tile is shifted back to end at the edge and overlaps its neighbour (unless C
// and D share memory: then only whole tiles).  Beyond that a problem may be cut into parts, each
// a GEMM of its own on a block of D (same leading dimensions and batch strides, offset
// pointers), launched one after the other on the caller's stream:
//   * a body of whole large tiles plus a bottom strip and a right strip, each planned again
//     (4160 rows: sixteen rows of 256 x 256 tiles and a strip of 64 x 64 tiles instead of
//     seventeen rows of large tiles, i.e. two rounds over the CUs).
// A cut is made only where the estimate says it pays.
struct gemm_part {
    int variant;  // 1-based; tiled_variant_count() + 1: the fragment-op kernel
    int c_type;
    miw::gemm_params p;
    long m0, n0, k0;  // where the part sits in the caller's problem
};

// The fragment-op kernels.  Up to 64 k-values with C laid out as D: the short-K kernel, which moves C
// and D at copy speed.  Otherwise every wavefront walks K alone, 16 k-values per step, straight
// from global memory.
double estimate_fragops_us(const miw::gemm_params &p, int c_type, int d_type)
{
    const double mn = (double)p.M * (double)p.N * (double)p.batch;
    const double cd_bytes = mn * (double)(dtype_size(d_type) + (p.use_c ? dtype_size(c_type) : 0));
    const double flop = 2.0 * mn * (double)p.K;
    if (p.K <= 64 && (!p.use_c || p.c_row == p.d_row)) return std::max(6.5, 3.0 + std::max(cd_bytes / 5.5e6, flop / 75e6));
    const int split = miw::fragops_ksplit(p, false);  // few tiles, long K: several wavefronts share a tile's K loop
    const double walk = 0.45 * (double)(p.K / 16) / split + (split > 1 ? 2.0 : 0.0);
    return 5.0 + std::max(walk, std::max(flop / 45e6, cd_bytes / 2.0e6));
}

miw::gemm_params sub_block(const miw::gemm_params &p, int c_type, int d_type, long m0, long m, long n0, long n)
{
    miw::gemm_params q = p;
    q.A = p.A + m0 * (p.a_row ? p.lda : 1);
    q.B = p.B + n0 * (p.b_row ? 1 : p.ldb);
    if (p.C) q.C = (const char *)p.C + (long)dtype_size(c_type) * (p.c_row ? m0 * p.ldc + n0 : n0 * p.ldc + m0);
    q.D = (char *)p.D + (long)dtype_size(d_type) * (p.d_row ? m0 * p.ldd + n0 : n0 * p.ldd + m0);
    q.M = m;
    q.N = n;
    return q;
}

struct gemm_planner {
    int d_type;
    bool in_place;  // C and D share memory
    int nt = miw::tiled_variant_count();

    double single(const miw::gemm_params &p, int c_type, long m0, long n0, long k0, std::vector<gemm_part> *out) const
    {
        const int v = pick_variant(p, c_type, d_type, false, 0, in_place);
        if (out) out->push_back(gemm_part{v, c_type, p, m0, n0, k0});
        return v == nt + 1 ? estimate_fragops_us(p, c_type, d_type) : estimate_us(v - 1, p, c_type, d_type);
    }

    // Appends the parts of p to *out (when given) and returns the estimated duration.
    double plan(const miw::gemm_params &p, int c_type, long m0, long n0, long k0, int depth, std::vector<gemm_part> *out) const
    {
        std::vector<gemm_part> best;
        double best_us = single(p, c_type, m0, n0, k0, &best);
        auto offer = [&](std::vector<gemm_part> &cand, double us) {
            if (us < 0.97 * best_us) { best_us = us; best.swap(cand); }
        };
        if (depth < 4) {
            if (p.K >= 64) {
                // whole large tiles, then what they leave at the bottom and on the right; a strip
                // is widened backwards to 64 rows (columns), over the body, where that is allowed
                for (int i : variant_order()) {
                    const miw::tiled_variant &v = miw::tiled_variant_at(i);
                    const long tm = p.d_row ? v.bn : v.bm, tn = p.d_row ? v.bm : v.bn;
                    const long mb = p.M / tm * tm, nb = p.N / tn * tn;
                    if (mb == 0 || nb == 0 || (mb == p.M && nb == p.N)) continue;
                    const miw::gemm_params body = sub_block(p, c_type, d_type, 0, mb, 0, nb);
                    if (!tiled_fits(i, body, c_type, d_type, false, 0, in_place)) continue;
                    if (v.kind == miw::KIND_WAVE128 && !wave128_pays(i, body)) continue;
                    std::vector<gemm_part> cand;
                    cand.push_back(gemm_part{i + 1, c_type, body, m0, n0, k0});
                    double us = estimate_us(i, body, c_type, d_type);
                    if (us >= best_us) continue;
                    const long sm = in_place || p.M < 64 ? mb : std::min(mb, p.M - 64);
                    const long sn = in_place || p.N < 64 ? nb : std::min(nb, p.N - 64);
                    if (mb != p.M)
                        us += plan(sub_block(p, c_type, d_type, sm, p.M - sm, 0, p.N), c_type, m0 + sm, n0, k0, depth + 1, &cand);
                    if (nb != p.N)
                        us += plan(sub_block(p, c_type, d_type, 0, mb, sn, p.N - sn), c_type, m0, n0 + sn, k0, depth + 1, &cand);
                    offer(cand, us);
                }
            }
        }
        if (out) out->insert(out->end(), best.begin(), best.end());
        return best_us;
    }
};

bool ranges_overlap(const void *a, size_t na, const void *b, size_t nb)
{
    const uintptr_t x = (uintptr_t)a, y = (uintptr_t)b;
    return x < y + nb && y < x + na;
}

// The launches of one miw_gemm call, validated.  A forced variant and fp16 accumulation (whose
// rounding points must not depend on where a cut falls) run as one launch.
int plan_gemm(const miw_gemm_desc *d, const miw::gemm_params &p, bool f16acc, bool in_place, std::vector<gemm_part> *parts)
{
    // The host thread's last plan is kept: a loop over one problem and one set of buffers plans once.
    struct cached_plan {
        miw_gemm_desc desc;
        const void *A, *B, *C;
        void *D;
        bool in_place, valid = false;
        std::vector<gemm_part> parts;
    };
    static thread_local cached_plan last;
    if (last.valid && memcmp(&last.desc, d, sizeof *d) == 0 && last.A == p.A && last.B == p.B && last.C == p.C && last.D == p.D &&
        last.in_place == in_place) {
        *parts = last.parts;
        return 0;
    }
    parts->clear();
    if (d->variant != 0 || f16acc) {
        int variant = 0;
        if (int rc = check_gemm(d, p, f16acc, in_place, &variant)) return rc;
        parts->push_back(gemm_part{variant, d->c_type, p, 0, 0, 0});
    } else {
        gemm_planner pl{d->d_type, in_place};
        pl.plan(p, d->c_type, 0, 0, 0, 0, parts);
        for (const gemm_part &part : *parts)
            if (part.variant == pl.nt + 1 && (part.p.M / 16) * (part.p.N / 16) / 4 >= (1l << 31))
                return fail(MIW_ERR_UNSUPPORTED, "gemm: %lld x %lld tiles of 16 x 16 do not fit the launch grid",
                            (long long)(part.p.M / 16), (long long)(part.p.N / 16));
    }
    last.desc = *d;
    last.A = p.A; last.B = p.B; last.C = p.C; last.D = p.D;
    last.in_place = in_place;
    last.parts = *parts;
    last.valid = true;
    return 0;
}

bool c_shares_d(const miw_gemm_desc *d, const miw::gemm_params &p)
{
    if (!p.use_c) return false;
    const size_t nc = (size_t)((p.batch - 1) * p.sc + p.ldc * (p.c_row ? p.M : p.N)) * dtype_size(d->c_type);
    const size_t nd = (size_t)((p.batch - 1) * p.sd + p.ldd * (p.d_row ? p.M : p.N)) * dtype_size(d->d_type);
    return ranges_overlap(p.C, nc, p.D, nd);
}

int launch_parts(const miw_gemm_desc *d, const std::vector<gemm_part> &parts, bool f16acc, hipStream_t s)
{
    for (const gemm_part &part : parts)
        if (int rc = launch_gemm(part.variant, part.p, part.c_type, d->d_type, f16acc, s)) return rc;
    return 0;
}

}  // namespace

extern "C" {

const char *miw_last_error(void) { return g_err; }

#ifndef MIW_BUILD_ID
#define MIW_BUILD_ID "unknown"
#endif
// The id follows a marker in the binary, so that a build script or test harness can read it from the
// file without loading the library into its own process.
static const char g_build_id[] = "miw-build-id:" MIW_BUILD_ID;
const char *miw_build_id(void) { return g_build_id + 13; }

int miw_init(int device)
{
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return fail(MIW_ERR_INVALID_VALUE, "init: device %d out of range (count %d)", device, n);
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(MIW_ERR_UNSUPPORTED, "init: kernels are built for gfx950, device is %s", prop.gcnArchName);
    g_cu_count = prop.multiProcessorCount;
    void *scratch = nullptr;
    if (int rc = splitk_scratch(&scratch)) return rc;  // once per device, with that device current
    g_initialized.store(true, std::memory_order_release);
    g_err[0] = 0;
    return 0;
}

int miw_device_info_get(miw_device_info *out)
{
    if (!out) return fail(MIW_ERR_NULL_POINTER, "device_info: null output");
    REQUIRE_INIT("device_info");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", prop.name);
    snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
    out->cu_count = prop.multiProcessorCount;
    out->wave_size = prop.warpSize;
    out->clock_mhz = prop.clockRate / 1000;
    out->mem_clock_mhz = prop.memoryClockRate / 1000;
    out->mem_bus_bits = prop.memoryBusWidth;
    out->l2_bytes = prop.l2CacheSize;
    out->max_threads_per_block = prop.maxThreadsPerBlock;
    out->lds_per_block = prop.sharedMemPerBlock;
    out->hbm_bytes = prop.totalGlobalMem;
    out->peak_f16_tflops = (double)out->cu_count * 4.0 * 1024.0 * (double)out->clock_mhz * 1e6 / 1e12;
    return 0;
}

int miw_malloc(void **out, size_t bytes)
{
    if (!out) return fail(MIW_ERR_NULL_POINTER, "malloc: null output");
    *out = nullptr;
    if (bytes == 0) return 0;
    REQUIRE_INIT("malloc");
    HIP_TRY(hipMalloc(out, bytes));
    return 0;
}

int miw_free(void *p)
{
    if (!p) return 0;
    REQUIRE_INIT("free");
    HIP_TRY(hipFree(p));
    return 0;
}

int miw_memcpy_h2d(void *dst, const void *src, size_t bytes)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(MIW_ERR_NULL_POINTER, "memcpy_h2d: null pointer");
    REQUIRE_INIT("memcpy_h2d");
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return 0;
}

int miw_memcpy_d2h(void *dst, const void *src, size_t bytes)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(MIW_ERR_NULL_POINTER, "memcpy_d2h: null pointer");
    REQUIRE_INIT("memcpy_d2h");
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return 0;
}

int miw_memcpy_d2d(void *dst, const void *src, size_t bytes)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(MIW_ERR_NULL_POINTER, "memcpy_d2d: null pointer");
    REQUIRE_INIT("memcpy_d2d");
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
    return 0;
}

int miw_memset(void *dst, int byte, size_t bytes)
{
    if (bytes == 0) return 0;
    if (!dst) return fail(MIW_ERR_NULL_POINTER, "memset: null pointer");
    REQUIRE_INIT("memset");
    HIP_TRY(hipMemset(dst, byte, bytes));
    return 0;
}

int miw_stream_create(void **out)
{
    if (!out) return fail(MIW_ERR_NULL_POINTER, "stream_create: null output");
    REQUIRE_INIT("stream_create");
    hipStream_t s;
    HIP_TRY(hipStreamCreate(&s));  // default priority only
    *out = (void *)s;
    return 0;
}

int miw_stream_destroy(void *stream)
{
    if (!stream) return 0;
    HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return 0;
}

int miw_sync(void *stream)
{
    REQUIRE_INIT("sync");
    if (stream) HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    else HIP_TRY(hipDeviceSynchronize());
    return 0;
}

int miw_event_create(void **out)
{
    if (!out) return fail(MIW_ERR_NULL_POINTER, "event_create: null output");
    REQUIRE_INIT("event_create");
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e));
    *out = (void *)e;
    return 0;
}

int miw_event_destroy(void *event)
{
    if (!event) return 0;
    HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int miw_event_record(void *event, void *stream)
{
    if (!event) return fail(MIW_ERR_NULL_POINTER, "event_record: null event");
    REQUIRE_INIT("event_record");
    HIP_TRY(hipEventRecord((hipEvent_t)event, as_stream(stream)));
    return 0;
}

int miw_event_synchronize(void *event)
{
    if (!event) return fail(MIW_ERR_NULL_POINTER, "event_synchronize: null event");
    HIP_TRY(hipEventSynchronize((hipEvent_t)event));
    return 0;
}

int miw_event_elapsed_ms(float *ms, void *start, void *stop)
{
    if (!ms || !start || !stop) return fail(MIW_ERR_NULL_POINTER, "event_elapsed_ms: null argument");
    HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

// ------------------------------------------------------------- fragments ---

int miw_frag_elems_per_lane(int use, int dtype)
{
    if (use < MIW_MATRIX_A || use > MIW_ACCUMULATOR) return fail(MIW_ERR_INVALID_VALUE, "Invalid fragment use %d", use);
    if (!valid_dtype(dtype)) return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: %d", dtype);
    if (use != MIW_ACCUMULATOR && dtype != MIW_F16)
        return fail(MIW_ERR_INVALID_TYPE, "Invalid type Float32 for matrix %s", use == MIW_MATRIX_A ? "a" : "b");
    return 4;
}

size_t miw_frag_image_bytes(int use, int dtype)
{
    int n = miw_frag_elems_per_lane(use, dtype);
    return n > 0 ? (size_t)n * 64 * dtype_size(dtype) : 0;
}

int miw_frag_load(int use, int dtype, int layout, int addr_space, int m, int n, int k, const void *addr,
                  int64_t stride, void *frag, void *stream)
{
    if (int rc = check_shape(m, n, k)) return rc;
    if (!valid_as(addr_space)) return fail(MIW_ERR_INVALID_AS, "Invalid address space for WMMA: %d", addr_space);
    if (!valid_layout(layout)) return fail(MIW_ERR_INVALID_LAYOUT, "Invalid layout for WMMA: %d", layout);
    if (int ne = miw_frag_elems_per_lane(use, dtype); ne < 0) return ne;
    if (!addr || !frag) return fail(MIW_ERR_NULL_POINTER, "frag_load: null pointer");
    if (stride < 16) return fail(MIW_ERR_INVALID_VALUE, "frag_load: stride %lld smaller than the tile", (long long)stride);
    if ((uintptr_t)addr & (dtype_size(dtype) - 1)) return fail(MIW_ERR_MISALIGNED, "frag_load: misaligned address");
    REQUIRE_INIT("frag_load");
    HIP_TRY(miw::launch_frag_load(use, dtype, layout == MIW_ROW_MAJOR, addr_space, addr, (long)stride, frag,
                                  as_stream(stream)));
    return 0;
}

int miw_frag_store(int dtype, int layout, int addr_space, int m, int n, int k, void *addr, const void *frag,
                   int64_t stride, void *stream)
{
    if (int rc = check_shape(m, n, k)) return rc;
    if (!valid_as(addr_space)) return fail(MIW_ERR_INVALID_AS, "Invalid address space for WMMA: %d", addr_space);
    if (!valid_layout(layout)) return fail(MIW_ERR_INVALID_LAYOUT, "Invalid layout for WMMA: %d", layout);
    if (!valid_dtype(dtype)) return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: %d", dtype);
    if (!addr || !frag) return fail(MIW_ERR_NULL_POINTER, "frag_store: null pointer");
    if (stride < 16) return fail(MIW_ERR_INVALID_VALUE, "frag_store: stride %lld smaller than the tile", (long long)stride);
    if ((uintptr_t)addr & (dtype_size(dtype) - 1)) return fail(MIW_ERR_MISALIGNED, "frag_store: misaligned address");
    REQUIRE_INIT("frag_store");
    HIP_TRY(miw::launch_frag_store(dtype, layout == MIW_ROW_MAJOR, addr_space, addr, frag, (long)stride,
                                   as_stream(stream)));
    return 0;
}

int miw_frag_fill(int dtype, float value, void *frag, void *stream)
{
    if (!valid_dtype(dtype)) return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: %d", dtype);
    if (!frag) return fail(MIW_ERR_NULL_POINTER, "frag_fill: null pointer");
    REQUIRE_INIT("frag_fill");
    HIP_TRY(miw::launch_frag_fill(dtype, value, frag, as_stream(stream)));
    return 0;
}

int miw_frag_map(int dtype, int op, float scalar, const void *in, void *out, size_t n_elems, void *stream)
{
    if (!valid_dtype(dtype)) return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: %d", dtype);
    if (op != MIW_OP_MUL && op != MIW_OP_ADD) return fail(MIW_ERR_INVALID_VALUE, "frag_map: unknown operator %d", op);
    if (n_elems && (!in || !out)) return fail(MIW_ERR_NULL_POINTER, "frag_map: null pointer");
    REQUIRE_INIT("frag_map");
    HIP_TRY(miw::launch_frag_map(dtype, op, scalar, in, out, n_elems, as_stream(stream)));
    return 0;
}

int miw_frag_mma(int a_layout, int b_layout, int c_type, int d_type, const void *a_frag, const void *b_frag,
                 const void *c_frag, void *d_frag, void *stream)
{
    if (!valid_layout(a_layout) || !valid_layout(b_layout))
        return fail(MIW_ERR_INVALID_LAYOUT, "Invalid layout for WMMA: a=%d b=%d", a_layout, b_layout);
    if (!valid_dtype(c_type) || !valid_dtype(d_type))
        return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: c=%d d=%d", c_type, d_type);
    if (!a_frag || !b_frag || !c_frag || !d_frag) return fail(MIW_ERR_NULL_POINTER, "frag_mma: null pointer");
    REQUIRE_INIT("frag_mma");
    HIP_TRY(miw::launch_frag_mma(c_type, d_type, a_frag, b_frag, c_frag, d_frag, as_stream(stream)));
    return 0;
}

int miw_wmma_mac(const miw_mac_desc *d, const void *A, const void *B, const void *C, void *D, void *stream)
{
    if (!d) return fail(MIW_ERR_NULL_POINTER, "wmma_mac: null descriptor");
    if (int rc = check_shape(d->m, d->n, d->k)) return rc;
    if (!valid_as(d->addr_space)) return fail(MIW_ERR_INVALID_AS, "Invalid address space for WMMA: %d", d->addr_space);
    if (!valid_layout(d->a_layout) || !valid_layout(d->b_layout) || !valid_layout(d->c_layout) ||
        !valid_layout(d->d_layout))
        return fail(MIW_ERR_INVALID_LAYOUT, "Invalid layout for WMMA: a=%d b=%d c=%d d=%d", d->a_layout, d->b_layout,
                    d->c_layout, d->d_layout);
    if (!valid_dtype(d->c_type) || !valid_dtype(d->d_type))
        return fail(MIW_ERR_INVALID_TYPE, "Invalid element type for WMMA: c=%d d=%d", d->c_type, d->d_type);
    if (!A || !B || !D || (d->use_c && !C)) return fail(MIW_ERR_NULL_POINTER, "wmma_mac: null operand pointer");
    const long lda = d->lda ? d->lda : 16, ldb = d->ldb ? d->ldb : 16, ldc = d->ldc ? d->ldc : 16,
               ldd = d->ldd ? d->ldd : 16;
    if (lda < 16 || ldb < 16 || ldc < 16 || ldd < 16)
        return fail(MIW_ERR_INVALID_VALUE, "wmma_mac: leading dimension smaller than the tile");
    if (((uintptr_t)A & 1) || ((uintptr_t)B & 1) || ((uintptr_t)D & (dtype_size(d->d_type) - 1)) ||
        (d->use_c && ((uintptr_t)C & (dtype_size(d->c_type) - 1))))
        return fail(MIW_ERR_MISALIGNED, "wmma_mac: operand pointer not aligned to its element type");
    REQUIRE_INIT("wmma_mac");
    HIP_TRY(miw::launch_wmma_mac(d->c_type, d->d_type, A, B, C, D, lda, ldb, ldc, ldd, d->a_layout == MIW_ROW_MAJOR,
                                 d->b_layout == MIW_ROW_MAJOR, d->c_layout == MIW_ROW_MAJOR,
                                 d->d_layout == MIW_ROW_MAJOR, d->use_c != 0, d->addr_space == MIW_AS_SHARED, d->alpha,
                                 d->beta, as_stream(stream)));
    return 0;
}

// ------------------------------------------------------------------ GEMM ---

int miw_gemm_variant_count(void) { return miw::tiled_variant_count() + 1; }

int miw_gemm_variant_info_get(int variant, miw_gemm_variant_info *out)
{
    if (!out) return fail(MIW_ERR_NULL_POINTER, "gemm_variant_info: null output");
    const int nt = miw::tiled_variant_count();
    if (variant < 1 || variant > nt + 1) return fail(MIW_ERR_INVALID_VALUE, "gemm_variant_info: unknown variant %d", variant);
    memset(out, 0, sizeof(*out));
    if (variant == nt + 1) {
        snprintf(out->name, sizeof(out->name), "fragment_ops");
        out->block_m = 16; out->block_n = 16; out->block_k = 16;
        out->waves_m = 1; out->waves_n = 1; out->stages = 1; out->lds_bytes = 0; out->fragment_ops = 1;
        out->f16_accumulate = 1;
        return 0;
    }
    const miw::tiled_variant &v = miw::tiled_variant_at(variant - 1);
    snprintf(out->name, sizeof(out->name), "%s", v.name);
    out->block_m = v.bm; out->block_n = v.bn; out->block_k = v.bk;
    out->waves_m = v.wm; out->waves_n = v.wn; out->stages = v.stages; out->lds_bytes = v.lds_bytes;
    out->f16_accumulate = miw::tiled_supports_f16acc(variant - 1) ? 1 : 0;
    out->pingpong = v.kind == miw::KIND_PINGPONG32 || v.kind == miw::KIND_PINGPONG64 ? 1 : v.kind == miw::KIND_WAVE128 ? 2 : 0;
    return 0;
}

int miw_gemm_variant_supports(const miw_gemm_desc *desc, int variant, int *supported)
{
    if (!supported) return fail(MIW_ERR_NULL_POINTER, "gemm_variant_supports: null output");
    const int nt = miw::tiled_variant_count();
    if (variant < 1 || variant > nt + 1) return fail(MIW_ERR_INVALID_VALUE, "gemm_variant_supports: unknown variant %d", variant);
    miw::gemm_params p;
    bool f16acc;
    static char dummy alignas(16);
    if (int rc = resolve_gemm(desc, &dummy, &dummy, &dummy, &dummy, &p, &f16acc)) return rc;
    if (variant == nt + 1) *supported = !(f16acc && desc->acc_chunk != 0 && desc->acc_chunk != 16);
    else *supported = tiled_fits(variant - 1, p, desc->c_type, desc->d_type, f16acc, desc->acc_chunk, false) ? 1 : 0;
    return 0;
}

int miw_gemm_pick_variant(const miw_gemm_desc *desc, int *variant)
{
    if (!variant) return fail(MIW_ERR_NULL_POINTER, "gemm_pick_variant: null output");
    miw::gemm_params p;
    bool f16acc;
    // Alignment of real pointers cannot be known here: assume aligned operands.
    static char dummy alignas(16);
    if (int rc = resolve_gemm(desc, &dummy, &dummy, &dummy, &dummy, &p, &f16acc)) return rc;
    *variant = pick_variant(p, desc->c_type, desc->d_type, f16acc, desc->acc_chunk, false);
    return 0;
}

int miw_gemm_plan(const miw_gemm_desc *desc, int in_place, miw_gemm_part *out, int capacity, int *count)
{
    if (!count || (capacity > 0 && !out)) return fail(MIW_ERR_NULL_POINTER, "gemm_plan: null output");
    miw::gemm_params p;
    bool f16acc;
    // Alignment of real pointers cannot be known here: assume 16-byte aligned operands far apart.
    char *const base = (char *)(uintptr_t)0x100000000ull;
    if (int rc = resolve_gemm(desc, base, base + (1ull << 40), base + (2ull << 40), base + (in_place ? 2ull << 40 : 3ull << 40), &p, &f16acc))
        return rc;
    std::vector<gemm_part> parts;
    if (int rc = plan_gemm(desc, p, f16acc, in_place != 0, &parts)) return rc;
    *count = (int)parts.size();
    for (int i = 0; i < (int)parts.size() && i < capacity; i++) {
        const gemm_part &g = parts[(size_t)i];
        out[i].variant = g.variant;
        out[i].reserved = 0;
        out[i].m0 = g.m0; out[i].n0 = g.n0; out[i].k0 = g.k0;
        out[i].m = g.p.M; out[i].n = g.p.N; out[i].k = g.p.K;
    }
    return 0;
}

int miw_gemm_acc_chunk(const miw_gemm_desc *desc, int *acc_chunk)
{
    if (!acc_chunk) return fail(MIW_ERR_NULL_POINTER, "gemm_acc_chunk: null output");
    int v = 0;
    if (int rc = miw_gemm_pick_variant(desc, &v)) return rc;
    if (desc->variant != 0) v = desc->variant;
    *acc_chunk = v == miw::tiled_variant_count() + 1 ? 16 : miw::tiled_f16acc_chunk();
    return 0;
}

int miw_gemm_resolve(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, const void *D, int *variant, int *acc_chunk)
{
    miw::gemm_params p;
    bool f16acc;
    if (int rc = resolve_gemm(desc, A, B, C, const_cast<void *>(D), &p, &f16acc)) return rc;
    std::vector<gemm_part> parts;
    if (int rc = plan_gemm(desc, p, f16acc, c_shares_d(desc, p), &parts)) return rc;
    const int v = parts.empty() ? 0 : parts[0].variant;
    if (variant) *variant = v;
    if (acc_chunk) *acc_chunk = !f16acc ? 0 : v == miw::tiled_variant_count() + 1 ? 16 : miw::tiled_f16acc_chunk();
    return 0;
}

int miw_gemm(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, void *stream)
{
    miw::gemm_params p;
    bool f16acc;
    if (int rc = resolve_gemm(desc, A, B, C, D, &p, &f16acc)) return rc;
    std::vector<gemm_part> parts;
    if (int rc = plan_gemm(desc, p, f16acc, c_shares_d(desc, p), &parts)) return rc;
    REQUIRE_INIT("gemm");
    return launch_parts(desc, parts, f16acc, as_stream(stream));
}

// ---- split-K ----

}  // extern "C"

namespace {

// Static workspace of miw_gemm_splitk_static: the Float32 partial products of one split-K GEMM.
// Every GPU the library runs on holds its own copy from the time the library's code is loaded
// there until the process ends.  In host code the array's name is not a device address: host code
// uses the address hipGetSymbolAddress returned for the current device.
constexpr size_t SPLITK_STATIC_BYTES = 32u << 20;
static __device__ __align__(256) unsigned char g_splitk_scratch[SPLITK_STATIC_BYTES];

constexpr int MAX_DEVICES = 64;
std::atomic<void *> g_splitk_scratch_ptr[MAX_DEVICES];

// Address of the current device's copy of the static workspace (looked up once per device).
int splitk_scratch(void **out)
{
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(MIW_ERR_UNSUPPORTED, "gemm_splitk_static: device index %d out of range", dev);
    void *ptr = g_splitk_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_splitk_scratch)));
        if (!ptr) return fail(MIW_ERR_UNSUPPORTED, "gemm_splitk_static: no address for the static workspace");
        g_splitk_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return 0;
}

struct splitk_plan {
    miw::gemm_params full;   // the caller's problem
    miw::gemm_params slice;  // first pass: `splits` independent products of K / splits k-values each
    int variant;             // tiled variant of the first pass (1-based)
    int splits;
    size_t bytes;            // workspace the first pass fills
};

// The first pass of a split-K GEMM as a strided-batched problem over the K slices.
miw::gemm_params splitk_slices(const miw::gemm_params &p, int splits, void *ws)
{
    miw::gemm_params q = p;
    const long klen = p.K / splits;
    q.K = klen;
    q.C = nullptr; q.use_c = 0; q.alpha = 1.0f; q.beta = 0.0f;
    q.D = ws;
    q.c_row = q.d_row = p.d_row;
    q.ldc = q.ldd = p.d_row ? p.N : p.M;
    q.sc = q.sd = p.M * p.N;
    q.sa = klen * (p.a_row ? 1 : p.lda);
    q.sb = klen * (p.b_row ? p.ldb : 1);
    q.batch = splits;
    return q;
}

int plan_splitk(const miw_gemm_desc *d, const void *A, const void *B, const void *C, void *D, int splits, splitk_plan *out,
                size_t workspace_cap = SIZE_MAX)
{
    bool f16acc;
    miw::gemm_params p;
    if (int rc = resolve_gemm(d, A, B, C, D, &p, &f16acc)) return rc;
    if (f16acc) return fail(MIW_ERR_UNSUPPORTED, "gemm_splitk: Float32 accumulation only (slices are added in Float32)");
    if (p.batch != 1) return fail(MIW_ERR_UNSUPPORTED, "gemm_splitk: one problem per call (batch %lld asked)", (long long)p.batch);
    if (d->variant != 0) return fail(MIW_ERR_INVALID_VALUE, "gemm_splitk: the variant is chosen per slice; desc.variant must be 0");
    if (splits < 0 || splits > 256) return fail(MIW_ERR_INVALID_VALUE, "gemm_splitk: splits must be 0 (choose) or 1..256, got %d", splits);
    const int nt = miw::tiled_variant_count();
    const bool in_place = c_shares_d(d, p);
    static char dummy alignas(16);
    // Variant and estimated duration of s slices (s = 1: the plain launch); false when no tiled kernel fits.
    auto try_splits = [&](int s, int *variant, double *us) {
        if (p.K % (64l * s)) return false;
        if (s == 1) {
            const int v = pick_variant(p, d->c_type, d->d_type, false, 0, in_place);
            if (v == nt + 1) return false;
            *variant = v;
            *us = estimate_us(v - 1, p, d->c_type, d->d_type);
            return true;
        }
        const miw::gemm_params q = splitk_slices(p, s, &dummy);
        const int v = pick_variant(q, MIW_F32, MIW_F32, false, 0, false);
        if (v == nt + 1) return false;
        *variant = v;
        // second kernel: launch, a quarter of a microsecond per slice (each thread adds its slices
        // in order), and the slices, C and D at the same pace as above
        const double mn = (double)p.M * (double)p.N;
        *us = estimate_us(v - 1, q, MIW_F32, MIW_F32) + 6.0 + 0.25 * s +
              mn * (4.0 * s + (double)dtype_size(d->d_type) + (p.use_c ? (double)dtype_size(d->c_type) : 0.0)) / 5.5e6;
        return true;
    };
    int variant = 0;
    double us = 0.0;
    if (splits == 0) {
        // The slice count with the shortest estimated duration, among 1 (no second pass) and the
        // counts up to 64 that leave every slice two LDS slots' worth of K or more.
        double best_us = 0.0;
        for (int s = 1; s <= 64 && (s == 1 || p.K / s >= 128); s++) {
            int v;
            // a caller with a bounded workspace is offered only the counts that fit in it
            if (s > 1 && (size_t)s * (size_t)p.M * (size_t)p.N * sizeof(float) > workspace_cap) break;
            if (!try_splits(s, &v, &us)) continue;
            if (splits == 0 || us < 0.97 * best_us) { splits = s; variant = v; best_us = us; }
        }
    } else if (!try_splits(splits, &variant, &us)) {
        splits = 0;
    }
    if (splits == 0)
        return fail(MIW_ERR_UNSUPPORTED,
                    "gemm_splitk: needs K divisible by 64 * splits, M and N of at least one LDS tile (64), "
                    "16-byte aligned operands and leading dimensions");
    out->full = p;
    out->splits = splits;
    out->variant = variant;
    // one slice is the plain launch: no workspace, no second kernel
    out->bytes = splits == 1 ? 0 : (size_t)splits * (size_t)p.M * (size_t)p.N * sizeof(float);
    out->slice = splitk_slices(p, splits, nullptr);
    return 0;
}

int run_splitk(const miw_gemm_desc *d, splitk_plan &plan, void *ws, hipStream_t s)
{
    if (plan.splits == 1) {
        if (!tiled_fits(plan.variant - 1, plan.full, d->c_type, d->d_type, false, 0, c_shares_d(d, plan.full)))
            return fail(MIW_ERR_MISALIGNED, "gemm_splitk: operands must be 16-byte aligned");
        HIP_TRY(miw::launch_gemm_tiled(plan.variant - 1, plan.full, d->c_type, d->d_type, false, s));
        return 0;
    }
    plan.slice.D = ws;
    // the slices are checked against the real operand pointers (plan_splitk assumed aligned ones)
    if (!tiled_fits(plan.variant - 1, plan.slice, MIW_F32, MIW_F32, false, 0, false))
        return fail(MIW_ERR_MISALIGNED, "gemm_splitk: operands and workspace must be 16-byte aligned");
    HIP_TRY(miw::launch_gemm_tiled(plan.variant - 1, plan.slice, MIW_F32, MIW_F32, false, s));
    HIP_TRY(miw::launch_splitk_reduce(plan.full, d->c_type, d->d_type, plan.splits, (const float *)ws, s));
    return 0;
}

}  // namespace

extern "C" {

int miw_gemm_splitk_workspace(const miw_gemm_desc *desc, int splits, int *splits_out, size_t *bytes)
{
    if (!bytes) return fail(MIW_ERR_NULL_POINTER, "gemm_splitk_workspace: null output");
    // Alignment of real pointers cannot be known here: assume 16-byte aligned operands far apart.
    char *const base = (char *)(uintptr_t)0x100000000ull;
    splitk_plan plan;
    if (int rc = plan_splitk(desc, base, base + (1ull << 40), base + (2ull << 40), base + (3ull << 40), splits, &plan)) return rc;
    if (splits_out) *splits_out = plan.splits;
    *bytes = plan.bytes;
    return 0;
}

int miw_gemm_splitk(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, int splits,
                    void *workspace, size_t workspace_bytes, void *stream)
{
    splitk_plan plan;
    if (int rc = plan_splitk(desc, A, B, C, D, splits, &plan)) return rc;
    if (!workspace && plan.bytes) return fail(MIW_ERR_NULL_POINTER, "gemm_splitk: null workspace");
    if (workspace_bytes < plan.bytes)
        return fail(MIW_ERR_INVALID_VALUE, "gemm_splitk: workspace of %zu bytes, %d slices need %zu", workspace_bytes,
                    plan.splits, plan.bytes);
    REQUIRE_INIT("gemm_splitk");
    return run_splitk(desc, plan, workspace, as_stream(stream));
}

int miw_gemm_splitk_static(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, int splits,
                           void *stream)
{
    splitk_plan plan;
    if (int rc = plan_splitk(desc, A, B, C, D, splits, &plan, SPLITK_STATIC_BYTES)) return rc;
    if (plan.bytes > SPLITK_STATIC_BYTES)
        return fail(MIW_ERR_UNSUPPORTED,
                    "gemm_splitk_static: %d slices of %lld x %lld Float32 need %zu bytes, the static workspace holds %zu; "
                    "use miw_gemm_splitk with a workspace of your own",
                    plan.splits, (long long)plan.full.M, (long long)plan.full.N, plan.bytes, SPLITK_STATIC_BYTES);
    REQUIRE_INIT("gemm_splitk_static");
    void *ws = nullptr;
    if (int rc = splitk_scratch(&ws)) return rc;
    return run_splitk(desc, plan, ws, as_stream(stream));
}

size_t miw_gemm_splitk_static_capacity(void) { return SPLITK_STATIC_BYTES; }

int miw_gemm_splitk_static_plan(const miw_gemm_desc *desc, int splits, int *splits_out, size_t *bytes)
{
    if (!bytes) return fail(MIW_ERR_NULL_POINTER, "gemm_splitk_static_plan: null output");
    char *const base = (char *)(uintptr_t)0x100000000ull;
    splitk_plan plan;
    if (int rc = plan_splitk(desc, base, base + (1ull << 40), base + (2ull << 40), base + (3ull << 40), splits, &plan, SPLITK_STATIC_BYTES))
        return rc;
    if (plan.bytes > SPLITK_STATIC_BYTES)
        return fail(MIW_ERR_UNSUPPORTED, "gemm_splitk_static: %d slices need %zu bytes, the static workspace holds %zu", plan.splits,
                    plan.bytes, SPLITK_STATIC_BYTES);
    if (splits_out) *splits_out = plan.splits;
    *bytes = plan.bytes;
    return 0;
}

int miw_mem_info(size_t *free_bytes, size_t *total_bytes)
{
    if (!free_bytes || !total_bytes) return fail(MIW_ERR_NULL_POINTER, "mem_info: null output");
    REQUIRE_INIT("mem_info");
    HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
    return 0;
}

int miw_gemm_bench(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, void *stream,
                   int warmup, int iters, float *ms_each)
{
    if (iters < 1 || iters > 100000 || warmup < 0 || !ms_each)
        return fail(MIW_ERR_INVALID_VALUE, "gemm_bench: bad warmup/iters/output (at most 100000 timed launches per call)");
    miw::gemm_params p;
    bool f16acc;
    if (int rc = resolve_gemm(desc, A, B, C, D, &p, &f16acc)) return rc;
    std::vector<gemm_part> parts;
    if (int rc = plan_gemm(desc, p, f16acc, c_shares_d(desc, p), &parts)) return rc;
    REQUIRE_INIT("gemm_bench");
    hipStream_t s = as_stream(stream);
    for (int i = 0; i < warmup; i++)
        if (int rc = launch_parts(desc, parts, f16acc, s)) return rc;
    std::vector<hipEvent_t> ev((size_t)iters + 1, nullptr);
    int rc = 0;
    hipError_t he = hipSuccess;
    for (auto &e : ev)
        if (he == hipSuccess) he = hipEventCreate(&e);
    if (he == hipSuccess) he = hipEventRecord(ev[0], s);
    for (int i = 0; i < iters && rc == 0 && he == hipSuccess; i++) {
        rc = launch_parts(desc, parts, f16acc, s);
        if (rc == 0) he = hipEventRecord(ev[(size_t)i + 1], s);
    }
    if (rc == 0 && he == hipSuccess) he = hipEventSynchronize(ev[(size_t)iters]);
    for (int i = 0; i < iters && rc == 0 && he == hipSuccess; i++)
        he = hipEventElapsedTime(&ms_each[i], ev[(size_t)i], ev[(size_t)i + 1]);
    for (auto &e : ev)
        if (e) (void)hipEventDestroy(e);
    if (rc) return rc;
    if (he != hipSuccess) return hip_fail(he, "gemm_bench");
    return 0;
}

int miw_launch_overhead_probe(int iters, int threads, float *cpu_us, float *gpu_us)
{
    if (!cpu_us || !gpu_us || iters < 1 || threads < 1 || threads > 1024)
        return fail(MIW_ERR_INVALID_VALUE, "launch_overhead_probe: bad arguments");
    REQUIRE_INIT("launch_overhead_probe");
    float *buf = nullptr;
    HIP_TRY(hipMalloc((void **)&buf, 4));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t he = hipEventCreate(&e0);
    if (he == hipSuccess) he = hipEventCreate(&e1);
    for (int i = 0; i < iters && he == hipSuccess; ++i) {
        timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        he = hipEventRecord(e0, nullptr);
        if (he == hipSuccess) he = miw::launch_dummy_store(buf, threads, nullptr);
        if (he == hipSuccess) he = hipEventRecord(e1, nullptr);
        if (he == hipSuccess) he = hipEventSynchronize(e1);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        float ms = 0.f;
        if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
        cpu_us[i] = (float)((t1.tv_sec - t0.tv_sec) * 1e6 + (t1.tv_nsec - t0.tv_nsec) * 1e-3);
        gpu_us[i] = ms * 1e3f;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(buf);
    if (he != hipSuccess) return hip_fail(he, "launch_overhead_probe");
    return 0;
}

int miw_mfma_power_probe(int iters, int random_operands, double *tflops, double *shader_mhz, void *stream)
{
    if (!tflops || !shader_mhz || iters < 1 || iters > 10000000)
        return fail(MIW_ERR_INVALID_VALUE, "mfma_power_probe: bad arguments (iters in 1..10000000)");
    REQUIRE_INIT("mfma_power_probe");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    int wall_khz = 0;
    HIP_TRY(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, dev));
    const int blocks = prop.multiProcessorCount;  // one 8-wavefront workgroup per CU
    float *sink = nullptr;
    long long *ticks = nullptr;
    HIP_TRY(hipMalloc((void **)&sink, 4));
    hipError_t he = hipMalloc((void **)&ticks, sizeof(long long) * 2 * blocks);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipStream_t s = as_stream(stream);
    const float scale = random_operands ? 1.0f : 0.0f;
    if (he == hipSuccess) he = hipEventCreate(&e0);
    if (he == hipSuccess) he = hipEventCreate(&e1);
    if (he == hipSuccess) he = miw::launch_mfma_power(blocks, iters / 4 + 1, scale, sink, ticks, s);  // warm-up
    if (he == hipSuccess) he = hipEventRecord(e0, s);
    if (he == hipSuccess) he = miw::launch_mfma_power(blocks, iters, scale, sink, ticks, s);
    if (he == hipSuccess) he = hipEventRecord(e1, s);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    float ms = 0.f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    std::vector<long long> host(2 * (size_t)blocks);
    if (he == hipSuccess) he = hipMemcpy(host.data(), ticks, sizeof(long long) * host.size(), hipMemcpyDeviceToHost);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    (void)hipFree(ticks);
    if (he != hipSuccess) return hip_fail(he, "mfma_power_probe");
    // per wavefront and iteration: 4 sets x 16 MFMAs of 16*16*32*2 flop
    const double flop = (double)blocks * 8.0 * (double)iters * 64.0 * 16384.0;
    *tflops = flop / ((double)ms * 1e-3) / 1e12;
    double mhz = 0.0;
    for (int b = 0; b < blocks; b++)
        mhz += (double)host[2 * b] / ((double)host[2 * b + 1] / ((double)wall_khz * 1e3)) / 1e6;
    *shader_mhz = mhz / blocks;
    return 0;
}

int miw_mfma_peak_probe(int iters, double *tflops, void *stream)
{
    if (!tflops || iters < 1 || iters > 10000000)
        return fail(MIW_ERR_INVALID_VALUE, "mfma_peak_probe: bad arguments (iters in 1..10000000)");
    REQUIRE_INIT("mfma_peak_probe");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev));
    const int blocks = prop.multiProcessorCount * 2;  // 8 wavefronts per CU
    float *sink = nullptr;
    HIP_TRY(hipMalloc((void **)&sink, 4));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipStream_t s = as_stream(stream);
    hipError_t he = hipEventCreate(&e0);
    if (he == hipSuccess) he = hipEventCreate(&e1);
    if (he == hipSuccess) he = miw::launch_mfma_peak(blocks, 16, sink, s);  // warm-up
    if (he == hipSuccess) he = hipEventRecord(e0, s);
    if (he == hipSuccess) he = miw::launch_mfma_peak(blocks, iters, sink, s);
    if (he == hipSuccess) he = hipEventRecord(e1, s);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    float ms = 0.f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (he != hipSuccess) return hip_fail(he, "mfma_peak_probe");
    // per wavefront and iteration: 4 x 8 MFMAs of 16*16*32*2 flop
    const double flop = (double)blocks * 4.0 * (double)iters * 32.0 * 16384.0;
    *tflops = flop / ((double)ms * 1e-3) / 1e12;
    return 0;
}

int miw_copy_probe(void *dst, const void *src, size_t bytes, void *stream)
{
    if (!dst || !src) return fail(MIW_ERR_NULL_POINTER, "copy_probe: null pointer");
    if (((uintptr_t)dst | (uintptr_t)src | bytes) & 15) return fail(MIW_ERR_MISALIGNED, "copy_probe: needs 16-byte multiples");
    REQUIRE_INIT("copy_probe");
    HIP_TRY(miw::launch_copy(dst, src, bytes, as_stream(stream)));
    return 0;
}

// -------------------------------------------------------- generic launch ---

int miw_kernel_count(void) { return (int)registry().size(); }

int miw_kernel_name(int index, char *buf, size_t buflen)
{
    if (!buf || buflen == 0) return fail(MIW_ERR_NULL_POINTER, "kernel_name: null buffer");
    if (index < 0 || index >= (int)registry().size()) return fail(MIW_ERR_INVALID_VALUE, "kernel_name: index %d out of range", index);
    snprintf(buf, buflen, "%s", registry()[(size_t)index].name.c_str());
    return 0;
}

int miw_kernel_lookup(const char *name, void **kernel)
{
    if (!name || !kernel) return fail(MIW_ERR_NULL_POINTER, "kernel_lookup: null argument");
    for (auto &k : registry())
        if (k.name == name) {
            *kernel = (void *)k.fn;
            return 0;
        }
    *kernel = nullptr;
    return fail(MIW_ERR_NOT_FOUND, "kernel_lookup: no kernel named '%s'", name);
}

int miw_kernel_attributes_get(void *kernel, miw_kernel_attributes *out)
{
    if (!kernel || !out) return fail(MIW_ERR_NULL_POINTER, "kernel_attributes: null argument");
    REQUIRE_INIT("kernel_attributes");
    if (is_module_kernel(kernel)) {
        hipFunction_t f = (hipFunction_t)kernel;
        int regs = 0, threads = 0, lds = 0, local = 0, cst = 0;
        HIP_TRY(hipFuncGetAttribute(&regs, HIP_FUNC_ATTRIBUTE_NUM_REGS, f));
        HIP_TRY(hipFuncGetAttribute(&threads, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, f));
        HIP_TRY(hipFuncGetAttribute(&lds, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, f));
        HIP_TRY(hipFuncGetAttribute(&local, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, f));
        HIP_TRY(hipFuncGetAttribute(&cst, HIP_FUNC_ATTRIBUTE_CONST_SIZE_BYTES, f));
        out->num_regs = regs;
        out->max_threads_per_block = threads;
        out->static_shared_bytes = (size_t)lds;
        out->local_bytes = (size_t)local;
        out->const_bytes = (size_t)cst;
        return 0;
    }
    hipFuncAttributes a;
    HIP_TRY(hipFuncGetAttributes(&a, kernel));
    out->num_regs = a.numRegs;
    out->max_threads_per_block = a.maxThreadsPerBlock;
    out->static_shared_bytes = a.sharedSizeBytes;
    out->local_bytes = a.localSizeBytes;
    out->const_bytes = a.constSizeBytes;
    return 0;
}

int miw_kernel_occupancy(void *kernel, size_t dynamic_shmem, int *min_grid, int *block)
{
    if (!kernel || !min_grid || !block) return fail(MIW_ERR_NULL_POINTER, "kernel_occupancy: null argument");
    REQUIRE_INIT("kernel_occupancy");
    if (is_module_kernel(kernel)) {
        HIP_TRY(hipModuleOccupancyMaxPotentialBlockSize(min_grid, block, (hipFunction_t)kernel, dynamic_shmem, 0));
        return 0;
    }
    HIP_TRY(hipOccupancyMaxPotentialBlockSize(min_grid, block, kernel, dynamic_shmem, 0));
    return 0;
}

int miw_module_load(const void *image, size_t bytes, void **module)
{
    if (!image || !module) return fail(MIW_ERR_NULL_POINTER, "module_load: null argument");
    *module = nullptr;
    // an ELF code object or a clang offload bundle that holds one
    static const char bundle_magic[] = "__CLANG_OFFLOAD_BUNDLE__";
    const bool elf = bytes >= 64 && memcmp(image, "\177ELF", 4) == 0;
    const bool bundle = bytes >= sizeof(bundle_magic) - 1 && memcmp(image, bundle_magic, sizeof(bundle_magic) - 1) == 0;
    if (!elf && !bundle)
        return fail(MIW_ERR_INVALID_VALUE, "module_load: %zu bytes that are neither an ELF code object nor an offload bundle", bytes);
    // hipModuleLoadData takes no size: it reads as far as the image's own headers say.  Check that they stay inside the buffer.
    if (!image_fits(image, bytes))
        return fail(MIW_ERR_INVALID_VALUE, "module_load: the image's headers describe more than the %zu bytes given (truncated file?)", bytes);
    REQUIRE_INIT("module_load");
    hipModule_t m = nullptr;
    HIP_TRY(hipModuleLoadData(&m, image));
    std::lock_guard<std::mutex> lock(g_module_mu);
    g_modules[(void *)m] = 1;
    *module = (void *)m;
    return 0;
}

int miw_module_get_kernel(void *module, const char *name, void **kernel)
{
    if (!module || !name || !kernel) return fail(MIW_ERR_NULL_POINTER, "module_get_kernel: null argument");
    *kernel = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_module_mu);
        if (!g_modules.count(module)) return fail(MIW_ERR_NOT_FOUND, "module_get_kernel: not a module of miw_module_load");
    }
    REQUIRE_INIT("module_get_kernel");
    hipFunction_t f = nullptr;
    hipError_t e = hipModuleGetFunction(&f, (hipModule_t)module, name);
    if (e == hipErrorNotFound) {
        (void)hipGetLastError();  // the runtime keeps the failure as its "last error": clear it, or the next launch would report it
        return fail(MIW_ERR_NOT_FOUND, "module_get_kernel: no kernel named '%s' in the module", name);
    }
    HIP_TRY(e);
    std::lock_guard<std::mutex> lock(g_module_mu);
    g_module_kernels[(void *)f] = module;
    *kernel = (void *)f;
    return 0;
}

int miw_module_unload(void *module)
{
    if (!module) return 0;
    {
        std::lock_guard<std::mutex> lock(g_module_mu);
        if (!g_modules.count(module)) return fail(MIW_ERR_NOT_FOUND, "module_unload: not a module of miw_module_load");
        for (auto it = g_module_kernels.begin(); it != g_module_kernels.end();)
            it = it->second == module ? g_module_kernels.erase(it) : std::next(it);
        g_modules.erase(module);
    }
    REQUIRE_INIT("module_unload");
    HIP_TRY(hipModuleUnload((hipModule_t)module));
    return 0;
}

int miw_launch(void *kernel, const unsigned grid[3], const unsigned block[3], unsigned shmem, void *stream, void **args)
{
    if (!kernel || !grid || !block) return fail(MIW_ERR_NULL_POINTER, "launch: null argument");
    if (is_module_kernel(kernel)) {
        const unsigned long nthreads = (unsigned long)block[0] * block[1] * block[2];
        if (nthreads == 0 || (unsigned long)grid[0] * grid[1] * grid[2] == 0)
            return fail(MIW_ERR_INVALID_VALUE, "launch: empty grid or block");
        if (shmem > 64u * 1024u)
            return fail(MIW_ERR_UNSUPPORTED, "launch: kernels of loaded code objects get at most 64 KiB of dynamic LDS (%u asked)", shmem);
        REQUIRE_INIT("launch");
        hipFunction_t f = (hipFunction_t)kernel;
        int max_threads = 0;
        HIP_TRY(hipFuncGetAttribute(&max_threads, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, f));
        if (nthreads > (unsigned long)max_threads)
            return fail((int)hipErrorInvalidConfiguration, "launch: %lu threads per block exceed the kernel's maximum %d",
                        nthreads, max_threads);
        HIP_TRY(hipModuleLaunchKernel(f, grid[0], grid[1], grid[2], block[0], block[1], block[2], shmem, as_stream(stream), args,
                                      nullptr));
        return 0;
    }
    bool known = false;
    for (auto &k : registry()) known = known || (void *)k.fn == kernel;
    if (!known) return fail(MIW_ERR_NOT_FOUND, "launch: not a kernel of this library");
    for (auto &k : registry())
        if ((void *)k.fn == kernel && k.launchable == 0)
            return fail(MIW_ERR_UNSUPPORTED,
                        "launch: '%s' takes a private argument block, a fixed workgroup size and up to 160 KiB of dynamic "
                        "LDS; it can be looked up and queried, and is launched through miw_gemm",
                        k.name.c_str());
    const unsigned long threads = (unsigned long)block[0] * block[1] * block[2];
    if (threads == 0 || (unsigned long)grid[0] * grid[1] * grid[2] == 0)
        return fail(MIW_ERR_INVALID_VALUE, "launch: empty grid or block");
    REQUIRE_INIT("launch");
    hipFuncAttributes a;
    HIP_TRY(hipFuncGetAttributes(&a, kernel));
    if (threads > (unsigned long)a.maxThreadsPerBlock)
        return fail((int)hipErrorInvalidConfiguration, "launch: %lu threads per block exceed the kernel's maximum %d", threads,
                    a.maxThreadsPerBlock);
    HIP_TRY(hipLaunchKernel(kernel, dim3(grid[0], grid[1], grid[2]), dim3(block[0], block[1], block[2]), args, shmem,
                            as_stream(stream)));
    return 0;
}

}  // extern "C"
