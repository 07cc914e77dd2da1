// oracle.cpp — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A single-threaded CPU restatement of catgrad's `NdArrayBackend`
// (reference: catgrad/src/interpreter/backend/ndarray.rs) behind the same C ABI
// as the HIP library (include/catgrad_hip.h), so that every parity test and the
// model driver can run unchanged against either.  Only tests, the smoke check
// and the benchmark's cpu_baseline leg may load this library; the product
// never does.
//
// Each function cites the reference lines it follows.  The arithmetic of the
// reference lives in two crates that are not vendored in the reference tree:
// `ndarray 0.17.1` and `matrixmultiply 0.3.10` (Cargo.lock).  Their published
// algorithms are restated here:
//   * sgemm  — matrixmultiply's Goto/BLIS loop nest: NC=1024, KC=256, MC=64,
//              8x8 FMA micro-kernel, C = (first K block ? 0 : C) + AB.
//   * sum    — ndarray `sum_axis`: 8-way unrolled fold on contiguous lanes,
//              sequential fold otherwise.
// What pins this file (see tests/test_oracle_*.py): the reference's own known
// answers (ndarray.rs:831-1022, tests/test_interpreter*.rs, helpers_tests.rs),
// numpy closed forms for integer/shape/index ops (bit-exact) and float64
// evaluation for f32 math.  PARITY UNPINNED at bit level (only to 1e-3 / 1e-4
// relative): the exact f32 accumulation order of sgemm and sum_axis and the last
// ulp of libm's expf/logf/sinf/cosf/powf — those could only be pinned by
// building the Rust reference, for which this image has no toolchain.  For the
// f16 / bf16 / fp8 dtypes (restated from CandleBackend's CPU path, further down):
// PARITY UNPINNED for Candle's accumulation in sum / matmul and for fp8 values
// beyond 464 (saturation per the float8 crate's documentation).
//
// Deliberate, documented differences from NdArrayBackend:
//   * element-wise operands of different shape are rejected ("Shape mismatch in
//     operation") as the trait demands (backend/mod.rs:22) and CandleBackend
//     does (candle.rs:1271-1297); ndarray's `+` would co-broadcast.
//   * results are always standard layout; ndarray's `x + y` keeps x's strides.
//   * panics become status codes.

#include "../include/catgrad_hip.h"

#include <immintrin.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <numeric>
#include <string>
#include <vector>

namespace {

thread_local std::string g_err;

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

// ArcArray's shared allocation (ndarray.rs:19-20).
// Large blocks are kept and handed out again instead of going back to the operating system: a model-sized run
// allocates and drops gigabytes per op (every op of the reference makes a fresh array), and first-touch page faults
// on fresh mappings cost several times the arithmetic.  Values are unaffected (vectors still zero-fill).
struct BlockCache {
    std::mutex mu;
    std::multimap<size_t, void *> free_;
    size_t cached = 0;
    static constexpr size_t kMin = 1u << 20, kMaxCached = (size_t)24 << 30;
    void *take(size_t bytes) {
        if (bytes >= kMin) {
            std::lock_guard<std::mutex> lk(mu);
            auto it = free_.lower_bound(bytes);
            if (it != free_.end() && it->first <= bytes + bytes / 4) {
                void *p = it->second;
                cached -= it->first;
                free_.erase(it);
                return p;
            }
        }
        void *p = malloc(bytes);
        if (!p) throw std::bad_alloc();
        return p;
    }
    void give(void *p, size_t bytes) {
        if (bytes >= kMin) {
            std::lock_guard<std::mutex> lk(mu);
            if (cached + bytes <= kMaxCached) {
                free_.emplace(bytes, p);
                cached += bytes;
                return;
            }
        }
        free(p);
    }
};
inline BlockCache &block_cache() {
    static BlockCache *c = new BlockCache; // never destroyed: vectors with static lifetime may outlive any order
    return *c;
}
template <class T> struct CachedAlloc {
    using value_type = T;
    CachedAlloc() = default;
    template <class U> CachedAlloc(const CachedAlloc<U> &) {}
    T *allocate(size_t n) { return static_cast<T *>(block_cache().take(n * sizeof(T))); }
    void deallocate(T *p, size_t n) { block_cache().give(p, n * sizeof(T)); }
    template <class U> bool operator==(const CachedAlloc<U> &) const { return true; }
    template <class U> bool operator!=(const CachedAlloc<U> &) const { return false; }
};
template <class T> using Vec = std::vector<T, CachedAlloc<T>>;

struct Storage {
    std::atomic<long> rc{1};
    Vec<uint32_t> data; // f32 and u32 are both stored as 4-byte words
};

} // namespace

struct cg_backend {
    std::atomic<size_t> live_bytes{0};
};

struct cg_tensor {
    std::atomic<long> rc{1};
    Storage *st = nullptr;
    cg_dtype dt = CG_F32;
    int rank = 0;
    size_t dims[CG_MAX_RANK] = {0};
    ptrdiff_t strides[CG_MAX_RANK] = {0};
    size_t offset = 0;
};

namespace {

size_t numel(const cg_tensor *t) {
    size_t n = 1;
    for (int i = 0; i < t->rank; i++) n *= t->dims[i];
    return n;
}

void set_contiguous_strides(cg_tensor *t) {
    ptrdiff_t s = 1;
    for (int i = t->rank - 1; i >= 0; i--) {
        t->strides[i] = s;
        s *= (ptrdiff_t)t->dims[i];
    }
}

// ndarray `is_standard_layout`: row-major contiguous, ignoring axes of length <= 1.
bool is_standard(const cg_tensor *t) {
    if (numel(t) == 0) return true;
    ptrdiff_t s = 1;
    for (int i = t->rank - 1; i >= 0; i--) {
        if (t->dims[i] != 1 && t->strides[i] != s) return false;
        s *= (ptrdiff_t)t->dims[i];
    }
    return true;
}

cg_tensor *new_tensor(cg_dtype dt, const size_t *dims, int rank) {
    cg_tensor *t = new cg_tensor;
    t->dt = dt;
    t->rank = rank;
    for (int i = 0; i < rank; i++) t->dims[i] = dims[i];
    set_contiguous_strides(t);
    t->st = new Storage;
    t->st->data.resize(numel(t));
    return t;
}

// A freshly computed (standard-layout, unshared) result of a 16-bit float dtype: every word rounded to the dtype.
uint32_t round_to(cg_dtype dt, uint32_t u);
void round_tensor(cg_tensor *t) {
    if (t->dt != CG_F16 && t->dt != CG_BF16 && t->dt != CG_F8) return;
    for (uint32_t &w : t->st->data) w = round_to(t->dt, w);
}

void release(cg_tensor *t) {
    if (!t) return;
    if (t->rc.fetch_sub(1) == 1) {
        if (t->st && t->st->rc.fetch_sub(1) == 1) delete t->st;
        delete t;
    }
}

struct Consume { // releases the consumed reference of an argument on scope exit
    cg_tensor *t;
    explicit Consume(cg_tensor *t) : t(t) {}
    ~Consume() { release(t); }
};

// View sharing t's storage.
cg_tensor *view_of(const cg_tensor *t) {
    cg_tensor *v = new cg_tensor;
    v->st = t->st;
    v->st->rc.fetch_add(1);
    v->dt = t->dt;
    v->rank = t->rank;
    memcpy(v->dims, t->dims, sizeof v->dims);
    memcpy(v->strides, t->strides, sizeof v->strides);
    v->offset = t->offset;
    return v;
}

// `TaggedArrayD::unwrap_{f32,u32}` = `ArcArray::into_owned` (ndarray.rs:24-36): when the
// allocation is shared the WHOLE allocation is cloned (strides kept); when unique it is
// taken as is.  The caller's consumed reference is the one being unwrapped, so "unique"
// means: this handle has one reference and the storage has one handle.
cg_tensor *unwrap_owned(cg_tensor *t) {
    if (t->rc.load() == 1 && t->st->rc.load() == 1) {
        t->rc.fetch_add(1); // result aliases the argument; Consume drops the other ref
        return t;
    }
    cg_tensor *o = new cg_tensor;
    o->st = new Storage;
    o->st->data = t->st->data; // deep copy of the full allocation
    o->dt = t->dt;
    o->rank = t->rank;
    memcpy(o->dims, t->dims, sizeof o->dims);
    memcpy(o->strides, t->strides, sizeof o->strides);
    o->offset = t->offset;
    return o;
}

// Logical (row-major) iteration of a strided view into a dense vector
// (ndarray `iter()` / `to_owned()` of a non-contiguous view).
template <typename T> void gather_logical(const cg_tensor *t, T *dst) {
    size_t n = numel(t);
    if (n == 0) return;
    const T *base = reinterpret_cast<const T *>(t->st->data.data()) + t->offset;
    if (is_standard(t)) {
        memcpy(dst, base, n * sizeof(T));
        return;
    }
    int r = t->rank;
    if (r == 0) {
        dst[0] = base[0];
        return;
    }
    // Same values, fewer cache misses (this is a checker, not a timing model of the reference): an outermost
    // stride-0 axis is gathered once and repeated, and a view whose unit stride sits on the second-to-last axis (a
    // transposed matrix, or a stack of them) is gathered in 32 x 32 tiles.
    if (r >= 2 && t->dims[0] > 1 && t->strides[0] == 0) {
        cg_tensor sub;
        sub.st = t->st;
        sub.dt = t->dt;
        sub.offset = t->offset;
        sub.rank = r - 1;
        for (int d = 1; d < r; d++) {
            sub.dims[d - 1] = t->dims[d];
            sub.strides[d - 1] = t->strides[d];
        }
        const size_t slab = n / t->dims[0];
        gather_logical<T>(&sub, dst);
        sub.st = nullptr;
        for (size_t i = 1; i < t->dims[0]; i++) memcpy(dst + i * slab, dst, slab * sizeof(T));
        return;
    }
    if (r >= 2 && t->strides[r - 2] == 1 && t->strides[r - 1] != 1 && t->dims[r - 1] >= 32 && t->dims[r - 2] >= 32) {
        const size_t R = t->dims[r - 2], Cn = t->dims[r - 1], mats = n / (R * Cn);
        const ptrdiff_t cs = t->strides[r - 1];
        size_t midx[CG_MAX_RANK] = {0};
        ptrdiff_t moff = 0;
        for (size_t m = 0; m < mats; m++) {
            const T *src = base + moff;
            T *out = dst + m * R * Cn;
            for (size_t i0 = 0; i0 < R; i0 += 32)
                for (size_t j0 = 0; j0 < Cn; j0 += 32) {
                    const size_t i1 = std::min(R, i0 + 32), j1 = std::min(Cn, j0 + 32);
                    for (size_t j = j0; j < j1; j++) {
                        const T *col = src + (ptrdiff_t)j * cs;
                        for (size_t i = i0; i < i1; i++) out[i * Cn + j] = col[i];
                    }
                }
            for (int d = r - 3; d >= 0; d--) { // odometer over the matrices
                midx[d]++;
                moff += t->strides[d];
                if (midx[d] < t->dims[d]) break;
                moff -= (ptrdiff_t)midx[d] * t->strides[d];
                midx[d] = 0;
            }
        }
        return;
    }
    size_t idx[CG_MAX_RANK] = {0};
    size_t inner = t->dims[r - 1];
    ptrdiff_t is = t->strides[r - 1];
    size_t rows = n / inner;
    ptrdiff_t off = 0;
    for (size_t row = 0; row < rows; row++) {
        const T *p = base + off;
        if (is == 1)
            memcpy(dst, p, inner * sizeof(T));
        else
            for (size_t i = 0; i < inner; i++) dst[i] = p[(ptrdiff_t)i * is];
        dst += inner;
        for (int d = r - 2; d >= 0; d--) { // odometer over the outer axes
            idx[d]++;
            off += t->strides[d];
            if (idx[d] < t->dims[d]) break;
            off -= (ptrdiff_t)idx[d] * t->strides[d];
            idx[d] = 0;
        }
    }
}

template <typename T> Vec<T> dense(const cg_tensor *t) {
    Vec<T> v(numel(t));
    gather_logical<T>(t, v.data());
    return v;
}

template <typename T> T *data_of(cg_tensor *t) { return reinterpret_cast<T *>(t->st->data.data()) + t->offset; }

bool same_shape(const cg_tensor *a, const cg_tensor *b) {
    if (a->rank != b->rank) return false;
    for (int i = 0; i < a->rank; i++)
        if (a->dims[i] != b->dims[i]) return false;
    return true;
}

bool supported(cg_dtype d) { return d == CG_F32 || d == CG_U32 || d == CG_F16 || d == CG_BF16 || d == CG_F8; }

// ---- the 16-bit float dtypes ------------------------------------------------------------------
// NdArrayBackend has `todo!()` for them (ndarray.rs:7-9, 98-120); what is restated here is the model of
// the `half` crate that CandleBackend's CPU path builds on (candle.rs:530-551, 575-599, 605-718): a value
// is widened to f32 exactly, the op runs in f32, the result is rounded to the dtype (nearest, ties to even;
// overflow to infinity; NaN stays NaN).  Sums and matrix products accumulate in f32 and round once: Candle's
// own accumulation order and width are NOT restated (PARITY UNPINNED for those two; conversions and
// element-wise results are pinned by numpy's float16 and by the closed form of bfloat16 rounding).
// Tensors of these dtypes hold 32-bit words whose values are exactly representable in the dtype.
bool isf(cg_dtype d) { return d == CG_F32 || d == CG_F16 || d == CG_BF16 || d == CG_F8; }
bool is_half(cg_dtype d) { return d == CG_F16 || d == CG_BF16; }

uint32_t bits_of(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
float float_of(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t f32_to_bf16_bits(uint32_t u) {
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); // NaN, made quiet
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// IEEE binary32 -> binary16, round to nearest even, written out on the bit patterns.
uint16_t f32_to_f16_bits(uint32_t u) {
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7E00u;  // NaN
    if (a >= 0x477FF000u) return sign | 0x7C00u; // >= 65520 rounds to infinity (and infinity itself)
    if (a >= 0x38800000u) {                      // normal in binary16: >= 2^-14
        uint32_t h = (((a >> 23) - 112u) << 10) | ((a & 0x7FFFFFu) >> 13);
        const uint32_t rest = a & 0x1FFFu;
        if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) h++; // a carry runs into the exponent, as it should
        return sign | (uint16_t)h;
    }
    // subnormal in binary16: the value in units of 2^-24, rounded to nearest even
    const float units = float_of(a) * 16777216.0f; // exact: a power of two
    return sign | (uint16_t)(uint32_t)nearbyintf(units);
}

uint32_t f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0x1F) return sign | 0x7F800000u | (m << 13);
    if (e != 0) return sign | ((e + 112u) << 23) | (m << 13);
    return sign | bits_of((float)m * (1.0f / 16777216.0f)); // subnormal or zero: m * 2^-24, exact in f32
}

// ---- fp8 --------------------------------------------------------------------------------------
// `Dtype::F8` is `float8::F8E4M3` (candle.rs:9, 382; crate float8 0.7.0 per Cargo.lock, not vendored): sign,
// 4 exponent bits (bias 7), 3 mantissa bits, no infinities, 0x7F / 0xFF the only NaNs, largest finite value
// 448 = 0x7E, subnormals m * 2^-9.  The crate documents its conversions as those of CUDA's cuda_fp8.hpp with
// saturation to the largest finite value (`__NV_SATFINITE`): round to nearest even; anything beyond 448,
// infinities included, becomes +-448; NaN stays NaN.  Element-wise ops are f32 ops on the widened values,
// narrowed again (the crate's operator impls), which is the same model as for the 16-bit dtypes above.
// Pinned: all 256 decodings and in-range rounding (ties, subnormals, the carry into 2^-6 and up to 448)
// against torch.float8_e4m3fn.  PARITY UNPINNED: what happens beyond 448 (torch makes NaN there, the crate's
// documentation says saturate; only the latter is restated), and the accumulation of sums and products.
uint8_t f32_to_f8e4m3_bits(uint32_t u) {
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7Fu;   // NaN
    if (a >= 0x43E00000u) return sign | 0x7Eu;  // >= 448, infinity too: the largest finite value
    if (a >= 0x3C800000u) {                     // normal in e4m3: >= 2^-6
        uint32_t h = (((a >> 23) - 120u) << 3) | ((a & 0x7FFFFFu) >> 20);
        const uint32_t rest = a & 0xFFFFFu;
        if (rest > 0x80000u || (rest == 0x80000u && (h & 1u))) h++; // a carry runs into the exponent
        return sign | (uint8_t)(h > 0x7Eu ? 0x7Eu : h);             // 464 and up would be 0x7F: saturate
    }
    const float units = float_of(a) * 512.0f; // subnormal: the value in units of 2^-9, nearest even
    return sign | (uint8_t)(uint32_t)nearbyintf(units);
}

uint32_t f8e4m3_bits_to_f32(uint8_t b) {
    const uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    const uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
    if (e == 0xF && m == 7) return sign | 0x7FC00000u;
    if (e != 0) return sign | ((e + 120u) << 23) | (m << 20);
    return sign | bits_of((float)m * (1.0f / 512.0f));
}

uint32_t round_to(cg_dtype dt, uint32_t u) {
    if (dt == CG_BF16) return (uint32_t)f32_to_bf16_bits(u) << 16;
    if (dt == CG_F16) return f16_bits_to_f32(f32_to_f16_bits(u));
    if (dt == CG_F8) return f8e4m3_bits_to_f32(f32_to_f8e4m3_bits(u));
    return u;
}


// Rust `f32 as u32`: truncate toward zero, saturating, NaN -> 0 (ndarray.rs:155).
inline uint32_t f32_as_u32(float v) {
    if (!(v == v)) return 0;
    if (v <= 0.0f) return 0;
    if (v >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)v;
}

// Rust `f32::total_cmp` key (ndarray.rs:676,708).
inline int32_t total_key(float f) {
    int32_t b;
    memcpy(&b, &f, 4);
    b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
    return b;
}

// ndarray `numeric_util::unrolled_fold` with zero/add, as used by `sum()` on a
// contiguous lane (called from `sum_axis`, ndarray.rs:729).
template <typename T> T unrolled_sum(const T *xs, size_t n) {
    T acc = 0, p0 = 0, p1 = 0, p2 = 0, p3 = 0, p4 = 0, p5 = 0, p6 = 0, p7 = 0;
    while (n >= 8) {
        p0 = p0 + xs[0];
        p1 = p1 + xs[1];
        p2 = p2 + xs[2];
        p3 = p3 + xs[3];
        p4 = p4 + xs[4];
        p5 = p5 + xs[5];
        p6 = p6 + xs[6];
        p7 = p7 + xs[7];
        xs += 8;
        n -= 8;
    }
    acc = acc + (p0 + p4);
    acc = acc + (p1 + p5);
    acc = acc + (p2 + p6);
    acc = acc + (p3 + p7);
    for (size_t i = 0; i < n; i++) acc = acc + xs[i];
    return acc;
}

// ---------------------------------------------------------------------------
// sgemm: restatement of matrixmultiply 0.3.10 `sgemm` (called by ndarray `dot`,
// ndarray.rs:747,806).  C[m,n] = A[m,k] B[k,n], arbitrary element strides.
// Loop nest and accumulation order: for each KC=256 block of k, an 8x8 micro-kernel
// accumulates ab += a*b with one fused multiply-add per k, sequentially, starting
// from zero; the block result is stored (first block) or added (later blocks) to C.
// ---------------------------------------------------------------------------
constexpr size_t SG_MR = 8, SG_NR = 8, SG_MC = 64, SG_KC = 256, SG_NC = 1024;

void pack_panels(size_t kc, size_t mc, float *pack, const float *a, ptrdiff_t rs, ptrdiff_t cs) {
    // Packs an mc x kc block (row stride rs, col stride cs) into MR-row panels, k-major
    // inside a panel, zero padded to a multiple of MR.
    for (size_t ir = 0; ir < mc; ir += SG_MR) {
        size_t rows = std::min(SG_MR, mc - ir);
        if (rows == SG_MR && rs == 1) {
            for (size_t p = 0; p < kc; p++) {
                memcpy(pack, a + (ptrdiff_t)ir + (ptrdiff_t)p * cs, SG_MR * sizeof(float));
                pack += SG_MR;
            }
        } else {
            for (size_t p = 0; p < kc; p++) {
                for (size_t i = 0; i < SG_MR; i++)
                    pack[i] = i < rows ? a[(ptrdiff_t)(ir + i) * rs + (ptrdiff_t)p * cs] : 0.0f;
                pack += SG_MR;
            }
        }
    }
}

inline void kernel_8x8(size_t kc, const float *ap, const float *bp, float *c, ptrdiff_t rsc, ptrdiff_t csc,
                       size_t rows, size_t cols, bool first) {
    __m256 ab[8];
    for (int i = 0; i < 8; i++) ab[i] = _mm256_setzero_ps();
    for (size_t p = 0; p < kc; p++) {
        __m256 bv = _mm256_loadu_ps(bp + p * 8);
        const float *av = ap + p * 8;
        for (int i = 0; i < 8; i++) ab[i] = _mm256_fmadd_ps(_mm256_broadcast_ss(av + i), bv, ab[i]);
    }
    if (rows == 8 && cols == 8 && csc == 1) {
        for (int i = 0; i < 8; i++) {
            float *cr = c + (ptrdiff_t)i * rsc;
            if (first)
                _mm256_storeu_ps(cr, ab[i]);
            else
                _mm256_storeu_ps(cr, _mm256_add_ps(_mm256_loadu_ps(cr), ab[i]));
        }
    } else {
        alignas(32) float tmp[8][8];
        for (int i = 0; i < 8; i++) _mm256_store_ps(tmp[i], ab[i]);
        for (size_t i = 0; i < rows; i++)
            for (size_t j = 0; j < cols; j++) {
                float *ce = c + (ptrdiff_t)i * rsc + (ptrdiff_t)j * csc;
                *ce = first ? tmp[i][j] : *ce + tmp[i][j];
            }
    }
}

void sgemm(size_t m, size_t k, size_t n, const float *a, ptrdiff_t rsa, ptrdiff_t csa, const float *b,
           ptrdiff_t rsb, ptrdiff_t csb, float *c, ptrdiff_t rsc, ptrdiff_t csc) {
    if (m == 0 || n == 0) return;
    if (k == 0) {
        for (size_t i = 0; i < m; i++)
            for (size_t j = 0; j < n; j++) c[(ptrdiff_t)i * rsc + (ptrdiff_t)j * csc] = 0.0f;
        return;
    }
    static thread_local std::vector<float> apack, bpack;
    apack.resize(((std::min(m, SG_MC) + SG_MR - 1) / SG_MR) * SG_MR * std::min(k, SG_KC));
    bpack.resize(((std::min(n, SG_NC) + SG_NR - 1) / SG_NR) * SG_NR * std::min(k, SG_KC));
    for (size_t l5 = 0; l5 < n; l5 += SG_NC) {
        size_t nc = std::min(SG_NC, n - l5);
        for (size_t l4 = 0; l4 < k; l4 += SG_KC) {
            size_t kc = std::min(SG_KC, k - l4);
            // B block kc x nc packed into NR-column panels (transpose roles of rs/cs)
            pack_panels(kc, nc, bpack.data(), b + (ptrdiff_t)l4 * rsb + (ptrdiff_t)l5 * csb, csb, rsb);
            bool first = l4 == 0;
            for (size_t l3 = 0; l3 < m; l3 += SG_MC) {
                size_t mc = std::min(SG_MC, m - l3);
                pack_panels(kc, mc, apack.data(), a + (ptrdiff_t)l3 * rsa + (ptrdiff_t)l4 * csa, rsa, csa);
                for (size_t jr = 0; jr < nc; jr += SG_NR) {
                    const float *bp = bpack.data() + (jr / SG_NR) * SG_NR * kc;
                    size_t cols = std::min(SG_NR, nc - jr);
                    for (size_t ir = 0; ir < mc; ir += SG_MR) {
                        const float *ap = apack.data() + (ir / SG_MR) * SG_MR * kc;
                        size_t rows = std::min(SG_MR, mc - ir);
                        kernel_8x8(kc, ap, bp, c + (ptrdiff_t)(l3 + ir) * rsc + (ptrdiff_t)(l5 + jr) * csc, rsc, csc,
                                   rows, cols, first);
                    }
                }
            }
        }
    }
}

// ndarray's generic (non f32/f64) `dot`: c[i,j] = fold over k, here with Rust
// release-mode wrapping u32 arithmetic (ndarray.rs:181).
void ugemm(size_t m, size_t k, size_t n, const uint32_t *a, ptrdiff_t rsa, ptrdiff_t csa, const uint32_t *b,
           ptrdiff_t rsb, ptrdiff_t csb, uint32_t *c) {
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            uint32_t s = 0;
            for (size_t p = 0; p < k; p++)
                s += a[(ptrdiff_t)i * rsa + (ptrdiff_t)p * csa] * b[(ptrdiff_t)p * rsb + (ptrdiff_t)j * csb];
            c[i * n + j] = s;
        }
}

// `to_shape((batch, r, c))` of an owned array (ndarray.rs:797-798): a view when the
// memory layout allows merging the leading axes, else a row-major copy.  Returns base
// pointer and the three strides; `tmp` holds the copy if one was needed.
template <typename T>
const T *as_batch3(cg_tensor *t, size_t batch, Vec<T> &tmp, ptrdiff_t &sb, ptrdiff_t &sr, ptrdiff_t &sc) {
    int r = t->rank;
    size_t R = t->dims[r - 2], C = t->dims[r - 1];
    // leading axes mergeable iff they are mutually row-major nested
    bool ok = true;
    ptrdiff_t bs = 0;
    bool have = false;
    size_t inner = 1;
    for (int d = r - 3; d >= 0; d--) {
        if (t->dims[d] == 1) continue;
        if (!have) {
            bs = t->strides[d];
            have = true;
            inner = t->dims[d];
        } else {
            if (t->strides[d] != bs * (ptrdiff_t)inner) ok = false;
            inner *= t->dims[d];
        }
    }
    if (ok || batch <= 1) {
        sb = have ? bs : 0;
        sr = t->strides[r - 2];
        sc = t->strides[r - 1];
        return data_of<T>(t);
    }
    tmp = dense<T>(t);
    sb = (ptrdiff_t)(R * C);
    sr = (ptrdiff_t)C;
    sc = 1;
    return tmp.data();
}

template <typename F> int for_each_dtype(cg_dtype dt, F &&f) {
    if (isf(dt)) return f(float{});
    if (dt == CG_U32) return f(uint32_t{});
    return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
}

} // namespace

extern "C" {

int cg_backend_create(int, cg_backend **out) {
    if (!out) return fail(CG_ERR_ARG, "null out");
    *out = new cg_backend;
    return CG_OK;
}
void cg_backend_destroy(cg_backend *b) { delete b; }
const char *cg_last_error(void) { return g_err.c_str(); }
const char *cg_backend_name(cg_backend *) { return "oracle:cpu (NdArrayBackend restated, 1 thread)"; }
int cg_sync(cg_backend *) { return CG_OK; }
int cg_pool_stats(cg_backend *, size_t *u, size_t *c) {
    if (u) *u = 0;
    if (c) *c = 0;
    return CG_OK;
}
int cg_pool_trim(cg_backend *) { return CG_OK; }
int cg_profile_enable(cg_backend *, cg_kernel_class, unsigned) { return CG_OK; } // no kernels to time
int cg_realize(cg_backend *, cg_tensor *) { return CG_OK; } // every result is already computed
int cg_program_stats(cg_backend *, uint64_t *compiled, uint64_t *interpreted, int) { // nothing is fused here
    if (compiled) *compiled = 0;
    if (interpreted) *interpreted = 0;
    return CG_OK;
}
int cg_profile_read(cg_backend *, cg_kernel_class, uint64_t *launches, double *milliseconds, double *work, int) {
    if (launches) *launches = 0;
    if (milliseconds) *milliseconds = 0.0;
    if (work) *work = 0.0;
    return CG_OK;
}

void cg_tensor_retain(cg_tensor *t) {
    if (t) t->rc.fetch_add(1);
}
void cg_tensor_release(cg_tensor *t) { release(t); }
size_t cg_tensor_rank(const cg_tensor *t) { return (size_t)t->rank; }
void cg_tensor_shape(const cg_tensor *t, size_t *dims) {
    for (int i = 0; i < t->rank; i++) dims[i] = t->dims[i];
}
cg_dtype cg_tensor_dtype(const cg_tensor *t) { return t->dt; }
size_t cg_tensor_numel(const cg_tensor *t) { return numel(t); }
int cg_tensor_is_contiguous(const cg_tensor *t) { return is_standard(t) ? 1 : 0; }

// ndarray.rs:71-84
int cg_zeros(cg_backend *, cg_dtype dtype, const size_t *dims, size_t rank, cg_tensor **out) {
    if (!out || rank > CG_MAX_RANK) return fail(CG_ERR_ARG, "bad arguments");
    if (!supported(dtype)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    *out = new_tensor(dtype, dims, (int)rank); // vector::resize zero-fills
    return CG_OK;
}

// ndarray.rs:86-96,122-132 (+ interpreter/mod.rs:28-30)
int cg_from_host(cg_backend *, cg_dtype dtype, const void *data, size_t len, const size_t *dims, size_t rank,
                 cg_tensor **out) {
    if (!out || rank > CG_MAX_RANK) return fail(CG_ERR_ARG, "bad arguments");
    if (!supported(dtype)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    size_t n = 1;
    for (size_t i = 0; i < rank; i++) n *= dims[i];
    if (n != len) return fail(CG_ERR_SHAPE, "ShapeError");
    cg_tensor *t = new_tensor(dtype, dims, (int)rank);
    if (n && is_half(dtype)) { // 2-byte elements, widened exactly (candle.rs:530-551)
        const uint16_t *h = static_cast<const uint16_t *>(data);
        uint32_t *d = t->st->data.data();
        for (size_t i = 0; i < n; i++) d[i] = dtype == CG_BF16 ? (uint32_t)h[i] << 16 : f16_bits_to_f32(h[i]);
    } else if (n && dtype == CG_F8) { // 1-byte elements (candle.rs:553-562)
        const uint8_t *h = static_cast<const uint8_t *>(data);
        uint32_t *d = t->st->data.data();
        for (size_t i = 0; i < n; i++) d[i] = f8e4m3_bits_to_f32(h[i]);
    } else if (n) {
        memcpy(t->st->data.data(), data, n * 4);
    }
    *out = t;
    return CG_OK;
}

// catgrad-llm/src/utils/mod.rs:158-168 (`decode_bf16_to_f32_into`: bf16::to_f32 is the bit
// pattern in the high half of an f32) followed by `interpreter::tensor` (mod.rs:23-33).
int cg_from_host_bf16_as_f32(cg_backend *b, const uint16_t *bits, size_t len, const size_t *dims, size_t rank,
                             cg_tensor **out) {
    if (!b || !out || (len && !bits)) return fail(CG_ERR_ARG, "bad arguments");
    size_t n = 1;
    for (size_t i = 0; i < rank; i++) n *= dims[i];
    if (n != len) return fail(CG_ERR_SHAPE, "ShapeError");
    cg_tensor *t = new_tensor(CG_F32, dims, (int)rank);
    uint32_t *dst = t->st->data.data();
    for (size_t i = 0; i < n; i++) dst[i] = (uint32_t)bits[i] << 16;
    *out = t;
    return CG_OK;
}

// ndarray.rs:134-138: `Array::range(0.0, end as f32, 1.0)` then cast to u32.  The f32
// detour is exact for end <= 2^24; above that the reference itself is inexact.
int cg_arange(cg_backend *, size_t end, cg_tensor **out) {
    if (!out) return fail(CG_ERR_ARG, "null out");
    float fe = (float)end;
    size_t n = (size_t)std::ceil(fe);
    size_t dims[1] = {n};
    cg_tensor *t = new_tensor(CG_U32, dims, 1);
    uint32_t *d = data_of<uint32_t>(t);
    for (size_t i = 0; i < n; i++) d[i] = f32_as_u32(0.0f + 1.0f * (float)i);
    *out = t;
    return CG_OK;
}

// ndarray.rs:50-58.  `as_slice().unwrap()` panics on a non-standard layout.
int cg_to_host(cg_backend *, const cg_tensor *t, void *dst, size_t len) {
    if (!t || (!dst && len)) return fail(CG_ERR_ARG, "null argument");
    if (len != numel(t)) return fail(CG_ERR_SHAPE, "to_vec: length mismatch");
    if (!is_standard(t)) return fail(CG_ERR_SHAPE, "to_vec: called `Option::unwrap()` on a `None` value (non-contiguous)");
    const uint32_t *src = reinterpret_cast<const uint32_t *>(t->st->data.data()) + t->offset;
    if (is_half(t->dt)) { // 2-byte elements out (candle.rs:463-470); exact, the words hold representable values
        uint16_t *h = static_cast<uint16_t *>(dst);
        for (size_t i = 0; i < len; i++) h[i] = t->dt == CG_BF16 ? (uint16_t)(src[i] >> 16) : f32_to_f16_bits(src[i]);
    } else if (t->dt == CG_F8) {
        uint8_t *h = static_cast<uint8_t *>(dst);
        for (size_t i = 0; i < len; i++) h[i] = f32_to_f8e4m3_bits(src[i]);
    } else if (len) {
        memcpy(dst, src, len * 4);
    }
    return CG_OK;
}

// ndarray.rs:140-149
int cg_to_bool(cg_backend *, const cg_tensor *t, int *out) {
    if (!t || !out) return fail(CG_ERR_ARG, "null argument");
    bool any = false;
    if (isf(t->dt)) {
        for (float v : dense<float>(t)) any |= v > 0.0f;
    } else {
        for (uint32_t v : dense<uint32_t>(t)) any |= v != 0;
    }
    *out = any;
    return CG_OK;
}

// ndarray.rs:534-541: derived PartialEq of ArcArray = same shape and element-wise ==.
int cg_compare(cg_backend *, const cg_tensor *x, const cg_tensor *y, int *out) {
    if (!x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "compare: dtype mismatch");
    bool eq = same_shape(x, y);
    if (eq) {
        if (isf(x->dt)) {
            auto a = dense<float>(x), b = dense<float>(y);
            for (size_t i = 0; i < a.size() && eq; i++) eq = a[i] == b[i];
        } else {
            eq = dense<uint32_t>(x) == dense<uint32_t>(y);
        }
    }
    *out = eq;
    return CG_OK;
}

// ndarray.rs:60-69
int cg_format_tensor(cg_backend *, const cg_tensor *t, char *buf, size_t cap) {
    if (!t || !buf || !cap) return fail(CG_ERR_ARG, "null argument");
    std::string s = t->dt == CG_F32 ? "f32[" : t->dt == CG_F16 ? "f16[" : t->dt == CG_BF16 ? "bf16[" : t->dt == CG_F8 ? "fp8[" : "u32[";
    for (int i = 0; i < t->rank; i++) s += (i ? "," : "") + std::to_string(t->dims[i]);
    s += "] [";
    size_t n = numel(t), shown = std::min<size_t>(n, 16);
    char tmp[48];
    if (isf(t->dt)) {
        auto v = dense<float>(t);
        for (size_t i = 0; i < shown; i++) {
            snprintf(tmp, sizeof tmp, "%s%.9g", i ? ", " : "", v[i]);
            s += tmp;
        }
    } else {
        auto v = dense<uint32_t>(t);
        for (size_t i = 0; i < shown; i++) {
            snprintf(tmp, sizeof tmp, "%s%u", i ? ", " : "", v[i]);
            s += tmp;
        }
    }
    s += n > shown ? ", ...]" : "]";
    snprintf(buf, cap, "%s", s.c_str());
    return CG_OK;
}

// ndarray.rs:151-174
int cg_cast(cg_backend *, cg_tensor *x, cg_dtype target, cg_tensor **out) {
    Consume cx(x);
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(target) || !supported(x->dt))
        return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (target == x->dt) { // (x @ F32, F32) => x
        x->rc.fetch_add(1);
        *out = x;
        return CG_OK;
    }
    cg_tensor *o = unwrap_owned(x);
    cg_tensor *r = new_tensor(target, o->dims, o->rank);
    size_t n = numel(o);
    if (target == CG_U32) {
        auto v = dense<float>(o);
        uint32_t *d = data_of<uint32_t>(r);
        for (size_t i = 0; i < n; i++) d[i] = f32_as_u32(v[i]);
    } else if (o->dt == CG_U32) {
        auto v = dense<uint32_t>(o);
        float *d = data_of<float>(r);
        for (size_t i = 0; i < n; i++) d[i] = (float)v[i]; // round to nearest even
    } else { // between floating-point dtypes (candle.rs:575-599): the value, rounded below if the target is narrower
        auto v = dense<uint32_t>(o);
        uint32_t *d = data_of<uint32_t>(r);
        for (size_t i = 0; i < n; i++) d[i] = v[i];
    }
    round_tensor(r);
    release(o);
    *out = r;
    return CG_OK;
}

// ndarray.rs:352-407, 630-648
int cg_unary(cg_backend *, cg_unary_op op, cg_tensor *x, cg_tensor **out) {
    Consume cx(x);
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (x->dt == CG_U32 && op != CG_NEG) {
        static const char *names[] = {"neg", "sin", "cos", "exp", "log", "floor", "round"};
        return fail(CG_ERR_DTYPE, "Invalid input types for %s", names[op]);
    }
    cg_tensor *o = unwrap_owned(x);
    cg_tensor *r = new_tensor(o->dt, o->dims, o->rank);
    size_t n = numel(o);
    if (o->dt == CG_U32) {
        auto v = dense<uint32_t>(o);
        uint32_t *d = data_of<uint32_t>(r);
        for (size_t i = 0; i < n; i++) d[i] = 0u - v[i]; // wrapping_neg
    } else {
        auto v = dense<float>(o);
        float *d = data_of<float>(r);
        switch (op) {
        case CG_NEG: for (size_t i = 0; i < n; i++) d[i] = -v[i]; break;
        case CG_SIN: for (size_t i = 0; i < n; i++) d[i] = sinf(v[i]); break;
        case CG_COS: for (size_t i = 0; i < n; i++) d[i] = cosf(v[i]); break;
        case CG_EXP: for (size_t i = 0; i < n; i++) d[i] = expf(v[i]); break;
        case CG_LOG: for (size_t i = 0; i < n; i++) d[i] = logf(v[i]); break;
        case CG_FLOOR: for (size_t i = 0; i < n; i++) d[i] = floorf(v[i]); break;
        case CG_ROUND: for (size_t i = 0; i < n; i++) d[i] = nearbyintf(v[i]); break; // default mode: ties to even
        default: release(o); release(r); return fail(CG_ERR_ARG, "unknown unary op");
        }
    }
    round_tensor(r);
    release(o);
    *out = r;
    return CG_OK;
}

static uint32_t wrapping_pow(uint32_t a, uint32_t e) { // Rust u32::pow in release mode
    uint32_t acc = 1;
    while (e) {
        if (e & 1) acc *= a;
        a *= a;
        e >>= 1;
    }
    return acc;
}

// ndarray.rs:185-323, 598-654
int cg_binary(cg_backend *, cg_binary_op op, cg_tensor *x, cg_tensor *y, cg_tensor **out) {
    Consume cx(x), cy(y);
    if (!x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt))
        return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "TypeError: mixed dtypes in a binary operation");
    if (!same_shape(x, y)) return fail(CG_ERR_SHAPE, "Shape mismatch in operation");
    cg_tensor *ox = unwrap_owned(x), *oy = unwrap_owned(y);
    cg_tensor *r = new_tensor(ox->dt, ox->dims, ox->rank);
    size_t n = numel(ox);
    int rc = CG_OK;
    if (isf(ox->dt)) {
        auto a = dense<float>(ox), b = dense<float>(oy);
        float *d = data_of<float>(r);
        switch (op) {
        case CG_ADD: for (size_t i = 0; i < n; i++) d[i] = a[i] + b[i]; break;
        case CG_SUB: for (size_t i = 0; i < n; i++) d[i] = a[i] - b[i]; break;
        case CG_MUL: for (size_t i = 0; i < n; i++) d[i] = a[i] * b[i]; break;
        case CG_DIV: for (size_t i = 0; i < n; i++) d[i] = a[i] / b[i]; break;
        case CG_POW: for (size_t i = 0; i < n; i++) d[i] = powf(a[i], b[i]); break;
        case CG_LT: for (size_t i = 0; i < n; i++) d[i] = a[i] < b[i] ? 1.0f : 0.0f; break;
        case CG_GT: for (size_t i = 0; i < n; i++) d[i] = a[i] > b[i] ? 1.0f : 0.0f; break;
        case CG_GTE: for (size_t i = 0; i < n; i++) d[i] = a[i] >= b[i] ? 1.0f : 0.0f; break;
        case CG_LTE: for (size_t i = 0; i < n; i++) d[i] = a[i] <= b[i] ? 1.0f : 0.0f; break;
        case CG_EQ: for (size_t i = 0; i < n; i++) d[i] = a[i] == b[i] ? 1.0f : 0.0f; break;
        default: rc = fail(CG_ERR_ARG, "unknown binary op");
        }
    } else {
        auto a = dense<uint32_t>(ox), b = dense<uint32_t>(oy);
        uint32_t *d = data_of<uint32_t>(r);
        switch (op) {
        case CG_ADD: for (size_t i = 0; i < n; i++) d[i] = a[i] + b[i]; break;
        case CG_SUB: for (size_t i = 0; i < n; i++) d[i] = a[i] - b[i]; break;
        case CG_MUL: for (size_t i = 0; i < n; i++) d[i] = a[i] * b[i]; break;
        case CG_DIV:
            for (size_t i = 0; i < n; i++) {
                if (b[i] == 0) {
                    rc = fail(CG_ERR_RANGE, "attempt to divide by zero");
                    break;
                }
                d[i] = a[i] / b[i];
            }
            break;
        case CG_POW: for (size_t i = 0; i < n; i++) d[i] = wrapping_pow(a[i], b[i]); break;
        case CG_LT: for (size_t i = 0; i < n; i++) d[i] = a[i] < b[i]; break;
        case CG_GT: for (size_t i = 0; i < n; i++) d[i] = a[i] > b[i]; break;
        case CG_GTE: for (size_t i = 0; i < n; i++) d[i] = a[i] >= b[i]; break;
        case CG_LTE: for (size_t i = 0; i < n; i++) d[i] = a[i] <= b[i]; break;
        case CG_EQ: for (size_t i = 0; i < n; i++) d[i] = a[i] == b[i]; break;
        default: rc = fail(CG_ERR_ARG, "unknown binary op");
        }
    }
    release(ox);
    release(oy);
    if (rc != CG_OK) {
        release(r);
        return rc;
    }
    round_tensor(r);
    *out = r;
    return CG_OK;
}

// ndarray.rs:325-350
int cg_where(cg_backend *, cg_tensor *mask, cg_tensor *x, cg_tensor *y, cg_tensor **out) {
    Consume cm(mask), cx(x), cy(y);
    if (!mask || !x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (mask->dt != x->dt || y->dt != x->dt) return fail(CG_ERR_DTYPE, "TypeError: mixed dtypes in where");
    if (!same_shape(mask, x) || !same_shape(x, y)) return fail(CG_ERR_SHAPE, "Shape mismatch in operation");
    cg_tensor *om = unwrap_owned(mask), *ox = unwrap_owned(x), *oy = unwrap_owned(y);
    cg_tensor *r = new_tensor(ox->dt, ox->dims, ox->rank);
    size_t n = numel(ox);
    if (isf(ox->dt)) {
        auto m = dense<float>(om), a = dense<float>(ox), b = dense<float>(oy);
        float *d = data_of<float>(r);
        for (size_t i = 0; i < n; i++) d[i] = m[i] > 0.0f ? a[i] : b[i];
    } else {
        auto m = dense<uint32_t>(om), a = dense<uint32_t>(ox), b = dense<uint32_t>(oy);
        uint32_t *d = data_of<uint32_t>(r);
        for (size_t i = 0; i < n; i++) d[i] = m[i] != 0 ? a[i] : b[i];
    }
    release(om);
    release(ox);
    release(oy);
    *out = r;
    return CG_OK;
}

// ndarray.rs:176-183, 732-816
int cg_matmul(cg_backend *, cg_tensor *x, cg_tensor *y, cg_tensor **out) {
    Consume cx(x), cy(y);
    if (!x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt))
        return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "TypeError: mixed dtypes in matmul");
    if (x->rank < 2) return fail(CG_ERR_SHAPE, "batched_matmul: lhs must be at least rank 2");
    if (y->rank < 2) return fail(CG_ERR_SHAPE, "batched_matmul: rhs must be at least rank 2");
    int rx = x->rank, ry = y->rank;
    if (x->dims[rx - 1] != y->dims[ry - 2]) return fail(CG_ERR_SHAPE, "batched_matmul: incompatible matrix dimensions");
    if (rx != ry) return fail(CG_ERR_SHAPE, "batched_matmul: batch dimensions must match");
    for (int i = 0; i < rx - 2; i++)
        if (x->dims[i] != y->dims[i]) return fail(CG_ERR_SHAPE, "batched_matmul: batch dimensions must match");
    size_t M = x->dims[rx - 2], K = x->dims[rx - 1], N = y->dims[ry - 1];
    size_t batch = 1;
    for (int i = 0; i < rx - 2; i++) batch *= x->dims[i];
    cg_tensor *ox = unwrap_owned(x), *oy = unwrap_owned(y);
    size_t odims[CG_MAX_RANK];
    for (int i = 0; i < rx - 2; i++) odims[i] = x->dims[i];
    odims[rx - 2] = M;
    odims[rx - 1] = N;
    cg_tensor *r = new_tensor(ox->dt, odims, rx);
    if (isf(ox->dt)) {
        Vec<float> ta, tb;
        ptrdiff_t sba, sra, sca, sbb, srb, scb;
        const float *a = as_batch3<float>(ox, batch, ta, sba, sra, sca);
        const float *b = as_batch3<float>(oy, batch, tb, sbb, srb, scb);
        float *c = data_of<float>(r);
        for (size_t bi = 0; bi < batch; bi++)
            sgemm(M, K, N, a + (ptrdiff_t)bi * sba, sra, sca, b + (ptrdiff_t)bi * sbb, srb, scb, c + bi * M * N,
                  (ptrdiff_t)N, 1);
    } else {
        Vec<uint32_t> ta, tb;
        ptrdiff_t sba, sra, sca, sbb, srb, scb;
        const uint32_t *a = as_batch3<uint32_t>(ox, batch, ta, sba, sra, sca);
        const uint32_t *b = as_batch3<uint32_t>(oy, batch, tb, sbb, srb, scb);
        uint32_t *c = data_of<uint32_t>(r);
        for (size_t bi = 0; bi < batch; bi++)
            ugemm(M, K, N, a + (ptrdiff_t)bi * sba, sra, sca, b + (ptrdiff_t)bi * sbb, srb, scb, c + bi * M * N);
    }
    round_tensor(r);
    release(ox);
    release(oy);
    *out = r;
    return CG_OK;
}

namespace {
// Shared frame of the last-axis reductions: rank must be >= 1 (`x.ndim() - 1`
// underflows on rank 0, ndarray.rs:658,672,728).
int reduce_frame(cg_tensor *x, cg_tensor **out, const char *what, cg_tensor **owned, size_t *rows, size_t *n) {
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (x->rank == 0) return fail(CG_ERR_SHAPE, "%s: rank-0 tensor has no last axis", what);
    *owned = unwrap_owned(x);
    *n = x->dims[x->rank - 1];
    size_t total = numel(x);
    *rows = *n ? total / *n : 0;
    if (*n == 0) {
        *rows = 1;
        for (int i = 0; i < x->rank - 1; i++) *rows *= x->dims[i];
    }
    return CG_OK;
}
} // namespace

// ndarray.rs:418-425, 723-730 — `sum_axis(last)`: on the minimum-stride axis each lane
// is summed with the 8-way unrolled fold when it is a contiguous slice and with a
// sequential fold otherwise; on any other axis sub-views are accumulated one by one,
// which is the same sequential order per output element.
int cg_sum(cg_backend *, cg_tensor *x, cg_tensor **out) {
    Consume cx(x);
    cg_tensor *o;
    size_t rows, n;
    int rc = reduce_frame(x, out, "sum", &o, &rows, &n);
    if (rc) return rc;
    int r = o->rank;
    bool last_is_min = true;
    {
        ptrdiff_t best = -1;
        int best_ax = r - 1;
        for (int d = r - 1; d >= 0; d--) { // reversed scan, first minimum wins
            if (o->dims[d] <= 1) continue;
            ptrdiff_t s = std::abs(o->strides[d]);
            if (best < 0 || s < best) {
                best = s;
                best_ax = d;
            }
        }
        last_is_min = best_ax == r - 1;
    }
    bool unrolled = last_is_min && (n <= 1 || o->strides[r - 1] == 1);
    size_t odims[CG_MAX_RANK];
    memcpy(odims, o->dims, sizeof odims);
    odims[r - 1] = 1;
    cg_tensor *res = new_tensor(o->dt, odims, r);
    for_each_dtype(o->dt, [&](auto tag) {
        using T = decltype(tag);
        auto v = dense<T>(o);
        T *d = data_of<T>(res);
        for (size_t i = 0; i < rows; i++) {
            const T *p = v.data() + i * n;
            if (unrolled) {
                d[i] = unrolled_sum<T>(p, n);
            } else {
                T s = 0;
                for (size_t j = 0; j < n; j++) s = s + p[j];
                d[i] = s;
            }
        }
        return CG_OK;
    });
    round_tensor(res);
    release(o);
    *out = res;
    return CG_OK;
}

// ndarray.rs:409-416, 656-668 — fold from f32::MIN with `f32::max` (NaN ignored); u32 from 0.
int cg_max(cg_backend *, cg_tensor *x, cg_tensor **out) {
    Consume cx(x);
    cg_tensor *o;
    size_t rows, n;
    int rc = reduce_frame(x, out, "max", &o, &rows, &n);
    if (rc) return rc;
    int r = o->rank;
    size_t odims[CG_MAX_RANK];
    memcpy(odims, o->dims, sizeof odims);
    odims[r - 1] = 1;
    cg_tensor *res = new_tensor(o->dt, odims, r);
    if (isf(o->dt)) {
        auto v = dense<float>(o);
        float *d = data_of<float>(res);
        for (size_t i = 0; i < rows; i++) {
            float acc = -std::numeric_limits<float>::max(); // f32::MIN
            for (size_t j = 0; j < n; j++) acc = fmaxf(acc, v[i * n + j]);
            d[i] = acc;
        }
    } else {
        auto v = dense<uint32_t>(o);
        uint32_t *d = data_of<uint32_t>(res);
        for (size_t i = 0; i < rows; i++) {
            uint32_t acc = 0;
            for (size_t j = 0; j < n; j++) acc = std::max(acc, v[i * n + j]);
            d[i] = acc;
        }
    }
    round_tensor(res); // the seed f32::MIN of an empty or all-NaN row is not a value of the 16-bit dtypes
    release(o);
    *out = res;
    return CG_OK;
}

// ndarray.rs:427-434, 670-694 — `max_by(total_cmp)`: the LAST of equal maxima wins.
int cg_argmax(cg_backend *, cg_tensor *x, cg_tensor **out) {
    Consume cx(x);
    cg_tensor *o;
    size_t rows, n;
    int rc = reduce_frame(x, out, "argmax", &o, &rows, &n);
    if (rc) return rc;
    if (n == 0) {
        release(o);
        return fail(CG_ERR_SHAPE, "argmax: called `Option::unwrap()` on a `None` value (empty axis)");
    }
    int r = o->rank;
    size_t odims[CG_MAX_RANK];
    memcpy(odims, o->dims, sizeof odims);
    odims[r - 1] = 1;
    cg_tensor *res = new_tensor(CG_U32, odims, r);
    uint32_t *d = data_of<uint32_t>(res);
    if (isf(o->dt)) {
        auto v = dense<float>(o);
        for (size_t i = 0; i < rows; i++) {
            size_t best = 0;
            int32_t bk = total_key(v[i * n]);
            for (size_t j = 1; j < n; j++) {
                int32_t k = total_key(v[i * n + j]);
                if (k >= bk) {
                    bk = k;
                    best = j;
                }
            }
            d[i] = (uint32_t)best;
        }
    } else {
        auto v = dense<uint32_t>(o);
        for (size_t i = 0; i < rows; i++) {
            size_t best = 0;
            for (size_t j = 1; j < n; j++)
                if (v[i * n + j] >= v[i * n + best]) best = j;
            d[i] = (uint32_t)best;
        }
    }
    release(o);
    *out = res;
    return CG_OK;
}

// The same rule on a dense [rows, n] array in plain memory (the checker's side of the entry point that the GPU
// library offers to callers that cannot allocate; `device` and `stream` mean nothing here).
int cg_noalloc_setup(int) { return CG_OK; } // nothing to set up in plain memory
int cg_argmax_rows_noalloc(int, cg_dtype dtype, const void *x, size_t rows, size_t n, uint32_t *out, void *) {
    if (n == 0) return fail(CG_ERR_SHAPE, "argmax: called `Option::unwrap()` on a `None` value (empty axis)");
    if (rows == 0) return CG_OK;
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    for (size_t i = 0; i < rows; i++) {
        size_t best = 0;
        if (dtype == CG_U32) {
            const uint32_t *v = static_cast<const uint32_t *>(x) + i * n;
            for (size_t j = 1; j < n; j++)
                if (v[j] >= v[best]) best = j;
        } else {
            const float *v = static_cast<const float *>(x) + i * n;
            int32_t bk = total_key(v[0]);
            for (size_t j = 1; j < n; j++) {
                const int32_t k = total_key(v[j]);
                if (k >= bk) {
                    bk = k;
                    best = j;
                }
            }
        }
        out[i] = (uint32_t)best;
    }
    return CG_OK;
}

// ndarray.rs:436-446, 696-721 — stable sort, descending by total_cmp, first k.
int cg_topk(cg_backend *, cg_tensor *x, size_t k, cg_tensor **values, cg_tensor **indices) {
    Consume cx(x);
    if (!x || !values || !indices) return fail(CG_ERR_ARG, "null argument");
    if (x->dt == CG_U32) return fail(CG_ERR_DTYPE, "Unsupported type for topk");
    if (!isf(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (x->rank == 0) return fail(CG_ERR_SHAPE, "topk: rank-0 tensor has no last axis");
    size_t n = x->dims[x->rank - 1];
    if (n == 0) return fail(CG_ERR_SHAPE, "topk: attempt to divide by zero (empty last axis)");
    cg_tensor *o = unwrap_owned(x);
    size_t rows = numel(o) / n;
    size_t kk = std::min(k, n); // truncate(k) keeps at most n
    if (kk != k) {
        // from_shape_vec with dims[last]=k would fail for k > n
        release(o);
        return fail(CG_ERR_SHAPE, "topk: k larger than the last axis");
    }
    size_t odims[CG_MAX_RANK];
    memcpy(odims, o->dims, sizeof odims);
    odims[o->rank - 1] = k;
    cg_tensor *vals = new_tensor(o->dt, odims, o->rank);
    cg_tensor *idxs = new_tensor(CG_U32, odims, o->rank);
    auto v = dense<float>(o);
    float *dv = data_of<float>(vals);
    uint32_t *di = data_of<uint32_t>(idxs);
    std::vector<size_t> order(n);
    for (size_t i = 0; i < rows; i++) {
        const float *lane = v.data() + i * n;
        std::iota(order.begin(), order.end(), 0);
        std::stable_sort(order.begin(), order.end(),
                         [&](size_t a, size_t b) { return total_key(lane[a]) > total_key(lane[b]); });
        for (size_t j = 0; j < k; j++) {
            dv[i * k + j] = lane[order[j]];
            di[i * k + j] = (uint32_t)order[j];
        }
    }
    release(o);
    *values = vals;
    *indices = idxs;
    return CG_OK;
}

// ndarray.rs:448-455, 553-559 — numpy-style right-aligned broadcast, MATERIALISED (`to_owned`).
int cg_broadcast(cg_backend *, cg_tensor *x, const size_t *dims, size_t rank, cg_tensor **out) {
    Consume cx(x);
    if (!x || !out || rank > CG_MAX_RANK) return fail(CG_ERR_ARG, "bad arguments");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if ((size_t)x->rank > rank) return fail(CG_ERR_SHAPE, "broadcast: called `Option::unwrap()` on a `None` value");
    int shift = (int)rank - x->rank;
    for (int i = 0; i < x->rank; i++)
        if (x->dims[i] != dims[i + shift] && x->dims[i] != 1)
            return fail(CG_ERR_SHAPE, "broadcast: called `Option::unwrap()` on a `None` value");
    cg_tensor *o = unwrap_owned(x);
    cg_tensor v; // stride-0 view, then densified
    v.st = o->st;
    v.dt = o->dt;
    v.rank = (int)rank;
    v.offset = o->offset;
    for (int i = 0; i < (int)rank; i++) {
        v.dims[i] = dims[i];
        int j = i - shift;
        v.strides[i] = (j >= 0 && o->dims[j] == dims[i]) ? o->strides[j] : 0;
    }
    cg_tensor *r = new_tensor(o->dt, dims, (int)rank);
    gather_logical<uint32_t>(&v, data_of<uint32_t>(r));
    v.st = nullptr;
    release(o);
    *out = r;
    return CG_OK;
}

// ndarray.rs:504-511, 545-551 — `to_shape(..).to_owned()`: row-major logical reshape, always a fresh array.
int cg_reshape(cg_backend *, cg_tensor *x, const size_t *dims, size_t rank, cg_tensor **out) {
    Consume cx(x);
    if (!x || !out || rank > CG_MAX_RANK) return fail(CG_ERR_ARG, "bad arguments");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    size_t n = 1;
    for (size_t i = 0; i < rank; i++) n *= dims[i];
    if (n != numel(x)) return fail(CG_ERR_SHAPE, "reshape: ShapeError/IncompatibleShape");
    cg_tensor *o = unwrap_owned(x);
    cg_tensor *r = new_tensor(o->dt, dims, (int)rank);
    gather_logical<uint32_t>(o, data_of<uint32_t>(r));
    release(o);
    *out = r;
    return CG_OK;
}

// ndarray.rs:457-464, 561-569 — `swap_axes`: a view.
int cg_transpose(cg_backend *, cg_tensor *x, size_t dim0, size_t dim1, cg_tensor **out) {
    Consume cx(x);
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (dim0 >= (size_t)x->rank || dim1 >= (size_t)x->rank) return fail(CG_ERR_RANGE, "transpose: axis out of range");
    cg_tensor *o = unwrap_owned(x);
    cg_tensor *v = view_of(o);
    std::swap(v->dims[dim0], v->dims[dim1]);
    std::swap(v->strides[dim0], v->strides[dim1]);
    release(o);
    *out = v;
    return CG_OK;
}

// ndarray.rs:489-502, 581-588 — `slice_axis_move`: a view.
int cg_slice(cg_backend *, cg_tensor *x, size_t dim, size_t start, size_t len, cg_tensor **out) {
    Consume cx(x);
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (dim >= (size_t)x->rank) return fail(CG_ERR_RANGE, "slice: axis out of range");
    if (start > x->dims[dim] || len > x->dims[dim] - start) return fail(CG_ERR_RANGE, "slice: range out of bounds");
    cg_tensor *o = unwrap_owned(x);
    cg_tensor *v = view_of(o);
    v->dims[dim] = len;
    v->offset = (size_t)((ptrdiff_t)v->offset + (ptrdiff_t)start * o->strides[dim]);
    release(o);
    *out = v;
    return CG_OK;
}

// ndarray.rs:513-532, 590-596 — `concatenate(Axis(dim), [a, b])`.
int cg_concat(cg_backend *, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out) {
    Consume cx(x), cy(y);
    if (!x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt))
        return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "Incompatible types for concatenation");
    if (x->rank != y->rank || dim >= (size_t)x->rank) return fail(CG_ERR_SHAPE, "concat: IncompatibleShape");
    for (int i = 0; i < x->rank; i++)
        if ((size_t)i != dim && x->dims[i] != y->dims[i]) return fail(CG_ERR_SHAPE, "concat: IncompatibleShape");
    cg_tensor *ox = unwrap_owned(x), *oy = unwrap_owned(y);
    size_t odims[CG_MAX_RANK];
    memcpy(odims, ox->dims, sizeof odims);
    odims[dim] = ox->dims[dim] + oy->dims[dim];
    cg_tensor *r = new_tensor(ox->dt, odims, ox->rank);
    auto a = dense<uint32_t>(ox), b = dense<uint32_t>(oy);
    size_t outer = 1, inner = 1;
    for (size_t i = 0; i < dim; i++) outer *= odims[i];
    for (int i = (int)dim + 1; i < ox->rank; i++) inner *= odims[i];
    size_t ca = ox->dims[dim] * inner, cb = oy->dims[dim] * inner;
    uint32_t *d = data_of<uint32_t>(r);
    for (size_t o = 0; o < outer; o++) {
        if (ca) memcpy(d + o * (ca + cb), a.data() + o * ca, ca * 4);
        if (cb) memcpy(d + o * (ca + cb) + ca, b.data() + o * cb, cb * 4);
    }
    release(ox);
    release(oy);
    *out = r;
    return CG_OK;
}

// ndarray.rs:466-487, 571-579 — `select(Axis(dim), idx)`; indices are read in logical order.
int cg_index(cg_backend *, cg_tensor *x, size_t dim, cg_tensor *indices, cg_tensor **out) {
    Consume cx(x), ci(indices);
    if (!x || !indices || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (indices->dt != CG_U32) return fail(CG_ERR_DTYPE, "Invalid input types for indexing");
    if (dim >= (size_t)x->rank) return fail(CG_ERR_RANGE, "index: axis out of range");
    cg_tensor *ox = unwrap_owned(x), *oi = unwrap_owned(indices);
    auto idx = dense<uint32_t>(oi);
    for (uint32_t i : idx)
        if (i >= ox->dims[dim]) {
            release(ox);
            release(oi);
            return fail(CG_ERR_RANGE, "index: index %u out of bounds for axis of length %zu", i, x->dims[dim]);
        }
    size_t odims[CG_MAX_RANK];
    memcpy(odims, ox->dims, sizeof odims);
    odims[dim] = idx.size();
    cg_tensor *r = new_tensor(ox->dt, odims, ox->rank);
    auto v = dense<uint32_t>(ox);
    size_t outer = 1, inner = 1;
    for (size_t i = 0; i < dim; i++) outer *= ox->dims[i];
    for (int i = (int)dim + 1; i < ox->rank; i++) inner *= ox->dims[i];
    size_t D = ox->dims[dim];
    uint32_t *d = data_of<uint32_t>(r);
    for (size_t o = 0; o < outer; o++)
        for (size_t j = 0; j < idx.size(); j++)
            if (inner) memcpy(d + (o * idx.size() + j) * inner, v.data() + (o * D + idx[j]) * inner, inner * 4);
    release(ox);
    release(oi);
    *out = r;
    return CG_OK;
}

} // extern "C"
