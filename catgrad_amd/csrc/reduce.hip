// Last-axis reductions for gfx950: sum, max, argmax, top-k, and the host-visible
// predicates behind to_bool / compare.
//
// Layout: a strided view is seen as rows x n; rows are addressed through the view's own
// outer strides, the reduced axis through its stride, so transposed / sliced inputs are
// reduced in place.  TPR lanes cooperate on one row (4, 16, 64 lanes of one wave, or the
// 256 lanes of a block); each lane strides over the row with 16-byte loads when the row
// is unit-stride and aligned; lanes combine with wave64 cross-lane shuffles and, for
// TPR = 256, a 4-entry LDS exchange.  HBM-bound: 4 B read per element, 4 B written per row.
//
// Semantics follow NdArrayBackend (catgrad/src/interpreter/backend/ndarray.rs:656-730):
//   max     folds from f32::MIN with NaN-ignoring max; u32 from 0
//   argmax  `max_by(total_cmp)`: the LAST of equal maxima; +0 > -0; +NaN greatest
//   topk    stable descending sort by total_cmp: ties in order of appearance
//   sum     f32 in tree order (the reference's own order is sequential/8-way; both are
//           within the 1e-3 relative contract), u32 wrapping
#include "common.hpp"
#include "device_utils.hpp"

#include <algorithm>
#include <mutex>

namespace cg {

namespace {

constexpr int kBlock = 256;
constexpr float kF32Min = -3.4028234663852886e38f;

struct RowsArgs {
    const char *x;
    uint32_t *out;
    uint32_t rows, n;
    int64_t sn;           // stride of the reduced axis (elements)
    uint32_t nouter;
    uint32_t od[kMaxOuter];
    FastDiv odiv[kMaxOuter];
    int64_t os[kMaxOuter];
    uint32_t vec;         // 4: rows are unit-stride and 16-byte aligned; 8: the same for rows of a narrow format (one access of
                          // 16 bytes, fp8 8 bytes, holds 8 elements)
    uint32_t fmt;         // how the elements lie in memory (kFmtWords, ...); narrow formats: reduce_rows_kernel only
};

__device__ __forceinline__ int32_t total_key(uint32_t bits) { // Rust f32::total_cmp
    int32_t b = (int32_t)bits;
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

// Accumulator per reduction kind.  K: 0 sum, 1 max, 2 argmax.  F: f32 input.
template <int K, bool F> struct Acc;

template <> struct Acc<kSum, true> {
    float v = 0.0f;
    __device__ void take(uint32_t w, uint32_t) { v += asf(w); }
    __device__ void merge(const Acc &o) { v += o.v; }
    __device__ uint32_t result() const { return asu(v); }
    __device__ Acc shfl(int m) const { Acc r; r.v = __shfl_xor(v, m); return r; }
    __device__ long long pack() const { return (long long)asu(v); }
    __device__ static Acc unpack(long long b) { Acc r; r.v = asf((uint32_t)b); return r; }
};
template <> struct Acc<kSum, false> {
    uint32_t v = 0;
    __device__ void take(uint32_t w, uint32_t) { v += w; }
    __device__ void merge(const Acc &o) { v += o.v; }
    __device__ uint32_t result() const { return v; }
    __device__ Acc shfl(int m) const { Acc r; r.v = __shfl_xor(v, m); return r; }
    __device__ long long pack() const { return (long long)v; }
    __device__ static Acc unpack(long long b) { Acc r; r.v = (uint32_t)b; return r; }
};
template <> struct Acc<kMax, true> {
    float v = kF32Min;
    __device__ void take(uint32_t w, uint32_t) { v = fmaxf(v, asf(w)); } // NaN operand ignored
    __device__ void merge(const Acc &o) { v = fmaxf(v, o.v); }
    __device__ uint32_t result() const { return asu(v); }
    __device__ Acc shfl(int m) const { Acc r; r.v = __shfl_xor(v, m); return r; }
    __device__ long long pack() const { return (long long)asu(v); }
    __device__ static Acc unpack(long long b) { Acc r; r.v = asf((uint32_t)b); return r; }
};
template <> struct Acc<kMax, false> {
    uint32_t v = 0;
    __device__ void take(uint32_t w, uint32_t) { v = w > v ? w : v; }
    __device__ void merge(const Acc &o) { v = o.v > v ? o.v : v; }
    __device__ uint32_t result() const { return v; }
    __device__ Acc shfl(int m) const { Acc r; r.v = __shfl_xor(v, m); return r; }
    __device__ long long pack() const { return (long long)v; }
    __device__ static Acc unpack(long long b) { Acc r; r.v = (uint32_t)b; return r; }
};
// argmax: (order key, index) packed so that a signed 64-bit max picks the greatest key
// and, among equal keys, the greatest index.
template <bool F> struct Acc<kArgmax, F> {
    long long c = (long long)0x8000000000000000ll;
    __device__ void take(uint32_t w, uint32_t idx) {
        int32_t key = F ? total_key(w) : (int32_t)(w ^ 0x80000000u);
        long long p = ((long long)key << 32) | (long long)idx;
        c = p > c ? p : c;
    }
    __device__ void merge(const Acc &o) { c = o.c > c ? o.c : c; }
    __device__ uint32_t result() const { return (uint32_t)(c & 0xFFFFFFFFll); }
    __device__ Acc shfl(int m) const {
        Acc r;
        int lo = __shfl_xor((int)(c & 0xFFFFFFFFll), m);
        int hi = __shfl_xor((int)(c >> 32), m);
        r.c = ((long long)hi << 32) | (long long)(uint32_t)lo;
        return r;
    }
    __device__ long long pack() const { return c; }
    __device__ static Acc unpack(long long b) { Acc r; r.c = b; return r; }
};

template <int K, bool F, int TPR> __global__ __launch_bounds__(kBlock) void reduce_rows_kernel(const RowsArgs a) {
    constexpr int RPB = kBlock / TPR; // rows per block
    const uint32_t lane = threadIdx.x % TPR;
    const uint32_t row = blockIdx.x * RPB + threadIdx.x / TPR;
    const bool live = row < a.rows;
    Acc<K, F> acc;
    if (live && a.fmt != kFmtWords) { // (the same for every lane: a launch parameter)
        Operand o;
        o.ptr = a.x;
        o.is = a.sn;
        o.uniform = 0;
        o.fmt = a.fmt;
        const int64_t base = row_offset(row, a.nouter, a.od, a.odiv, a.os);
        if (a.vec == 8) {
            const uint32_t nv = a.n / 8;
            uint32_t i = lane;
            for (; i + TPR < nv; i += 2 * TPR) { // two independent loads in flight per lane per trip
                uint32_t t0[8], t1[8];
                load_narrow<8>(o, base + 8 * (int64_t)i, t0);
                load_narrow<8>(o, base + 8 * (int64_t)(i + TPR), t1);
#pragma unroll
                for (int j = 0; j < 8; j++) acc.take(t0[j], 8 * i + j);
#pragma unroll
                for (int j = 0; j < 8; j++) acc.take(t1[j], 8 * (i + TPR) + j);
            }
            if (i < nv) {
                uint32_t t0[8];
                load_narrow<8>(o, base + 8 * (int64_t)i, t0);
#pragma unroll
                for (int j = 0; j < 8; j++) acc.take(t0[j], 8 * i + j);
            }
        } else {
            for (uint32_t i = lane; i < a.n; i += TPR) {
                uint32_t t[1];
                load_narrow<1>(o, base + (int64_t)i * a.sn, t);
                acc.take(t[0], i);
            }
        }
    } else if (live) {
        const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + row_offset(row, a.nouter, a.od, a.odiv, a.os);
        if (a.vec == 4) {
            const uint32_t nv = a.n / 4;
            // two independent 16-byte loads in flight per lane per trip
            uint32_t i = lane;
            for (; i + TPR < nv; i += 2 * TPR) {
                uint4 t0 = reinterpret_cast<const uint4 *>(p)[i];
                uint4 t1 = reinterpret_cast<const uint4 *>(p)[i + TPR];
                acc.take(t0.x, 4 * i);
                acc.take(t0.y, 4 * i + 1);
                acc.take(t0.z, 4 * i + 2);
                acc.take(t0.w, 4 * i + 3);
                acc.take(t1.x, 4 * (i + TPR));
                acc.take(t1.y, 4 * (i + TPR) + 1);
                acc.take(t1.z, 4 * (i + TPR) + 2);
                acc.take(t1.w, 4 * (i + TPR) + 3);
            }
            if (i < nv) {
                uint4 t0 = reinterpret_cast<const uint4 *>(p)[i];
                acc.take(t0.x, 4 * i);
                acc.take(t0.y, 4 * i + 1);
                acc.take(t0.z, 4 * i + 2);
                acc.take(t0.w, 4 * i + 3);
            }
        } else {
            for (uint32_t i = lane; i < a.n; i += TPR) acc.take(p[(int64_t)i * a.sn], i);
        }
    }
    constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
    for (int m = W / 2; m >= 1; m >>= 1) acc.merge(acc.shfl(m));
    if constexpr (TPR > 64) {
        __shared__ long long part[kBlock / 64];
        if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = acc.pack();
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int w = 1; w < kBlock / 64; w++) acc.merge(Acc<K, F>::unpack(part[w]));
        }
    }
    if (live && lane == 0) a.out[row] = acc.result();
}

// top-k by repeated selection: element e precedes f when key(e) > key(f), or the keys
// are equal and e appears first.  One block per row; k passes over the row.
__global__ __launch_bounds__(kBlock) void topk_kernel(const RowsArgs a, uint32_t k, uint32_t *idx_out) {
    const uint32_t row = blockIdx.x;
    const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + row_offset(row, a.nouter, a.od, a.odiv, a.os);
    __shared__ long long part[kBlock / 64];
    __shared__ long long chosen;
    long long prev = 0x7FFFFFFFFFFFFFFFll;
    for (uint32_t j = 0; j < k; j++) {
        long long best = (long long)0x8000000000000000ll;
        for (uint32_t i = threadIdx.x; i < a.n; i += kBlock) {
            uint32_t w = p[(int64_t)i * a.sn];
            long long c = ((long long)total_key(w) << 32) | (long long)(0xFFFFFFFFu - i);
            if (c < prev && c > best) best = c;
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            int lo = __shfl_xor((int)(best & 0xFFFFFFFFll), m);
            int hi = __shfl_xor((int)(best >> 32), m);
            long long o = ((long long)hi << 32) | (long long)(uint32_t)lo;
            best = o > best ? o : best;
        }
        if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = best;
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < kBlock / 64; w++) best = part[w] > best ? part[w] : best;
            uint32_t i = 0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFll);
            a.out[(uint64_t)row * k + j] = p[(int64_t)i * a.sn];
            idx_out[(uint64_t)row * k + j] = i;
            chosen = best;
        }
        __syncthreads();
        prev = chosen;
        __syncthreads();
    }
}

struct AnyArgs {
    EwGeom g;
    Operand x, y;
    uint32_t *flag;
};

// MODE 0: any(x > 0) (f32) / any(x != 0) (u32).  MODE 1: any(x != y) with IEEE
// inequality for f32 (NaN differs from everything, -0 equals +0).
template <int MODE, bool F, int VEC> __global__ __launch_bounds__(kBlock) void any_kernel(const AnyArgs a) {
    uint64_t v64 = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v64 >= a.g.total) return;
    uint32_t v = (uint32_t)v64;
    uint32_t row = fastdiv(v, a.g.ipr_div);
    int64_t e = (int64_t)(v - row * a.g.ipr) * VEC;
    int64_t ox = e * a.x.is, oy = e * a.y.is;
    for (uint32_t d = 0; d < a.g.nouter; d++) {
        uint32_t q = fastdiv(row, a.g.odiv[d]);
        int64_t i = (int64_t)(row - q * a.g.od[d]);
        row = q;
        ox += i * a.x.os[d];
        oy += i * a.y.os[d];
    }
    uint32_t xs[VEC], ys[VEC];
    load_words<VEC>(a.x, ox, xs);
    if (MODE == 1) load_words<VEC>(a.y, oy, ys);
    bool hit = false;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        if (MODE == 0)
            hit |= F ? asf(xs[j]) > 0.0f : xs[j] != 0u;
        else
            hit |= F ? !(asf(xs[j]) == asf(ys[j])) : xs[j] != ys[j];
    }
    if (hit) *a.flag = 1u;
}

// native: a view of a narrow buffer is described as it lies in memory (for reduce_rows_kernel); else as 32-bit words
int fill_rows_args(const cg_tensor *x, RowsArgs *a, bool native = false) {
    memset(a, 0, sizeof *a);
    const void *p;
    int fmt = kFmtWords;
    int rc = native ? device_ptr_fmt(x, &p, &fmt) : device_ptr(x, &p);
    if (rc) return rc;
    a->fmt = (uint32_t)fmt;
    a->x = static_cast<const char *>(p);
    int r = x->rank;
    int64_t n = x->dims[r - 1];
    a->sn = x->uniform ? 0 : x->strides[r - 1];
    // collapse the outer axes of this one view
    int64_t dims[kMaxRank], st[kMaxRank];
    int w = 0;
    for (int i = 0; i < r - 1; i++) {
        if (x->dims[i] == 1) continue;
        int64_t s = x->uniform ? 0 : x->strides[i];
        if (w > 0 && st[w - 1] == s * x->dims[i]) {
            dims[w - 1] *= x->dims[i];
            st[w - 1] = s;
        } else {
            dims[w] = x->dims[i];
            st[w] = s;
            w++;
        }
    }
    int64_t rows = 1;
    for (int i = 0; i < w; i++) rows *= dims[i];
    if (rows > 0xFFFFFFFFll || n > 0x3FFFFFFFll) return fail(CG_ERR_UNSUPPORTED, "reduction extents above 2^32-1");
    a->rows = (uint32_t)rows;
    a->n = (uint32_t)n;
    a->nouter = (uint32_t)w;
    const int64_t per = fmt == kFmtWords ? 4 : 8; // elements per vector access
    bool vec = !x->uniform && a->sn == 1 && n % per == 0 && reinterpret_cast<uintptr_t>(p) % (fmt == kFmtF8 ? 8 : 16) == 0;
    for (int d = 0; d < w; d++) {
        a->od[d] = (uint32_t)dims[w - 1 - d];
        a->odiv[d] = make_fastdiv(a->od[d]);
        a->os[d] = st[w - 1 - d];
        if (a->os[d] % per) vec = false;
    }
    a->vec = vec ? (uint32_t)per : 1;
    return CG_OK;
}

// Few, long rows (the arg-max over a 128 K vocabulary for a handful of sequences): a row per
// workgroup would leave most of the chip idle, so every row is cut into segments, a workgroup
// reduces one segment to a packed accumulator, and a second small kernel merges a row's segments.
template <int K, bool F>
__global__ __launch_bounds__(kBlock) void reduce_segments_kernel(const RowsArgs a, long long *part, uint32_t seglen) {
    const uint32_t row = blockIdx.y, seg = blockIdx.x;
    const uint32_t lo = seg * seglen, hi = min(a.n, lo + seglen);
    const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + row_offset(row, a.nouter, a.od, a.odiv, a.os);
    Acc<K, F> acc;
    if (a.vec == 4) { // seglen is a multiple of 4
        for (uint32_t i = lo / 4 + threadIdx.x; i < hi / 4; i += kBlock) {
            const uint4 t = reinterpret_cast<const uint4 *>(p)[i];
            acc.take(t.x, 4 * i);
            acc.take(t.y, 4 * i + 1);
            acc.take(t.z, 4 * i + 2);
            acc.take(t.w, 4 * i + 3);
        }
        for (uint32_t i = hi / 4 * 4 + threadIdx.x; i < hi; i += kBlock) acc.take(p[i], i); // tail of the last segment
    } else {
        for (uint32_t i = lo + threadIdx.x; i < hi; i += kBlock) acc.take(p[(int64_t)i * a.sn], i);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc.merge(acc.shfl(m));
    __shared__ long long wpart[kBlock / 64];
    if (threadIdx.x % 64 == 0) wpart[threadIdx.x / 64] = acc.pack();
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kBlock / 64; w++) acc.merge(Acc<K, F>::unpack(wpart[w]));
        part[(uint64_t)row * gridDim.x + seg] = acc.pack();
    }
}

template <int K, bool F>
__global__ __launch_bounds__(64) void reduce_segments_final_kernel(const long long *part, uint32_t *out, uint32_t segs) {
    const uint32_t row = blockIdx.x;
    Acc<K, F> acc;
    for (uint32_t s = threadIdx.x; s < segs; s += 64) acc.merge(Acc<K, F>::unpack(part[(uint64_t)row * segs + s]));
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc.merge(acc.shfl(m));
    if (threadIdx.x == 0) out[row] = acc.result();
}

// The reduced axis is not the unit-stride one, the innermost of the other axes is (the last axis of a transposed view:
// a sum over the rows of a row-major matrix).  A lane per output would read 4 bytes per 128-byte line; here the lanes of a
// wave sit on neighbouring OUTPUTS (16 bytes each when aligned) and every lane walks the reduced axis, so each step of a
// wave reads one contiguous kilobyte.  The four waves of a workgroup split the steps and meet in LDS; few outputs with a
// long axis are also cut into segments over grid.y, merged by a second small kernel.  HBM-bound: 4 bytes per element.
template <int K, bool F, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_cols_kernel(const RowsArgs a, uint32_t tiles0, uint32_t seglen, uint32_t segs,
                                                             long long *part) {
    constexpr uint32_t CH = 64 * VEC; // outputs per workgroup
    const uint32_t lx = threadIdx.x % 64, ly = threadIdx.x / 64;
    const uint32_t tile = blockIdx.x % tiles0;
    uint32_t rest = blockIdx.x / tiles0;
    const uint32_t rest_index = rest;
    int64_t base = 0;
    for (uint32_t d = 1; d < a.nouter; d++) {
        const uint32_t q = fastdiv(rest, a.odiv[d]);
        base += (int64_t)(rest - q * a.od[d]) * a.os[d];
        rest = q;
    }
    const uint32_t r0 = tile * CH + lx * VEC;
    const uint32_t lo = blockIdx.y * seglen, hi = min(a.n, lo + seglen);
    const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + base + r0;
    Acc<K, F> acc[VEC];
    if (r0 < a.od[0]) {
        if constexpr (VEC == 4) {
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            uint32_t i = lo + ly;
            for (; i + 28 < hi; i += 32) { // eight loads in flight per lane
                u4 t[8];
#pragma unroll
                for (int u = 0; u < 8; u++) t[u] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p + (int64_t)(i + 4 * u) * a.sn));
#pragma unroll
                for (int u = 0; u < 8; u++)
#pragma unroll
                    for (int v = 0; v < 4; v++) acc[v].take(t[u][v], i + 4 * u);
            }
            for (; i < hi; i += 4) {
                const u4 t = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p + (int64_t)i * a.sn));
#pragma unroll
                for (int v = 0; v < 4; v++) acc[v].take(t[v], i);
            }
        } else {
            for (uint32_t i = lo + ly; i < hi; i += 4) acc[0].take(p[(int64_t)i * a.sn], i);
        }
    }
    __shared__ long long meet[3][CH];
    if (ly > 0) {
#pragma unroll
        for (int v = 0; v < VEC; v++) meet[ly - 1][lx * VEC + v] = acc[v].pack();
    }
    __syncthreads();
    if (ly == 0 && r0 < a.od[0]) {
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            for (int w = 0; w < 3; w++) acc[v].merge(Acc<K, F>::unpack(meet[w][lx * VEC + v]));
            if (r0 + v < a.od[0]) {
                const uint64_t row = (uint64_t)rest_index * a.od[0] + r0 + v;
                if (segs == 1) a.out[row] = acc[v].result();
                else part[(uint64_t)blockIdx.y * a.rows + row] = acc[v].pack();
            }
        }
    }
}

// The same in ONE launch when there are outputs enough for every compute unit: a workgroup owns 32 neighbouring outputs (a
// 128-byte line per step of the reduced axis), eight lanes of 16 bytes side by side and 32 groups of lanes that take the
// steps in turn, eight loads in flight per lane; the groups meet in LDS and are merged in a fixed order.  No segments, no
// partial results in memory, no second launch.
template <int K, bool F>
__global__ __launch_bounds__(kBlock) void reduce_cols_narrow_kernel(const RowsArgs a, uint32_t tiles0) {
    constexpr uint32_t CH = 32, G = kBlock / 8; // outputs per workgroup, groups of lanes
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint32_t lx = threadIdx.x % 8, ly = threadIdx.x / 8;
    const uint32_t tile = blockIdx.x % tiles0;
    uint32_t rest = blockIdx.x / tiles0;
    const uint32_t rest_index = rest;
    int64_t base = 0;
    for (uint32_t d = 1; d < a.nouter; d++) {
        const uint32_t q = fastdiv(rest, a.odiv[d]);
        base += (int64_t)(rest - q * a.od[d]) * a.os[d];
        rest = q;
    }
    const uint32_t r0 = tile * CH + lx * 4; // (od[0] is a multiple of 32)
    const uint32_t *p = reinterpret_cast<const uint32_t *>(a.x) + base + r0;
    Acc<K, F> acc[4];
    uint32_t i = ly;
    for (; i + 7 * G < a.n; i += 8 * G) {
        u4 t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p + (int64_t)(i + u * G) * a.sn));
#pragma unroll
        for (int u = 0; u < 8; u++)
#pragma unroll
            for (int v = 0; v < 4; v++) acc[v].take(t[u][v], i + u * G);
    }
    for (; i < a.n; i += G) {
        const u4 t = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p + (int64_t)i * a.sn));
#pragma unroll
        for (int v = 0; v < 4; v++) acc[v].take(t[v], i);
    }
    __shared__ long long meet[G][CH];
#pragma unroll
    for (int v = 0; v < 4; v++) meet[ly][lx * 4 + v] = acc[v].pack();
    __syncthreads();
    if (threadIdx.x < CH) {
        Acc<K, F> r = Acc<K, F>::unpack(meet[0][threadIdx.x]);
        for (uint32_t g = 1; g < G; g++) r.merge(Acc<K, F>::unpack(meet[g][threadIdx.x]));
        a.out[(uint64_t)rest_index * a.od[0] + tile * CH + threadIdx.x] = r.result();
    }
}

template <int K, bool F>
__global__ __launch_bounds__(kBlock) void reduce_cols_final_kernel(const long long *part, uint32_t *out, uint32_t segs, uint32_t rows) {
    // 64 neighbouring outputs per workgroup; the four waves split the segments (independent loads) and meet in LDS
    const uint32_t lx = threadIdx.x % 64, ly = threadIdx.x / 64;
    const uint32_t row = blockIdx.x * 64 + lx;
    Acc<K, F> acc;
    if (row < rows)
        for (uint32_t s = ly; s < segs; s += 4) acc.merge(Acc<K, F>::unpack(part[(uint64_t)s * rows + row]));
    __shared__ long long meet[3][64];
    if (ly > 0) meet[ly - 1][lx] = acc.pack();
    __syncthreads();
    if (ly == 0 && row < rows) {
        for (int w = 0; w < 3; w++) acc.merge(Acc<K, F>::unpack(meet[w][lx]));
        out[row] = acc.result();
    }
}

template <int K, bool F> int launch_cols(cg_backend *be, const RowsArgs &a) {
    const uint32_t R0 = a.od[0];
    bool vec = R0 % 4 == 0 && reinterpret_cast<uintptr_t>(a.x) % 16 == 0 && a.sn % 4 == 0;
    for (uint32_t d = 1; d < a.nouter; d++) vec = vec && a.os[d] % 4 == 0;
    const uint32_t ch = vec ? 256 : 64, tiles0 = (R0 + ch - 1) / ch;
    const uint64_t blocks = (uint64_t)tiles0 * (a.rows / R0);
    if (blocks > 0x7FFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "reduction extents above 2^31-1 workgroups");
    // outputs enough for a workgroup of 32 on every compute unit and a long axis: one launch (env CG_COLS_NARROW=0: never)
    static const bool narrow_allowed = [] { const char *e = getenv("CG_COLS_NARROW"); return !(e && e[0] == '0'); }();
    if (narrow_allowed && vec && R0 % 32 == 0 && (uint64_t)(R0 / 32) * (a.rows / R0) >= 256 && a.n >= 1024) {
        const uint64_t nblocks = (uint64_t)(R0 / 32) * (a.rows / R0);
        if (nblocks <= 0x7FFFFFFFull) {
            hipLaunchKernelGGL((reduce_cols_narrow_kernel<K, F>), dim3((uint32_t)nblocks), dim3(kBlock), 0, be->stream, a, R0 / 32);
            hipError_t ne = hipGetLastError();
            return ne == hipSuccess ? CG_OK : hip_fail(ne, "column reduction launch");
        }
    }
    // segments along the reduced axis until about 1024 workgroups are in flight (measured best on 8192 x 8192: 54.5 us against
    // 60 at 512 and 56.5 at 2048 and 4096; env CG_COLS_BLOCKS for measurements), at least 64 steps each
    static const uint64_t want = [] { const char *e = getenv("CG_COLS_BLOCKS"); return e ? (uint64_t)atoll(e) : 1024ull; }();
    uint32_t segs = (uint32_t)std::min<uint64_t>(std::min<uint64_t>((want + blocks - 1) / blocks, (a.n + 63) / 64), 64);
    if (segs < 1) segs = 1;
    const uint32_t seglen = ((a.n + segs - 1) / segs + 3) / 4 * 4;
    segs = (a.n + seglen - 1) / seglen;
    void *part = nullptr;
    size_t cls = 0;
    if (segs > 1) {
        int rc = be->pool.alloc((size_t)segs * a.rows * sizeof(long long), &part, &cls);
        if (rc) return rc;
    }
    const dim3 grid((uint32_t)blocks, segs);
    if (vec)
        hipLaunchKernelGGL((reduce_cols_kernel<K, F, 4>), grid, dim3(kBlock), 0, be->stream, a, tiles0, seglen, segs, static_cast<long long *>(part));
    else
        hipLaunchKernelGGL((reduce_cols_kernel<K, F, 1>), grid, dim3(kBlock), 0, be->stream, a, tiles0, seglen, segs, static_cast<long long *>(part));
    if (segs > 1) {
        hipLaunchKernelGGL((reduce_cols_final_kernel<K, F>), dim3((a.rows + 63) / 64), dim3(kBlock), 0, be->stream,
                           static_cast<const long long *>(part), a.out, segs, a.rows);
        be->pool.free(part, cls); // stream-ordered: later users queue behind the merge
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "column reduction launch");
}

// Which kernels launch_rows picks: 1 the column kernels, 2 the segmented ones, 0 a row per 4 .. 256 lanes.
static int rows_route(const RowsArgs &a) {
    if (a.sn != 1 && a.nouter >= 1 && a.os[0] == 1 && a.od[0] >= 16 && a.n >= 8) return 1;
    return a.rows <= 64 && a.n >= 32768 ? 2 : 0;
}

template <int K, bool F> int launch_rows(cg_backend *be, const RowsArgs &a) {
    if (rows_route(a) != 0 && a.fmt != kFmtWords) return fail(CG_ERR_ARG, "internal error: a narrow operand in a reduction kernel that reads words");
    if (rows_route(a) == 1) return launch_cols<K, F>(be, a);
    if (rows_route(a) == 2) {
        uint32_t segs = std::min<uint32_t>(256, (a.n + 1023) / 1024);
        const uint32_t seglen = ((a.n + segs - 1) / segs + 3) / 4 * 4;
        segs = (a.n + seglen - 1) / seglen;
        void *part = nullptr;
        size_t cls = 0;
        int rc = be->pool.alloc((size_t)a.rows * segs * sizeof(long long), &part, &cls);
        if (rc) return rc;
        hipLaunchKernelGGL((reduce_segments_kernel<K, F>), dim3(segs, a.rows), dim3(kBlock), 0, be->stream, a,
                           static_cast<long long *>(part), seglen);
        hipLaunchKernelGGL((reduce_segments_final_kernel<K, F>), dim3(a.rows), dim3(64), 0, be->stream,
                           static_cast<const long long *>(part), a.out, segs);
        be->pool.free(part, cls); // stream-ordered: later users queue behind the merge
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? CG_OK : hip_fail(e, "segmented reduction launch");
    }
    // lanes per row: enough that a lane sees about eight elements, within {4,16,64,256}
    uint32_t want = (a.n + 7) / 8;
    int tpr = want <= 4 ? 4 : want <= 16 ? 16 : want <= 64 ? 64 : 256;
    uint32_t rpb = kBlock / tpr;
    dim3 grid((a.rows + rpb - 1) / rpb), block(kBlock);
    switch (tpr) {
    case 4: hipLaunchKernelGGL((reduce_rows_kernel<K, F, 4>), grid, block, 0, be->stream, a); break;
    case 16: hipLaunchKernelGGL((reduce_rows_kernel<K, F, 16>), grid, block, 0, be->stream, a); break;
    case 64: hipLaunchKernelGGL((reduce_rows_kernel<K, F, 64>), grid, block, 0, be->stream, a); break;
    default: hipLaunchKernelGGL((reduce_rows_kernel<K, F, 256>), grid, block, 0, be->stream, a); break;
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "reduction launch");
}

} // namespace

// ---- arg-max for callers that cannot allocate -------------------------------------------------------------------
// The segmented arg-max above takes its per-segment results from the pool.  This variant keeps them in a fixed array
// in device memory instead, so that the call allocates nothing: every GPU the library runs on holds one copy of the
// array (128 KiB) until the process ends.  In host code the array's name stands for no device address; the address
// on a given device comes from hipGetSymbolAddress, asked once per device with that device current.
constexpr uint32_t kNoAllocMaxParts = 16384; // rows x segments
static __device__ __align__(256) long long scratch[kNoAllocMaxParts];

constexpr int kNoAllocMaxDevices = 64;
static std::mutex g_scratch_mu;
static std::atomic<long long *> g_scratch_ptr[kNoAllocMaxDevices] = {};

// Set-up (loads the code object on `device` if need be, so it is not for code under stream capture): leaves the
// calling thread's current device as it found it.
int noalloc_setup(int device) {
    if (device < 0 || device >= kNoAllocMaxDevices) return fail(CG_ERR_ARG, "device %d out of range", device);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return CG_OK;
    int prev = -1;
    CG_HIP(hipGetDevice(&prev));
    CG_HIP(hipSetDevice(device));
    long long *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (prev != device) (void)hipSetDevice(prev);
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!ptr) return fail(CG_ERR_DEVICE, "no device address for the scratch array on device %d", device);
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
    return CG_OK;
}

int launch_reduce(cg_backend *be, int kind, const cg_tensor *x, cg_tensor *out) {
    if (int frc = flush_deferred(be)) return frc;
    RowsArgs a;
    int rc = fill_rows_args(x, &a, true);
    if (!rc && a.fmt != kFmtWords && rows_route(a) != 0) rc = fill_rows_args(x, &a); // those kernels read words
    if (rc) return rc;
    a.out = static_cast<uint32_t *>(out->buf->ptr);
    bool f = is_f(x->dt);
    ProfScope prof(be, CG_K_REDUCE, distinct_bytes(x) + distinct_bytes(out));
    switch (kind) {
    case kSum: return f ? launch_rows<kSum, true>(be, a) : launch_rows<kSum, false>(be, a);
    case kMax: return f ? launch_rows<kMax, true>(be, a) : launch_rows<kMax, false>(be, a);
    case kArgmax: return f ? launch_rows<kArgmax, true>(be, a) : launch_rows<kArgmax, false>(be, a);
    default: return fail(CG_ERR_ARG, "unknown reduction %d", kind);
    }
}

int launch_topk(cg_backend *be, const cg_tensor *x, int64_t k, cg_tensor *vals, cg_tensor *idxs) {
    if (int frc = flush_deferred(be)) return frc;
    RowsArgs a;
    int rc = fill_rows_args(x, &a);
    if (rc) return rc;
    a.out = static_cast<uint32_t *>(vals->buf->ptr);
    hipLaunchKernelGGL(topk_kernel, dim3(a.rows), dim3(kBlock), 0, be->stream, a, (uint32_t)k,
                       static_cast<uint32_t *>(idxs->buf->ptr));
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "topk launch");
}

static int launch_any(cg_backend *be, int mode, const cg_tensor *x, const cg_tensor *y) {
    if (int frc = flush_deferred(be)) return frc;
    int rc = launch_fill_word(be, be->flag_dev, 0);
    if (rc) return rc;
    const cg_tensor *views[2] = {x, y ? y : x};
    AnyArgs a;
    memset(&a, 0, sizeof a);
    Operand ops[2];
    rc = plan_elementwise(views, 2, &a.g, ops);
    if (rc) return rc;
    a.x = ops[0];
    a.y = ops[1];
    a.flag = be->flag_dev;
    dim3 grid((uint32_t)((a.g.total + kBlock - 1) / kBlock)), block(kBlock);
    bool f = is_f(x->dt);
#define CG_ANY(MODE, F, VEC) hipLaunchKernelGGL((any_kernel<MODE, F, VEC>), grid, block, 0, be->stream, a)
    if (mode == 0) {
        if (a.g.vec == 4) { if (f) CG_ANY(0, true, 4); else CG_ANY(0, false, 4); }
        else { if (f) CG_ANY(0, true, 1); else CG_ANY(0, false, 1); }
    } else {
        if (a.g.vec == 4) { if (f) CG_ANY(1, true, 4); else CG_ANY(1, false, 4); }
        else { if (f) CG_ANY(1, true, 1); else CG_ANY(1, false, 1); }
    }
#undef CG_ANY
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "predicate launch");
}

int launch_any_positive(cg_backend *be, const cg_tensor *x) { return launch_any(be, 0, x, nullptr); }
int launch_any_diff(cg_backend *be, const cg_tensor *x, const cg_tensor *y) { return launch_any(be, 1, x, y); }

} // namespace cg

extern "C" int cg_noalloc_setup(int device) { return cg::noalloc_setup(device); }

// Arg-max over the rows of a dense [rows, n] array of 32-bit words at `x` (device memory) into out[rows] (device
// memory), queued on `stream`; nothing is allocated and nothing waits.  Same kernels as the segmented arg-max behind
// cg_argmax, with the per-segment results in the library's fixed scratch array, whose address on `device` set-up
// (cg_noalloc_setup, or cg_backend_create on that device) must have asked for before: the call itself resolves nothing.
extern "C" int cg_argmax_rows_noalloc(int device, cg_dtype dtype, const void *x, size_t rows, size_t n, uint32_t *out,
                                      void *stream) {
    using namespace cg;
    if (dtype != CG_F32 && dtype != CG_U32 && dtype != CG_F16 && dtype != CG_BF16 && dtype != CG_F8)
        return fail(CG_ERR_UNSUPPORTED, "unknown dtype");
    if (n == 0) return fail(CG_ERR_SHAPE, "argmax: called `Option::unwrap()` on a `None` value (empty axis)");
    if (rows == 0) return CG_OK;
    if (!x || !out) return fail(CG_ERR_ARG, "null argument");
    if (n > 0x3FFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "argmax without allocation: rows longer than 2^30-1 elements");
    uint32_t segs = std::min<uint32_t>(256, (uint32_t)((n + 1023) / 1024));
    const uint32_t seglen = (uint32_t)(((n + segs - 1) / segs + 3) / 4 * 4);
    segs = (uint32_t)((n + seglen - 1) / seglen);
    if (rows > 65535 || rows * segs > kNoAllocMaxParts)
        return fail(CG_ERR_UNSUPPORTED,
                    "argmax without allocation: %zu rows x %u segments exceed the fixed scratch of %u partial results "
                    "(rows x ceil(n / 1024), segments capped at 256)",
                    rows, segs, kNoAllocMaxParts);
    if (device < 0 || device >= kNoAllocMaxDevices) return fail(CG_ERR_ARG, "device %d out of range", device);
    long long *part = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!part)
        return fail(CG_ERR_ARG, "argmax without allocation: device %d is not set up (call cg_noalloc_setup or cg_backend_create "
                                "on it first, outside any stream capture)", device);
    // the launches go to `device`; the calling thread's current device is put back before the call returns
    int prev = -1;
    CG_HIP(hipGetDevice(&prev));
    if (prev != device) CG_HIP(hipSetDevice(device));
    RowsArgs a;
    memset(&a, 0, sizeof a);
    a.x = static_cast<const char *>(x);
    a.out = out;
    a.rows = (uint32_t)rows;
    a.n = (uint32_t)n;
    a.sn = 1;
    a.nouter = 1;
    a.od[0] = (uint32_t)rows;
    a.odiv[0] = make_fastdiv(a.od[0]);
    a.os[0] = (int64_t)n;
    a.vec = (n % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) ? 4 : 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // every partial result the second kernel reads is written by the first: nothing has to start at zero
    if (dtype == CG_U32) {
        hipLaunchKernelGGL((reduce_segments_kernel<kArgmax, false>), dim3(segs, a.rows), dim3(kBlock), 0, s, a, part, seglen);
        hipLaunchKernelGGL((reduce_segments_final_kernel<kArgmax, false>), dim3(a.rows), dim3(64), 0, s, part, out, segs);
    } else {
        hipLaunchKernelGGL((reduce_segments_kernel<kArgmax, true>), dim3(segs, a.rows), dim3(kBlock), 0, s, a, part, seglen);
        hipLaunchKernelGGL((reduce_segments_final_kernel<kArgmax, true>), dim3(a.rows), dim3(64), 0, s, part, out, segs);
    }
    hipError_t e = hipGetLastError();
    if (prev != device) (void)hipSetDevice(prev);
    return e == hipSuccess ? CG_OK : hip_fail(e, "argmax without allocation: launch");
}
