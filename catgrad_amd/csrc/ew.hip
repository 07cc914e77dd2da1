// Element-wise, cast, strided-copy, gather and iota kernels for gfx950.
//
// One kernel shape serves every map over views of a common logical shape: the host
// collapses the iteration space (plan_elementwise) to "rows x inner"; a work item is
// one 16-byte vector (or one element) of the output; each lane handles UNROLL items a
// block-stride apart so that every wave keeps several 16-byte loads per operand in
// flight; operands are addressed through their own strides, so broadcast (stride 0),
// transposed and sliced views are consumed in place and constants arrive as kernel
// arguments.  All of these kernels are HBM-bound: 4 B read per operand element + 4 B
// written per output element.
//
// Arithmetic follows NdArrayBackend (catgrad/src/interpreter/backend/ndarray.rs):
// IEEE f32 with one rounding per operation (the file is compiled with
// -ffp-contract=off), accurate libm-grade sin/cos/exp/log/pow, wrapping u32.
#include "ew_kernel.hpp"

#include <algorithm>
#include <type_traits>

namespace cg {

namespace {

__global__ void arange_kernel(uint32_t *out, uint32_t n) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = i;
}

__global__ void fill_word_kernel(uint32_t *p, uint32_t bits) { *p = bits; }

// 8 bfloat16 per lane and trip: one 16-byte load, two 16-byte stores.  HBM-bound: 2 B read + 4 B written per element.
__global__ __launch_bounds__(kBlock) void bf16_widen_kernel(const uint16_t *__restrict__ src, uint32_t *__restrict__ dst,
                                                            uint64_t n) {
    const uint64_t groups = n / 8;
    for (uint64_t g = (uint64_t)blockIdx.x * kBlock + threadIdx.x; g < groups; g += (uint64_t)gridDim.x * kBlock) {
        const uint4 v = reinterpret_cast<const uint4 *>(src)[g];
        uint4 lo, hi;
        lo.x = v.x << 16; lo.y = v.x & 0xFFFF0000u; lo.z = v.y << 16; lo.w = v.y & 0xFFFF0000u;
        hi.x = v.z << 16; hi.y = v.z & 0xFFFF0000u; hi.z = v.w << 16; hi.w = v.w & 0xFFFF0000u;
        reinterpret_cast<uint4 *>(dst)[2 * g] = lo;
        reinterpret_cast<uint4 *>(dst)[2 * g + 1] = hi;
    }
    if (blockIdx.x == 0 && threadIdx.x < n % 8) { // ragged tail
        const uint64_t i = groups * 8 + threadIdx.x;
        dst[i] = (uint32_t)src[i] << 16;
    }
}

// out[o, j, :] = x[o, idx[j], :]  with x row-major [outer, D, inner]
template <int VEC>
__global__ __launch_bounds__(kBlock) void gather_kernel(const uint32_t *__restrict__ x, const uint32_t *__restrict__ idx,
                                                        int64_t idx_stride, uint32_t *__restrict__ out, uint32_t D,
                                                        uint32_t inner, FastDiv ipr_div, uint32_t ipr, FastDiv j_div,
                                                        uint32_t J, uint64_t total, uint32_t *fault) {
    uint64_t v64 = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v64 >= total) return;
    uint32_t v = (uint32_t)v64;
    uint32_t row = fastdiv(v, ipr_div);
    uint32_t c = (v - row * ipr) * VEC;
    uint32_t o = fastdiv(row, j_div);
    uint32_t j = row - o * J;
    uint32_t id = idx[(int64_t)j * idx_stride];
    uint32_t *dst = out + (uint64_t)row * inner + c;
    if (id >= D) { // the reference panics (ndarray `select`); report and write zeros
        *fault = kFaultIndexRange;
        if (VEC == 4)
            *reinterpret_cast<uint4 *>(dst) = make_uint4(0, 0, 0, 0);
        else
            *dst = 0;
        return;
    }
    const uint32_t *src = x + ((uint64_t)o * D + id) * inner + c;
    if (VEC == 4)
        *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src);
    else
        *dst = *src;
}

} // namespace

// ---- copies that transpose ------------------------------------------------------------------------------------------
// A strided copy whose source is unit-stride along another axis than its destination (the row-major copy of a
// transposed view: `reshape` of [B, h, S, hd] seen as [B, S, h, hd], ndarray.rs:545-569) would read 4 bytes per 128-byte
// line with one of the two.  Here a workgroup moves a 64 x 64 tile through LDS: 16-byte loads along the source's
// unit-stride axis, 16-byte stores along the destination's.  HBM-bound: 8 bytes per element.
struct TransposeArgs {
    const char *src;
    char *dst;
    uint32_t I, T;            // extents of the destination's fast axis (i) and of the source's fast axis (t)
    int64_t src_is, dst_ts;   // source stride along i, destination stride along t (the other two are 1), in elements
    uint32_t tiles_i, tiles_t;
    uint32_t nrest;           // further axes, innermost first
    uint32_t rd[kMaxOuter];
    FastDiv rdiv[kMaxOuter];
    int64_t src_rs[kMaxOuter], dst_rs[kMaxOuter];
    uint32_t vec;             // 1: every 16-byte access of a whole tile is aligned
};

// EB: bytes per element (4: 32-bit words; 2 / 1: the narrow formats, moved as they lie).  A 16-byte piece holds 16 / EB
// elements; in LDS every element has a 32-bit word of its own, so the exchange is the same for every width.
template <int EB> __global__ __launch_bounds__(kBlock) void transpose_copy_kernel(const TransposeArgs a) {
    constexpr int TS = 64, PITCH = TS + 1;
    constexpr int PER = 16 / EB, PIECES = TS / PER, RPP = kBlock / PIECES, PASSES = TS / RPP;
    typedef typename std::conditional<EB == 4, uint32_t, typename std::conditional<EB == 2, uint16_t, uint8_t>::type>::type E;
    __shared__ uint32_t tile[TS][PITCH]; // [i][t]
    // tiles are walked along diagonals: neighbouring workgroups then differ in BOTH their source rows and their
    // destination rows, which spreads the strided side of the copy over the memory channels
    uint32_t blk = blockIdx.x;
    const uint32_t tt = blk % a.tiles_t;
    blk /= a.tiles_t;
    const uint32_t ti = (blk % a.tiles_i + tt) % a.tiles_i;
    uint32_t rest = blk / a.tiles_i;
    int64_t so = 0, dofs = 0;
    for (uint32_t d = 0; d < a.nrest; d++) {
        const uint32_t q = fastdiv(rest, a.rdiv[d]);
        const int64_t i = (int64_t)(rest - q * a.rd[d]);
        rest = q;
        so += i * a.src_rs[d];
        dofs += i * a.dst_rs[d];
    }
    const E *const src = reinterpret_cast<const E *>(a.src);
    E *const dst = reinterpret_cast<E *>(a.dst);
    const uint32_t i0 = ti * TS, t0 = tt * TS;
    const bool whole = a.vec && i0 + TS <= a.I && t0 + TS <= a.T;
    const uint32_t q = threadIdx.x % PIECES, r = threadIdx.x / PIECES; // a row of 16-byte pieces, RPP rows per pass
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    if (whole) {
        u4 v[PASSES];
#pragma unroll
        for (int k = 0; k < PASSES; k++) // row i0 + r + RPP k of the source, elements t0 + PER q .. + PER - 1
            v[k] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(src + so + (int64_t)(i0 + r + RPP * k) * a.src_is + t0 + PER * q));
#pragma unroll
        for (int k = 0; k < PASSES; k++) {
            uint32_t *row = tile[r + RPP * k];
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const uint32_t word = v[k][j * EB / 4];
                row[PER * q + j] = EB == 4 ? word : EB == 2 ? (word >> (16 * (j % 2))) & 0xFFFFu : (word >> (8 * (j % 4))) & 0xFFu;
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < PASSES; k++) { // row t0 + r + RPP k of the destination, elements i0 + PER q .. + PER - 1
            const uint32_t t = r + RPP * k;
            u4 o = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const uint32_t e = tile[PER * q + j][t];
                o[j * EB / 4] |= EB == 4 ? e : EB == 2 ? e << (16 * (j % 2)) : e << (8 * (j % 4));
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u4 *>(dst + dofs + (int64_t)(t0 + t) * a.dst_ts + i0 + PER * q));
        }
        return;
    }
    // ragged or unaligned tile: element by element, still along the fast axis of each side
    const uint32_t c = threadIdx.x % 64, w = threadIdx.x / 64;
    for (uint32_t k = w; k < TS; k += 4)
        if (i0 + k < a.I && t0 + c < a.T) tile[k][c] = src[so + (int64_t)(i0 + k) * a.src_is + t0 + c];
    __syncthreads();
    for (uint32_t k = w; k < TS; k += 4)
        if (t0 + k < a.T && i0 + c < a.I) dst[dofs + (int64_t)(t0 + k) * a.dst_ts + i0 + c] = (E)tile[c][k];
}

// Takes a planned copy (a.out, a.in[0]) when it is a transposition worth tiling; kDeclined otherwise.
static int try_transpose_copy(cg_backend *be, const EwArgs &a) {
    const EwGeom &g = a.g;
    if (a.in[0].uniform || a.out.is != 1 || a.in[0].is == 1 || a.in[0].is == 0 || g.nouter < 1) return kDeclined;
    if (a.in[0].fmt != a.out.fmt || a.round) return kDeclined; // (elements are moved as they lie)
    const int64_t eb = (int64_t)fmt_bytes((int)a.out.fmt), per = 16 / eb; // bytes per element, elements per 16-byte access
    int td = -1; // the outer axis along which the source is unit-stride
    for (uint32_t d = 0; d < g.nouter; d++)
        if (a.in[0].os[d] == 1 && g.od[d] >= 16) td = (int)d;
    if (td < 0 || g.inner < 16) return kDeclined;
    TransposeArgs t;
    memset(&t, 0, sizeof t);
    t.src = a.in[0].ptr;
    t.dst = const_cast<char *>(a.out.ptr);
    t.I = g.inner;
    t.T = g.od[td];
    t.src_is = a.in[0].is;
    t.dst_ts = a.out.os[td];
    if (t.src_is < 0 || t.dst_ts <= 0) return kDeclined;
    t.tiles_i = (t.I + 63) / 64;
    t.tiles_t = (t.T + 63) / 64;
    uint64_t blocks = (uint64_t)t.tiles_i * t.tiles_t;
    bool vec = reinterpret_cast<uintptr_t>(t.src) % 16 == 0 && reinterpret_cast<uintptr_t>(t.dst) % 16 == 0 && t.src_is % per == 0 &&
               t.dst_ts % per == 0;
    for (uint32_t d = 0; d < g.nouter; d++) {
        if ((int)d == td) continue;
        t.rd[t.nrest] = g.od[d];
        t.rdiv[t.nrest] = make_fastdiv(g.od[d]);
        t.src_rs[t.nrest] = a.in[0].os[d];
        t.dst_rs[t.nrest] = a.out.os[d];
        if (a.in[0].os[d] % per || a.out.os[d] % per) vec = false;
        blocks *= g.od[d];
        t.nrest++;
    }
    if (blocks == 0 || blocks > 0x7FFFFFFFull) return kDeclined;
    t.vec = vec ? 1u : 0u;
    if (eb == 4) hipLaunchKernelGGL(transpose_copy_kernel<4>, dim3((uint32_t)blocks), dim3(kBlock), 0, be->stream, t);
    else if (eb == 2) hipLaunchKernelGGL(transpose_copy_kernel<2>, dim3((uint32_t)blocks), dim3(kBlock), 0, be->stream, t);
    else hipLaunchKernelGGL(transpose_copy_kernel<1>, dim3((uint32_t)blocks), dim3(kBlock), 0, be->stream, t);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "transposing copy launch");
}

int launch_elementwise(cg_backend *be, int op, cg_dtype dt, const cg_tensor *out, const cg_tensor *const *ins, int nin, int round_op) {
    if (int frc = flush_deferred(be)) return frc;
    const cg_tensor *views[4] = {out, nullptr, nullptr, nullptr};
    for (int k = 0; k < nin; k++) views[k + 1] = ins[k];
    EwArgs a;
    memset(&a, 0, sizeof a);
    Operand ops[4];
    int rc = plan_elementwise(views, nin + 1, &a.g, ops, true);
    if (rc) return rc;
    a.out = ops[0];
    for (int k = 0; k < nin; k++) a.in[k] = ops[k + 1];
    a.fault = be->fault_dev;
    a.round = (uint32_t)round_op;
    double work = distinct_bytes(out);
    for (int k = 0; k < nin; k++) work += distinct_bytes(ins[k]);
    ProfScope prof(be, CG_K_ELEMENTWISE, work);
    if (op == kCopy && nin == 1) {
        const int trc = try_transpose_copy(be, a);
        if (trc != kDeclined) return trc;
    }
    return a.g.vec == 8   ? launch_ew_vec<8>(be, op, dt, a)
           : a.g.vec == 4 ? launch_ew_vec<4>(be, op, dt, a)
                          : launch_ew_vec<1>(be, op, dt, a);
}

__global__ void small_readback_kernel(const uint32_t *src, uint32_t n, uint32_t *dst, uint32_t seq) {
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) dst[i] = src[i];
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(dst + kReadbackWords, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

struct UploadWords {
    uint32_t w[kUploadWords];
};
__global__ void small_upload_kernel(uint32_t *dst, const UploadWords v, uint32_t n) {
    if (threadIdx.x < n) dst[threadIdx.x] = v.w[threadIdx.x];
}

int launch_small_upload(cg_backend *be, uint32_t *dst, const uint32_t *host_words, uint32_t n) {
    UploadWords v;
    memset(&v, 0, sizeof v);
    memcpy(v.w, host_words, (size_t)n * 4);
    hipLaunchKernelGGL(small_upload_kernel, dim3(1), dim3(kUploadWords), 0, be->stream, dst, v, n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "upload launch");
}

int launch_small_readback(cg_backend *be, const uint32_t *src, uint32_t n, uint32_t seq) {
    hipLaunchKernelGGL(small_readback_kernel, dim3(1), dim3(256), 0, be->stream, src, n, be->rb_dev, seq);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "read-back launch");
}

int launch_arange(cg_backend *be, cg_tensor *out) {
    uint32_t n = (uint32_t)out->dims[0];
    hipLaunchKernelGGL(arange_kernel, dim3((n + 255) / 256), dim3(256), 0, be->stream,
                       static_cast<uint32_t *>(out->buf->ptr), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "arange launch");
}

int launch_bf16_widen(cg_backend *be, const void *src, void *dst, uint64_t n) {
    if (n == 0) return CG_OK;
    const uint64_t groups = n / 8;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>(std::max<uint64_t>((groups + kBlock - 1) / kBlock, 1), 8192);
    hipLaunchKernelGGL(bf16_widen_kernel, dim3(blocks), dim3(kBlock), 0, be->stream, static_cast<const uint16_t *>(src),
                       static_cast<uint32_t *>(dst), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "bf16 widen launch");
}

__global__ __launch_bounds__(kBlock) void f16_widen_kernel(const uint16_t *src, uint32_t *dst, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock)
        dst[i] = asu(__half2float(__ushort_as_half(src[i])));
}
// BF16: the upper halves; else binary16 conversion (exact: the words hold representable values)
template <bool BF16> __global__ __launch_bounds__(kBlock) void narrow16_kernel(const uint32_t *src, uint16_t *dst, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock)
        dst[i] = BF16 ? (uint16_t)(src[i] >> 16) : __half_as_ushort(__float2half_rn(asf(src[i])));
}

int launch_f16_widen(cg_backend *be, const void *src, void *dst, uint64_t n) {
    if (n == 0) return CG_OK;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + kBlock - 1) / kBlock, 16384);
    hipLaunchKernelGGL(f16_widen_kernel, dim3(blocks), dim3(kBlock), 0, be->stream, static_cast<const uint16_t *>(src),
                       static_cast<uint32_t *>(dst), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "f16 widen launch");
}

int launch_narrow16(cg_backend *be, cg_dtype dt, const void *src, void *dst, uint64_t n) {
    if (n == 0) return CG_OK;
    if (int frc = flush_deferred(be)) return frc;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + kBlock - 1) / kBlock, 16384);
    if (dt == CG_BF16)
        hipLaunchKernelGGL((narrow16_kernel<true>), dim3(blocks), dim3(kBlock), 0, be->stream, static_cast<const uint32_t *>(src),
                           static_cast<uint16_t *>(dst), n);
    else
        hipLaunchKernelGGL((narrow16_kernel<false>), dim3(blocks), dim3(kBlock), 0, be->stream, static_cast<const uint32_t *>(src),
                           static_cast<uint16_t *>(dst), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "16-bit narrowing launch");
}

__global__ __launch_bounds__(kBlock) void f8_widen_kernel(const uint8_t *src, uint32_t *dst, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) dst[i] = f8_word_of(src[i]);
}
__global__ __launch_bounds__(kBlock) void narrow8_kernel(const uint32_t *src, uint8_t *dst, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) dst[i] = f8_byte_of(src[i]);
}
int launch_f8_widen(cg_backend *be, const void *src, void *dst, uint64_t n) {
    if (n == 0) return CG_OK;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + kBlock - 1) / kBlock, 16384);
    hipLaunchKernelGGL(f8_widen_kernel, dim3(blocks), dim3(kBlock), 0, be->stream, static_cast<const uint8_t *>(src),
                       static_cast<uint32_t *>(dst), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fp8 widen launch");
}
int launch_narrow8(cg_backend *be, const void *src, void *dst, uint64_t n) {
    if (n == 0) return CG_OK;
    if (int frc = flush_deferred(be)) return frc;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((n + kBlock - 1) / kBlock, 16384);
    hipLaunchKernelGGL(narrow8_kernel, dim3(blocks), dim3(kBlock), 0, be->stream, static_cast<const uint32_t *>(src),
                       static_cast<uint8_t *>(dst), n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fp8 narrowing launch");
}

int launch_widen(cg_backend *be, int fmt, const void *src, void *dst, uint64_t n) {
    return fmt == kFmtBF16 ? launch_bf16_widen(be, src, dst, n) : fmt == kFmtF16 ? launch_f16_widen(be, src, dst, n) : launch_f8_widen(be, src, dst, n);
}

int launch_fill_word(cg_backend *be, void *ptr, uint32_t bits) {
    hipLaunchKernelGGL(fill_word_kernel, dim3(1), dim3(1), 0, be->stream, static_cast<uint32_t *>(ptr), bits);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fill launch");
}

int launch_gather(cg_backend *be, const cg_tensor *x, int dim, const cg_tensor *idx, cg_tensor *out) {
    if (int frc = flush_deferred(be)) return frc;
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < dim; i++) outer *= x->dims[i];
    for (int i = dim + 1; i < x->rank; i++) inner *= x->dims[i];
    int64_t D = x->dims[dim], J = out->dims[dim];
    if (D > 0xFFFFFFFFll || inner > 0xFFFFFFFFll || outer * J > 0xFFFFFFFFll)
        return fail(CG_ERR_UNSUPPORTED, "index: extents above 2^32-1");
    const void *xp, *ip;
    int rc = device_ptr(idx, &ip);
    if (rc) return rc;
    // Rows of a narrow source that are whole 32-bit words long and start on one are gathered as those words (2 or 1 bytes
    // per element moved); the result keeps the format, or, a small one, is widened afterwards.  Other narrow sources are
    // read through their widened copy.
    const int xf = x->buf ? x->buf->fmt : kFmtWords, of = out->buf->fmt;
    const int64_t eb = (int64_t)fmt_bytes(xf);
    const bool as_bytes = xf != kFmtWords && inner * eb % 4 == 0 && x->offset * eb % 4 == 0;
    if (of != kFmtWords && !(as_bytes && of == xf)) return fail(CG_ERR_ARG, "internal error: gather into a narrow buffer of another layout");
    void *tmp = nullptr;
    size_t tmp_cls = 0;
    uint32_t *op = static_cast<uint32_t *>(out->buf->ptr);
    const int64_t out_elems = outer * J * inner;
    if (as_bytes) {
        int f;
        rc = device_ptr_fmt(x, &xp, &f);
        if (rc) return rc;
        inner = inner * eb / 4;
        if (of == kFmtWords) {
            rc = be->pool.alloc((size_t)(out_elems * eb), &tmp, &tmp_cls);
            if (rc) return rc;
            op = static_cast<uint32_t *>(tmp);
        }
    } else {
        rc = device_ptr(x, &xp);
        if (rc) return rc;
    }
    int64_t istride = idx->uniform ? 0 : (idx->rank == 1 ? idx->strides[0] : 1);
    bool vec4 = inner % 4 == 0 && reinterpret_cast<uintptr_t>(xp) % 16 == 0 && reinterpret_cast<uintptr_t>(op) % 16 == 0;
    uint32_t vec = vec4 ? 4 : 1;
    uint32_t ipr = (uint32_t)(inner / vec);
    uint64_t total = (uint64_t)outer * J * ipr;
    if (total > 0xFFFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "index: launch above 2^32-1 work items");
    dim3 grid((uint32_t)((total + kBlock - 1) / kBlock)), block(kBlock);
    ProfScope prof(be, CG_K_GATHER, 2.0 * distinct_bytes(out) + distinct_bytes(idx));
    if (vec4)
        hipLaunchKernelGGL((gather_kernel<4>), grid, block, 0, be->stream, static_cast<const uint32_t *>(xp),
                           static_cast<const uint32_t *>(ip), istride, op, (uint32_t)D, (uint32_t)inner,
                           make_fastdiv(ipr), ipr, make_fastdiv((uint32_t)J), (uint32_t)J, total, be->fault_dev);
    else
        hipLaunchKernelGGL((gather_kernel<1>), grid, block, 0, be->stream, static_cast<const uint32_t *>(xp),
                           static_cast<const uint32_t *>(ip), istride, op, (uint32_t)D, (uint32_t)inner,
                           make_fastdiv(ipr), ipr, make_fastdiv((uint32_t)J), (uint32_t)J, total, be->fault_dev);
    hipError_t e = hipGetLastError();
    if (tmp) { // stream-ordered free: the widening kernel queued here reads it first
        if (e == hipSuccess) rc = launch_widen(be, xf, tmp, out->buf->ptr, (uint64_t)out_elems);
        be->pool.free(tmp, tmp_cls);
        if (e == hipSuccess) return rc;
    }
    return e == hipSuccess ? CG_OK : hip_fail(e, "gather launch");
}

} // namespace cg
