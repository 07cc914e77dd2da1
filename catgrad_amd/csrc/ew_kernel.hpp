// The element-wise kernel and the table of its instantiations, shared by the translation units
// that compile them: one per vector width (ew_vec1.hip, ew_vec4.hip, ew_vec8.hip), so that the
// three thirds of the table build side by side.  ew.hip plans a launch and calls launch_ew_vec<VEC>.
#pragma once
#include "common.hpp"
#include "device_utils.hpp"

namespace cg {

constexpr int kBlock = 256;
constexpr int kUnroll = 4;
constexpr uint64_t kStreamItems = 4u << 20; // work items (64 MiB of 16-byte vectors) from which outputs stream past the caches

struct EwArgs {
    EwGeom g;
    Operand out;
    Operand in[3];
    uint32_t *fault;
    uint32_t round; // kRoundBF16 / kRoundF16 / kRoundF8: the result is rounded to that format before it is stored; 0: not
};

// FLAT: the iteration space collapsed to a single axis (no index arithmetic at all).
template <int OP, bool F, int NIN, int VEC, bool FLAT>
__global__ __launch_bounds__(kBlock) void ew_kernel(const EwArgs a) {
    const uint64_t base = (uint64_t)blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
    int64_t off[kUnroll][4];
    bool live[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        uint64_t v64 = base + (uint64_t)u * kBlock;
        live[u] = v64 < a.g.total;
        uint32_t v = (uint32_t)v64;
        if (FLAT) {
            int64_t e = (int64_t)v * VEC;
            off[u][0] = e * a.out.is;
#pragma unroll
            for (int k = 0; k < NIN; k++) off[u][k + 1] = e * a.in[k].is;
        } else {
            uint32_t row = fastdiv(v, a.g.ipr_div);
            int64_t e = (int64_t)(v - row * a.g.ipr) * VEC;
            int64_t oo = e * a.out.is;
            int64_t oi[3];
#pragma unroll
            for (int k = 0; k < NIN; k++) oi[k] = e * a.in[k].is;
            for (uint32_t d = 0; d < a.g.nouter; d++) {
                uint32_t q = fastdiv(row, a.g.odiv[d]);
                int64_t i = (int64_t)(row - q * a.g.od[d]);
                row = q;
                oo += i * a.out.os[d];
#pragma unroll
                for (int k = 0; k < NIN; k++) oi[k] += i * a.in[k].os[d];
            }
            off[u][0] = oo;
#pragma unroll
            for (int k = 0; k < NIN; k++) off[u][k + 1] = oi[k];
        }
    }
    uint32_t x[kUnroll][3][VEC];
#pragma unroll
    for (int u = 0; u < kUnroll; u++)
        if (live[u]) {
#pragma unroll
            for (int k = 0; k < NIN; k++) {
                // fully collapsed space: a unit-stride operand is read exactly once, so it need not
                // displace anything from the caches either
                if (FLAT && a.g.total >= kStreamItems) load_words<VEC, true>(a.in[k], off[u][k + 1], x[u][k]);
                else load_words<VEC>(a.in[k], off[u][k + 1], x[u][k]);
            }
        }
#pragma unroll
    for (int u = 0; u < kUnroll; u++)
        if (live[u]) {
            uint32_t r[VEC];
#pragma unroll
            for (int j = 0; j < VEC; j++)
                r[j] = apply<OP, F>(x[u][0][j], NIN > 1 ? x[u][1 % NIN][j] : 0u, NIN > 2 ? x[u][2 % NIN][j] : 0u, a.fault);
            if (F && a.round) { // (the same for every lane: a launch parameter)
#pragma unroll
                for (int j = 0; j < VEC; j++)
                    r[j] = a.round == kRoundBF16 ? apply<kRoundBF16, true>(r[j], 0u, 0u, a.fault)
                           : a.round == kRoundF16 ? apply<kRoundF16, true>(r[j], 0u, 0u, a.fault)
                                                  : apply<kRoundF8, true>(r[j], 0u, 0u, a.fault);
            }
            if (a.g.total >= kStreamItems) store_words<VEC, true>(a.out, off[u][0], r);
            else store_words<VEC>(a.out, off[u][0], r);
        }
}

template <int VEC, int OP, bool F, int NIN> int launch_variants(cg_backend *be, const EwArgs &a) {
    uint64_t per_block = (uint64_t)kBlock * kUnroll;
    uint64_t blocks = (a.g.total + per_block - 1) / per_block;
    if (blocks == 0) return CG_OK;
    dim3 grid((uint32_t)blocks), block(kBlock);
    if (a.g.nouter == 0)
        hipLaunchKernelGGL((ew_kernel<OP, F, NIN, VEC, true>), grid, block, 0, be->stream, a);
    else
        hipLaunchKernelGGL((ew_kernel<OP, F, NIN, VEC, false>), grid, block, 0, be->stream, a);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "element-wise kernel launch");
}

template <int VEC, int OP, int NIN> int launch_by_dtype(cg_backend *be, cg_dtype dt, const EwArgs &a) {
    return is_f(dt) ? launch_variants<VEC, OP, true, NIN>(be, a) : launch_variants<VEC, OP, false, NIN>(be, a);
}

// The kernel for `op` at vector width VEC (1, 4 or 8 elements per work item); a.g.vec says which to call.
// The table comes in two parts, so that the widest kernels compile as two translation units: the
// operations of two operands, and all others.
template <int VEC> int launch_ew_binary(cg_backend *be, int op, cg_dtype dt, const EwArgs &a) {
    switch (op) {
#define CG_EW2(OP) case OP: return launch_by_dtype<VEC, OP, 2>(be, dt, a);
    CG_EW2(kAdd) CG_EW2(kSub) CG_EW2(kMul) CG_EW2(kDiv) CG_EW2(kPow)
    CG_EW2(kLt) CG_EW2(kGt) CG_EW2(kGte) CG_EW2(kLte) CG_EW2(kEq)
#undef CG_EW2
    default: return fail(CG_ERR_ARG, "unknown element-wise op %d", op);
    }
}

template <int VEC> int launch_ew_other(cg_backend *be, int op, cg_dtype dt, const EwArgs &a) {
    switch (op) {
    case kNeg: return launch_by_dtype<VEC, kNeg, 1>(be, dt, a);
    case kSin: return launch_variants<VEC, kSin, true, 1>(be, a);
    case kCos: return launch_variants<VEC, kCos, true, 1>(be, a);
    case kExp: return launch_variants<VEC, kExp, true, 1>(be, a);
    case kLog: return launch_variants<VEC, kLog, true, 1>(be, a);
    case kFloor: return launch_variants<VEC, kFloor, true, 1>(be, a);
    case kRound: return launch_variants<VEC, kRound, true, 1>(be, a);
    case kRoundBF16: return launch_variants<VEC, kRoundBF16, true, 1>(be, a);
    case kRoundF16: return launch_variants<VEC, kRoundF16, true, 1>(be, a);
    case kRoundF8: return launch_variants<VEC, kRoundF8, true, 1>(be, a);
    case kWhere: return launch_by_dtype<VEC, kWhere, 3>(be, dt, a);
    case kCastF2U: return launch_variants<VEC, kCastF2U, true, 1>(be, a);
    case kCastU2F: return launch_variants<VEC, kCastU2F, false, 1>(be, a);
    case kCopy: return launch_variants<VEC, kCopy, false, 1>(be, a);
    default: return fail(CG_ERR_ARG, "unknown element-wise op %d", op);
    }
}

#define CG_EW_TABLE(KEYWORD, VEC)                                                             \
    KEYWORD template int launch_ew_binary<VEC>(cg_backend *, int, cg_dtype, const EwArgs &); \
    KEYWORD template int launch_ew_other<VEC>(cg_backend *, int, cg_dtype, const EwArgs &);
CG_EW_TABLE(extern, 1)
CG_EW_TABLE(extern, 4)
CG_EW_TABLE(extern, 8)
#undef CG_EW_TABLE

inline bool ew_is_binary(int op) {
    switch (op) {
    case kAdd: case kSub: case kMul: case kDiv: case kPow: case kLt: case kGt: case kGte: case kLte: case kEq: return true;
    default: return false;
    }
}

template <int VEC> int launch_ew_vec(cg_backend *be, int op, cg_dtype dt, const EwArgs &a) {
    return ew_is_binary(op) ? launch_ew_binary<VEC>(be, op, dt, a) : launch_ew_other<VEC>(be, op, dt, a);
}

} // namespace cg
