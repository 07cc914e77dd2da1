// The interpreter's device code and the host code that fills its arguments, shared by the two
// translation units that launch it: fused.hip (programs as maps, reductions and row programs) and
// attention.hip (the attention kernels, which run a program's score and weight phases).
//
// A program is a short list of instructions over a register file of 16 values per
// element: the leaves (strided views or immediates, loaded once) occupy the first
// registers, every instruction names its destination (allocated on the host).  Every lane runs the same program, so the
// register numbers and op codes are wave-uniform: the register file lives in VGPRs and is
// indexed with scalar (uniform) indices, and the op switch is a scalar branch.  Arithmetic
// is the same `apply<OP, F>` the single-op kernels use, applied in the same order, so a
// fused chain is bit-identical to the chain of separate kernels — it just reads every leaf
// once and writes once.
#pragma once
#include "common.hpp"
#include "device_utils.hpp"

#include <algorithm>
#include <mutex>
#include <set>
#include <string>

namespace cg {

namespace {

constexpr int kBlock = 256;
constexpr float kF32Min = -3.4028234663852886e38f;

typedef uint32_t regfile __attribute__((ext_vector_type(16)));

} // namespace

// Program after register allocation: leaves sit in registers 0..nleaf-1, each instruction
// names its destination.
struct PInstr {
    uint8_t op, a, b, c, dst, pad[3];
};

struct FusedArgs {
    EwGeom g;
    Operand out;
    Operand leaf[kMaxLeaves];
    uint32_t nleaf, ninstr;
    PInstr ins[kMaxInstr];
    uint32_t *fault;
    // reductions only
    uint32_t rows, n;
    // programs with row-reduce instructions only
    uint32_t nred, reduced;
    uint8_t red_op[4]; // op code of the k-th row reduce
    // the piecewise leaf, if any (pw_leaf < 0: none): elements of the row at or beyond pw_split come
    // from `leaf2`, addressed with (position - pw_split); pw_neg bit 0 / 1: negate part 1 / 2
    int32_t pw_leaf;
    uint32_t pw_split, pw_neg;
    Operand leaf2;
};

// A row program that has a kernel compiled for it (aot_rows.hip) is launched with it: true.  `tpr` is the
// number of lanes per row, 16 / 64 / 256; `grid` the launch's workgroups of 256 / tpr rows each.
bool launch_compiled_rows(const Pending &p, const FusedArgs &a, uint32_t *rowout, int tpr, dim3 grid, hipStream_t s);

// Any row program through the interpreter, at four elements or one per work item (fused_rows_vec4.hip,
// fused_rows_vec1.hip): `tpr` lanes per row, 4 / 16 / 64 / 256; `full`: no lane of the grid is idle.
void launch_interpreted_rows4(const FusedArgs &a, uint32_t *rowout, int tpr, bool full, dim3 grid, hipStream_t s);
void launch_interpreted_rows1(const FusedArgs &a, uint32_t *rowout, int tpr, bool full, dim3 grid, hipStream_t s);

namespace {

// Leaf `l` of the work item that starts at position `e` of its row: `off` is the element offset
// in the leaf's (first) view, `off2` the offset in the second part of the piecewise leaf.
template <int VEC>
__device__ __forceinline__ void load_leaf(const FusedArgs &a, int l, int64_t off, int64_t off2, uint32_t e,
                                          uint32_t (&t)[VEC]) {
    if (l != a.pw_leaf) {
        load_words<VEC>(a.leaf[l], off, t);
        return;
    }
    const bool second = e >= a.pw_split; // a vector never straddles the split (it is a multiple of VEC)
    if (second) load_words<VEC>(a.leaf2, off2, t);
    else load_words<VEC>(a.leaf[l], off, t);
    if ((a.pw_neg >> (second ? 1 : 0)) & 1u) {
#pragma unroll
        for (int j = 0; j < VEC; j++) t[j] ^= 0x80000000u;
    }
}

// One instruction on the VEC elements of a work item.  op is wave-uniform, so the switch is
// a scalar branch, and the VEC applications inside a case are independent (they interleave
// in the pipeline).  FULL adds the long routines (sin, cos, log, pow, u32 pow); programs
// without them run the lean instantiation, which needs fewer registers and less code.
template <int VEC, bool FULL>
__device__ __forceinline__ void apply_rt(uint32_t op, const uint32_t (&x)[VEC], const uint32_t (&y)[VEC],
                                         const uint32_t (&z)[VEC], uint32_t (&o)[VEC], uint32_t *fault) {
#define CG_CASE(CODE, OP, F)                                                        \
    case CODE:                                                                      \
        _Pragma("unroll") for (int j = 0; j < VEC; j++) o[j] = apply<OP, F>(x[j], y[j], z[j], fault); \
        return;
#define CG_F(OP) CG_CASE(OP, OP, true)
#define CG_U(OP) CG_CASE((OP | kInstrU32), OP, false)
    if (FULL) {
        switch (op) {
            CG_F(kSin) CG_F(kCos) CG_F(kLog) CG_F(kPow) CG_U(kPow)
        default: break;
        }
    }
    switch (op) {
        CG_F(kNeg) CG_F(kExp) CG_F(kFloor) CG_F(kRound) CG_F(kRoundBF16) CG_F(kRoundF16) CG_F(kRoundF8)
        CG_F(kAdd) CG_F(kSub) CG_F(kMul) CG_F(kDiv)
        CG_F(kLt) CG_F(kGt) CG_F(kGte) CG_F(kLte) CG_F(kEq) CG_F(kWhere) CG_F(kCastF2U)
        CG_U(kNeg) CG_U(kAdd) CG_U(kSub) CG_U(kMul) CG_U(kDiv)
        CG_U(kLt) CG_U(kGt) CG_U(kGte) CG_U(kLte) CG_U(kEq) CG_U(kWhere) CG_U(kCastU2F)
    default:
#pragma unroll
        for (int j = 0; j < VEC; j++) o[j] = x[j]; // kCopy
        return;
    }
#undef CG_F
#undef CG_U
#undef CG_CASE
}

// Loads the leaves of one work item and runs the program; result in res[VEC].
template <int VEC, bool FULL>
__device__ __forceinline__ void eval_program(const FusedArgs &a, const int64_t (&off)[kMaxLeaves], int64_t off2, uint32_t e,
                                             uint32_t (&res)[VEC]) {
    regfile r[VEC];
#pragma unroll
    for (int l = 0; l < kMaxLeaves; l++) {
        if ((uint32_t)l < a.nleaf) {
            uint32_t t[VEC];
            load_leaf<VEC>(a, l, off[l], off2, e, t);
#pragma unroll
            for (int j = 0; j < VEC; j++) r[j][l] = t[j];
        }
    }
    PInstr in = a.ins[0];
    for (uint32_t i = 0; i < a.ninstr; i++) {
        const PInstr cur = in;
        if (i + 1 < a.ninstr) in = a.ins[i + 1]; // next instruction word on its way while this one runs
        uint32_t x[VEC], y[VEC], z[VEC], o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            x[j] = r[j][cur.a];
            y[j] = r[j][cur.b];
            z[j] = r[j][cur.c];
        }
        apply_rt<VEC, FULL>(cur.op, x, y, z, o, a.fault);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            r[j][cur.dst] = o[j];
            res[j] = o[j];
        }
    }
}

template <int VEC, bool FULL> __global__ __launch_bounds__(kBlock) void fused_kernel(const FusedArgs a) {
    const uint64_t v64 = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v64 >= a.g.total) return;
    const uint32_t v = (uint32_t)v64;
    uint32_t row = fastdiv(v, a.g.ipr_div);
    const int64_t e = (int64_t)(v - row * a.g.ipr) * VEC;
    int64_t oo = e * a.out.is;
    int64_t off[kMaxLeaves];
#pragma unroll
    for (int l = 0; l < kMaxLeaves; l++) off[l] = (uint32_t)l < a.nleaf ? e * a.leaf[l].is : 0;
    int64_t off2 = (e - (int64_t)a.pw_split) * a.leaf2.is;
    for (uint32_t d = 0; d < a.g.nouter; d++) {
        const uint32_t q = fastdiv(row, a.g.odiv[d]);
        const int64_t i = (int64_t)(row - q * a.g.od[d]);
        row = q;
        oo += i * a.out.os[d];
        off2 += i * a.leaf2.os[d];
#pragma unroll
        for (int l = 0; l < kMaxLeaves; l++)
            if ((uint32_t)l < a.nleaf) off[l] += i * a.leaf[l].os[d];
    }
    uint32_t res[VEC];
    eval_program<VEC, FULL>(a, off, off2, (uint32_t)e, res);
    store_words<VEC>(a.out, oo, res);
}

// ---- reduction over the last axis of a program's value --------------------------------------
__device__ __forceinline__ int32_t total_key(uint32_t bits) { // Rust f32::total_cmp
    int32_t b = (int32_t)bits;
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

// kind 0 sum, 1 max, 2 argmax; f32 flag picks the arithmetic.  One 64-bit accumulator serves
// all six cases so that the kernel is not instantiated per case.
struct RedAcc {
    long long c;
    __device__ static RedAcc init(int kind, bool f) {
        RedAcc r;
        if (kind == kSum) r.c = 0;
        else if (kind == kMax) r.c = f ? (long long)asu(kF32Min) : 0;
        else r.c = (long long)0x8000000000000000ll;
        return r;
    }
    __device__ void take(int kind, bool f, uint32_t w, uint32_t idx) {
        if (kind == kSum) {
            c = f ? (long long)asu(asf((uint32_t)c) + asf(w)) : (long long)(uint32_t)((uint32_t)c + w);
        } else if (kind == kMax) {
            if (f) c = (long long)asu(fmaxf(asf((uint32_t)c), asf(w)));
            else c = w > (uint32_t)c ? (long long)w : c;
        } else {
            int32_t key = f ? total_key(w) : (int32_t)(w ^ 0x80000000u);
            long long p = ((long long)key << 32) | (long long)idx;
            c = p > c ? p : c;
        }
    }
    __device__ void merge(int kind, bool f, const RedAcc &o) {
        if (kind == kSum) {
            c = f ? (long long)asu(asf((uint32_t)c) + asf((uint32_t)o.c)) : (long long)(uint32_t)((uint32_t)c + (uint32_t)o.c);
        } else if (kind == kMax) {
            if (f) c = (long long)asu(fmaxf(asf((uint32_t)c), asf((uint32_t)o.c)));
            else c = (uint32_t)o.c > (uint32_t)c ? o.c : c;
        } else {
            c = o.c > c ? o.c : c;
        }
    }
    __device__ RedAcc shfl(int m) const {
        RedAcc r;
        int lo = __shfl_xor((int)(c & 0xFFFFFFFFll), m);
        int hi = __shfl_xor((int)(c >> 32), m);
        r.c = ((long long)hi << 32) | (long long)(uint32_t)lo;
        return r;
    }
};

template <int VEC, int TPR, bool FULL>
__global__ __launch_bounds__(kBlock) void fused_reduce_kernel(const FusedArgs a, uint32_t *out, int kind, int f32) {
    constexpr int RPB = kBlock / TPR;
    const uint32_t lane = threadIdx.x % TPR;
    const uint32_t row = blockIdx.x * RPB + threadIdx.x / TPR;
    const bool live = row < a.rows;
    const bool f = f32 != 0;
    RedAcc acc = RedAcc::init(kind, f);
    if (live) {
        int64_t base[kMaxLeaves];
#pragma unroll
        for (int l = 0; l < kMaxLeaves; l++) base[l] = 0;
        uint32_t rr = row;
        int64_t base2 = 0;
        for (uint32_t d = 0; d < a.g.nouter; d++) {
            const uint32_t q = fastdiv(rr, a.g.odiv[d]);
            const int64_t i = (int64_t)(rr - q * a.g.od[d]);
            rr = q;
            base2 += i * a.leaf2.os[d];
#pragma unroll
            for (int l = 0; l < kMaxLeaves; l++)
                if ((uint32_t)l < a.nleaf) base[l] += i * a.leaf[l].os[d];
        }
        const uint32_t items = a.n / VEC;
        for (uint32_t it = lane; it < items; it += TPR) {
            int64_t off[kMaxLeaves];
#pragma unroll
            for (int l = 0; l < kMaxLeaves; l++)
                off[l] = (uint32_t)l < a.nleaf ? base[l] + (int64_t)it * VEC * a.leaf[l].is : 0;
            const int64_t off2 = base2 + ((int64_t)it * VEC - (int64_t)a.pw_split) * a.leaf2.is;
            uint32_t res[VEC];
            eval_program<VEC, FULL>(a, off, off2, it * VEC, res);
#pragma unroll
            for (int j = 0; j < VEC; j++) acc.take(kind, f, res[j], it * VEC + j);
        }
    }
    constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
    for (int m = W / 2; m >= 1; m >>= 1) acc.merge(kind, f, acc.shfl(m));
    if constexpr (TPR > 64) {
        __shared__ long long part[kBlock / 64];
        if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = acc.c;
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int w = 1; w < kBlock / 64; w++) {
                RedAcc o;
                o.c = part[w];
                acc.merge(kind, f, o);
            }
        }
    }
    if (live && lane == 0) out[row] = (uint32_t)(acc.c & 0xFFFFFFFFll);
}

// ---- programs with row-reduce instructions -----------------------------------------------------
__device__ __forceinline__ uint32_t row_init(bool is_max, bool f) { return is_max && f ? asu(kF32Min) : 0u; }
__device__ __forceinline__ uint32_t row_merge(bool is_max, bool f, uint32_t c, uint32_t w) {
    if (is_max) return f ? asu(fmaxf(asf(c), asf(w))) : (w > c ? w : c);
    return f ? asu(asf(c) + asf(w)) : c + w;
}

// Runs the program on one work item up to row reduce number `phase`: earlier reduces take
// their finished row value from rs, the operand of reduce `phase` is returned in res (true),
// and with phase == nred the whole program runs and res is its value (false).
template <int VEC, bool FULL>
__device__ __forceinline__ bool eval_rows(const FusedArgs &a, const int64_t (&off)[kMaxLeaves], int64_t off2, uint32_t e,
                                          const uint32_t (&rs)[kMaxRowReduce], uint32_t phase, uint32_t (&res)[VEC]) {
    regfile r[VEC];
#pragma unroll
    for (int l = 0; l < kMaxLeaves; l++) {
        if ((uint32_t)l < a.nleaf) {
            uint32_t t[VEC];
            load_leaf<VEC>(a, l, off[l], off2, e, t);
#pragma unroll
            for (int j = 0; j < VEC; j++) r[j][l] = t[j];
        }
    }
    uint32_t seen = 0;
    PInstr in = a.ins[0];
    for (uint32_t i = 0; i < a.ninstr; i++) {
        const PInstr cur = in;
        if (i + 1 < a.ninstr) in = a.ins[i + 1];
        if (is_row_reduce(cur.op)) {
            if (seen == phase) {
#pragma unroll
                for (int j = 0; j < VEC; j++) res[j] = r[j][cur.a];
                return true;
            }
            const uint32_t v = seen == 0 ? rs[0] : seen == 1 ? rs[1] : rs[2];
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                r[j][cur.dst] = v;
                res[j] = v;
            }
            seen++;
            continue;
        }
        uint32_t x[VEC], y[VEC], z[VEC], o[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            x[j] = r[j][cur.a];
            y[j] = r[j][cur.b];
            z[j] = r[j][cur.c];
        }
        apply_rt<VEC, FULL>(cur.op, x, y, z, o, a.fault);
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            r[j][cur.dst] = o[j];
            res[j] = o[j];
        }
    }
    return false;
}

// TPR lanes share a row.  For each row reduce in program order the lanes walk the row,
// evaluate the program up to that reduce and combine; a last walk evaluates the whole
// program and stores the row (or, for a reduced result, lane 0 stores the row's value).
// Leaves are re-read on every walk: a row is a few KiB and stays in L1/L2.
template <int VEC, int TPR, bool FULL>
__global__ __launch_bounds__(kBlock) void fused_rows_kernel(const FusedArgs a, uint32_t *rowout) {
    constexpr int RPB = kBlock / TPR;
    const uint32_t lane = threadIdx.x % TPR;
    const uint32_t row = blockIdx.x * RPB + threadIdx.x / TPR;
    const bool live = row < a.rows;
    int64_t base[kMaxLeaves];
#pragma unroll
    for (int l = 0; l < kMaxLeaves; l++) base[l] = 0;
    int64_t obase = 0, base2 = 0;
    if (live) {
        uint32_t rr = row;
        for (uint32_t d = 0; d < a.g.nouter; d++) {
            const uint32_t q = fastdiv(rr, a.g.odiv[d]);
            const int64_t i = (int64_t)(rr - q * a.g.od[d]);
            rr = q;
            obase += i * a.out.os[d];
            base2 += i * a.leaf2.os[d];
#pragma unroll
            for (int l = 0; l < kMaxLeaves; l++)
                if ((uint32_t)l < a.nleaf) base[l] += i * a.leaf[l].os[d];
        }
    }
    const uint32_t items = a.n / VEC;
    uint32_t rs[kMaxRowReduce] = {0, 0, 0};
    for (uint32_t phase = 0; phase < a.nred; phase++) {
        const uint32_t rop = a.red_op[phase];
        const bool is_max = (rop & ~kInstrU32) == kRowMax, f = !(rop & kInstrU32);
        uint32_t acc = row_init(is_max, f);
        if (live) {
            for (uint32_t it = lane; it < items; it += TPR) {
                int64_t off[kMaxLeaves];
#pragma unroll
                for (int l = 0; l < kMaxLeaves; l++)
                    off[l] = (uint32_t)l < a.nleaf ? base[l] + (int64_t)it * VEC * a.leaf[l].is : 0;
                const int64_t off2 = base2 + ((int64_t)it * VEC - (int64_t)a.pw_split) * a.leaf2.is;
                uint32_t res[VEC];
                eval_rows<VEC, FULL>(a, off, off2, it * VEC, rs, phase, res);
#pragma unroll
                for (int j = 0; j < VEC; j++) acc = row_merge(is_max, f, acc, res[j]);
            }
        }
        // xor butterfly: both partners add the same two values, so every lane of the row ends
        // with the same bits
        constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
        for (int m = W / 2; m >= 1; m >>= 1) acc = row_merge(is_max, f, acc, (uint32_t)__shfl_xor((int)acc, m));
        if constexpr (TPR > 64) {
            __shared__ uint32_t part[kBlock / 64];
            if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = acc;
            __syncthreads();
            acc = part[0];
#pragma unroll
            for (int w = 1; w < kBlock / 64; w++) acc = row_merge(is_max, f, acc, part[w]);
            __syncthreads();
        }
        if (phase == 0) rs[0] = acc;
        else if (phase == 1) rs[1] = acc;
        else rs[2] = acc;
    }
    if (!live) return;
    if (a.reduced) {
        if (lane == 0) {
            int64_t off[kMaxLeaves];
#pragma unroll
            for (int l = 0; l < kMaxLeaves; l++) off[l] = base[l];
            uint32_t res[VEC];
            eval_rows<VEC, FULL>(a, off, base2 - (int64_t)a.pw_split * a.leaf2.is, 0, rs, a.nred, res);
            rowout[row] = res[0];
        }
        return;
    }
    for (uint32_t it = lane; it < items; it += TPR) {
        int64_t off[kMaxLeaves];
#pragma unroll
        for (int l = 0; l < kMaxLeaves; l++)
            off[l] = (uint32_t)l < a.nleaf ? base[l] + (int64_t)it * VEC * a.leaf[l].is : 0;
        const int64_t off2 = base2 + ((int64_t)it * VEC - (int64_t)a.pw_split) * a.leaf2.is;
        uint32_t res[VEC];
        eval_rows<VEC, FULL>(a, off, off2, it * VEC, rs, a.nred, res);
        store_words<VEC>(a.out, obase + (int64_t)it * VEC * a.out.is, res);
    }
}

template <int VEC>
void launch_interpreted_rows(const FusedArgs &a, uint32_t *rowout, int tpr, bool full, dim3 grid, hipStream_t s) {
#define CG_LAUNCH(TPR)                                                                                  \
    do {                                                                                                \
        if (full)                                                                                       \
            hipLaunchKernelGGL((fused_rows_kernel<VEC, TPR, true>), grid, dim3(kBlock), 0, s, a, rowout);  \
        else                                                                                            \
            hipLaunchKernelGGL((fused_rows_kernel<VEC, TPR, false>), grid, dim3(kBlock), 0, s, a, rowout); \
    } while (0)
    switch (tpr) {
    case 4: CG_LAUNCH(4); break;
    case 16: CG_LAUNCH(16); break;
    case 64: CG_LAUNCH(64); break;
    default: CG_LAUNCH(256); break;
    }
#undef CG_LAUNCH
}

#include "aot_programs.hpp"

// Linear-scan register allocation over the 16-entry register file: leaves take 0..nleaf-1,
// an instruction's destination is any register whose value has no later use (an operand's
// own register qualifies: it is read before the result is written).  False if 16 do not suffice.
bool allocate_registers(const Pending &p, uint8_t *phys) {
    constexpr int kRegs = 16;
    int last_use[kMaxLeaves + kMaxInstr];
    for (int i = 0; i < kMaxLeaves + kMaxInstr; i++) last_use[i] = -1;
    for (int i = 0; i < p.ninstr; i++) {
        last_use[p.ins[i].a] = i;
        last_use[p.ins[i].b] = i;
        last_use[p.ins[i].c] = i;
    }
    if (p.ninstr > 0) last_use[kMaxLeaves + p.ninstr - 1] = p.ninstr; // the result
    int owner[kRegs];
    for (int r = 0; r < kRegs; r++) owner[r] = -1;
    for (int l = 0; l < p.nleaf; l++) {
        phys[l] = (uint8_t)l;
        owner[l] = l;
    }
    for (int i = 0; i < p.ninstr; i++) {
        int pick = -1;
        for (int r = 0; r < kRegs && pick < 0; r++)
            if (owner[r] < 0 || last_use[owner[r]] <= i) pick = r;
        if (pick < 0) return false;
        owner[pick] = kMaxLeaves + i;
        phys[kMaxLeaves + i] = (uint8_t)pick;
    }
    return true;
}

int fill_args(cg_backend *be, const Pending &p, const int64_t *dims, int rank, const cg_tensor *out, bool keep_last,
              FusedArgs *a, double *leaf_bytes, bool *full, int ninstr = -1, bool skip_lazy = false) {
    if (ninstr < 0) ninstr = p.ninstr;
    memset(a, 0, sizeof *a);
    ViewDesc v[kMaxViews + 1];
    int64_t out_strides[kMaxRank];
    if (out) {
        const void *op;
        int rc = device_ptr_fmt(out, &op, &v[0].fmt); // (a destination: the buffer itself, in its own format)
        if (rc) return rc;
        v[0].strides = out->strides;
        v[0].uniform = false;
        v[0].ubits = 0;
        v[0].ptr = static_cast<const char *>(op);
    } else { // reductions plan over the leaves only; a stand-in output keeps the planner's shape
        int64_t s = 1;
        for (int i = rank - 1; i >= 0; i--) {
            out_strides[i] = s;
            s *= dims[i];
        }
        v[0].strides = out_strides;
        v[0].uniform = false;
        v[0].ubits = 0;
        v[0].ptr = nullptr;
    }
    double bytes = 0.0;
    int pw_leaf = -1;
    for (int l = 0; l < p.nleaf; l++) {
        const LeafView &lv = p.leaf[l];
        v[l + 1].strides = lv.strides;
        v[l + 1].uniform = lv.uniform;
        v[l + 1].ubits = lv.ubits;
        const Buffer *src = lv.buf;
        if (lv.lazy && !skip_lazy) { // a product that has been put off until now
            int lrc = lazy_mm_force(be, lv.lazy);
            if (lrc) return lrc;
            src = lv.lazy->result;
        }
        v[l + 1].fmt = lv.uniform || !src ? kFmtWords : src->fmt;
        v[l + 1].ptr = lv.uniform || !src ? nullptr : static_cast<const char *>(src->ptr) + lv.offset * (int64_t)fmt_bytes(v[l + 1].fmt);
        v[l + 1].vec_period = 0;
        if (lv.pw) { // its second part is planned as one more view, and the row axis stays on its own
            pw_leaf = l;
            v[l + 1].vec_period = lv.pw_split;
            ViewDesc &w = v[p.nleaf + 1];
            w.strides = lv.strides2;
            w.uniform = false;
            w.ubits = 0;
            const Buffer *src2 = lv.buf2;
            if (lv.lazy2) { // the second part is a view of a product that has been put off until now
                int lrc = lazy_mm_force(be, lv.lazy2);
                if (lrc) return lrc;
                src2 = lv.lazy2->result;
            }
            w.fmt = src2->fmt;
            w.ptr = static_cast<const char *>(src2->ptr) + lv.offset2 * (int64_t)fmt_bytes(w.fmt);
            w.vec_period = lv.pw_split;
        }
        if (!lv.uniform) {
            double n = 1.0;
            for (int i = 0; i < rank; i++)
                if (lv.strides[i] != 0 || dims[i] <= 1) n *= (double)dims[i];
            if (!(lv.lazy && skip_lazy)) bytes += (double)fmt_bytes(v[l + 1].fmt) * n;
        }
    }
    Operand ops[kMaxViews + 1];
    // Small problems are latency-bound: one element per lane keeps each lane's serial chain
    // (operand moves, long routines) four times shorter and still fills the chip.
    int64_t elems = 1;
    for (int i = 0; i < rank; i++) elems *= dims[i];
    int rc = plan_views(dims, rank, v, p.nleaf + 1 + (pw_leaf >= 0 ? 1 : 0), keep_last || pw_leaf >= 0, &a->g, ops,
                        keep_last || elems > 32768);
    if (rc) return rc;
    a->out = ops[0];
    for (int l = 0; l < p.nleaf; l++) a->leaf[l] = ops[l + 1];
    a->pw_leaf = pw_leaf;
    if (pw_leaf >= 0) {
        const LeafView &lv = p.leaf[pw_leaf];
        if (lv.pw_split > 0xFFFFFFFFll) return fail(CG_ERR_UNSUPPORTED, "concat: last axis above 2^32-1 elements");
        a->leaf2 = ops[p.nleaf + 1];
        a->pw_split = (uint32_t)lv.pw_split;
        a->pw_neg = (lv.neg1 ? 1u : 0u) | (lv.neg2 ? 2u : 0u);
    }
    a->nleaf = (uint32_t)p.nleaf;
    a->ninstr = (uint32_t)ninstr;
    uint8_t phys[kMaxLeaves + kMaxInstr];
    if (!allocate_registers(p, phys)) return fail(CG_ERR_ARG, "internal error: fused program needs too many registers");
    *full = false;
    for (int i = 0; i < ninstr; i++) {
        const Instr &in = p.ins[i];
        PInstr q;
        memset(&q, 0, sizeof q);
        q.op = in.op;
        q.a = phys[in.a];
        q.b = phys[in.b];
        q.c = phys[in.c];
        q.dst = phys[kMaxLeaves + i];
        a->ins[i] = q;
        const int op = in.op & ~kInstrU32;
        *full = *full || op == kSin || op == kCos || op == kLog || op == kPow;
        if (is_row_reduce(op)) {
            if (a->nred >= (uint32_t)kMaxRowReduce) return fail(CG_ERR_ARG, "internal error: too many row reduces");
            a->red_op[a->nred++] = in.op;
        }
    }
    a->fault = be->fault_dev;
    *leaf_bytes = bytes;
    return CG_OK;
}

// CG_TRACE_PROGRAMS=1: each distinct program, once, in the order of first execution.
void trace_program(cg_backend *be, const Pending &p, int ninstr, const char *how, const int64_t *dims, int rank) {
    if (!be->trace_programs) return;
    static std::mutex mu;
    static std::set<std::string> seen;
    std::string key = how;
    char buf[64];
    snprintf(buf, sizeof buf, " nleaf=%d ninstr=%d code=", p.nleaf, ninstr);
    key += buf;
    for (int i = 0; i < ninstr; i++) {
        snprintf(buf, sizeof buf, "{%d,%d,%d,%d},", p.ins[i].op, p.ins[i].a, p.ins[i].b, p.ins[i].c);
        key += buf;
    }
    std::lock_guard<std::mutex> lk(mu);
    if (!seen.insert(key).second) return;
    std::string where = " uniform=";
    for (int l = 0; l < p.nleaf; l++) where += p.leaf[l].pw ? 'p' : p.leaf[l].lazy ? 'm' : p.leaf[l].uniform ? '1' : '0';
    where += " dims=[";
    for (int i = 0; i < rank; i++) {
        snprintf(buf, sizeof buf, "%s%lld", i ? "," : "", (long long)dims[i]);
        where += buf;
    }
    fprintf(stderr, "[cg program] %s%s]\n", key.c_str(), where.c_str());
}
} // namespace

} // namespace cg
