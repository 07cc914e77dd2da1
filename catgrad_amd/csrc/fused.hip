// Interpreter kernels for deferred element-wise expressions (see `Pending` in common.hpp).
//
// A program is a short list of instructions over a register file of 16 values per
// element: the leaves (strided views or immediates, loaded once) occupy the first
// registers, every instruction names its destination (allocated on the host).  Every lane runs the same program, so the
// register numbers and op codes are wave-uniform: the register file lives in VGPRs and is
// indexed with scalar (uniform) indices, and the op switch is a scalar branch.  Arithmetic
// is the same `apply<OP, F>` the single-op kernels use, applied in the same order, so a
// fused chain is bit-identical to the chain of separate kernels — it just reads every leaf
// once and writes once.
//
//   fused_kernel         value of the program -> dense or strided output      (HBM-bound:
//                        4 B per distinct leaf element + 4 B per output element)
//   fused_reduce_kernel  sum / max / argmax over the last axis of the value   (HBM-bound:
//                        4 B per distinct leaf element + 4 B per row)
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

#include "attention.hpp"

} // namespace

static int64_t attn_blocks() {
    static const int64_t n = [] { const char *e = getenv("CG_ATTN_BLOCKS"); return e ? atoll(e) : 1024ll; }();
    return n;
}

// Longest cache that the one-workgroup-per-KV-head attention kernel takes (env CG_ATTN_WHOLE_T, for measurements).
static int64_t attn_whole_limit() {
    static const int64_t n = [] { const char *e = getenv("CG_ATTN_WHOLE_T"); return e ? atoll(e) : 4096ll; }();
    return n;
}

// Longest cache that the one-workgroup-per-row attention kernel takes in segments (env CG_ATTN_SEGMENT_T, for measurements).
// Measured at 128 query rows: 6000 positions in 25.9 + 4.1 us against 33.0 + 7.6 for the chunked pair, 12000 positions (three
// segments, one and a half rounds of workgroups) in 56 + 4 against 47 + 11.
static int64_t attn_segment_limit() {
    static const int64_t n = [] { const char *e = getenv("CG_ATTN_SEGMENT_T"); return e ? atoll(e) : 8192ll; }();
    return n;
}

// Launches of the one-workgroup-per-row attention kernel with fewer workgroups than this split each row's output in
// two halves (env CG_ATTN_HALVES_BELOW, for measurements; 0: never).
static int64_t attn_row_halves_below() {
    static const int64_t n = [] { const char *e = getenv("CG_ATTN_HALVES_BELOW"); return e ? atoll(e) : 256ll; }();
    return n;
}

// Most segments per KV head (env CG_ATTN_SEG_MAX, for measurements).  With few (batch entry, KV head) groups many segments
// pay: one group of 8 KV heads with head_dim 128 at 4500 positions 18.7 us with up to 32 segments, 24.0 with up to 16.
static int64_t attn_seg_max() {
    static const int64_t n = [] { const char *e = getenv("CG_ATTN_SEG_MAX"); return e ? atoll(e) : 32ll; }();
    return n;
}

template <class P, int LPT, int MM, int PASSES, bool LOOP>
static int launch_seg_kernel(cg_backend *be, const AttnArgs &g, const FusedArgs &a, uint32_t batch) {
    const size_t lds = seg_lds_bytes(MM, LPT * 4, g.chunk);
    static const bool lds_ok = hipFuncSetAttribute(reinterpret_cast<const void *>(&decode_attention_seg_kernel<P, LPT, MM, PASSES, LOOP>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                                   (int)seg_lds_bytes(MM, LPT * 4, kSegMaxChunk)) == hipSuccess;
    if (!lds_ok) return fail(CG_ERR_DEVICE, "decode attention: cannot reserve %zu bytes of LDS", seg_lds_bytes(MM, LPT * 4, kSegMaxChunk));
    hipLaunchKernelGGL((decode_attention_seg_kernel<P, LPT, MM, PASSES, LOOP>), dim3(g.splits, batch), dim3(kSegBlock), lds, be->stream, g, a);
    return CG_OK;
}

int launch_decode_attention(cg_backend *be, const Pending &p, const int64_t *pdims, int prank, const cg_tensor *q,
                            const cg_tensor *kt, const cg_tensor *v, cg_tensor *out) {
    if (int frc = flush_deferred(be)) return frc;
    using P = RowsSoftmaxCausal;
    if (!be->aot || !program_matches<P>(p) || !p.leaf[0].lazy || p.leaf[0].lazy->result || p.reduced) return kDeclined;
    cg_tensor pd; // the soft-max result as a dense descriptor: the left operand of p.V
    pd.rank = prank;
    int64_t st = 1;
    for (int i = prank - 1; i >= 0; i--) {
        pd.dims[i] = pdims[i];
        pd.strides[i] = st;
        st *= pdims[i];
    }
    if (p.leaf[0].offset != 0) return kDeclined;
    for (int i = 0; i < prank; i++)
        if (pdims[i] > 1 && p.leaf[0].strides[i] != pd.strides[i]) return kDeclined;
    MmFold f1, f2;
    if (fold_matmul(q, kt, &f1) || fold_matmul(&pd, v, &f2)) return kDeclined;
    const int64_t T = f1.N, hd = f1.K;
    if (f1.M != f2.M || f1.M < 1 || f1.M > kAttnRows || f1.nb != f2.nb || f2.K != T || f2.N != hd) return kDeclined;
    if (hd != 64 && hd != 128) return kDeclined;
    if (f1.a_sk != 1 || f1.b_sk != 1 || f2.b_sn != 1 || f2.a_sk != 1 || f2.a_sm != T) return kDeclined;
    if (f1.batch < 1 || f1.batch > 65535 || T < 1 || T > 0x7FFFFFFFll) return kDeclined;
    for (int d = 0; d < f1.nb; d++)
        if (f1.bd[d] != f2.bd[d] || f2.a_bs[d] % T || f1.a_bs[d] % 4 || f1.b_bs[d] % 4 || f2.b_bs[d] % 4) return kDeclined;
    if (f1.a_sm % 4 || f1.b_sn % 4 || f2.b_sk % 4) return kDeclined;
    const void *pq, *pk, *pv;
    int rc = device_ptr(q, &pq);
    if (!rc) rc = device_ptr(kt, &pk);
    if (!rc) rc = device_ptr(v, &pv);
    if (rc) return rc;
    if (reinterpret_cast<uintptr_t>(pq) % 16 || reinterpret_cast<uintptr_t>(pk) % 16 || reinterpret_cast<uintptr_t>(pv) % 16)
        return kDeclined;
    FusedArgs a;
    double leaf_bytes;
    bool full;
    rc = fill_args(be, p, pdims, prank, nullptr, true, &a, &leaf_bytes, &full, -1, true);
    if (rc) return rc;
    uint64_t rows = 1;
    for (uint32_t d = 0; d < a.g.nouter; d++) rows *= a.g.od[d];
    if (a.g.inner != (uint32_t)T || rows != (uint64_t)f1.batch * (uint64_t)f1.M) return kDeclined;

    AttnArgs g;
    memset(&g, 0, sizeof g);
    g.Q = static_cast<const uint32_t *>(pq);
    g.Kc = static_cast<const uint32_t *>(pk);
    g.V = static_cast<const uint32_t *>(pv);
    g.M = (uint32_t)f1.M;
    g.T = (uint32_t)T;
    g.hd = (uint32_t)hd;
    // enough workgroups for every CU twice over, chunks of 64..256 positions
    const int64_t cap = attn_chunk_cap(hd == 64 ? 16 : 32);
    const int64_t want = std::max<int64_t>(1, attn_blocks() / f1.batch);
    int64_t chunk = std::min<int64_t>(cap, std::max<int64_t>(32, (T + want - 1) / want));
    chunk = std::min<int64_t>(cap, (chunk + 15) / 16 * 16);
    g.chunk = (uint32_t)chunk;
    g.splits = (uint32_t)((T + chunk - 1) / chunk);
    g.nb = (uint32_t)f1.nb;
    for (int d = 0; d < f1.nb; d++) {
        g.bd[d] = (uint32_t)f1.bd[d];
        g.bdiv[d] = make_fastdiv(g.bd[d]);
        g.q_bs[d] = f1.a_bs[d];
        g.k_bs[d] = f1.b_bs[d];
        g.v_bs[d] = f2.b_bs[d];
        g.p_bs[d] = f2.a_bs[d];
    }
    g.q_sm = f1.a_sm;
    g.k_st = f1.b_sn;
    g.v_st = f2.b_sk;
    // One workgroup per query row: a cache of up to kRowMaxT positions in one launch with nothing to combine (beyond
    // 1024 positions only while the workgroups fit the compute units in one round: a row costs its compute unit
    // T x head_dim x 4 multiply-adds); longer caches in segments of at most kRowMaxT positions per workgroup, merged by the
    // combine kernel.  Everything else goes to the chunked kernel below, which spreads a KV head over many workgroups.
    const int64_t qrows = f1.batch * f1.M;
    // A workgroup per (batch entry, KV head) and segment of the cache, all of the group's rows together: every byte of K and
    // V is pulled into a compute unit once.  As many segments as put a workgroup on every compute unit, at most
    // attn_seg_max() (each segment is one more partial result to merge), each a whole number of passes.  Taken for long
    // caches, and from 1024 positions when there are more query rows than compute units.  Measured with its combine launch
    // against the kernels below (batch 4 x 8 KV heads x 4 rows, head_dim 64): 2100 positions 20.4 against 19.7 us (the segment
    // kernel alone 13.6 against 19.7: what it saves, the combine launch and the hand-over to it cost again), 6000 positions 34.9
    // against 34.9, 9000 positions 44 against 55, 12000 positions 53 against 64; batch 16 at 2100 positions 42 against 46.
    // With at most 8 groups (a single sequence) the kernels below leave most of the device idle and the segments win from 2560
    // positions on: 8 KV heads, head_dim 128: 3000 positions 17.2 against 28.3 us, 12000 positions 31.7 against 59.0; 3 KV
    // heads, head_dim 64: 4500 positions 16.7 against 20.0, 12000 positions 22.1 against 40.5 (2100 positions: 15.8 against 15.8).
    // (Merging the segments inside the kernel — the workgroup that counts itself last at a device-scope counter reads the
    // others' results — was measured and costs what the combine launch costs: the stores must reach memory, the count must come
    // back and the loads go out again, 6 to 7 us in all; with a release / acquire fence per workgroup 24.0 against 19.3 us.)
    if (be->attn_seg_from > 0 && (T >= be->attn_seg_from || (qrows > 256 && T >= 1024) || (f1.batch <= 8 && T >= 2560))) {
        const int64_t tpb = hd == 64 ? kSegBlock / 16 : kSegBlock / 32;
        int64_t want = std::min<int64_t>(attn_seg_max(), std::max<int64_t>(1, 256 / f1.batch));
        want = std::max<int64_t>(1, std::min<int64_t>(want, T / 64));
        const int64_t chunk = ((T + want - 1) / want + tpb - 1) / tpb * tpb;
        if (chunk <= kSegMaxChunk) {
            g.chunk = (uint32_t)chunk;
            g.splits = (uint32_t)((T + chunk - 1) / chunk);
            const size_t o_b = (size_t)f1.batch * g.splits * g.M * hd * 4, ml_b = (size_t)f1.batch * g.splits * g.M * 2 * 4;
            void *so = nullptr, *sml = nullptr;
            size_t cso = 0, csml = 0;
            rc = be->pool.alloc(o_b, &so, &cso);
            if (rc) return rc;
            rc = be->pool.alloc(ml_b, &sml, &csml);
            if (rc) {
                be->pool.free(so, cso);
                return rc;
            }
            g.part_o = static_cast<float *>(so);
            g.part_ml = static_cast<float *>(sml);
            be->programs_compiled++;
            {
                ProfScope prof(be, CG_K_GEMM_SKINNY, distinct_bytes(q) + distinct_bytes(kt) + distinct_bytes(v) + distinct_bytes(out));
                const bool one_trip = chunk <= 5 * tpb;
                const uint32_t nb = (uint32_t)f1.batch;
#define CG_SEG_KERNEL(LPT, MMV)                                                                    \
    rc = one_trip ? launch_seg_kernel<P, LPT, MMV, 5, false>(be, g, a, nb) : launch_seg_kernel<P, LPT, MMV, 4, true>(be, g, a, nb)
                if (hd == 64 && g.M <= 4) CG_SEG_KERNEL(16, 4);
                else if (hd == 64) CG_SEG_KERNEL(16, 8);
                else if (g.M <= 4) CG_SEG_KERNEL(32, 4);
                else CG_SEG_KERNEL(32, 8);
#undef CG_SEG_KERNEL
                if (!rc) {
                    const uint64_t nrows = (uint64_t)f1.batch * g.M, waves = kBlock / 64;
                    hipLaunchKernelGGL(decode_attention_combine_kernel, dim3((uint32_t)((nrows + waves - 1) / waves)), dim3(kBlock), 0,
                                       be->stream, g.part_o, g.part_ml, static_cast<uint32_t *>(out->buf->ptr), g.splits, g.M,
                                       (uint32_t)hd, nrows);
                }
            }
            be->pool.free(so, cso); // stream-ordered: later users queue behind the combine
            be->pool.free(sml, csml);
            if (rc) return rc;
            hipError_t e = hipGetLastError();
            return e == hipSuccess ? CG_OK : hip_fail(e, "decode attention launch");
        }
    }
    const bool one_launch = T <= std::min<int64_t>(attn_whole_limit(), kRowMaxT) && (T <= 1024 || qrows <= 256);
    const bool segmented = !one_launch && attn_whole_limit() > 0 && T > kRowMaxT && T <= attn_segment_limit() && qrows <= 256;
    if (one_launch || segmented) {
        be->programs_compiled++;
        ProfScope prof(be, CG_K_GEMM_SKINNY, distinct_bytes(q) + distinct_bytes(kt) + distinct_bytes(v) + distinct_bytes(out));
        uint32_t *const po = static_cast<uint32_t *>(out->buf->ptr);
        const uint32_t nseg = segmented ? (uint32_t)((T + kRowMaxT - 1) / kRowMaxT) : 1u;
        const int64_t seglen = segmented ? ((T + nseg - 1) / nseg + 63) / 64 * 64 : T;
        g.chunk = (uint32_t)seglen;
        g.splits = (uint32_t)f1.batch; // (this kernel has no chunks: the field carries the number of batch entries)
        void *part_o = nullptr, *part_ml = nullptr;
        size_t co = 0, cml = 0;
        if (segmented) {
            rc = be->pool.alloc((size_t)f1.batch * nseg * g.M * hd * 4, &part_o, &co);
            if (rc) return rc;
            rc = be->pool.alloc((size_t)f1.batch * nseg * g.M * 2 * 4, &part_ml, &cml);
            if (rc) {
                be->pool.free(part_o, co);
                return rc;
            }
        }
        g.part_o = static_cast<float *>(part_o);
        g.part_ml = static_cast<float *>(part_ml);
        const int64_t per_pass = hd == 64 ? kRowBlock / 16 : kRowBlock / 32;
        const int passes = seglen <= 5 * per_pass ? 5 : seglen <= 10 * per_pass ? 10 : seglen <= 16 * per_pass ? 16 : 0;
        const bool halves = qrows * nseg * 2 <= attn_row_halves_below(); // two workgroups per row still leave compute units idle
        const dim3 grid((uint32_t)((f1.batch + 7) / 8 * 8 * g.M * (halves ? 2 : 1)), nseg), block(kRowBlock);
#define CG_ROW_KERNEL(LPT, VS)                                                                                                     \
    do {                                                                                                                           \
        if (passes == 5) hipLaunchKernelGGL((decode_attention_row_kernel<P, LPT, 5, false, VS>), grid, block, 0, be->stream, g, a, po);   \
        else if (passes == 10) hipLaunchKernelGGL((decode_attention_row_kernel<P, LPT, 10, false, VS>), grid, block, 0, be->stream, g, a, po); \
        else if (passes == 16) hipLaunchKernelGGL((decode_attention_row_kernel<P, LPT, 16, false, VS>), grid, block, 0, be->stream, g, a, po); \
        else hipLaunchKernelGGL((decode_attention_row_kernel<P, LPT, 6, true, VS>), grid, block, 0, be->stream, g, a, po);          \
    } while (0)
        if (hd == 64 && halves) CG_ROW_KERNEL(16, 2);
        else if (hd == 64) CG_ROW_KERNEL(16, 1);
        else if (halves) CG_ROW_KERNEL(32, 2);
        else CG_ROW_KERNEL(32, 1);
#undef CG_ROW_KERNEL
        if (segmented) {
            const uint64_t nrows = (uint64_t)f1.batch * g.M, waves = kBlock / 64;
            hipLaunchKernelGGL(decode_attention_combine_kernel, dim3((uint32_t)((nrows + waves - 1) / waves)), dim3(kBlock), 0,
                               be->stream, g.part_o, g.part_ml, po, nseg, g.M, (uint32_t)hd, nrows);
            be->pool.free(part_o, co); // stream-ordered: later users queue behind the combine
            be->pool.free(part_ml, cml);
        }
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? CG_OK : hip_fail(e, "decode attention launch");
    }
    const size_t o_bytes = (size_t)f1.batch * g.splits * g.M * hd * 4, ml_bytes = (size_t)f1.batch * g.splits * g.M * 2 * 4;
    void *po = nullptr, *pml = nullptr;
    size_t co = 0, cml = 0;
    rc = be->pool.alloc(o_bytes, &po, &co);
    if (rc) return rc;
    rc = be->pool.alloc(ml_bytes, &pml, &cml);
    if (rc) {
        be->pool.free(po, co);
        return rc;
    }
    g.part_o = static_cast<float *>(po);
    g.part_ml = static_cast<float *>(pml);
    be->programs_compiled++;
    {
        ProfScope prof(be, CG_K_GEMM_SKINNY, distinct_bytes(q) + distinct_bytes(kt) + distinct_bytes(v) + distinct_bytes(out));
        dim3 grid(g.splits, (uint32_t)f1.batch);
        if (hd == 64)
            hipLaunchKernelGGL((decode_attention_kernel<P, 16>), grid, dim3(kBlock), 0, be->stream, g, a);
        else
            hipLaunchKernelGGL((decode_attention_kernel<P, 32>), grid, dim3(kBlock), 0, be->stream, g, a);
        const uint64_t rows = (uint64_t)f1.batch * g.M, waves = kBlock / 64;
        hipLaunchKernelGGL(decode_attention_combine_kernel, dim3((uint32_t)((rows + waves - 1) / waves)), dim3(kBlock), 0,
                           be->stream, g.part_o, g.part_ml, static_cast<uint32_t *>(out->buf->ptr), g.splits, g.M,
                           (uint32_t)hd, rows);
    }
    be->pool.free(po, co); // stream-ordered: later users queue behind the combine
    be->pool.free(pml, cml);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "decode attention launch");
}

// q.K^T -> causal soft-max -> p.V for many query rows per KV head (a prefill), in one pass: see
// prefill_attention_kernel.  Declines unless the program is the listed soft-max with a causal mask built
// from the backend's iota (query position against key position), head_dim is 64 and the operands are laid
// out as the decoder graphs lay them out.
// With CG_TRACE_PROGRAMS=1: which check made the one-pass prefill attention decline (the number counts the
// checks of launch_prefill_attention from the top).
static int pf_declined(const cg_backend *be, int check) {
    if (be->trace_programs) fprintf(stderr, "[cg program] prefill attention declined at check %d\n", check);
    return kDeclined;
}

int launch_prefill_attention(cg_backend *be, const Pending &p, const int64_t *pdims, int prank, const cg_tensor *q,
                             const cg_tensor *kt, const cg_tensor *v, cg_tensor *out) {
    if (int frc = flush_deferred(be)) return frc;
    using P = RowsSoftmaxCausal;
    if (!be->aot || prank != 4 || !program_matches<P>(p) || !p.leaf[0].lazy || p.leaf[0].lazy->result || p.reduced) return pf_declined(be, 1);
    cg_tensor pd; // the soft-max result as a dense descriptor: the left operand of p.V
    pd.rank = prank;
    int64_t st = 1;
    for (int i = prank - 1; i >= 0; i--) {
        pd.dims[i] = pdims[i];
        pd.strides[i] = st;
        st *= pdims[i];
    }
    if (p.leaf[0].offset != 0) return pf_declined(be, 2);
    for (int i = 0; i < prank; i++)
        if (pdims[i] > 1 && p.leaf[0].strides[i] != pd.strides[i]) return pf_declined(be, 3);
    // the mask: f32(l2 < l3) * l4 with l2 = position of the query (iota along axis 2, from some offset) and
    // l3 = position of the key (iota along axis 3, from 0); l4 hugely negative
    const LeafView &lq = p.leaf[2], &lk = p.leaf[3];
    const int64_t S = pdims[2], T = pdims[3];
    if (!be->iota || lq.buf != be->iota || lk.buf != be->iota || lk.offset != 0 || lq.offset < 0 || lq.offset + S > be->iota_len ||
        T > be->iota_len)
        return pf_declined(be, 4);
    for (int i = 0; i < 4; i++) {
        const int64_t want_q = i == 2 ? 1 : 0, want_k = i == 3 ? 1 : 0;
        if (pdims[i] > 1 && (lq.strides[i] != want_q || lk.strides[i] != want_k)) return pf_declined(be, 5);
    }
    float mask_mul;
    memcpy(&mask_mul, &p.leaf[4].ubits, 4);
    if (!(mask_mul <= -1e30f)) return pf_declined(be, 6);
    MmFold f1, f2;
    if (fold_matmul(q, kt, &f1) || fold_matmul(&pd, v, &f2)) return pf_declined(be, 7);
    const int64_t hd = f1.K;
    if (f1.N != T || f1.M != f2.M || f1.M <= kAttnRows || f1.M % S != 0 || f1.batch != f2.batch || f2.K != T || f2.N != hd) return pf_declined(be, 8);
    if (hd != 64 && hd != 128) return pf_declined(be, 9);
    if (f1.a_sk != 1 || f1.b_sk != 1 || f2.b_sn != 1 || f2.a_sk != 1 || f2.a_sm != T) return pf_declined(be, 10);
    if (f1.batch < 1 || f1.batch > 65535 || T < 1 || T > 0x7FFFFFFFll || f1.M > 0x7FFFFFFFll) return pf_declined(be, 11);
    for (int d = 0; d < f1.nb; d++)
        if (f1.a_bs[d] % 4 || f1.b_bs[d] % 4) return pf_declined(be, 12);
    for (int d = 0; d < f2.nb; d++)
        if (f2.b_bs[d] % 4) return pf_declined(be, 12);
    if (f1.a_sm % 4 || f1.b_sn % 4 || f2.b_sk % 4) return pf_declined(be, 13);
    // rows of the folded group must land in `out` in order: out is [batch][M][hd]
    if ((int64_t)f1.batch * f1.M * hd != numel(out) || !is_contiguous(out)) return pf_declined(be, 14);
    const void *pq, *pk, *pv;
    int rc = device_ptr(q, &pq);
    if (!rc) rc = device_ptr(kt, &pk);
    if (!rc) rc = device_ptr(v, &pv);
    if (rc) return rc;
    if (reinterpret_cast<uintptr_t>(pq) % 16 || reinterpret_cast<uintptr_t>(pk) % 16 || reinterpret_cast<uintptr_t>(pv) % 16)
        return pf_declined(be, 15);
    static const bool lds_ok = hipFuncSetAttribute(reinterpret_cast<const void *>(&prefill_attention_kernel<64>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                                   (int)prefill_lds_bytes(64)) == hipSuccess &&
                               hipFuncSetAttribute(reinterpret_cast<const void *>(&prefill_attention_kernel<128>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                                   (int)prefill_lds_bytes(128)) == hipSuccess;
    if (!lds_ok) return pf_declined(be, 16);
    AttnArgs g;
    memset(&g, 0, sizeof g);
    g.Q = static_cast<const uint32_t *>(pq);
    g.Kc = static_cast<const uint32_t *>(pk);
    g.V = static_cast<const uint32_t *>(pv);
    g.M = (uint32_t)f1.M;
    g.T = (uint32_t)T;
    g.hd = (uint32_t)hd;
    g.nb = (uint32_t)f1.nb;
    for (int d = 0; d < f1.nb; d++) {
        g.bd[d] = (uint32_t)f1.bd[d];
        g.bdiv[d] = make_fastdiv(g.bd[d]);
        g.q_bs[d] = f1.a_bs[d];
        g.k_bs[d] = f1.b_bs[d];
    }
    g.nbv = (uint32_t)f2.nb;
    for (int d = 0; d < f2.nb; d++) {
        g.vbd[d] = (uint32_t)f2.bd[d];
        g.vbdiv[d] = make_fastdiv(g.vbd[d]);
        g.v_bs[d] = f2.b_bs[d];
    }
    g.q_sm = f1.a_sm;
    g.k_st = f1.b_sn;
    g.v_st = f2.b_sk;
    PrefillArgs e;
    e.out = static_cast<uint32_t *>(out->buf->ptr);
    e.S = (uint32_t)S;
    e.pos0 = (uint32_t)lq.offset;
    e.scale = p.leaf[1].ubits;
    e.mask_mul = p.leaf[4].ubits;
    e.batch = (uint32_t)f1.batch;
    e.tiles_per_head = S % kPfRows == 0 ? (uint32_t)(S / kPfRows) : 0;
    const uint64_t nblocks = (uint64_t)((f1.M + kPfRows - 1) / kPfRows) * (uint64_t)f1.batch;
    if (nblocks > 0x7FFFFFFFull) return pf_declined(be, 17);
    // Fewer workgroups than the device takes at once (one sequence; a short prompt): what bounds the launch is the chain of
    // matrix instructions of the workgroup with the most keys, so the keys of every row tile are cut into parts (at least two
    // key tiles each, about two workgroups per compute unit in all) and a small second kernel merges the parts.
    // (env CG_PREFILL_KSPLIT=n forces n parts, 1 = never)
    static const int forced_split = [] { const char *ev = getenv("CG_PREFILL_KSPLIT"); return ev ? atoi(ev) : 0; }();
    const int64_t key_tiles = (std::min<int64_t>(T, (int64_t)e.pos0 + S) + kPfKeys - 1) / kPfKeys;
    int64_t ksplit = forced_split > 0 ? forced_split : std::min<int64_t>((512 + (int64_t)nblocks - 1) / (int64_t)nblocks, 8);
    ksplit = std::max<int64_t>(1, std::min<int64_t>(ksplit, key_tiles / 2));
    if (forced_split <= 0 && nblocks >= 256) ksplit = 1;
    e.ksplit = (uint32_t)ksplit;
    e.part_o = e.part_ml = nullptr;
    void *po = nullptr, *pml = nullptr;
    size_t cpo = 0, cpml = 0;
    const uint64_t rows = (uint64_t)f1.batch * (uint64_t)f1.M;
    if (ksplit > 1) {
        rc = be->pool.alloc((size_t)ksplit * rows * hd * 4, &po, &cpo);
        if (rc) return rc;
        rc = be->pool.alloc((size_t)ksplit * rows * 2 * 4, &pml, &cpml);
        if (rc) {
            be->pool.free(po, cpo);
            return rc;
        }
        e.part_o = static_cast<float *>(po);
        e.part_ml = static_cast<float *>(pml);
    }
    be->programs_compiled++;
    {
        // flop: the visible half of the [rows, T] rectangle, twice (scores and weighted sum)
        const double flop = 2.0 * 2.0 * (double)f1.batch * (double)f1.M * (double)hd * ((double)e.pos0 + 0.5 * (double)S);
        ProfScope prof(be, CG_K_ATTENTION, flop);
        dim3 grid((uint32_t)nblocks, (uint32_t)ksplit);
        if (hd == 64)
            hipLaunchKernelGGL((prefill_attention_kernel<64>), grid, dim3(kBlock), prefill_lds_bytes(64), be->stream, g, e);
        else
            hipLaunchKernelGGL((prefill_attention_kernel<128>), grid, dim3(kBlock), prefill_lds_bytes(128), be->stream, g, e);
        if (ksplit > 1) {
            const uint64_t items = rows * (uint64_t)(hd / 4);
            hipLaunchKernelGGL(prefill_attention_combine_kernel, dim3((uint32_t)((items + kBlock - 1) / kBlock)), dim3(kBlock), 0, be->stream,
                               e.part_o, e.part_ml, e.out, (uint32_t)ksplit, (uint32_t)hd, rows);
        }
    }
    if (ksplit > 1) {
        be->pool.free(po, cpo); // stream-ordered: later users queue behind the combine
        be->pool.free(pml, cpml);
    }
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? CG_OK : hip_fail(err, "prefill attention launch");
}

bool fused_program_fits(const Pending &p) {
    uint8_t phys[kMaxLeaves + kMaxInstr];
    return allocate_registers(p, phys);
}

int launch_fused(cg_backend *be, const cg_tensor *out, const Pending &p) {
    if (int frc = flush_deferred(be)) return frc;
    FusedArgs a;
    double bytes;
    bool full;
    int rc = fill_args(be, p, out->dims, out->rank, out, false, &a, &bytes, &full);
    if (rc) return rc;
    if (a.g.total == 0) return CG_OK;
    trace_program(be, p, p.ninstr, "map", out->dims, out->rank);
    ProfScope prof(be, CG_K_ELEMENTWISE, bytes + distinct_bytes(out));
    dim3 grid((uint32_t)((a.g.total + kBlock - 1) / kBlock)), block(kBlock);
    if (be->aot && aot_map_dispatch(p, a, grid, be->stream, MapPrograms{})) {
        be->programs_compiled++;
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? CG_OK : hip_fail(e, "compiled element-wise launch");
    }
    be->programs_interpreted++;
    if (a.g.vec == 4) {
        if (full)
            hipLaunchKernelGGL((fused_kernel<4, true>), grid, block, 0, be->stream, a);
        else
            hipLaunchKernelGGL((fused_kernel<4, false>), grid, block, 0, be->stream, a);
    } else {
        if (full)
            hipLaunchKernelGGL((fused_kernel<1, true>), grid, block, 0, be->stream, a);
        else
            hipLaunchKernelGGL((fused_kernel<1, false>), grid, block, 0, be->stream, a);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fused element-wise launch");
}

// Two or three element-wise results in one launch; declines unless every program is one the
// grouped kernel holds (rotary embedding, strided copy).
int launch_fused_group(cg_backend *be, const cg_tensor *const *outs, const Pending *const *ps, int n) {
    if (!be->aot || n < 2 || n > kMaxMapGroup) return kDeclined;
    FusedGroup g;
    double bytes = 0;
    uint32_t blocks = 0;
    for (int i = 0; i < n; i++) {
        const Pending &p = *ps[i];
        if (program_matches<MapRope>(p))
            g.prog[i] = 0;
        else if (p.nleaf == 1 && p.ninstr == 1 && p.nred == 0 && (p.ins[0].op & ~kInstrU32) == kCopy && p.ins[0].a == 0 &&
                 !p.leaf[0].uniform && !p.leaf[0].pw)
            g.prog[i] = 1;
        else
            return kDeclined;
        double b;
        bool full;
        int rc = fill_args(be, p, outs[i]->dims, outs[i]->rank, outs[i], false, &g.p[i], &b, &full);
        if (rc) return rc;
        if (g.p[i].g.total == 0) return kDeclined;
        bytes += b + distinct_bytes(outs[i]);
        g.first[i] = blocks;
        blocks += (uint32_t)((g.p[i].g.total + kBlock - 1) / kBlock);
    }
    g.first[n] = blocks;
    g.n = (uint32_t)n;
    for (int i = 0; i < n; i++) trace_program(be, *ps[i], ps[i]->ninstr, "map (grouped)", outs[i]->dims, outs[i]->rank);
    ProfScope prof(be, CG_K_ELEMENTWISE, bytes);
    hipLaunchKernelGGL(aot_map_group_kernel, dim3(blocks), dim3(kBlock), 0, be->stream, g);
    be->programs_compiled += n;
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "grouped element-wise launch");
}

int launch_fused_reduce(cg_backend *be, int kind, bool f32, const Pending &p, int ninstr, const int64_t *dims, int rank,
                        cg_tensor *out) {
    if (int frc = flush_deferred(be)) return frc;
    FusedArgs a;
    double bytes;
    bool full;
    int rc = fill_args(be, p, dims, rank, nullptr, true, &a, &bytes, &full, ninstr);
    if (rc) return rc;
    a.n = a.g.inner;
    uint64_t rows = 1;
    for (uint32_t d = 0; d < a.g.nouter; d++) rows *= a.g.od[d];
    if (rows > 0xFFFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "reduction extents above 2^32-1");
    a.rows = (uint32_t)rows;
    uint32_t *op = static_cast<uint32_t *>(out->buf->ptr);
    be->programs_interpreted++;
    trace_program(be, p, ninstr, kind == kSum ? "reduce-sum" : kind == kMax ? "reduce-max" : "reduce-argmax", dims, rank);
    ProfScope prof(be, CG_K_REDUCE, bytes + distinct_bytes(out));
    uint32_t want = (a.n + 7) / 8;
    int tpr = want <= 4 ? 4 : want <= 16 ? 16 : want <= 64 ? 64 : 256;
    uint32_t rpb = kBlock / tpr;
    dim3 grid((a.rows + rpb - 1) / rpb), block(kBlock);
    const int f = f32 ? 1 : 0;
#define CG_LAUNCH(VEC, TPR)                                                                                  \
    do {                                                                                                     \
        if (full)                                                                                            \
            hipLaunchKernelGGL((fused_reduce_kernel<VEC, TPR, true>), grid, block, 0, be->stream, a, op, kind, f);  \
        else                                                                                                 \
            hipLaunchKernelGGL((fused_reduce_kernel<VEC, TPR, false>), grid, block, 0, be->stream, a, op, kind, f); \
    } while (0)
    if (a.g.vec == 4) {
        switch (tpr) {
        case 4: CG_LAUNCH(4, 4); break;
        case 16: CG_LAUNCH(4, 16); break;
        case 64: CG_LAUNCH(4, 64); break;
        default: CG_LAUNCH(4, 256); break;
        }
    } else {
        switch (tpr) {
        case 4: CG_LAUNCH(1, 4); break;
        case 16: CG_LAUNCH(1, 16); break;
        case 64: CG_LAUNCH(1, 64); break;
        default: CG_LAUNCH(1, 256); break;
        }
    }
#undef CG_LAUNCH
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fused reduction launch");
}

int launch_fused_rows(cg_backend *be, const cg_tensor *out, const Pending &p, const int64_t *dims, int rank) {
    if (int frc = flush_deferred(be)) return frc;
    FusedArgs a;
    double bytes;
    bool full;
    int rc = fill_args(be, p, dims, rank, p.reduced ? nullptr : out, true, &a, &bytes, &full);
    if (rc) return rc;
    a.n = a.g.inner;
    a.reduced = p.reduced ? 1 : 0;
    uint64_t rows = 1;
    for (uint32_t d = 0; d < a.g.nouter; d++) rows *= a.g.od[d];
    if (rows > 0xFFFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "reduction extents above 2^32-1");
    a.rows = (uint32_t)rows;
    if (a.rows == 0 || a.n == 0) return CG_OK;
    uint32_t *rowout = nullptr;
    if (p.reduced) {
        if (!is_contiguous(out)) return fail(CG_ERR_ARG, "internal error: row results need a dense destination");
        const void *op;
        rc = device_ptr(out, &op);
        if (rc) return rc;
        rowout = static_cast<uint32_t *>(const_cast<void *>(op));
    }
    trace_program(be, p, p.ninstr, p.reduced ? "rows-reduced" : "rows", dims, rank);
    ProfScope prof(be, CG_K_ELEMENTWISE, bytes + distinct_bytes(out));
    uint32_t want = (a.n + 7) / 8;
    int tpr = want <= 4 ? 4 : want <= 16 ? 16 : want <= 64 ? 64 : 256;
    uint32_t rpb = kBlock / tpr;
    dim3 grid((a.rows + rpb - 1) / rpb), block(kBlock);
    if (be->aot && tpr >= 16 && aot_rows_dispatch(p, a, rowout, tpr, grid, be->stream, RowsPrograms{})) {
        be->programs_compiled++;
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? CG_OK : hip_fail(e, "compiled row-program launch");
    }
    be->programs_interpreted++;
#define CG_LAUNCH(VEC, TPR)                                                                           \
    do {                                                                                              \
        if (full)                                                                                     \
            hipLaunchKernelGGL((fused_rows_kernel<VEC, TPR, true>), grid, block, 0, be->stream, a, rowout);  \
        else                                                                                          \
            hipLaunchKernelGGL((fused_rows_kernel<VEC, TPR, false>), grid, block, 0, be->stream, a, rowout); \
    } while (0)
    if (a.g.vec == 4) {
        switch (tpr) {
        case 4: CG_LAUNCH(4, 4); break;
        case 16: CG_LAUNCH(4, 16); break;
        case 64: CG_LAUNCH(4, 64); break;
        default: CG_LAUNCH(4, 256); break;
        }
    } else {
        switch (tpr) {
        case 4: CG_LAUNCH(1, 4); break;
        case 16: CG_LAUNCH(1, 16); break;
        case 64: CG_LAUNCH(1, 64); break;
        default: CG_LAUNCH(1, 256); break;
        }
    }
#undef CG_LAUNCH
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fused row-program launch");
}

} // namespace cg
