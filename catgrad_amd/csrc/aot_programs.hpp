// Ahead-of-time specialised kernels for deferred programs (included by fused.hip, inside
// its anonymous namespace, after FusedArgs and the row helpers).
//
// The interpreter kernels run any program, but pay for decoding: operand moves through an
// indexed register file and a branch per instruction.  The decoder graphs of the model
// families produce only a handful of distinct programs (RMS norm with and without the
// residual adds in front, soft-max over masked scores, SiLU gating, rotary embedding, the
// residual sums), and they produce them for every layer of every step.  Each of those is
// listed here in the very encoding `Pending` uses, and the compiler turns it into
// straight-line code: `apply<OP, F>` per instruction, in program order, so results are
// bit-identical to the interpreter and to unfused execution.  A program that is not listed
// runs in the interpreter; CG_TRACE_PROGRAMS=1 prints programs in this notation.
#pragma once

#include <utility>

#define CG_PROGRAM(NAME, NLEAF, UNIFORM, PW, ...)                      \
    struct NAME {                                                      \
        static constexpr int nleaf = NLEAF;                            \
        static constexpr unsigned uniform = UNIFORM; /* bit l: leaf l is a constant */ \
        static constexpr int pw = PW; /* the piecewise leaf (a deferred last-axis concat), -1: none */ \
        static constexpr uint8_t code[][4] = {__VA_ARGS__};            \
        static constexpr int ninstr = (int)(sizeof(code) / 4);         \
    };

// op codes: 0 neg, 3 exp, 16 add, 17 sub, 18 mul, 19 div, 20 pow, 42 copy, 48 row-sum, 49 row-max;
// +128 = u32 operands (149 = u32 lt, 169 = cast u32 -> f32).  Registers 0..7 are leaves,
// 8 + i is the result of instruction i.  Which leaves are constants is part of a program's
// identity: the compiler then sees that whatever depends only on constants and row results
// (the square root of an RMS norm) does not change along a row and computes it once.

// ---- element-wise ------------------------------------------------------------------------
// cos * x + sin * rotate_half(x), rotate_half(x) = concat(-x2, x1) read in place as the
// piecewise leaf 3                                        (rotary embedding)
CG_PROGRAM(MapRope, 4, 0x0, 3, {18, 0, 1, 0}, {18, 2, 3, 2}, {16, 8, 9, 8})
// a strided copy (only used inside grouped launches; alone it is the single-op copy kernel)
CG_PROGRAM(MapCopy, 1, 0x0, -1, {42, 0, 0, 0})
// g * (1 / (1 + exp(-g))) * u                            (SiLU gate times up projection)
CG_PROGRAM(MapSiluMul, 3, 0x2, -1, {0, 0, 0, 0}, {3, 8, 8, 8}, {16, 1, 9, 1}, {19, 1, 10, 1}, {18, 0, 11, 0}, {18, 12, 2, 12})
// residual stream after three adds, in the two operand orders the layer loop produces
CG_PROGRAM(MapResidual3a, 4, 0x0, -1, {16, 1, 2, 1}, {16, 0, 8, 0}, {16, 9, 3, 9})
CG_PROGRAM(MapResidual3b, 4, 0x0, -1, {16, 1, 2, 1}, {16, 8, 3, 8}, {16, 0, 9, 0})

// ---- with row reduces ------------------------------------------------------------------------
// x / sqrt(sum(x*x)/n + eps) * gamma                     (RMS norm)
CG_PROGRAM(RowsRmsNorm, 5, 0xE, -1, {18, 0, 0, 0}, {48, 8, 8, 8}, {19, 9, 1, 9}, {16, 10, 2, 10}, {20, 11, 3, 11},
           {19, 0, 12, 0}, {18, 13, 4, 13})
// the same on h = a + b, and on h = a + (b + c) / (a + b) + c
CG_PROGRAM(RowsRmsNormAdd, 6, 0x1C, -1, {16, 0, 1, 0}, {18, 8, 8, 8}, {48, 9, 9, 9}, {19, 10, 2, 10}, {16, 11, 3, 11},
           {20, 12, 4, 12}, {19, 8, 13, 8}, {18, 14, 5, 14})
CG_PROGRAM(RowsRmsNormAdd2a, 7, 0x38, -1, {16, 1, 2, 1}, {16, 0, 8, 0}, {18, 9, 9, 9}, {48, 10, 10, 10}, {19, 11, 3, 11},
           {16, 12, 4, 12}, {20, 13, 5, 13}, {19, 9, 14, 9}, {18, 15, 6, 15})
CG_PROGRAM(RowsRmsNormAdd2b, 7, 0x38, -1, {16, 0, 1, 0}, {16, 8, 2, 8}, {18, 9, 9, 9}, {48, 10, 10, 10}, {19, 11, 3, 11},
           {16, 12, 4, 12}, {20, 13, 5, 13}, {19, 9, 14, 9}, {18, 15, 6, 15})
// softmax(s / d + f32(j < i) * m): attention scores, causal mask built from two index vectors
CG_PROGRAM(RowsSoftmaxCausal, 5, 0x12, -1, {19, 0, 1, 0}, {149, 2, 3, 2}, {169, 9, 9, 9}, {18, 10, 4, 10}, {16, 8, 11, 8},
           {49, 12, 12, 12}, {17, 12, 13, 12}, {3, 14, 14, 14}, {48, 15, 15, 15}, {19, 15, 16, 15})

// The same program for launches whose leaves and result all lie in 32-bit words (every tensor of an f32 model): the kernels
// compiled for WordsOnly<P> carry no code for the narrow formats.
template <class P> struct WordsOnly : P {
    static constexpr bool words_only = true;
};
template <class P, class = void> struct words_only_of : std::false_type {};
template <class P> struct words_only_of<P, std::void_t<decltype(P::words_only)>> : std::true_type {};

template <class... P> struct ProgramList {};
using MapPrograms = ProgramList<MapRope, MapSiluMul, MapResidual3a, MapResidual3b>;
using RowsPrograms = ProgramList<RowsRmsNorm, RowsRmsNormAdd, RowsRmsNormAdd2a, RowsRmsNormAdd2b, RowsSoftmaxCausal>;

template <class P> bool program_matches(const Pending &p) {
    if (p.nleaf != P::nleaf || p.ninstr != P::ninstr) return false;
    for (int l = 0; l < P::nleaf; l++)
        if (p.leaf[l].uniform != (((P::uniform >> l) & 1u) != 0) || p.leaf[l].pw != (l == P::pw)) return false;
    for (int i = 0; i < P::ninstr; i++) {
        const Instr &in = p.ins[i];
        if (in.op != P::code[i][0] || in.a != P::code[i][1] || in.b != P::code[i][2] || in.c != P::code[i][3])
            return false;
    }
    return true;
}

// ---- compile-time evaluation ------------------------------------------------------------------
template <class P> constexpr int reduces_before(int i) {
    int n = 0;
    for (int k = 0; k < i; k++) n += is_row_reduce(P::code[k][0]) ? 1 : 0;
    return n;
}
// index of row reduce number `phase`; ninstr when the program has no such reduce
template <class P> constexpr int reduce_index(int phase) {
    int n = 0;
    for (int k = 0; k < P::ninstr; k++)
        if (is_row_reduce(P::code[k][0]) && n++ == phase) return k;
    return P::ninstr;
}

template <class P, int VEC> struct Values {
    uint32_t v[kMaxLeaves + P::ninstr][VEC];
};

template <class P, int VEC, int I>
__device__ __forceinline__ void aot_step(Values<P, VEC> &s, const uint32_t (&rs)[kMaxRowReduce], uint32_t *fault) {
    constexpr int op = P::code[I][0];
    constexpr int a = P::code[I][1], b = P::code[I][2], c = P::code[I][3];
    if constexpr (is_row_reduce(op)) {
        constexpr int k = reduces_before<P>(I);
#pragma unroll
        for (int j = 0; j < VEC; j++) s.v[kMaxLeaves + I][j] = rs[k];
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++)
            s.v[kMaxLeaves + I][j] = apply<(op & ~kInstrU32), !(op & kInstrU32)>(s.v[a][j], s.v[b][j], s.v[c][j], fault);
    }
}

template <class P, int VEC, int... I>
__device__ __forceinline__ void aot_run(Values<P, VEC> &s, const uint32_t (&rs)[kMaxRowReduce], uint32_t *fault,
                                        std::integer_sequence<int, I...>) {
    (aot_step<P, VEC, I>(s, rs, fault), ...);
}

// Leaf l of the work item at position e of its row; off[nleaf] is the offset into the second
// part of the piecewise leaf (unused when the program has none).
template <class P, int VEC, int L>
__device__ __forceinline__ void aot_load_leaf(const FusedArgs &a, const int64_t (&off)[P::nleaf + 1], uint32_t e,
                                              uint32_t (&t)[VEC]) {
    if constexpr ((P::uniform >> L) & 1u) {
#pragma unroll
        for (int j = 0; j < VEC; j++) t[j] = a.leaf[L].ubits;
    } else if constexpr (L == P::pw) {
        const bool second = e >= a.pw_split;
        if (second) load_words<VEC, false, words_only_of<P>::value>(a.leaf2, off[P::nleaf], t);
        else load_words<VEC, false, words_only_of<P>::value>(a.leaf[L], off[L], t);
        if ((a.pw_neg >> (second ? 1 : 0)) & 1u) {
#pragma unroll
            for (int j = 0; j < VEC; j++) t[j] ^= 0x80000000u;
        }
    } else {
        load_words<VEC, false, words_only_of<P>::value>(a.leaf[L], off[L], t);
    }
}

template <class P, int VEC, int... L>
__device__ __forceinline__ void aot_load_all(const FusedArgs &a, const int64_t (&off)[P::nleaf + 1], uint32_t e,
                                             uint32_t (&v)[P::nleaf][VEC], std::integer_sequence<int, L...>) {
    (aot_load_leaf<P, VEC, L>(a, off, e, v[L]), ...);
}

// ---- element-wise kernel: the geometry of fused_kernel, the program compiled in ----------------------
template <class P, int VEC> __device__ __forceinline__ void aot_map_body(const FusedArgs &a, const uint32_t block) {
    const uint64_t v64 = (uint64_t)block * kBlock + threadIdx.x;
    if (v64 >= a.g.total) return;
    const uint32_t v = (uint32_t)v64;
    uint32_t row = fastdiv(v, a.g.ipr_div);
    const int64_t e = (int64_t)(v - row * a.g.ipr) * VEC;
    int64_t oo = e * a.out.is;
    int64_t off[P::nleaf + 1];
#pragma unroll
    for (int l = 0; l < P::nleaf; l++) off[l] = e * a.leaf[l].is;
    off[P::nleaf] = (e - (int64_t)a.pw_split) * a.leaf2.is;
    for (uint32_t d = 0; d < a.g.nouter; d++) {
        const uint32_t q = fastdiv(row, a.g.odiv[d]);
        const int64_t i = (int64_t)(row - q * a.g.od[d]);
        row = q;
        oo += i * a.out.os[d];
#pragma unroll
        for (int l = 0; l < P::nleaf; l++) off[l] += i * a.leaf[l].os[d];
        if constexpr (P::pw >= 0) off[P::nleaf] += i * a.leaf2.os[d];
    }
    Values<P, VEC> s;
    {
        uint32_t lw[P::nleaf][VEC];
        aot_load_all<P, VEC>(a, off, (uint32_t)e, lw, std::make_integer_sequence<int, P::nleaf>{});
#pragma unroll
        for (int l = 0; l < P::nleaf; l++)
#pragma unroll
            for (int j = 0; j < VEC; j++) s.v[l][j] = lw[l][j];
    }
    const uint32_t rs[kMaxRowReduce] = {0, 0, 0};
    aot_run<P, VEC>(s, rs, a.fault, std::make_integer_sequence<int, P::ninstr>{});
    store_words<VEC, false, words_only_of<P>::value>(a.out, oo, s.v[kMaxLeaves + P::ninstr - 1]);
}
template <class P, int VEC> __global__ __launch_bounds__(kBlock) void aot_map_kernel(const FusedArgs a) {
    aot_map_body<P, VEC>(a, blockIdx.x);
}

// Up to three small element-wise launches in one: the writes of a decode step that nobody reads
// before the attention does (rotary embedding of k into the cache, v into the cache, rotary
// embedding of q).  Each workgroup finds its entry from the table of first workgroups.
constexpr int kMaxMapGroup = 3;
struct FusedGroup {
    FusedArgs p[kMaxMapGroup];
    uint32_t first[kMaxMapGroup + 1]; // first workgroup of each entry; first[n] = grid size
    uint32_t n;
    uint32_t prog[kMaxMapGroup]; // 0: MapRope, 1: MapCopy
};
static_assert(sizeof(FusedGroup) <= 4096, "kernel arguments are limited to 4 KiB");
__global__ __launch_bounds__(kBlock) void aot_map_group_kernel(const FusedGroup g) {
    uint32_t e = 0;
    while (e + 1 < g.n && blockIdx.x >= g.first[e + 1]) e++;
    const uint32_t block = blockIdx.x - g.first[e];
    const FusedArgs &a = g.p[e];
    if (g.prog[e] == 0) {
        if (a.g.vec == 4) aot_map_body<MapRope, 4>(a, block);
        else aot_map_body<MapRope, 1>(a, block);
    } else {
        if (a.g.vec == 4) aot_map_body<MapCopy, 4>(a, block);
        else aot_map_body<MapCopy, 1>(a, block);
    }
}

// ---- row kernel: the phases of fused_rows_kernel, unrolled at compile time -----------------------------
// CI > 0: a lane keeps the leaf words of its (at most CI) work items in registers, so the
// row is read from memory once however many reduces the program has.  CI == 0: rows too long
// for that; every walk re-reads the leaves (from L1/L2).
template <class P, int VEC> struct LeafWords {
    uint32_t v[P::nleaf][VEC];
};

template <class P, int VEC>
__device__ __forceinline__ void aot_fetch(const FusedArgs &a, const int64_t (&base)[P::nleaf + 1], uint32_t it,
                                          LeafWords<P, VEC> &w) {
    int64_t off[P::nleaf + 1];
#pragma unroll
    for (int l = 0; l < P::nleaf; l++) off[l] = base[l] + (int64_t)it * VEC * a.leaf[l].is;
    off[P::nleaf] = base[P::nleaf] + ((int64_t)it * VEC - (int64_t)a.pw_split) * a.leaf2.is;
    aot_load_all<P, VEC>(a, off, it * VEC, w.v, std::make_integer_sequence<int, P::nleaf>{});
}

// Value of instructions [0, UPTO) on one work item; returns the register file.
template <class P, int VEC, int UPTO>
__device__ __forceinline__ Values<P, VEC> aot_eval(const LeafWords<P, VEC> &w, const uint32_t (&rs)[kMaxRowReduce],
                                                   uint32_t *fault) {
    Values<P, VEC> s;
#pragma unroll
    for (int l = 0; l < P::nleaf; l++)
#pragma unroll
        for (int j = 0; j < VEC; j++) s.v[l][j] = w.v[l][j];
    aot_run<P, VEC>(s, rs, fault, std::make_integer_sequence<int, UPTO>{});
    return s;
}

template <bool IS_MAX, bool F, int TPR> __device__ __forceinline__ uint32_t aot_row_combine(uint32_t acc) {
    constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
    for (int m = W / 2; m >= 1; m >>= 1) acc = row_merge(IS_MAX, F, acc, (uint32_t)__shfl_xor((int)acc, m));
    if constexpr (TPR > 64) {
        __shared__ uint32_t part[kBlock / 64];
        if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = acc;
        __syncthreads();
        acc = part[0];
#pragma unroll
        for (int w = 1; w < kBlock / 64; w++) acc = row_merge(IS_MAX, F, acc, part[w]);
        __syncthreads();
    }
    return acc;
}

template <class P, int VEC, int TPR, int CI, int PHASE>
__device__ __forceinline__ void aot_rows_phase(const FusedArgs &a, const int64_t (&base)[P::nleaf + 1], uint32_t lane, bool live,
                                               uint32_t items, const LeafWords<P, VEC> (&cache)[CI > 0 ? CI : 1],
                                               uint32_t (&rs)[kMaxRowReduce]) {
    constexpr int ri = reduce_index<P>(PHASE);
    constexpr int rop = P::code[ri][0];
    constexpr bool is_max = (rop & ~kInstrU32) == kRowMax, f = !(rop & kInstrU32);
    constexpr int src = P::code[ri][1];
    uint32_t acc = row_init(is_max, f);
    if constexpr (CI > 0) {
#pragma unroll
        for (int c = 0; c < CI; c++) {
            if (live && lane + c * TPR < items) {
                const Values<P, VEC> s = aot_eval<P, VEC, ri>(cache[c], rs, a.fault);
#pragma unroll
                for (int j = 0; j < VEC; j++) acc = row_merge(is_max, f, acc, s.v[src][j]);
            }
        }
    } else if (live) {
        for (uint32_t it = lane; it < items; it += TPR) {
            LeafWords<P, VEC> w;
            aot_fetch<P, VEC>(a, base, it, w);
            const Values<P, VEC> s = aot_eval<P, VEC, ri>(w, rs, a.fault);
#pragma unroll
            for (int j = 0; j < VEC; j++) acc = row_merge(is_max, f, acc, s.v[src][j]);
        }
    }
    rs[PHASE] = aot_row_combine<is_max, f, TPR>(acc);
}

template <class P, int VEC, int TPR, int CI, int... PH>
__device__ __forceinline__ void aot_rows_phases(const FusedArgs &a, const int64_t (&base)[P::nleaf + 1], uint32_t lane, bool live,
                                                uint32_t items, const LeafWords<P, VEC> (&cache)[CI > 0 ? CI : 1],
                                                uint32_t (&rs)[kMaxRowReduce], std::integer_sequence<int, PH...>) {
    (aot_rows_phase<P, VEC, TPR, CI, PH>(a, base, lane, live, items, cache, rs), ...);
}

template <class P, int VEC, int TPR, int CI>
__global__ __launch_bounds__(kBlock) void aot_rows_kernel(const FusedArgs a, uint32_t *rowout) {
    constexpr int RPB = kBlock / TPR;
    constexpr int NRED = reduces_before<P>(P::ninstr);
    const uint32_t lane = threadIdx.x % TPR;
    const uint32_t row = blockIdx.x * RPB + threadIdx.x / TPR;
    const bool live = row < a.rows;
    int64_t base[P::nleaf + 1];
#pragma unroll
    for (int l = 0; l <= P::nleaf; l++) base[l] = 0;
    int64_t obase = 0;
    if (live) {
        uint32_t rr = row;
        for (uint32_t d = 0; d < a.g.nouter; d++) {
            const uint32_t q = fastdiv(rr, a.g.odiv[d]);
            const int64_t i = (int64_t)(rr - q * a.g.od[d]);
            rr = q;
            obase += i * a.out.os[d];
#pragma unroll
            for (int l = 0; l < P::nleaf; l++) base[l] += i * a.leaf[l].os[d];
            if constexpr (P::pw >= 0) base[P::nleaf] += i * a.leaf2.os[d];
        }
    }
    const uint32_t items = a.n / VEC;
    LeafWords<P, VEC> cache[CI > 0 ? CI : 1];
    if constexpr (CI > 0) {
#pragma unroll
        for (int c = 0; c < CI; c++)
            if (live && lane + c * TPR < items) aot_fetch<P, VEC>(a, base, lane + c * TPR, cache[c]);
    }
    uint32_t rs[kMaxRowReduce] = {0, 0, 0};
    aot_rows_phases<P, VEC, TPR, CI>(a, base, lane, live, items, cache, rs, std::make_integer_sequence<int, NRED>{});
    if (!live) return;
    if (a.reduced) {
        if (lane == 0) {
            LeafWords<P, VEC> w;
            aot_fetch<P, VEC>(a, base, 0, w);
            const Values<P, VEC> s = aot_eval<P, VEC, P::ninstr>(w, rs, a.fault);
            rowout[row] = s.v[kMaxLeaves + P::ninstr - 1][0];
        }
        return;
    }
    if constexpr (CI > 0) {
#pragma unroll
        for (int c = 0; c < CI; c++) {
            const uint32_t it = lane + c * TPR;
            if (it < items) {
                const Values<P, VEC> s = aot_eval<P, VEC, P::ninstr>(cache[c], rs, a.fault);
                store_words<VEC, false, words_only_of<P>::value>(a.out, obase + (int64_t)it * VEC * a.out.is, s.v[kMaxLeaves + P::ninstr - 1]);
            }
        }
    } else {
        for (uint32_t it = lane; it < items; it += TPR) {
            LeafWords<P, VEC> w;
            aot_fetch<P, VEC>(a, base, it, w);
            const Values<P, VEC> s = aot_eval<P, VEC, P::ninstr>(w, rs, a.fault);
            store_words<VEC, false, words_only_of<P>::value>(a.out, obase + (int64_t)it * VEC * a.out.is, s.v[kMaxLeaves + P::ninstr - 1]);
        }
    }
}

// ---- dispatch ---------------------------------------------------------------------------------------
inline bool all_words(const FusedArgs &a) {
    bool words = a.out.fmt == kFmtWords && a.leaf2.fmt == kFmtWords;
    for (uint32_t l = 0; l < a.nleaf; l++) words &= a.leaf[l].fmt == kFmtWords;
    return words;
}
template <class P> void aot_map_launch(const FusedArgs &a, dim3 grid, hipStream_t s) {
    const bool words = all_words(a);
    if (a.g.vec == 4 && words)
        hipLaunchKernelGGL((aot_map_kernel<WordsOnly<P>, 4>), grid, dim3(kBlock), 0, s, a);
    else if (a.g.vec == 4)
        hipLaunchKernelGGL((aot_map_kernel<P, 4>), grid, dim3(kBlock), 0, s, a);
    else if (words)
        hipLaunchKernelGGL((aot_map_kernel<WordsOnly<P>, 1>), grid, dim3(kBlock), 0, s, a);
    else
        hipLaunchKernelGGL((aot_map_kernel<P, 1>), grid, dim3(kBlock), 0, s, a);
}
inline bool aot_map_dispatch(const Pending &, const FusedArgs &, dim3, hipStream_t, ProgramList<>) { return false; }
template <class P, class... Rest>
bool aot_map_dispatch(const Pending &p, const FusedArgs &a, dim3 grid, hipStream_t s, ProgramList<P, Rest...>) {
    if (program_matches<P>(p)) {
        aot_map_launch<P>(a, grid, s);
        return true;
    }
    return aot_map_dispatch(p, a, grid, s, ProgramList<Rest...>{});
}

// Cached items per lane: 3 vectors of four (rows up to 12 * TPR elements) or 10 single
// elements (rows up to 10 * TPR); longer rows take the re-reading instantiation.
template <class P, int VEC> void aot_rows_launch(const FusedArgs &a, uint32_t *rowout, int tpr, dim3 grid, hipStream_t s) {
    constexpr int CI = VEC == 4 ? 3 : 10;
    const bool fits = (uint64_t)(a.n / VEC) <= (uint64_t)CI * (uint32_t)tpr;
#define CG_ROWS(TPR)                                                                                        \
    do {                                                                                                    \
        if (fits)                                                                                           \
            hipLaunchKernelGGL((aot_rows_kernel<P, VEC, TPR, CI>), grid, dim3(kBlock), 0, s, a, rowout);     \
        else                                                                                                \
            hipLaunchKernelGGL((aot_rows_kernel<P, VEC, TPR, 0>), grid, dim3(kBlock), 0, s, a, rowout);      \
    } while (0)
    if (tpr == 16) CG_ROWS(16);
    else if (tpr == 64) CG_ROWS(64);
    else CG_ROWS(256);
#undef CG_ROWS
}
inline bool aot_rows_dispatch(const Pending &, const FusedArgs &, uint32_t *, int, dim3, hipStream_t, ProgramList<>) {
    return false;
}
// tpr: lanes per row, one of 16 / 64 / 256 (shorter rows stay with the interpreter)
template <class P, class... Rest>
bool aot_rows_dispatch(const Pending &p, const FusedArgs &a, uint32_t *rowout, int tpr, dim3 grid, hipStream_t s,
                       ProgramList<P, Rest...>) {
    if (program_matches<P>(p)) {
        const bool words = all_words(a);
        if (a.g.vec == 4 && words)
            aot_rows_launch<WordsOnly<P>, 4>(a, rowout, tpr, grid, s);
        else if (a.g.vec == 4)
            aot_rows_launch<P, 4>(a, rowout, tpr, grid, s);
        else if (words)
            aot_rows_launch<WordsOnly<P>, 1>(a, rowout, tpr, grid, s);
        else
            aot_rows_launch<P, 1>(a, rowout, tpr, grid, s);
        return true;
    }
    return aot_rows_dispatch(p, a, rowout, tpr, grid, s, ProgramList<Rest...>{});
}
