// Decode-time attention in one pass (included by attention.hip after interp.hpp).
//
// A decode step issues, per layer, q.K^T (at most 8 query rows per KV head after the GQA
// group is folded into rows), the soft-max program over the scores, and p.V.  Each of the
// three reads or writes the [rows, T] score matrix and the two products each stream the
// cache once from a launch of their own.  When the scores product is still lazy at the
// moment its soft-max becomes the left operand of p.V (see LazyMm), the three run here
// instead: a workgroup takes one KV head and one chunk of the T cached positions, computes
// its scores from K, runs the soft-max program on them with the chunk as the row (local
// maximum m_c, local sum l_c of exp(x - m_c)), multiplies the un-normalised weights with its
// chunk of V, and writes (m_c, l_c, o_c).  A second small kernel combines the chunks:
//     out = sum_c e^(m_c - g) o_c / sum_c e^(m_c - g) l_c,   g = max_c m_c,
// which is the soft-max-weighted sum written with another grouping of the same terms.
// The program is the compiled RowsSoftmaxCausal; its instructions before the row maximum
// (scale, causal mask) and between maximum and sum (subtract, exp) are evaluated by the
// same template code as in aot_rows_kernel, the final division is replaced by the combine.
// HBM-bound: K and V once (2 x 4 x T x head_dim bytes per KV head) + the chunk results.
#pragma once

#include <type_traits>

typedef float float4v __attribute__((ext_vector_type(4)));

// Leaf words of leaves FIRST.. of one work item (leaf 0 of the attention program has no memory).
template <class P, int VEC, int FIRST, int... L>
__device__ __forceinline__ void aot_load_from(const FusedArgs &a, const int64_t (&off)[P::nleaf + 1], uint32_t e,
                                              uint32_t (&v)[P::nleaf][VEC], std::integer_sequence<int, L...>) {
    (aot_load_leaf<P, VEC, FIRST + L>(a, off, e, v[FIRST + L]), ...);
}
template <class P, int FIRST>
__device__ __forceinline__ void aot_fetch_from(const FusedArgs &a, const int64_t (&base)[P::nleaf + 1], uint32_t it,
                                               LeafWords<P, 1> &w) {
    int64_t off[P::nleaf + 1];
#pragma unroll
    for (int l = 0; l < P::nleaf; l++) off[l] = base[l] + (int64_t)it * a.leaf[l].is;
    off[P::nleaf] = 0;
    aot_load_from<P, 1, FIRST>(a, off, it, w.v, std::make_integer_sequence<int, P::nleaf - FIRST>{});
}

// Sum over the 16 lanes of a DPP row (lanes 16i..16i+15), left in every lane of the row: four
// rotate-and-add steps inside the vector ALU instead of four trips through the LDS crossbar.
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, false)); // row_ror:8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, false)); // row_ror:4
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xF, 0xF, false)); // row_ror:2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xF, 0xF, false)); // row_ror:1
    return v;
}

struct AttnArgs {
    const uint32_t *Q, *Kc, *V;
    float *part_o;  // [batch][splits][M][hd]
    float *part_ml; // [batch][splits][M][2]
    uint32_t M, T, hd, splits, chunk;
    uint32_t nb;
    uint32_t bd[kMaxBatchAxes];
    FastDiv bdiv[kMaxBatchAxes];
    int64_t q_bs[kMaxBatchAxes], k_bs[kMaxBatchAxes], v_bs[kMaxBatchAxes], p_bs[kMaxBatchAxes];
    int64_t q_sm; // stride between the query rows of a group
    int64_t k_st; // stride between cached positions of K (head_dim contiguous)
    int64_t v_st; // stride between cached positions of V (head_dim contiguous)
    // prefill only: the batch axes as p.V collapsed them (same number of entries, possibly another split)
    uint32_t nbv;
    uint32_t vbd[kMaxBatchAxes];
    FastDiv vbdiv[kMaxBatchAxes];
};

constexpr int kAttnRows = 8;    // most query rows per KV head
constexpr int kAttnPasses = 8; // cached positions per lane group and workgroup
// most cached positions per workgroup: 128 for head_dim 64, 64 for head_dim 128
constexpr int attn_chunk_cap(int lpt) { return kAttnPasses * (kBlock / lpt); }

// LPT lanes share a cached position (head_dim / 4): 16 or 32.  Every lane first asks for all of
// its K and V pieces of the chunk (at most 2 x 8 sixteen-byte loads in flight), so the chunk
// costs one trip to memory; scores, soft-max and the weighted sum then run out of registers and LDS.
template <class P, int LPT>
__global__ __launch_bounds__(kBlock) void decode_attention_kernel(const AttnArgs g, const FusedArgs a) {
    constexpr int HD = LPT * 4;
    constexpr int TPB = kBlock / LPT; // positions per pass
    constexpr int CAP = attn_chunk_cap(LPT);
    constexpr int IPL = CAP / 64; // chunk positions per lane in the soft-max phase
    constexpr int ri0 = reduce_index<P>(0), ri1 = reduce_index<P>(1);
    constexpr int src0 = P::code[ri0][1], src1 = P::code[ri1][1];
    static_assert((P::code[ri0][0] & ~kInstrU32) == kRowMax && (P::code[ri1][0] & ~kInstrU32) == kRowSum,
                  "a soft-max: row maximum, then row sum");
    __shared__ float sc[kAttnRows][CAP];
    __shared__ float red[TPB][kAttnRows * LPT + 1][4];
    const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const uint32_t split = blockIdx.x, b = blockIdx.y;
    const uint32_t t0 = split * g.chunk, t1 = min(g.T, t0 + g.chunk);
    // operand offsets of this batch entry
    int64_t oq = 0, ok = 0, ov = 0, op = 0;
    {
        uint32_t bb = b;
        // (every axis slot is visited, so that the fields are read from the argument block at once instead of one
        // dependent scalar load after the other)
#pragma unroll
        for (uint32_t d = 0; d < (uint32_t)kMaxBatchAxes; d++) {
            if (d >= g.nb) break;
            const uint32_t q = fastdiv(bb, g.bdiv[d]);
            const int64_t i = (int64_t)(bb - q * g.bd[d]);
            bb = q;
            oq += i * g.q_bs[d];
            ok += i * g.k_bs[d];
            ov += i * g.v_bs[d];
            op += i * g.p_bs[d];
        }
    }
    const uint32_t row0 = (uint32_t)(op / g.T); // first row of this group in the program's [rows, T] space
    const uint32_t l = tid % LPT, sub = tid / LPT;

    float4v kf[kAttnPasses], vf[kAttnPasses];
#pragma unroll
    for (int ps = 0; ps < kAttnPasses; ps++) {
        const uint32_t t = t0 + sub + ps * TPB;
        kf[ps] = (float4v){0.f, 0.f, 0.f, 0.f};
        vf[ps] = (float4v){0.f, 0.f, 0.f, 0.f};
        if (t < t1) {
            kf[ps] = *reinterpret_cast<const float4v *>(g.Kc + ok + (int64_t)t * g.k_st + l * 4);
            vf[ps] = *reinterpret_cast<const float4v *>(g.V + ov + (int64_t)t * g.v_st + l * 4);
        }
    }

    // ---- scores of the chunk: LPT lanes per position, one 16-byte piece of head_dim each
    {
        float4v qf[kAttnRows];
#pragma unroll
        for (int m = 0; m < kAttnRows; m++) {
            qf[m] = (float4v){0.f, 0.f, 0.f, 0.f};
            if ((uint32_t)m < g.M) qf[m] = *reinterpret_cast<const float4v *>(g.Q + oq + (int64_t)m * g.q_sm + l * 4);
        }
        const uint32_t passes = (t1 - t0 + TPB - 1) / TPB;
#pragma unroll
        for (int ps = 0; ps < kAttnPasses; ps++) {
            if ((uint32_t)ps < passes) {
                const uint32_t t = t0 + sub + ps * TPB;
#pragma unroll
                for (int m = 0; m < kAttnRows; m++) {
                    if ((uint32_t)m < g.M) {
                        float v = fmaf(qf[m][3], kf[ps][3], fmaf(qf[m][2], kf[ps][2], fmaf(qf[m][1], kf[ps][1], qf[m][0] * kf[ps][0])));
                        v = row16_sum(v);
                        if (LPT == 32) v += __shfl_xor(v, 16);
                        if (l == 0 && t < t1) sc[m][t - t0] = v;
                    }
                }
            }
        }
    }
    __syncthreads();

    // ---- the soft-max program on the chunk: a wave per query row, IPL positions per lane
    for (uint32_t m = wave; m < g.M; m += kBlock / 64) {
        const uint32_t row = row0 + m;
        int64_t base[P::nleaf + 1];
#pragma unroll
        for (int i = 0; i <= P::nleaf; i++) base[i] = 0;
        {
            uint32_t rr = row;
#pragma unroll
            for (uint32_t d = 0; d < (uint32_t)kMaxOuter; d++) {
                if (d >= a.g.nouter) break;
                const uint32_t q = fastdiv(rr, a.g.odiv[d]);
                const int64_t i = (int64_t)(rr - q * a.g.od[d]);
                rr = q;
#pragma unroll
                for (int lf = 1; lf < P::nleaf; lf++) base[lf] += i * a.leaf[lf].os[d];
            }
        }
        LeafWords<P, 1> w[IPL];
#pragma unroll
        for (int c = 0; c < IPL; c++) {
            const uint32_t i = lane + c * 64;
            if (i < t1 - t0) {
                aot_fetch_from<P, 1>(a, base, t0 + i, w[c]); // leaf 0 is the score
                w[c].v[0][0] = asu(sc[m][i]);
            }
        }
        uint32_t rs[kMaxRowReduce] = {0, 0, 0};
        uint32_t acc = row_init(true, true);
#pragma unroll
        for (int c = 0; c < IPL; c++) {
            if (lane + c * 64 < t1 - t0) {
                const Values<P, 1> s = aot_eval<P, 1, ri0>(w[c], rs, a.fault);
                acc = row_merge(true, true, acc, s.v[src0][0]);
            }
        }
#pragma unroll
        for (int sft = 32; sft >= 1; sft >>= 1) acc = row_merge(true, true, acc, (uint32_t)__shfl_xor((int)acc, sft));
        rs[0] = acc;
        uint32_t sum = row_init(false, true);
#pragma unroll
        for (int c = 0; c < IPL; c++) {
            const uint32_t i = lane + c * 64;
            if (i < t1 - t0) {
                const Values<P, 1> s = aot_eval<P, 1, ri1>(w[c], rs, a.fault);
                sum = row_merge(false, true, sum, s.v[src1][0]);
                sc[m][i] = asf(s.v[src1][0]); // the un-normalised weight
            }
        }
#pragma unroll
        for (int sft = 32; sft >= 1; sft >>= 1) sum = row_merge(false, true, sum, (uint32_t)__shfl_xor((int)sum, sft));
        if (lane == 0) {
            float *ml = g.part_ml + (((uint64_t)b * g.splits + split) * g.M + m) * 2;
            ml[0] = asf(acc);
            ml[1] = asf(sum);
        }
    }
    __syncthreads();

    // ---- weights times V: the lane's V pieces are those of its positions, head_dim piece l
    {
        float4v o[kAttnRows];
#pragma unroll
        for (int m = 0; m < kAttnRows; m++) o[m] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ps = 0; ps < kAttnPasses; ps++) {
            const uint32_t t = t0 + sub + ps * TPB;
            if (t < t1) {
#pragma unroll
                for (int m = 0; m < kAttnRows; m++) {
                    if ((uint32_t)m < g.M) {
                        const float wgt = sc[m][t - t0];
                        o[m][0] = fmaf(wgt, vf[ps][0], o[m][0]);
                        o[m][1] = fmaf(wgt, vf[ps][1], o[m][1]);
                        o[m][2] = fmaf(wgt, vf[ps][2], o[m][2]);
                        o[m][3] = fmaf(wgt, vf[ps][3], o[m][3]);
                    }
                }
            }
        }
#pragma unroll
        for (int m = 0; m < kAttnRows; m++)
            if ((uint32_t)m < g.M) {
#pragma unroll
                for (int j = 0; j < 4; j++) red[sub][m * LPT + l][j] = o[m][j];
            }
        __syncthreads();
        for (uint32_t e = tid; e < g.M * HD; e += kBlock) {
            const uint32_t m = e / HD, n = e % HD;
            float v = 0.0f;
#pragma unroll
            for (int k = 0; k < TPB; k++) v += red[k][m * LPT + n / 4][n % 4];
            g.part_o[(((uint64_t)b * g.splits + split) * g.M + m) * HD + n] = v;
        }
    }
}

// The same attention with ONE workgroup of 1024 threads per query row (and per half of head_dim, see VS) walking all
// T cached positions: no chunk results, no second launch.  At decode time a KV head's cache is a few hundred KiB to
// a few MiB, and the chunked pair of kernels spends most of its 20 us waiting (launch, operand offsets, a trip to
// memory, the hand-over to the combine, its trip).  Here the loads of K are asked for as far ahead as registers
// allow, the scores of the row wait in LDS, the soft-max program runs once over all of them (the row's maximum and
// sum cross the waves through LDS), V is on its way while that happens, and the weighted sum is divided by the
// row's sum where it is stored.  The workgroups of a batch entry (its query rows read the same K and V) get block
// indices a multiple of eight apart, which lands them on the same XCD: the second to last read hit in its L2.
// What bounds a workgroup is its compute unit's path to L2: measured, a compute unit streams about 60 GB/s (25 bytes a
// clock) out of L2 however many loads it keeps in flight (a ring of 16 passes per lane instead of two alternating trips
// of six was no faster), and a workgroup pulls all of K plus its half of V through it (835 KB at T = 2176: 14 us).
// Taken up to T = 4096 in one launch and, in
// two segments per row whose results decode_attention_combine_kernel merges, up to 8192; longer caches go to the chunked
// kernels, which spread a KV head over many workgroups.
// PASSES x (1024 / LPT) positions per trip to memory.  LOOP: several trips, the next always asked for before the
// current one is used (PASSES registers twice); else one trip covers T, the soft-max program's other leaves are
// asked for before K, and with at most ten passes V right behind K (the registers hold both).
// VS = 2: the workgroup computes all scores but only one half of head_dim of the output, so that twice as many compute
// units pull on V (used when the launch would otherwise leave half of them idle).
constexpr int kRowBlock = 1024;
constexpr int kRowMaxT = 4096;
template <class P, int LPT, int PASSES, bool LOOP, int VS>
__global__ __launch_bounds__(kRowBlock) void decode_attention_row_kernel(const AttnArgs g, const FusedArgs a, uint32_t *out) {
    constexpr int HD = LPT * 4;
    constexpr int TPB = kRowBlock / LPT; // positions per pass
    constexpr int SPAN = TPB * PASSES;    // positions per trip to memory
    constexpr int LPV = LPT / VS;         // lanes per position in the V phase
    constexpr int TPV = kRowBlock / LPV, PASSES_V = (PASSES + VS - 1) / VS, SPAN_V = TPV * PASSES_V;
    constexpr int WAVES = kRowBlock / 64;
    constexpr int IPL = LOOP ? kRowMaxT / kRowBlock : 1; // positions per thread in the soft-max phase
    constexpr bool V_EARLY = !LOOP && PASSES + PASSES_V <= 20;
    constexpr int ri0 = reduce_index<P>(0), ri1 = reduce_index<P>(1);
    constexpr int src0 = P::code[ri0][1], src1 = P::code[ri1][1];
    static_assert((P::code[ri0][0] & ~kInstrU32) == kRowMax && (P::code[ri1][0] & ~kInstrU32) == kRowSum,
                  "a soft-max: row maximum, then row sum");
    static_assert(LOOP || SPAN <= kRowBlock, "one position per thread in the soft-max phase");
    __shared__ float sc[LOOP ? kRowMaxT : kRowBlock];
    __shared__ float red[WAVES][HD / VS];
    __shared__ uint32_t cross[2][WAVES];
    const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    // a cache beyond kRowMaxT positions is cut into segments over grid.y: a workgroup then leaves its segment's maximum,
    // sum and un-normalised weighted sum for decode_attention_combine_kernel
    const uint32_t seg = blockIdx.y, t_first = seg * g.chunk;
    const uint32_t T = min(g.T, t_first + g.chunk) - t_first; // positions of this workgroup
    // block -> (batch entry, query row, half): the workgroups of an entry eight blocks apart
    const uint32_t rest = blockIdx.x / 8, inner = rest % (g.M * VS), m = inner / VS, part = inner % VS;
    const uint32_t b = rest / (g.M * VS) * 8 + blockIdx.x % 8;
    if (b >= g.splits) return; // (the number of batch entries; the same for the whole workgroup)
    int64_t oq = 0, ok = 0, ov = 0, op = 0;
    {
        uint32_t bb = b;
        // (every axis slot is visited, so that the fields are read from the argument block up front and at once
        // instead of one dependent scalar load after the other)
#pragma unroll
        for (uint32_t d = 0; d < (uint32_t)kMaxBatchAxes; d++) {
            if (d >= g.nb) break;
            const uint32_t q = fastdiv(bb, g.bdiv[d]);
            const int64_t i = (int64_t)(bb - q * g.bd[d]);
            bb = q;
            oq += i * g.q_bs[d];
            ok += i * g.k_bs[d];
            ov += i * g.v_bs[d];
            op += i * g.p_bs[d];
        }
    }
    const uint32_t l = tid % LPT, sub = tid / LPT, lv = tid % LPV, subv = tid / LPV;
    const uint32_t *kbase = g.Kc + ok + (int64_t)t_first * g.k_st + l * 4;
    const uint32_t *vbase = g.V + ov + (int64_t)t_first * g.v_st + (part * LPV + lv) * 4;
    // FULL (a tag type): the trip lies inside the T positions, nothing is checked
    const int64_t k_step = (int64_t)TPB * g.k_st, v_step = (int64_t)TPV * g.v_st;
    auto ask_k = [&](float4v (&f)[PASSES], uint32_t first, auto full) {
        const uint32_t *p = kbase + (int64_t)(first + sub) * g.k_st;
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            if constexpr (decltype(full)::value) {
                f[ps] = *reinterpret_cast<const float4v *>(p);
            } else {
                f[ps] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (first + sub + ps * TPB < T) f[ps] = *reinterpret_cast<const float4v *>(p);
            }
            p += k_step;
        }
    };
    auto ask_v = [&](float4v (&f)[PASSES_V], uint32_t first, auto full) {
        const uint32_t *p = vbase + (int64_t)(first + subv) * g.v_st;
#pragma unroll
        for (int ps = 0; ps < PASSES_V; ps++) {
            if constexpr (decltype(full)::value) {
                f[ps] = *reinterpret_cast<const float4v *>(p);
            } else {
                f[ps] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (first + subv + ps * TPV < T) f[ps] = *reinterpret_cast<const float4v *>(p);
            }
            p += v_step;
        }
    };
    constexpr std::true_type whole_trip{};
    constexpr std::false_type ragged{};
    // the trip that starts at `first`, checked only when it reaches beyond T
    auto ask_k_at = [&](float4v (&f)[PASSES], uint32_t first) {
        if (first + SPAN <= T) ask_k(f, first, whole_trip);
        else ask_k(f, first, ragged);
    };
    auto ask_v_at = [&](float4v (&f)[PASSES_V], uint32_t first) {
        if (first + SPAN_V <= T) ask_v(f, first, whole_trip);
        else ask_v(f, first, ragged);
    };
    float4v ka[PASSES], kb[LOOP ? PASSES : 1];
    float4v va[PASSES_V], vb[LOOP ? PASSES_V : 1];
    ask_k_at(ka, 0);
    if constexpr (V_EARLY) ask_v_at(va, 0);
    const float4v qf = *reinterpret_cast<const float4v *>(g.Q + oq + (int64_t)m * g.q_sm + l * 4);
    // the soft-max program's other leaves at this thread's positions (tid, tid + 1024, ...)
    LeafWords<P, 1> w[IPL];
    int64_t base[P::nleaf + 1];
    {
#pragma unroll
        for (int i = 0; i <= P::nleaf; i++) base[i] = 0;
        uint32_t rr = (uint32_t)(op / g.T) + m; // the row in the program's [rows, T] space
#pragma unroll
        for (uint32_t d = 0; d < (uint32_t)kMaxOuter; d++) {
            if (d >= a.g.nouter) break;
            const uint32_t q = fastdiv(rr, a.g.odiv[d]);
            const int64_t i = (int64_t)(rr - q * a.g.od[d]);
            rr = q;
#pragma unroll
            for (int lf = 1; lf < P::nleaf; lf++) base[lf] += i * a.leaf[lf].os[d];
        }
    }
    auto fetch_leaves = [&]() {
#pragma unroll
        for (int c = 0; c < IPL; c++)
            if (tid + c * kRowBlock < T) aot_fetch_from<P, 1>(a, base, t_first + tid + c * kRowBlock, w[c]);
    };
    if constexpr (!LOOP) fetch_leaves(); // nothing waits for them yet

    // ---- scores of the whole row
    auto score = [&](const float4v (&f)[PASSES], uint32_t first, auto full) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            const uint32_t t = first + sub + ps * TPB;
            if (decltype(full)::value || first + ps * TPB < T) { // the same for the whole workgroup
                float v = fmaf(qf[3], f[ps][3], fmaf(qf[2], f[ps][2], fmaf(qf[1], f[ps][1], qf[0] * f[ps][0])));
                v = row16_sum(v);
                if (LPT == 32) v += __shfl_xor(v, 16);
                if (l == 0 && (decltype(full)::value || t < T)) sc[t] = v;
            }
        }
    };
    auto score_at = [&](const float4v (&f)[PASSES], uint32_t first) {
        if (first + SPAN <= T) score(f, first, whole_trip);
        else score(f, first, ragged);
    };
    if constexpr (LOOP) {
        for (uint32_t first = 0; first < T; first += 2 * SPAN) {
            if (first + SPAN < T) ask_k_at(kb, first + SPAN);
            score_at(ka, first);
            if (first + 2 * SPAN < T) ask_k_at(ka, first + 2 * SPAN);
            if (first + SPAN < T) score_at(kb, first + SPAN);
        }
    } else {
        score_at(ka, 0);
    }
    if constexpr (!V_EARLY) ask_v_at(va, 0); // on its way through the soft-max
    if constexpr (LOOP) fetch_leaves();
    __syncthreads();

    // ---- the soft-max program over the row
    float total, row_max;
    {
        uint32_t rs[kMaxRowReduce] = {0, 0, 0};
        uint32_t acc = row_init(true, true);
#pragma unroll
        for (int c = 0; c < IPL; c++) {
            const uint32_t i = tid + c * kRowBlock;
            if (i < T) {
                w[c].v[0][0] = asu(sc[i]); // leaf 0 is the score
                const Values<P, 1> s = aot_eval<P, 1, ri0>(w[c], rs, a.fault);
                acc = row_merge(true, true, acc, s.v[src0][0]);
            }
        }
#pragma unroll
        for (int sft = 32; sft >= 1; sft >>= 1) acc = row_merge(true, true, acc, (uint32_t)__shfl_xor((int)acc, sft));
        if (lane == 0) cross[0][wave] = acc;
        __syncthreads();
        acc = cross[0][0];
#pragma unroll
        for (int k = 1; k < WAVES; k++) acc = row_merge(true, true, acc, cross[0][k]);
        rs[0] = acc;
        row_max = asf(acc);
        uint32_t sum = row_init(false, true);
#pragma unroll
        for (int c = 0; c < IPL; c++) {
            const uint32_t i = tid + c * kRowBlock;
            if (i < T) {
                const Values<P, 1> s = aot_eval<P, 1, ri1>(w[c], rs, a.fault);
                sum = row_merge(false, true, sum, s.v[src1][0]);
                sc[i] = asf(s.v[src1][0]); // the un-normalised weight
            }
        }
#pragma unroll
        for (int sft = 32; sft >= 1; sft >>= 1) sum = row_merge(false, true, sum, (uint32_t)__shfl_xor((int)sum, sft));
        if (lane == 0) cross[1][wave] = sum;
        __syncthreads();
        sum = cross[1][0];
#pragma unroll
        for (int k = 1; k < WAVES; k++) sum = row_merge(false, true, sum, cross[1][k]);
        total = asf(sum);
    }

    // ---- weights times V (this workgroup's columns)
    float4v o = {0.f, 0.f, 0.f, 0.f};
    auto weigh = [&](const float4v (&f)[PASSES_V], uint32_t first, auto full) {
#pragma unroll
        for (int ps = 0; ps < PASSES_V; ps++) {
            const uint32_t t = first + subv + ps * TPV;
            if (decltype(full)::value || t < T) {
                const float wgt = sc[t];
                o[0] = fmaf(wgt, f[ps][0], o[0]);
                o[1] = fmaf(wgt, f[ps][1], o[1]);
                o[2] = fmaf(wgt, f[ps][2], o[2]);
                o[3] = fmaf(wgt, f[ps][3], o[3]);
            }
        }
    };
    auto weigh_at = [&](const float4v (&f)[PASSES_V], uint32_t first) {
        if (first + SPAN_V <= T) weigh(f, first, whole_trip);
        else weigh(f, first, ragged);
    };
    if constexpr (LOOP) {
        for (uint32_t first = 0; first < T; first += 2 * SPAN_V) {
            if (first + SPAN_V < T) ask_v_at(vb, first + SPAN_V);
            weigh_at(va, first);
            if (first + 2 * SPAN_V < T) ask_v_at(va, first + 2 * SPAN_V);
            if (first + SPAN_V < T) weigh_at(vb, first + SPAN_V);
        }
    } else {
        weigh_at(va, 0);
    }
    // the wave's position groups (lanes lv, lv + LPV, ...) first, then the waves through LDS
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float v = o[j];
#pragma unroll
        for (int sft = LPV; sft < 64; sft <<= 1) v += __shfl_xor(v, sft);
        o[j] = v;
    }
    if (lane < LPV) *reinterpret_cast<float4v *>(&red[wave][lv * 4]) = o;
    __syncthreads();
    if (tid < HD / VS) {
        float v = 0.0f;
#pragma unroll
        for (int k = 0; k < WAVES; k++) v += red[k][tid];
        if (g.part_o) {
            const uint64_t at = ((uint64_t)b * gridDim.y + seg) * g.M + m;
            g.part_o[at * HD + part * (HD / VS) + tid] = v;
            if (tid == 0 && part == 0) {
                g.part_ml[at * 2] = row_max;
                g.part_ml[at * 2 + 1] = total;
            }
        } else {
            out[((uint64_t)b * g.M + m) * HD + part * (HD / VS) + tid] = asu(v / total);
        }
    }
}

// The same attention with a workgroup of 1024 threads per (batch entry, KV head) x SEGMENT of the cached positions,
// all of the group's query rows together: every byte of K and V crosses the path from L2 into a compute unit once
// (one workgroup per query row pulls K through it once per row and per half of head_dim: six times the traffic, and
// that path, 25 bytes a clock per unit, is what bounds a launch of this size).  With 256 / (batch entries x KV heads)
// segments a launch puts one workgroup on every compute unit, each with T / segments positions: 134 KB of K and V at
// the 1B shape's T = 2100, in flight at once (PASSES x 1024 / LPT positions per trip, K and V of a trip in 2 x PASSES
// sixteen-byte loads per lane).  A segment leaves its rows' maximum, sum and un-normalised weighted sum of V, as the
// chunked kernel does; decode_attention_combine_kernel — or the load of the product that reads the result, see
// AttnPartials — merges the segments.
// LOOP: several trips, the next always asked for before the current one is used; else one trip covers the segment and
// the soft-max program's other leaves are asked for before K.  MM: most query rows per KV head (4 or 8).
constexpr int kSegBlock = 1024;
constexpr int kSegMaxChunk = 2048; // most positions per workgroup: their scores wait in LDS, MM x 8 KiB
constexpr size_t seg_lds_bytes(int mm, int hd, uint32_t chunk) {
    return ((size_t)mm * ((chunk + 63) / 64 * 64) + (size_t)(kSegBlock / 64) * mm * hd) * sizeof(float);
}
template <class P, int LPT, int MM, int PASSES, bool LOOP>
__global__ __launch_bounds__(kSegBlock) void decode_attention_seg_kernel(const AttnArgs g, const FusedArgs a) {
    constexpr int HD = LPT * 4;
    constexpr int TPB = kSegBlock / LPT; // positions per pass
    constexpr int SPAN = TPB * PASSES;    // positions per trip to memory
    constexpr int WAVES = kSegBlock / 64;
    constexpr int IPL = LOOP ? 1 : (SPAN + 63) / 64; // positions per lane in the soft-max phase whose leaves wait in registers
    constexpr int ri0 = reduce_index<P>(0), ri1 = reduce_index<P>(1);
    constexpr int src0 = P::code[ri0][1], src1 = P::code[ri1][1];
    static_assert((P::code[ri0][0] & ~kInstrU32) == kRowMax && (P::code[ri1][0] & ~kInstrU32) == kRowSum,
                  "a soft-max: row maximum, then row sum");
    extern __shared__ float seg_lds[];
    const uint32_t cap = (g.chunk + 63) / 64 * 64;
    float *sc = seg_lds;              // [MM][cap]: scores, then un-normalised weights
    float *red = seg_lds + MM * cap;  // [WAVES][MM * HD]
    const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const uint32_t split = blockIdx.x, b = blockIdx.y;
    const uint32_t t0 = split * g.chunk, n = min(g.T, t0 + g.chunk) - t0; // (the host makes no empty segment)
    int64_t oq = 0, ok = 0, ov = 0, op = 0;
    {
        uint32_t bb = b;
        // (every axis slot is visited, so that the fields are read from the argument block at once instead of one
        // dependent scalar load after the other)
#pragma unroll
        for (uint32_t d = 0; d < (uint32_t)kMaxBatchAxes; d++) {
            if (d >= g.nb) break;
            const uint32_t q = fastdiv(bb, g.bdiv[d]);
            const int64_t i = (int64_t)(bb - q * g.bd[d]);
            bb = q;
            oq += i * g.q_bs[d];
            ok += i * g.k_bs[d];
            ov += i * g.v_bs[d];
            op += i * g.p_bs[d];
        }
    }
    const uint32_t l = tid % LPT, sub = tid / LPT;
    const uint32_t *kbase = g.Kc + ok + (int64_t)t0 * g.k_st + l * 4;
    const uint32_t *vbase = g.V + ov + (int64_t)t0 * g.v_st + l * 4;
    const int64_t k_step = (int64_t)TPB * g.k_st, v_step = (int64_t)TPB * g.v_st;
    // the trip that starts at `first`: FULL (a tag type) when it lies inside the segment, nothing is checked then
    auto ask = [&](float4v (&f)[PASSES], const uint32_t *base, int64_t st, int64_t step, uint32_t first, auto full) {
        const uint32_t *p = base + (int64_t)(first + sub) * st;
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            if constexpr (decltype(full)::value) {
                f[ps] = *reinterpret_cast<const float4v *>(p);
            } else {
                f[ps] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (first + sub + ps * TPB < n) f[ps] = *reinterpret_cast<const float4v *>(p);
            }
            p += step;
        }
    };
    constexpr std::true_type whole_trip{};
    constexpr std::false_type ragged{};
    auto ask_k = [&](float4v (&f)[PASSES], uint32_t first) {
        if (first + SPAN <= n) ask(f, kbase, g.k_st, k_step, first, whole_trip);
        else ask(f, kbase, g.k_st, k_step, first, ragged);
    };
    auto ask_v = [&](float4v (&f)[PASSES], uint32_t first) {
        if (first + SPAN <= n) ask(f, vbase, g.v_st, v_step, first, whole_trip);
        else ask(f, vbase, g.v_st, v_step, first, ragged);
    };
    float4v ka[PASSES], kb[LOOP ? PASSES : 1];
    float4v va[PASSES], vb[LOOP ? PASSES : 1];
    ask_k(ka, 0);
    if constexpr (!LOOP) ask_v(va, 0); // the whole segment is in flight from the start: the registers hold both
    float4v qf[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) {
        qf[m] = (float4v){0.f, 0.f, 0.f, 0.f};
        if ((uint32_t)m < g.M) qf[m] = *reinterpret_cast<const float4v *>(g.Q + oq + (int64_t)m * g.q_sm + l * 4);
    }
    // the soft-max phase gives a wave a query row (waves M.. have none); its lanes take positions lane, lane + 64, ...
    const uint32_t my_row = wave; // < g.M: this wave runs the program on row my_row
    int64_t base[P::nleaf + 1];
    LeafWords<P, 1> w[IPL];
    if (my_row < g.M) {
#pragma unroll
        for (int i = 0; i <= P::nleaf; i++) base[i] = 0;
        uint32_t rr = (uint32_t)(op / g.T) + my_row; // the row in the program's [rows, T] space
#pragma unroll
        for (uint32_t d = 0; d < (uint32_t)kMaxOuter; d++) {
            if (d >= a.g.nouter) break;
            const uint32_t q = fastdiv(rr, a.g.odiv[d]);
            const int64_t i = (int64_t)(rr - q * a.g.od[d]);
            rr = q;
#pragma unroll
            for (int lf = 1; lf < P::nleaf; lf++) base[lf] += i * a.leaf[lf].os[d];
        }
        if constexpr (!LOOP) { // nothing waits for them yet
#pragma unroll
            for (int c = 0; c < IPL; c++)
                if (lane + c * 64 < n) aot_fetch_from<P, 1>(a, base, t0 + lane + c * 64, w[c]);
        }
    }

    // ---- scores of the segment, all rows of the group
    auto score = [&](const float4v (&f)[PASSES], uint32_t first, auto full) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            const uint32_t t = first + sub + ps * TPB;
            if (decltype(full)::value || first + ps * TPB < n) { // the same for the whole workgroup
#pragma unroll
                for (int m = 0; m < MM; m++) {
                    if ((uint32_t)m < g.M) {
                        float v = fmaf(qf[m][3], f[ps][3], fmaf(qf[m][2], f[ps][2], fmaf(qf[m][1], f[ps][1], qf[m][0] * f[ps][0])));
                        v = row16_sum(v);
                        if (LPT == 32) v += __shfl_xor(v, 16);
                        if (l == 0 && (decltype(full)::value || t < n)) sc[m * cap + t] = v;
                    }
                }
            }
        }
    };
    auto score_at = [&](const float4v (&f)[PASSES], uint32_t first) {
        if (first + SPAN <= n) score(f, first, whole_trip);
        else score(f, first, ragged);
    };
    if constexpr (LOOP) {
        for (uint32_t first = 0; first < n; first += 2 * SPAN) {
            if (first + SPAN < n) ask_k(kb, first + SPAN);
            score_at(ka, first);
            if (first + 2 * SPAN < n) ask_k(ka, first + 2 * SPAN);
            if (first + SPAN < n) score_at(kb, first + SPAN);
        }
    } else {
        score_at(ka, 0);
    }
    if constexpr (LOOP) ask_v(va, 0); // on its way through the soft-max
    __syncthreads();

    // ---- the soft-max program on the segment: local maximum, local sum, un-normalised weights
    if (my_row < g.M) {
        const uint32_t m = my_row;
        uint32_t rs[kMaxRowReduce] = {0, 0, 0};
        uint32_t acc = row_init(true, true);
        if constexpr (!LOOP) {
#pragma unroll
            for (int c = 0; c < IPL; c++) {
                const uint32_t i = lane + c * 64;
                if (i < n) {
                    w[c].v[0][0] = asu(sc[m * cap + i]); // leaf 0 is the score
                    const Values<P, 1> s = aot_eval<P, 1, ri0>(w[c], rs, a.fault);
                    acc = row_merge(true, true, acc, s.v[src0][0]);
                }
            }
        } else {
            for (uint32_t i = lane; i < n; i += 64) {
                aot_fetch_from<P, 1>(a, base, t0 + i, w[0]);
                w[0].v[0][0] = asu(sc[m * cap + i]);
                const Values<P, 1> s = aot_eval<P, 1, ri0>(w[0], rs, a.fault);
                acc = row_merge(true, true, acc, s.v[src0][0]);
            }
        }
#pragma unroll
        for (int sft = 32; sft >= 1; sft >>= 1) acc = row_merge(true, true, acc, (uint32_t)__shfl_xor((int)acc, sft));
        rs[0] = acc;
        uint32_t sum = row_init(false, true);
        if constexpr (!LOOP) {
#pragma unroll
            for (int c = 0; c < IPL; c++) {
                const uint32_t i = lane + c * 64;
                if (i < n) {
                    const Values<P, 1> s = aot_eval<P, 1, ri1>(w[c], rs, a.fault);
                    sum = row_merge(false, true, sum, s.v[src1][0]);
                    sc[m * cap + i] = asf(s.v[src1][0]); // the un-normalised weight
                }
            }
        } else {
            for (uint32_t i = lane; i < n; i += 64) {
                aot_fetch_from<P, 1>(a, base, t0 + i, w[0]);
                w[0].v[0][0] = asu(sc[m * cap + i]);
                const Values<P, 1> s = aot_eval<P, 1, ri1>(w[0], rs, a.fault);
                sum = row_merge(false, true, sum, s.v[src1][0]);
                sc[m * cap + i] = asf(s.v[src1][0]);
            }
        }
#pragma unroll
        for (int sft = 32; sft >= 1; sft >>= 1) sum = row_merge(false, true, sum, (uint32_t)__shfl_xor((int)sum, sft));
        if (lane == 0) {
            float *ml = g.part_ml + (((uint64_t)b * g.splits + split) * g.M + m) * 2;
            ml[0] = asf(acc);
            ml[1] = asf(sum);
        }
    }
    __syncthreads();

    // ---- weights times V: the lane's pieces of V are those of its positions, piece l of head_dim
    float4v o[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) o[m] = (float4v){0.f, 0.f, 0.f, 0.f};
    auto weigh = [&](const float4v (&f)[PASSES], uint32_t first, auto full) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            const uint32_t t = first + sub + ps * TPB;
            if (decltype(full)::value || t < n) {
#pragma unroll
                for (int m = 0; m < MM; m++) {
                    if ((uint32_t)m < g.M) {
                        const float wgt = sc[m * cap + t];
                        o[m][0] = fmaf(wgt, f[ps][0], o[m][0]);
                        o[m][1] = fmaf(wgt, f[ps][1], o[m][1]);
                        o[m][2] = fmaf(wgt, f[ps][2], o[m][2]);
                        o[m][3] = fmaf(wgt, f[ps][3], o[m][3]);
                    }
                }
            }
        }
    };
    auto weigh_at = [&](const float4v (&f)[PASSES], uint32_t first) {
        if (first + SPAN <= n) weigh(f, first, whole_trip);
        else weigh(f, first, ragged);
    };
    if constexpr (LOOP) {
        for (uint32_t first = 0; first < n; first += 2 * SPAN) {
            if (first + SPAN < n) ask_v(vb, first + SPAN);
            weigh_at(va, first);
            if (first + 2 * SPAN < n) ask_v(va, first + 2 * SPAN);
            if (first + SPAN < n) weigh_at(vb, first + SPAN);
        }
    } else {
        weigh_at(va, 0);
    }
    // the wave's position groups (lanes l, l + LPT, ...) first, then the waves through LDS
#pragma unroll
    for (int m = 0; m < MM; m++) {
        if ((uint32_t)m < g.M) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = o[m][j];
#pragma unroll
                for (int sft = LPT; sft < 64; sft <<= 1) v += __shfl_xor(v, sft);
                o[m][j] = v;
            }
            if (lane < LPT) *reinterpret_cast<float4v *>(&red[(wave * MM + m) * HD + l * 4]) = o[m];
        }
    }
    __syncthreads();
    for (uint32_t e = tid; e < g.M * HD; e += kSegBlock) {
        const uint32_t m = e / HD, d = e % HD;
        float v = 0.0f;
#pragma unroll
        for (int k = 0; k < WAVES; k++) v += red[(k * MM + m) * HD + d];
        g.part_o[(((uint64_t)b * g.splits + split) * g.M + m) * HD + d] = v;
    }
}

// out[b][m][n] = sum_c e^(m_c - g) o_c[n] / sum_c e^(m_c - g) l_c.  A wave per (batch entry, query
// row): lane c first holds the statistics of chunk c (so each weight e^(m_c - g) is computed once
// and handed round by lane broadcast), then lane n sums output element n (and n + 64) over the chunks.
__global__ __launch_bounds__(kBlock) void decode_attention_combine_kernel(const float *part_o, const float *part_ml,
                                                                          uint32_t *out, uint32_t splits, uint32_t M,
                                                                          uint32_t hd, uint64_t rows) {
    const uint32_t lane = threadIdx.x % 64;
    const uint64_t r = (uint64_t)blockIdx.x * (kBlock / 64) + threadIdx.x / 64;
    if (r >= rows) return;
    const uint32_t m = (uint32_t)(r % M);
    const uint64_t b = r / M;
    const float *ml = part_ml + (b * splits * M + m) * 2; // chunk c at + c * M * 2
    const float *po = part_o + (b * splits * M + m) * (uint64_t)hd; // chunk c at + c * M * hd
    constexpr uint32_t kGroup = 32; // chunks per trip to memory
    const bool wide = lane + 64 < hd;
    float gmax = kF32Min;
    float num0 = 0.0f, num1 = 0.0f, den = 0.0f;
    for (uint32_t c0 = 0; c0 < splits; c0 += kGroup) {
        // every load of the group is asked for before anything is used
        float v0[kGroup], v1[kGroup];
#pragma unroll
        for (uint32_t k = 0; k < kGroup; k++) {
            v0[k] = 0.0f;
            v1[k] = 0.0f;
            if (c0 + k < splits) {
                const float *o = po + (uint64_t)(c0 + k) * M * hd;
                if (lane < hd) v0[k] = o[lane];
                if (wide) v1[k] = o[lane + 64];
            }
        }
        const uint32_t c = c0 + lane;
        const bool mine = lane < kGroup && c < splits;
        const float cm = mine ? ml[(uint64_t)c * M * 2] : kF32Min, cl = mine ? ml[(uint64_t)c * M * 2 + 1] : 0.0f;
        float m2 = fmaxf(gmax, cm);
#pragma unroll
        for (int sft = 16; sft >= 1; sft >>= 1) m2 = fmaxf(m2, __shfl_xor(m2, sft));
        m2 = __shfl(m2, 0);
        // what was summed so far is relative to the old maximum
        const float rescale = expf(gmax - m2);
        num0 *= rescale;
        num1 *= rescale;
        den *= rescale;
        gmax = m2;
        const float w = mine ? expf(cm - gmax) : 0.0f;
        den = fmaf(w, cl, den);
#pragma unroll
        for (uint32_t k = 0; k < kGroup; k++) {
            const float wk = __shfl(w, (int)k);
            num0 = fmaf(wk, v0[k], num0);
            num1 = fmaf(wk, v1[k], num1);
        }
    }
#pragma unroll
    for (int sft = 32; sft >= 1; sft >>= 1) den += __shfl_xor(den, sft);
    if (lane < hd) out[r * hd + lane] = asu(num0 / den);
    if (lane + 64 < hd) out[r * hd + lane + 64] = asu(num1 / den);
}

// ---- prefill: causal attention of many query rows in one pass ---------------------------------------------------
// The same three ops as above with thousands of query rows per KV head: unfused they write and re-read the
// [rows, T] score matrix four times (2 GiB per layer of the 1B-shape prefill).  Here a workgroup takes 128
// query rows of one KV head (a wave 32 of them) and walks the cached positions in tiles of 64, never going
// beyond the last position its rows may see.  Everything is computed TRANSPOSED, so that a query is a lane:
//     S^T[t][m] = K[t] . Q[m] / scale  first MFMA operand K (from LDS), second Q / scale (registers, loaded once)
//     running maximum / sum per query  = per lane: in-register over its 32 values + one exchange with lane ^ 32
//     O^T[d][m] += V^T[d][t] P^T[t][m] first operand V^T (columns of the LDS tile), second P^T — which, in the accumulator
//                                      layout of v_mfma_f32_32x32x2 (column = lane % 32, rows 8*(v/4) + 4*(lane/32)
//                                      + v%4), already is the operand layout: no trip through LDS, no transposition
// The scores are divided by the scale and masked exactly as the soft-max program does (x / d + f32(i < j) * m with
// i the query's position, j the key's); masked keys get weight zero, which is what exp(x - max) rounds to for them.
// out = O / l at the end (the program divides the weights first: same value up to rounding).
// MFMA-bound: 2 x 2 x 32 x 64 x 64 flop per wave and tile over ~half of the [rows, T] rectangle.
struct PrefillArgs {
    uint32_t *out;      // [batch][M][hd], dense
    uint32_t S;         // query positions per head: row m of a group is position m % S
    uint32_t pos0;      // position of the first query row (length of the cache before this chunk)
    uint32_t scale;     // f32 bits of the divisor of the scores
    uint32_t mask_mul;  // f32 bits of the multiplier of the 0/1 mask
    uint32_t batch;     // folded batch entries (KV heads)
    uint32_t tiles_per_head; // S / 128 when that is whole and heads are whole in M, else 0
    // Few workgroups (one sequence, a short prompt): the keys of a row tile are cut into `ksplit` parts over grid.y; a part
    // leaves its rows' running maximum, sum and un-normalised O for prefill_attention_combine_kernel.
    uint32_t ksplit;    // 1: none
    float *part_o;      // [ksplit][batch][M][hd]
    float *part_ml;     // [ksplit][batch][M][2]
};

constexpr int kPfRows = 128, kPfKeys = 64;
// K and V tiles, [64 keys][head_dim + 4] each (a row starts 4 banks after the one before), double buffered:
// 68 KiB for head_dim 64 (two workgroups per CU), 132 KiB for 128 (one)
constexpr size_t prefill_lds_bytes(int hd) { return 2 * 2 * (size_t)kPfKeys * (hd + 4) * sizeof(float); }

template <int HD>
__global__ __launch_bounds__(kBlock) void prefill_attention_kernel(const AttnArgs g, const PrefillArgs e) {
    static_assert(HD == 64 || HD == 128, "head_dim 64 or 128");
    constexpr int kPfPitch = HD + 4;
    typedef float float16v __attribute__((ext_vector_type(16)));
    extern __shared__ float pf_lds[]; // above the static limit
    float (*Ks)[kPfKeys][kPfPitch] = reinterpret_cast<float (*)[kPfKeys][kPfPitch]>(pf_lds);                       // [2][t][d]
    float (*Vs)[kPfKeys][kPfPitch] = reinterpret_cast<float (*)[kPfKeys][kPfPitch]>(pf_lds + 2 * kPfKeys * kPfPitch); // [2][t][d]
    const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64, li = lane % 32, lg = lane / 32;
    // Work per workgroup grows with the position of its rows inside their head (more visible keys), so the grid
    // is walked longest first over ALL batch entries and heads: the tail of the launch is made of short ones.
    const uint32_t ntile_rows = (g.M + kPfRows - 1) / kPfRows;
    uint32_t rt, b;
    if (e.tiles_per_head) {
        const uint32_t per_step = e.batch * (ntile_rows / e.tiles_per_head); // workgroups with the same row position
        const uint32_t step = blockIdx.x / per_step, rest = blockIdx.x % per_step;
        rt = (rest / e.batch) * e.tiles_per_head + (e.tiles_per_head - 1 - step);
        b = rest % e.batch;
    } else { // heads are not whole numbers of row tiles
        rt = ntile_rows - 1 - blockIdx.x / e.batch;
        b = blockIdx.x % e.batch;
    }
    int64_t oq = 0, ok = 0, ov = 0;
    {
        uint32_t bb = b;
        for (uint32_t d = 0; d < g.nb; d++) {
            const uint32_t q = fastdiv(bb, g.bdiv[d]);
            const int64_t i = (int64_t)(bb - q * g.bd[d]);
            bb = q;
            oq += i * g.q_bs[d];
            ok += i * g.k_bs[d];
        }
        bb = b;
        for (uint32_t d = 0; d < g.nbv; d++) {
            const uint32_t q = fastdiv(bb, g.vbdiv[d]);
            const int64_t i = (int64_t)(bb - q * g.vbd[d]);
            bb = q;
            ov += i * g.v_bs[d];
        }
    }
    const uint32_t m0 = rt * kPfRows;
    const uint32_t m = m0 + wave * 32 + li; // this lane's query row (both halves of the wave hold the same 32 queries)
    const bool live = m < g.M;
    const uint32_t iq = e.pos0 + (live ? m % e.S : 0); // position of the query: keys up to iq are visible
    // last key any row of the workgroup may see
    uint32_t kmax;
    {
        const uint32_t s0 = m0 % e.S, last = min(m0 + kPfRows, g.M) - 1 - m0; // rows m0 .. m0 + last
        const uint32_t smax = s0 + last < e.S ? s0 + last : e.S - 1;            // the tile may run into the next head
        kmax = min(g.T - 1, e.pos0 + smax);
    }
    const uint32_t ntiles_all = kmax / kPfKeys + 1;
    // this workgroup's share of the key tiles (all of them without a split)
    const uint32_t per_part = (ntiles_all + e.ksplit - 1) / e.ksplit;
    const uint32_t it_first = blockIdx.y * per_part, ntiles = min(ntiles_all, it_first + per_part);

    // the query rows, as second MFMA operands: chunk c covers d = 8c .. 8c+7, this lane holds 4*lg .. 4*lg+3 of them.
    // The program divides every score by the scale; dividing the query once instead is the same value up to
    // rounding and takes the division out of the loop.
    const float scale = asf(e.scale);
    float4v qf[HD / 8];
#pragma unroll
    for (int c = 0; c < HD / 8; c++) {
        qf[c] = (float4v){0.f, 0.f, 0.f, 0.f};
        if (live) qf[c] = *reinterpret_cast<const float4v *>(g.Q + oq + (int64_t)m * g.q_sm + c * 8 + lg * 4);
#pragma unroll
        for (int r = 0; r < 4; r++) qf[c][r] = qf[c][r] / scale;
    }
    float16v acc_o[HD / 32];
#pragma unroll
    for (int db = 0; db < HD / 32; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc_o[db][v] = 0.0f;
    float run_max = -INFINITY, run_sum = 0.0f;
    constexpr float kLog2e = 1.4426950408889634f;

    // K / V tile: 64 positions x HD floats each = 16 * HD float4 per operand, HD / 16 per thread
    constexpr int kSlots = kPfKeys * (HD / 4) / kBlock, kQpr = HD / 4;
    float4v kr[kSlots], vr[kSlots];
    auto load_kv = [&](uint32_t t0) {
#pragma unroll
        for (int h = 0; h < kSlots; h++) {
            const uint32_t slot = tid + h * kBlock, t = t0 + slot / kQpr, dq = slot % kQpr;
            kr[h] = (float4v){0.f, 0.f, 0.f, 0.f};
            vr[h] = (float4v){0.f, 0.f, 0.f, 0.f};
            if (t < g.T) {
                kr[h] = *reinterpret_cast<const float4v *>(g.Kc + ok + (int64_t)t * g.k_st + dq * 4);
                vr[h] = *reinterpret_cast<const float4v *>(g.V + ov + (int64_t)t * g.v_st + dq * 4);
            }
        }
    };
    auto store_kv = [&](uint32_t buf) {
#pragma unroll
        for (int h = 0; h < kSlots; h++) {
            const uint32_t slot = tid + h * kBlock, t = slot / kQpr, dq = slot % kQpr;
            *reinterpret_cast<float4v *>(&Ks[buf][t][dq * 4]) = kr[h];
            *reinterpret_cast<float4v *>(&Vs[buf][t][dq * 4]) = vr[h];
        }
    };
    if (it_first < ntiles) { // (a part beyond the last key tile of these rows has nothing to do but to say so)
        load_kv(it_first * kPfKeys);
        store_kv(it_first & 1);
    }
    __syncthreads();

    for (uint32_t it = it_first; it < ntiles; it++) {
        const uint32_t cur = it & 1, t0 = it * kPfKeys;
        const bool more = it + 1 < ntiles;
        if (more) load_kv(t0 + kPfKeys);
        // ---- S^T = K Q^T for the tile: two blocks of 32 keys x this wave's 32 queries
        float16v acc_s[kPfKeys / 32];
#pragma unroll
        for (int tb = 0; tb < kPfKeys / 32; tb++) {
#pragma unroll
            for (int v = 0; v < 16; v++) acc_s[tb][v] = 0.0f;
#pragma unroll
            for (int c = 0; c < HD / 8; c++) {
                const float4v kf = *reinterpret_cast<const float4v *>(&Ks[cur][tb * 32 + li][c * 8 + lg * 4]);
#pragma unroll
                for (int r = 0; r < 4; r++) acc_s[tb] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[r], qf[c][r], acc_s[tb], 0, 0, 0);
            }
        }
        // ---- mask, running soft-max statistics of this lane's query.  Weights are 2^((x - max) log2 e) on the
        // hardware's exp2 (relative error ~1e-6 for the arguments that matter: inside the 1e-4 of element-wise math).
        // A tile that every query of the wave sees whole (the common case below the diagonal) needs no per-key test.
        const bool whole = __all((int)(live && t0 + kPfKeys - 1 <= iq && t0 + kPfKeys <= g.T));
        float tile_max = -INFINITY;
        if (whole) {
#pragma unroll
            for (int tb = 0; tb < kPfKeys / 32; tb++)
#pragma unroll
                for (int v = 0; v < 16; v++) tile_max = fmaxf(tile_max, acc_s[tb][v]);
        } else {
#pragma unroll
            for (int tb = 0; tb < kPfKeys / 32; tb++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    // the program's x / d + f32(i < j) * m: nothing is added to a visible key, and an invisible one
                    // (m is hugely negative: the host checks) ends with weight exp(-huge) = 0, so it is left out
                    const uint32_t t = t0 + tb * 32 + 8 * (v / 4) + 4 * lg + (v % 4);
                    const bool seen = t <= iq && t < g.T && live;
                    acc_s[tb][v] = seen ? acc_s[tb][v] : -INFINITY;
                    tile_max = fmaxf(tile_max, acc_s[tb][v]);
                }
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
        const float new_max = fmaxf(run_max, tile_max);
        const float base = new_max == -INFINITY ? 0.0f : new_max; // a lane without a live query: keep NaN out
        const float alpha = __builtin_amdgcn_exp2f((run_max - base) * kLog2e);
        float tile_sum = 0.0f;
#pragma unroll
        for (int tb = 0; tb < kPfKeys / 32; tb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float p = __builtin_amdgcn_exp2f((acc_s[tb][v] - base) * kLog2e); // 2^-inf = 0 for a hidden key
                acc_s[tb][v] = p;
                tile_sum += p;
            }
        tile_sum += __shfl_xor(tile_sum, 32);
        run_sum = run_sum * alpha + tile_sum;
        run_max = new_max;
        // ---- O^T = alpha O^T + V^T P^T: the V operand is read column-wise from the [t][d] tile (32 lanes, 32 banks)
#pragma unroll
        for (int db = 0; db < HD / 32; db++) {
#pragma unroll
            for (int v = 0; v < 16; v++) acc_o[db][v] *= alpha;
#pragma unroll
            for (int tb = 0; tb < kPfKeys / 32; tb++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float vf = Vs[cur][tb * 32 + q * 8 + lg * 4 + r][db * 32 + li];
                        acc_o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf, acc_s[tb][q * 4 + r], acc_o[db], 0, 0, 0);
                    }
                }
        }
        if (more) store_kv(cur ^ 1);
        __syncthreads();
    }
    if (e.ksplit > 1) { // the part's statistics and un-normalised O; lane group 0 of a wave writes the statistics
        if (live) {
            const uint64_t row = ((uint64_t)blockIdx.y * e.batch + b) * g.M + m;
            float *orow = e.part_o + row * HD;
#pragma unroll
            for (int db = 0; db < HD / 32; db++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    float4v o;
#pragma unroll
                    for (int r = 0; r < 4; r++) o[r] = acc_o[db][j * 4 + r];
                    *reinterpret_cast<float4v *>(orow + db * 32 + j * 8 + lg * 4) = o;
                }
            if (lg == 0) {
                e.part_ml[row * 2] = run_max;
                e.part_ml[row * 2 + 1] = run_sum;
            }
        }
        return;
    }
    // ---- out[m][d] = O^T[d][m] / l[m]
    if (live) {
        uint32_t *orow = e.out + ((uint64_t)b * g.M + m) * HD;
#pragma unroll
        for (int db = 0; db < HD / 32; db++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4v o;
#pragma unroll
                for (int r = 0; r < 4; r++) o[r] = acc_o[db][j * 4 + r] / run_sum;
                *reinterpret_cast<float4v *>(orow + db * 32 + j * 8 + lg * 4) = o;
            }
    }
}

// out[row][d] = sum_p 2^((m_p - g) log2 e) O_p[row][d] / sum_p 2^((m_p - g) log2 e) l_p, g = max_p m_p: the parts of a
// prefill attention whose keys were cut over several workgroups, merged in the order of the parts.  A thread per four
// consecutive d of a row.  A part that saw no key of a row has m_p = -inf, l_p = 0 and O_p = 0: weight zero.
__global__ __launch_bounds__(kBlock) void prefill_attention_combine_kernel(const float *part_o, const float *part_ml, uint32_t *out,
                                                                           uint32_t parts, uint32_t hd, uint64_t rows) {
    const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x, q = hd / 4;
    if (i >= rows * q) return;
    const uint64_t row = i / q;
    const uint32_t d = (uint32_t)(i % q) * 4;
    constexpr float kLog2e = 1.4426950408889634f;
    float g = -INFINITY;
    for (uint32_t p = 0; p < parts; p++) g = fmaxf(g, part_ml[((uint64_t)p * rows + row) * 2]);
    float4v num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.0f;
    for (uint32_t p = 0; p < parts; p++) {
        const float *ml = part_ml + ((uint64_t)p * rows + row) * 2;
        const float w = __builtin_amdgcn_exp2f((ml[0] - g) * kLog2e);
        const float4v o = *reinterpret_cast<const float4v *>(part_o + ((uint64_t)p * rows + row) * hd + d);
        den = fmaf(w, ml[1], den);
        num[0] = fmaf(w, o[0], num[0]);
        num[1] = fmaf(w, o[1], num[1]);
        num[2] = fmaf(w, o[2], num[2]);
        num[3] = fmaf(w, o[3], num[3]);
    }
    float4v r;
#pragma unroll
    for (int k = 0; k < 4; k++) r[k] = num[k] / den;
    *reinterpret_cast<float4v *>(out + row * hd + d) = r;
}
