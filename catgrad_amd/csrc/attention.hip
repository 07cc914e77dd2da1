// Launchers of the attention kernels (attention.hpp): decode-time attention over a KV cache in one
// pass, in segments or in chunks with a combine, and prefill attention on the matrix cores.
#include "interp.hpp"

namespace cg {

namespace {

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
    using P = WordsOnly<RowsSoftmaxCausal>; // (the scores of an open product are f32, and so is all that meets them)
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
    if (!all_words(a)) return kDeclined;
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
    // So a single sequence takes the segments from 128 Ki cached values per KV head on (1024 positions of head_dim 128, 2048
    // of 64): the Qwen3-0.6B shape's decode step (8 KV heads, head_dim 128, 16 query rows, 1024 to 1152 positions) takes 1.45
    // to 1.53 ms with them against 1.64 to 1.66 ms with its 32 workgroups of the kernel below.
    // (Merging the segments inside the kernel — the workgroup that counts itself last at a device-scope counter reads the
    // others' results — was measured and costs what the combine launch costs: the stores must reach memory, the count must come
    // back and the loads go out again, 6 to 7 us in all; with a release / acquire fence per workgroup 24.0 against 19.3 us.)
    if (be->attn_seg_from > 0 && (T >= be->attn_seg_from || (qrows > 256 && T >= 1024) || (f1.batch <= 8 && T * hd >= 131072))) {
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

} // namespace cg
