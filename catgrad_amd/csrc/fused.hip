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
#include "interp.hpp"

namespace cg {

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

} // namespace cg
