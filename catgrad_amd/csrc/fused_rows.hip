// Launcher of programs with reductions over the last axis inside them (soft-max, the norms): one
// team of lanes per row, through the kernels compiled for known programs or the interpreter.
#include "interp.hpp"

namespace cg {

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
    dim3 grid((a.rows + rpb - 1) / rpb);
    if (be->aot && tpr >= 16 && launch_compiled_rows(p, a, rowout, tpr, grid, be->stream)) {
        be->programs_compiled++;
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? CG_OK : hip_fail(e, "compiled row-program launch");
    }
    be->programs_interpreted++;
    if (a.g.vec == 4) launch_interpreted_rows4(a, rowout, tpr, full, grid, be->stream);
    else launch_interpreted_rows1(a, rowout, tpr, full, grid, be->stream);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "fused row-program launch");
}

} // namespace cg
