// The row-program kernels compiled ahead of time for the programs of a decoder block (the norms, the
// causal soft-max): the phases of the interpreter's row kernel unrolled at compile time.
#include "interp.hpp"

namespace cg {

bool launch_compiled_rows(const Pending &p, const FusedArgs &a, uint32_t *rowout, int tpr, dim3 grid, hipStream_t s) {
    return aot_rows_dispatch(p, a, rowout, tpr, grid, s, RowsPrograms{});
}

} // namespace cg
