// The interpreter's row kernels at four elements per work item.
#include "interp.hpp"

namespace cg {

void launch_interpreted_rows4(const FusedArgs &a, uint32_t *rowout, int tpr, bool full, dim3 grid, hipStream_t s) {
    launch_interpreted_rows<4>(a, rowout, tpr, full, grid, s);
}

} // namespace cg
