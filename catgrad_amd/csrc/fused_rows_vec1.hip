// The interpreter's row kernels at one element per work item.
#include "interp.hpp"

namespace cg {

void launch_interpreted_rows1(const FusedArgs &a, uint32_t *rowout, int tpr, bool full, dim3 grid, hipStream_t s) {
    launch_interpreted_rows<1>(a, rowout, tpr, full, grid, s);
}

} // namespace cg
