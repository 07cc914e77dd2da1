// Element-wise kernels at 8 elements per work item: the operations of two operands.
#include "ew_kernel.hpp"

namespace cg {
template int launch_ew_binary<8>(cg_backend *, int, cg_dtype, const EwArgs &);
} // namespace cg
