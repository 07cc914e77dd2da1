// Element-wise kernels at 4 elements per work item.
#include "ew_kernel.hpp"

namespace cg {
template int launch_ew_binary<4>(cg_backend *, int, cg_dtype, const EwArgs &);
template int launch_ew_other<4>(cg_backend *, int, cg_dtype, const EwArgs &);
} // namespace cg
