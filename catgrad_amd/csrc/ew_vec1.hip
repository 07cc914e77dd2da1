// Element-wise kernels at 1 element per work item.
#include "ew_kernel.hpp"

namespace cg {
template int launch_ew_binary<1>(cg_backend *, int, cg_dtype, const EwArgs &);
template int launch_ew_other<1>(cg_backend *, int, cg_dtype, const EwArgs &);
} // namespace cg
