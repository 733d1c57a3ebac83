// The interpreter's row kernels at 8 elements per vector (see rows_kernels.hpp); launched from rows.hip.
#include "rows_kernels.hpp"

namespace axhip {
template int launch_plan_e<8>(const AxhipRowsProgram &, const RowsPlan &, hipStream_t);
} // namespace axhip
