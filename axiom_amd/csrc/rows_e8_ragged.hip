// The interpreter's resident row kernels at 8 elements per vector for rows that are not whole, aligned vectors
// (see rows_kernels.hpp); launched through launch_plan_e<8>.
#include "rows_kernels.hpp"

namespace axhip {
template int launch_resident_plan<8, true>(const AxhipRowsProgram &, int, int, hipStream_t);
} // namespace axhip
