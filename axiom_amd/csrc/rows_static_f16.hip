// Specialised fused-row kernels, f16 element type.
#define AXHIP_STATIC_DT AXHIP_DTYPE_F16
#define AXHIP_STATIC_LAUNCH rows_static_launch_f16
#include "rows_static.inc"
