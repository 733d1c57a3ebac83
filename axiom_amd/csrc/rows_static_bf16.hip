// Specialised fused-row kernels, bf16 element type.
#define AXHIP_STATIC_DT AXHIP_DTYPE_BF16
#define AXHIP_STATIC_LAUNCH rows_static_launch_bf16
#include "rows_static.inc"
