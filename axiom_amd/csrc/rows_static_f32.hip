// Specialised fused-row kernels, f32 element type.
#define AXHIP_STATIC_DT AXHIP_DTYPE_F32
#define AXHIP_STATIC_LAUNCH rows_static_launch_f32
#include "rows_static.inc"
