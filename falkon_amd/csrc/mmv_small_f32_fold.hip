// Register-resident fp32 product kernel: instantiations for odd feature counts (half norm of the
// output rows folded into the padding feature).
#define FLK_FOLD true
#define FLK_LAUNCH_NAME launch_mmv_small_f32_fold
#include "mmv_small_f32_dispatch.inc"
