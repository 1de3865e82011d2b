// Register-resident fp32 product kernel: instantiations for odd feature counts (half norm of the
// output rows folded into the padding feature).  Compiled once per kernel function (-DFLK_KF=0..4).
#ifndef FLK_KF
#define FLK_KF 0
#endif
#define FLK_FOLD true
#define FLK_PASTE2(a, b) a##b
#define FLK_PASTE(a, b) FLK_PASTE2(a, b)
#define FLK_LAUNCH_NAME FLK_PASTE(launch_mmv_small_f32_fold_kf, FLK_KF)
#include "mmv_small_f32_dispatch.inc"
