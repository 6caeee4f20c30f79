#include "moe_gemm_mxn_kernel.h"

namespace tk {

int32_t gemm_launch_mxn(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  //                                  BLKM MFW NFW G WD XD
  if (block_m == 64) return launch_mxn<64, 2, 2, 1, 4, 2, false>(p, grid_m, swiglu, st);
  if (block_m == 256) return launch_mxn<256, 5, 2, 1, 2, 1, false>(p, grid_m, swiglu, st);
  return launch_mxn<128, 4, 2, 1, 4, 2, false>(p, grid_m, swiglu, st);
}

}  // namespace tk
