// MX-quantised output (matmul_details/_matmul.py:593-637) of the bf16-activation prefill kernel: the epilogue quantises the fp32
// accumulator.  Instantiated apart from the bf16-output variants to keep the build's longest compile short.
#include "moe_gemm_mxn_kernel.h"

namespace tk {

int32_t gemm_launch_mxn_mx(const GemmParams& p, int block_m, int grid_m, bool swiglu, hipStream_t st) {
  //                                   BLKM MFW NFW G WD XD
  if (block_m == 256) return launch_mxn<256, 5, 2, 1, 2, 1, true>(p, grid_m, swiglu, st);
  return launch_mxn<128, 4, 2, 1, 4, 2, true>(p, grid_m, swiglu, st);
}

}  // namespace tk
