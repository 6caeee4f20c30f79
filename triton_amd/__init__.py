"""MI355X (gfx950) implementation of the quantized mixture-of-experts hot path of `triton_kernels`.

The modules mirror the reference's module paths (`topk`, `matmul`, `swiglu`, `reduce`, `tensor`,
`numerics_details.mxfp`, ...); the top-level `triton_kernels` package aliases them so that
`from triton_kernels.matmul import matmul` resolves here.  All device work goes through the C ABI of
`include/triton_amd.h` (`libtriton_amd.so`, hand-written HIP); there is no CPU or PyTorch fallback.
"""
__version__ = "0.1.0"
