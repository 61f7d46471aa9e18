"""MI355X (gfx950) back-end for MatConvNet's convolution / batch-normalisation / pooling operators.

The product is native: HIP kernels behind a C ABI (``include/mcn_hip.h`` -> ``libmcn_hip.so``) and a C++
operator layer with the reference's ``vl::nn`` interface (``bits/`` -> ``libmcn_vl.so``).  This Python
package only builds those libraries (``matconvnet_amd.build``) and binds them with ctypes for tests and
benchmarks (``matconvnet_amd.capi``); PyTorch is used for device memory and streams, nothing else.
"""
