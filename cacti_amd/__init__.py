"""cacti_amd: MI355X-native kernels and host runtime for cacti's LLaMA backward pass.

The product is the C-ABI library `libcacti_gpu_hip_ffi.so` (see include/cacti_gpu_hip_ffi.h);
this package loads it (`cacti_amd.ffi`) and mirrors the reference's thunk interface on top.
"""
