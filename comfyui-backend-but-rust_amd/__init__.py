"""MI355X-native quantized-linear path (W8A8 / W6A8) behind the reference's C ABI.

Submodules: `ffi` (ctypes view of libgpu_kernels.so), `qlinear` (the host-side call pattern on torch device memory),
`synth` (counter-hashed synthetic workloads), `build` (hipcc driver).
"""
