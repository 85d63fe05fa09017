"""pie_amd — MI355X (gfx950) kernels and host driver for the Pie forward pass.

The compute lives in `libpie_hip_kernels.so` (hand-written HIP, C ABI declared in
`include/pie_hip_kernels.h`).  `pie_amd.ops` is the Python mirror of the
reference's launcher interface over torch-ROCm device buffers; torch is used for
device memory and streams only.
"""
__version__ = "0.1.0"
