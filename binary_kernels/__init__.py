"""Drop-in for the reference's `binary_kernels` extension module.

The reference builds a torch extension of this name whose import registers
`torch.ops.binary_kernels.*` (src/nanoquant/kernel/pybind.cpp:83-131) and its callers do
`import binary_kernels` before touching the ops (src/nanoquant/kernel/utils.py:33-38,
src/nanoquant/modules/linear.py:201).  Importing this package does the same with the gfx950
implementation.
"""
import nanoquant_amd.ops  # noqa: F401
