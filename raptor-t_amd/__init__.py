"""MI355X-native block-sparse (BigBird-pattern) encoder layer.

`capi` binds the C-ABI library (HIP kernels, host metadata, pipeline, GEMM);
`raptor_t` (built from `layers/`) is the pybind module with the reference's class
surface; `modeling_bert` / `util` are the Python callers on top of it.  There is no CPU
implementation of the GPU path: every op raises if the library is missing.
"""
from . import capi  # noqa: F401
