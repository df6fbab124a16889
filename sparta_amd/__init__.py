"""sparta_amd: block-sparse operators for AMD Instinct MI355X (gfx950).

Same user-facing API as microsoft/SparTA's block-sparse operator path
(`nn.SparseLinear / SparseBatchMatMul / SparseSoftmax / SparseAttention /
DynamicSparseMoE`, `nn.tune`, `nn.build`, `testing.*`, `tesa.*`), backed by
hand-written HIP kernels in libsparta_hip.so (C ABI in include/sparta_hip.h).
Use `import sparta_amd as sparta` to switch an existing script over.
"""
from sparta_amd import _lib

__env_ready__ = True
__version__ = '0.1.0'

from sparta_amd import nn, testing, tesa  # noqa: E402
