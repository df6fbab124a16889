"""Tensor-with-sparsity-attribute indexes (BCSR / BCSC), as exported by the
reference's sparta.tesa (sparta/tesa/__init__.py:4-5)."""
from sparta_amd.tesa.tesa_base import TeSAIndexes, TeSAFunctionContext
from sparta_amd.tesa.block_compressed import (
    get_bcs_function, build_indexes_batch, BCSIndexes, BCSRIndexes, BCSCIndexes, BCSRCIndexes, BCSFunctionContext,
)
