"""Mask generator, masked-dense reference functions, profile / check helpers.
Same exports as the reference's sparta.testing (sparta/testing/__init__.py:4-6)."""
from sparta_amd.testing.mask import block_mask
from sparta_amd.testing.utils import check, profile
from sparta_amd.testing.math import (
    sparse_softmax_forward_reference,
    sparse_softmax_backward_reference,
    sparse_multi_head_attention_reference,
)
