"""User-facing namespace: the sparse operators plus tune() / build()
(same exports as the reference's sparta.nn, sparta/nn/__init__.py:4-5)."""
from sparta_amd.specializer import (
    OperatorBase, SparseLinear, SparseBatchMatMul, SparseSoftmax, SparseAttention, DynamicSparseMoE,
    SeqlenDynamicSparseAttention,
)
from sparta_amd.specializer.operators.operator_base import update_masks
from sparta_amd.nn.module_tuner import tune_combined_module as tune, build_combined_module as build
