from sparta_amd.specializer.operators import (
    OperatorBase, SparseLinear, SparseBatchMatMul, SparseSoftmax, SparseAttention, DynamicSparseMoE,
    SeqlenDynamicSparseAttention,
)
