from sparta_amd.specializer.kernels.kernel_base import KernelBase, PortConfig
from sparta_amd.specializer.kernels.matmul import (
    SparseMatMulKernel, SparTASparseMatMulKernel, OpenAISparseMatMulKernel,
)
from sparta_amd.specializer.kernels.softmax import (
    SparseSoftmaxForwardKernel, SparTASparseSoftmaxForwardKernel,
    SparseSoftmaxBackwardKernel, SparTASparseSoftmaxBackwardKernel,
)
