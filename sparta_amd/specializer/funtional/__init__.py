"""Function contexts and autograd functions.  The package keeps the reference's
spelling ("funtional", sparta/specializer/funtional/) so import paths carry over."""
from sparta_amd.specializer.funtional.sparse_ctx_base import KernelPlaceholder, SparseCtxBase
from sparta_amd.specializer.funtional.batch_matmul import SparseBatchMatMulCtx, SparseBatchMatMulFunc
from sparta_amd.specializer.funtional.batch_softmax import SparseBatchSoftmaxCtx, SparseBatchSoftmaxFunc
