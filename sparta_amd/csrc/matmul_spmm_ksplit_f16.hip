// f16 instantiations of the K-split sparse-operand matmul kernel.
#include "matmul_spmm_ksplit.hpp"
namespace spx {
template <>
int launch_spmm_ksplit<_Float16>(const SpmmParams& p, int BN, int batch, hipStream_t st) {
    if (!spmm_ksplit_supported<_Float16>(BN, p.BK)) return fail(SPX_E_CONFIG, "block (%d,%d) not supported by the K-split kernel", p.BK, BN);
    return launch_spmm_ksplit_impl<_Float16>(p, BN, batch, st);
}
}  // namespace spx
