// f16 instantiations of the register-direct sparse-operand matmul kernel.
#include "matmul_spmm_direct.hpp"
namespace spx {
template <>
int launch_spmm_direct<_Float16>(const SpmmParams& p, int BN, int batch, int wm, hipStream_t st) {
    return launch_spmm_direct_impl<_Float16>(p, BN, batch, wm, st);
}
}  // namespace spx
