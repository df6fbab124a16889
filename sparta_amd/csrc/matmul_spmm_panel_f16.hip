// f16 instantiations of the panel sparse-operand matmul kernel.
#include "matmul_spmm_panel.hpp"
namespace spx {
template <>
int launch_spmm_panel<_Float16>(const SpmmParams& p, int BN, int batch, int nst, hipStream_t st) {
    if (!spmm_panel_supported<_Float16>(BN, p.BK)) return fail(SPX_E_CONFIG, "block (%d,%d) not supported by the panel kernel", p.BK, BN);
    if (nst == 3) return launch_spmm_panel_impl<_Float16, 3>(p, BN, batch, st);
    return launch_spmm_panel_impl<_Float16, 2>(p, BN, batch, st);
}
}  // namespace spx
