// f32 instantiations of the panel sparse-operand matmul kernels (one workgroup per tile, and persistent).
#include "matmul_spmm_stream.hpp"
namespace spx {
template <>
int launch_spmm_panel<float>(const SpmmParams& p, int BN, int batch, int nst, hipStream_t st) {
    if (!spmm_panel_supported<float>(BN, p.BK)) return fail(SPX_E_CONFIG, "block (%d,%d) not supported by the panel kernel", p.BK, BN);
    if (nst == 3) return launch_spmm_panel_impl<float, 3, false>(p, BN, batch, st);
    if (nst == 12) {  // shared S tile; the dense operand may be stored with m contiguous
        if (!p.d_kcontig) return launch_spmm_panel_impl<float, 2, true, true>(p, BN, batch, st);
        return launch_spmm_panel_impl<float, 2, true>(p, BN, batch, st);
    }
    return launch_spmm_panel_impl<float, 2, false>(p, BN, batch, st);
}
template <>
int launch_spmm_stream<float>(const SpmmParams& p, int BN, int batch, hipStream_t st) {
    if (!spmm_stream_supported<float>(p, BN)) return fail(SPX_E_CONFIG, "the persistent panel kernel needs a k-contiguous dense operand and 64-byte block rows");
    return launch_spmm_stream_impl<float>(p, BN, batch, st);
}
}  // namespace spx
