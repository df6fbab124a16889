// Instantiations of the thin-dense-operand sparse matmul kernel (16-bit types).
#include "matmul_spmm_thin.hpp"
namespace spx {
template <> bool spmm_thin_supported<_Float16>(const SpmmParams& p, int BN) { return spmm_thin_ok<_Float16>(p, BN); }
template <> bool spmm_thin_supported<bf16_t>(const SpmmParams& p, int BN) { return spmm_thin_ok<bf16_t>(p, BN); }
template <> bool spmm_thin_supported<float>(const SpmmParams&, int) { return false; }
template <> int launch_spmm_thin<_Float16>(const SpmmParams& p, int batch, hipStream_t st) { return launch_spmm_thin_impl<_Float16>(p, batch, st); }
template <> int launch_spmm_thin<bf16_t>(const SpmmParams& p, int batch, hipStream_t st) { return launch_spmm_thin_impl<bf16_t>(p, batch, st); }
template <> int launch_spmm_thin<float>(const SpmmParams& p, int batch, hipStream_t st) { return launch_spmm_thin_impl<float>(p, batch, st); }
}  // namespace spx
