// f32 instantiations of the sparse-operand matmul kernel.
#include "matmul_spmm.hpp"
namespace spx {
template <>
int launch_spmm<float>(const SpmmParams& p, int BN, int batch, int tile_cfg, hipStream_t st) {
    return launch_spmm_impl<float>(p, BN, batch, tile_cfg, st);
}
}  // namespace spx
