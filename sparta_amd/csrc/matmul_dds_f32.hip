// f32 instantiations of the sparse-output matmul kernel.
#include "matmul_dds.hpp"
namespace spx {
template <>
int launch_dds<float>(const DdsParams& p, int BM, int BN, int nnz_bound, int batch, int tile_cfg, hipStream_t st) {
    return launch_dds_impl<float>(p, BM, BN, nnz_bound, batch, tile_cfg, st);
}
}  // namespace spx
