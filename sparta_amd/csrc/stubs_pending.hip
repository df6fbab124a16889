// Entry points whose kernels are not built yet report so instead of computing.
#include "common.hpp"
extern "C" int spx_num_tile_cfgs(int) { return 0; }
extern "C" int spx_tile_cfg_info(int, int, spx_tile_cfg*) { return spx::fail(SPX_E_CONFIG, "no tile configs"); }
