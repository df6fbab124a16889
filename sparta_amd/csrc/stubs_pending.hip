// Entry points whose kernels are not built yet report so instead of computing.
#include "common.hpp"
extern "C" int spx_attention_forward(int, const void*, const void*, const void*, void*, const int32_t*,
                                     const int32_t*, const uint8_t*, float, int, int, int, int, int, int,
                                     int, spx_stream_t) {
    return spx::fail(SPX_E_NO_DEVICE, "spx_attention_forward is not built in this library");
}
extern "C" int spx_num_tile_cfgs(int) { return 0; }
extern "C" int spx_tile_cfg_info(int, int, spx_tile_cfg*) { return spx::fail(SPX_E_CONFIG, "no tile configs"); }
