// Table of the pre-instantiated tile configurations that tune() may enumerate.
// It takes the place of the reference's Jinja template parameters and of its
// thread-tile look-up table (sparta/specializer/kernels/look_up_tables/
// sparta_matmul_lut.csv): nothing is generated at run time, a configuration id
// selects one of the kernels compiled into this library.
#include "common.hpp"
#include <string.h>

namespace spx {

static const spx_tile_cfg kSpmmCfgs[] = {
    // id, tile_m, tile_n, waves, lds_stages, min_block, dtype_mask, name
    {0, 0, 0, 4, 0, 16, 7, "auto"},
    {1, 64, 0, 4, 1, 16, 7, "lds-64"},
    {2, 128, 0, 4, 1, 16, 7, "lds-128"},
    {3, 64, 0, 4, 2, 16, 7, "direct-64"},
    {4, 256, 0, 4, 2, 16, 7, "direct-256"},
    {5, 256, 0, 4, 2, 16, 7, "panel-256x2"},
    {6, 256, 0, 4, 3, 16, 7, "panel-256x3"},
    {7, 256, 0, 4, 2, 16, 7, "panel-256-sharedS"},
    {8, 64, 0, 4, 2, 16, 7, "panel-64-ksplit"},
    {9, 64, 0, 4, 2, 64, 6, "thin-dense-operand"},
    {10, 256, 0, 4, 2, 16, 7, "panel-256-persistent"},
};
static const spx_tile_cfg kDdsCfgs[] = {
    {0, 0, 0, 4, 1, 16, 7, "auto"},
    {1, 0, 0, 4, 1, 16, 7, "block-per-workgroup"},
    {2, 0, 0, 4, 3, 16, 7, "block-per-workgroup-pipelined"},
    {3, 0, 0, 4, 2, 32, 7, "block-row-per-workgroup-short-k"},
    {4, 0, 0, 4, 2, 32, 6, "wave-per-16-rows-short-k"},
};
static const spx_tile_cfg kSoftmaxCfgs[] = {
    {0, 4, 0, 4, 0, 4, 7, "auto"},
    {1, 4, 0, 4, 0, 4, 7, "wave-per-row"},
    {2, 4, 0, 4, 0, 8, 7, "wave-per-row-16-byte"},
    {3, 16, 0, 4, 0, 8, 7, "16-lanes-per-row-16-byte"},
};
static const spx_tile_cfg kAttentionCfgs[] = {
    {0, 0, 0, 0, 1, 16, 6, "auto"},
    {1, 0, 0, 0, 1, 16, 6, "fused-online-softmax"},
    {2, 0, 0, 0, 2, 32, 6, "fused-pipelined"},
    {3, 0, 0, 0, 2, 32, 6, "fused-pipelined-32x32-mfma"},
};
static const spx_tile_cfg kMoeCfgs[] = {
    {0, 0, 0, 4, 0, 0, 7, "auto"},
    {1, 128, 128, 4, 1, 0, 7, "gather-128x128"},
    {2, 128, 128, 4, 2, 0, 7, "gather-128x128-lds-direct"},
    {3, 256, 256, 8, 2, 0, 7, "gather-256x256-lds-direct"},
    {4, 256, 256, 16, 2, 0, 7, "gather-256x256-direct-16-waves"},
    {5, 256, 256, 16, 2, 0, 7, "gather-256x256-plus-128-tail"},
    {6, 256, 256, 16, 4, 0, 6, "gather-256x256-cross-stage"},
};

static const spx_tile_cfg* table(int op, int* n) {
    switch (op) {
        case 0: *n = sizeof(kSpmmCfgs) / sizeof(spx_tile_cfg); return kSpmmCfgs;
        case 1: *n = sizeof(kDdsCfgs) / sizeof(spx_tile_cfg); return kDdsCfgs;
        case 2: *n = sizeof(kSoftmaxCfgs) / sizeof(spx_tile_cfg); return kSoftmaxCfgs;
        case 3: *n = sizeof(kAttentionCfgs) / sizeof(spx_tile_cfg); return kAttentionCfgs;
        case 4: *n = sizeof(kMoeCfgs) / sizeof(spx_tile_cfg); return kMoeCfgs;
        default: *n = 0; return nullptr;
    }
}

}  // namespace spx

extern "C" int spx_num_tile_cfgs(int op) {
    int n = 0;
    spx::table(op, &n);
    return n;
}

extern "C" int spx_tile_cfg_info(int op, int id, spx_tile_cfg* out) {
    using namespace spx;
    SPX_REQUIRE(out, SPX_E_NULL, "out is NULL");
    int n = 0;
    const spx_tile_cfg* t = table(op, &n);
    SPX_REQUIRE(t, SPX_E_CONFIG, "unknown op %d", op);
    SPX_REQUIRE(id >= 0 && id < n, SPX_E_CONFIG, "tile config %d out of range [0,%d) for op %d", id, n, op);
    memcpy(out, &t[id], sizeof(spx_tile_cfg));
    return 0;
}
