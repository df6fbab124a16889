// BCSR / BCSC index build for a uint8 element mask.
//
// Two launches, no host round trip, no atomics, canonical (sorted) order:
//   1. liveness_kernel: streams the mask once with 16-byte loads and writes one
//      byte per block ("any byte of the tile non-zero").  HBM-bound: H*W bytes in.
//   2. emit_kernel (one workgroup): turns the byte map into 64-block words with
//      wavefront ballots, prefix-scans the word popcounts (which directly yields
//      row_ptr / col_ptr and every block's rank), and writes the index arrays.
// Replaces bcs_index_1 / bcs_index_2 of the reference
// (sparta/tesa/templates/block_compressed.cu.j2:67-170) and the cumsum + .item()
// glue of sparta/tesa/block_compressed.py:242-309.
#include "common.hpp"

namespace spx {

struct LiveParams {
    const uint8_t* mask;
    uint8_t* live;
    int H, W, BH, BW, Cn;
    int segw;      // bytes of a mask row covered by one workgroup (power of two)
    int log_tcols; // log2(segw / VEC)
    int log_bw;
};

template <int VEC>
__global__ __launch_bounds__(256) void liveness_kernel(LiveParams p) {
    __shared__ uint32_t flags[256];
    const int tid = threadIdx.x;
    flags[tid] = 0;
    __syncthreads();

    const int tcols = 1 << p.log_tcols;
    const int trows = 256 >> p.log_tcols;
    const int tx = tid & (tcols - 1);
    const int ty = tid >> p.log_tcols;
    const int seg = blockIdx.x;
    const int r = blockIdx.y;
    const int64_t col_byte = (int64_t)seg * p.segw + (int64_t)tx * VEC;

    if (col_byte < p.W) {
        const uint8_t* src = p.mask + ((int64_t)r * p.BH) * p.W + col_byte;
        if constexpr (VEC == 16) {
            uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
            for (int row = ty; row < p.BH; row += trows) {
                const vec16 v = *reinterpret_cast<const vec16*>(src + (int64_t)row * p.W);
                a0 |= v.x; a1 |= v.y; a2 |= v.z; a3 |= v.w;
            }
            if (p.BW >= 16) {
                if (a0 | a1 | a2 | a3) flags[(tx * 16) >> p.log_bw] = 1;
            } else if (p.BW == 8) {
                if (a0 | a1) flags[tx * 2] = 1;
                if (a2 | a3) flags[tx * 2 + 1] = 1;
            } else {  // BW == 4
                if (a0) flags[tx * 4] = 1;
                if (a1) flags[tx * 4 + 1] = 1;
                if (a2) flags[tx * 4 + 2] = 1;
                if (a3) flags[tx * 4 + 3] = 1;
            }
        } else if constexpr (VEC == 4) {
            uint32_t a = 0;
            for (int row = ty; row < p.BH; row += trows)
                a |= *reinterpret_cast<const uint32_t*>(src + (int64_t)row * p.W);
            if (a) flags[(tx * 4) >> p.log_bw] = 1;
        } else {
            uint32_t a = 0;
            for (int row = ty; row < p.BH; row += trows) a |= src[(int64_t)row * p.W];
            if (a) flags[tx >> p.log_bw] = 1;
        }
    }
    __syncthreads();
    const int blk_per_seg = p.segw >> p.log_bw;
    if (tid < blk_per_seg) {
        const int c = seg * blk_per_seg + tid;
        if (c < p.Cn) p.live[(int64_t)r * p.Cn + c] = (uint8_t)flags[tid];
    }
}

struct EmitParams {
    const uint8_t* live;
    unsigned long long* wbits;  // [R * WPR] row words
    int* wbase;                 // [R * WPR] exclusive prefix of row-word popcounts
    int* cbase;                 // [Cn * WPC] exclusive prefix of column-word popcounts
    int32_t* row_ptr;
    int32_t* bcsr_idx;
    int32_t* col_ptr;
    void* bcsc_idx;
    int bcsc_i64;
    int32_t* nnz_dev;
    int cap;
    int R, Cn, WPR, WPC;
};

// Exclusive prefix sum of a[0..n) in place by one workgroup; returns the total.
__device__ int block_scan_inplace(int* a, int n, int* lds) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    int carry = 0;
    for (int base = 0; base < n; base += blockDim.x) {
        const int i = base + threadIdx.x;
        const int v = i < n ? a[i] : 0;
        const int inc = wave_inclusive_scan(v);
        if (lane == 63) lds[wave] = inc;
        __syncthreads();
        int before = 0, total = 0;
        for (int w = 0; w < nwaves; ++w) {
            const int t = lds[w];
            if (w < wave) before += t;
            total += t;
        }
        if (i < n) a[i] = carry + before + inc - v;
        carry += total;
        __syncthreads();
    }
    return carry;
}

__global__ __launch_bounds__(1024) void emit_kernel(EmitParams p) {
    __shared__ int lds[32];
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

    // ---- row words -----------------------------------------------------------
    const int NW = p.R * p.WPR;
    for (int g = wave; g < NW; g += nwaves) {
        const int r = g / p.WPR;
        const int c = (g - r * p.WPR) * 64 + lane;
        const bool flag = c < p.Cn && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (lane == 0) {
            p.wbits[g] = word;
            p.wbase[g] = __popcll(word);
        }
    }
    __syncthreads();
    const int nnz = block_scan_inplace(p.wbase, NW, lds);
    if (threadIdx.x == 0) p.nnz_dev[0] = nnz;

    if (p.row_ptr) {
        for (int r = threadIdx.x; r < p.R; r += blockDim.x) p.row_ptr[r] = p.wbase[r * p.WPR];
        if (threadIdx.x == 0) p.row_ptr[p.R] = nnz;
    }
    if (p.bcsr_idx) {
        for (int g = wave; g < NW; g += nwaves) {
            const int r = g / p.WPR;
            const int c = (g - r * p.WPR) * 64 + lane;
            const unsigned long long word = p.wbits[g];
            if ((word >> lane) & 1ull) {
                const int pos = p.wbase[g] + __popcll(word & lt_mask);
                if (pos < p.cap) p.bcsr_idx[pos] = (r << 16) | c;
            }
        }
    }
    if (!p.col_ptr) return;  // uniform over the workgroup

    // ---- column words --------------------------------------------------------
    const int NWC = p.Cn * p.WPC;
    for (int g = wave; g < NWC; g += nwaves) {
        const int c = g / p.WPC;
        const int r = (g - c * p.WPC) * 64 + lane;
        const bool flag = r < p.R && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (lane == 0) p.cbase[g] = __popcll(word);
    }
    __syncthreads();
    const int nnz2 = block_scan_inplace(p.cbase, NWC, lds);
    for (int c = threadIdx.x; c < p.Cn; c += blockDim.x) p.col_ptr[c] = p.cbase[c * p.WPC];
    if (threadIdx.x == 0) p.col_ptr[p.Cn] = nnz2;

    if (p.bcsc_idx) {
        for (int g = wave; g < NWC; g += nwaves) {
            const int c = g / p.WPC;
            const int r = (g - c * p.WPC) * 64 + lane;
            const bool flag = r < p.R && p.live[(int64_t)r * p.Cn + c] != 0;
            const unsigned long long word = __ballot(flag);
            if (flag) {
                const int pos = p.cbase[g] + __popcll(word & lt_mask);
                if (pos < p.cap) {
                    if (p.bcsc_i64) {
                        const int gw = r * p.WPR + (c >> 6);
                        const int cl = c & 63;
                        const unsigned long long below =
                            cl == 0 ? 0ull : (p.wbits[gw] & (~0ull >> (64 - cl)));
                        const long long bpos = p.wbase[gw] + __popcll(below);
                        reinterpret_cast<long long*>(p.bcsc_idx)[pos] =
                            (bpos << 32) | ((long long)c << 16) | (long long)r;
                    } else {
                        reinterpret_cast<int32_t*>(p.bcsc_idx)[pos] = (c << 16) | r;
                    }
                }
            }
        }
    }
}

struct IndexWorkspace {
    size_t live_off, wbits_off, wbase_off, cbase_off, total;
    int R, Cn, WPR, WPC;
};

static IndexWorkspace index_workspace(int H, int W, int BH, int BW) {
    IndexWorkspace w;
    w.R = H / BH;
    w.Cn = W / BW;
    w.WPR = (w.Cn + 63) / 64;
    w.WPC = (w.R + 63) / 64;
    size_t off = 0;
    w.live_off = off;  off += round_up((size_t)w.R * w.Cn, 256);
    w.wbits_off = off; off += round_up((size_t)w.R * w.WPR * 8, 256);
    w.wbase_off = off; off += round_up((size_t)w.R * w.WPR * 4, 256);
    w.cbase_off = off; off += round_up((size_t)w.Cn * w.WPC * 4, 256);
    w.total = off;
    return w;
}

static int check_index_shape(int H, int W, int BH, int BW) {
    SPX_REQUIRE(valid_block_edge(BH) && valid_block_edge(BW), SPX_E_CONFIG,
                "block size (%d,%d) must be a power of two in [4,256]", BH, BW);
    SPX_REQUIRE(H > 0 && W > 0 && H % BH == 0 && W % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a positive multiple of the block (%d,%d)", H, W, BH, BW);
    SPX_REQUIRE(H / BH <= 65535 && W / BW <= 65535, SPX_E_SHAPE,
                "more than 65535 blocks per dimension do not fit the 16-bit index fields");
    return 0;
}

}  // namespace spx

extern "C" size_t spx_bcs_index_workspace_bytes(int H, int W, int BH, int BW) {
    if (spx::check_index_shape(H, W, BH, BW) != 0) return 0;
    return spx::index_workspace(H, W, BH, BW).total;
}

extern "C" int spx_bcs_index(const uint8_t* mask, int H, int W, int BH, int BW,
                             int32_t* row_ptr, int32_t* bcsr_idx,
                             int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                             int32_t* nnz_dev, int cap,
                             void* workspace, size_t workspace_bytes, spx_stream_t stream) {
    using namespace spx;
    int rc = check_index_shape(H, W, BH, BW);
    if (rc) return rc;
    SPX_REQUIRE(mask && nnz_dev && workspace, SPX_E_NULL, "mask, nnz_dev and workspace are required");
    SPX_REQUIRE((row_ptr != nullptr) == (bcsr_idx != nullptr), SPX_E_NULL,
                "row_ptr and bcsr_idx must be given together");
    SPX_REQUIRE((col_ptr != nullptr) == (bcsc_idx != nullptr), SPX_E_NULL,
                "col_ptr and bcsc_idx must be given together");
    SPX_REQUIRE(row_ptr || col_ptr, SPX_E_NULL, "neither a BCSR nor a BCSC index was requested");
    SPX_REQUIRE(!(bcsc_i64 && !bcsc_idx), SPX_E_NULL, "bcsc_i64 set without a bcsc_idx buffer");
    SPX_REQUIRE(cap >= 0, SPX_E_SHAPE, "negative index capacity");
    const IndexWorkspace ws = index_workspace(H, W, BH, BW);
    SPX_REQUIRE(workspace_bytes >= ws.total, SPX_E_WORKSPACE,
                "workspace of %zu bytes is smaller than the %zu required", workspace_bytes, ws.total);
    SPX_REQUIRE(aligned(workspace, 256), SPX_E_ALIGN, "workspace must be 256-byte aligned");
    SPX_REQUIRE(!bcsc_i64 || aligned(bcsc_idx, 8), SPX_E_ALIGN, "int64 bcsc_idx must be 8-byte aligned");

    char* wsb = reinterpret_cast<char*>(workspace);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);

    // Widest load the mask's address and row pitch allow.
    int vec = 1;
    if (W % 16 == 0 && aligned(mask, 16)) vec = 16;
    else if (W % 4 == 0 && aligned(mask, 4)) vec = 4;

    // Segment width: at most 256 threads * vec bytes, at least one block wide;
    // narrowed while that buys more workgroups (the launch wants >> 256 of them).
    int segw = 256 * vec;
    if (segw > 1024) segw = 1024;
    int wpow = 1;
    while (wpow < W) wpow <<= 1;
    if (segw > wpow) segw = wpow;
    const int min_seg = BW > vec ? BW : vec;
    while (segw > min_seg && (int64_t)ws.R * ((W + segw - 1) / segw) < 2048) segw >>= 1;
    if (segw < min_seg) segw = min_seg;

    LiveParams lp;
    lp.mask = mask;
    lp.live = reinterpret_cast<uint8_t*>(wsb + ws.live_off);
    lp.H = H; lp.W = W; lp.BH = BH; lp.BW = BW; lp.Cn = ws.Cn;
    lp.segw = segw;
    lp.log_tcols = ilog2(segw / vec);
    lp.log_bw = ilog2(BW);
    dim3 grid((W + segw - 1) / segw, ws.R, 1);
    if (vec == 16) hipLaunchKernelGGL(liveness_kernel<16>, grid, dim3(256), 0, st, lp);
    else if (vec == 4) hipLaunchKernelGGL(liveness_kernel<4>, grid, dim3(256), 0, st, lp);
    else hipLaunchKernelGGL(liveness_kernel<1>, grid, dim3(256), 0, st, lp);
    SPX_LAUNCH_CHECK("liveness_kernel");

    EmitParams ep;
    ep.live = lp.live;
    ep.wbits = reinterpret_cast<unsigned long long*>(wsb + ws.wbits_off);
    ep.wbase = reinterpret_cast<int*>(wsb + ws.wbase_off);
    ep.cbase = reinterpret_cast<int*>(wsb + ws.cbase_off);
    ep.row_ptr = row_ptr; ep.bcsr_idx = bcsr_idx;
    ep.col_ptr = col_ptr; ep.bcsc_idx = bcsc_idx; ep.bcsc_i64 = bcsc_i64;
    ep.nnz_dev = nnz_dev; ep.cap = cap;
    ep.R = ws.R; ep.Cn = ws.Cn; ep.WPR = ws.WPR; ep.WPC = ws.WPC;
    hipLaunchKernelGGL(emit_kernel, dim3(1), dim3(1024), 0, st, ep);
    SPX_LAUNCH_CHECK("emit_kernel");
    return 0;
}
