// dense <-> compressed block values, and row/column sums of compressed values.
// Pure data movement: one workgroup per (live block, batch), widest vector the
// tile pitch allows.  Replaces dense_to_bcs_val / bcs_val_to_dense /
// bcsr_val_sum_row / bcsr_val_sum_col of the reference
// (sparta/tesa/templates/block_compressed.cu.j2:172-288) for every element size.
#include "common.hpp"

namespace spx {

struct ConvParams {
    const char* src;
    char* dst;
    const void* idx;
    const int32_t* nnz_dev;
    int idx_kind;
    int H, W, BH, BW;
    int log_vpr;  // log2(vectors per tile row)
    int64_t sparse_batch_stride;  // in vectors
    int64_t dense_row_pitch;      // in vectors
};

__device__ __forceinline__ void decode_block(const void* idx, int kind, int i, int& br, int& bc) {
    if (kind == SPX_IDX_BCSR_I32) {
        const int v = reinterpret_cast<const int32_t*>(idx)[i];
        br = (v >> 16) & 0xffff; bc = v & 0xffff;
    } else if (kind == SPX_IDX_BCSC_I32) {
        const int v = reinterpret_cast<const int32_t*>(idx)[i];
        bc = (v >> 16) & 0xffff; br = v & 0xffff;
    } else {
        const long long v = reinterpret_cast<const long long*>(idx)[i];
        bc = (int)((v >> 16) & 0xffff); br = (int)(v & 0xffff);
    }
}

// V: vector type moved per thread; GATHER: dense -> sparse, else sparse -> dense.
template <typename V, bool GATHER>
__global__ __launch_bounds__(256) void convert_kernel(ConvParams p) {
    const int i = blockIdx.x;
    if (p.nnz_dev && i >= p.nnz_dev[0]) return;
    int br, bc;
    decode_block(p.idx, p.idx_kind, i, br, bc);
    const int vpr = 1 << p.log_vpr;
    const int nvec = p.BH << p.log_vpr;
    const V* src = reinterpret_cast<const V*>(p.src);
    V* dst = reinterpret_cast<V*>(p.dst);
    const int64_t b = blockIdx.y;
    const int64_t dense_base = (b * p.H + (int64_t)br * p.BH) * p.dense_row_pitch + (int64_t)bc * vpr;
    const int64_t sparse_base = b * p.sparse_batch_stride + (int64_t)i * nvec;
    for (int v = threadIdx.x; v < nvec; v += 256) {
        const int r = v >> p.log_vpr;
        const int c = v & (vpr - 1);
        const int64_t d = dense_base + (int64_t)r * p.dense_row_pitch + c;
        if (GATHER) dst[sparse_base + v] = src[d];
        else dst[d] = src[sparse_base + v];
    }
}

template <bool GATHER>
static int launch_convert(const void* src, void* dst, const void* idx, int idx_kind,
                          int nnz_bound, const int32_t* nnz_dev, int batch, int H, int W,
                          int BH, int BW, int elem_bytes, int64_t sparse_batch_stride,
                          hipStream_t st) {
    SPX_REQUIRE((src && dst && idx) || nnz_bound == 0 || batch == 0, SPX_E_NULL,
                "dense, sparse and index buffers are required");
    SPX_REQUIRE(idx_kind >= 0 && idx_kind <= 2, SPX_E_CONFIG, "unknown idx_kind %d", idx_kind);
    SPX_REQUIRE(valid_block_edge(BH) && valid_block_edge(BW), SPX_E_CONFIG,
                "block size (%d,%d) must be a power of two in [4,256]", BH, BW);
    SPX_REQUIRE(H > 0 && W > 0 && H % BH == 0 && W % BW == 0, SPX_E_SHAPE,
                "shape (%d,%d) is not a positive multiple of the block (%d,%d)", H, W, BH, BW);
    SPX_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
                SPX_E_DTYPE, "element size %d not in {1,2,4,8}", elem_bytes);
    SPX_REQUIRE(batch >= 0 && nnz_bound >= 0, SPX_E_SHAPE, "negative batch or nnz");
    SPX_REQUIRE(batch <= 65535, SPX_E_SHAPE, "batch %d exceeds the 65535 grid limit", batch);
    if (batch == 0 || nnz_bound == 0) return 0;

    // Widest vector that divides a tile row and keeps every access aligned.
    const int64_t row_bytes = (int64_t)BW * elem_bytes;
    const int64_t pitch_bytes = (int64_t)W * elem_bytes;
    const int64_t sbs_bytes = sparse_batch_stride * elem_bytes;
    int vb = 16;
    while (vb > elem_bytes &&
           (row_bytes % vb || pitch_bytes % vb || sbs_bytes % vb || !aligned(src, vb) || !aligned(dst, vb)))
        vb >>= 1;
    SPX_REQUIRE(aligned(src, vb) && aligned(dst, vb), SPX_E_ALIGN, "buffers are not element-aligned");

    ConvParams p;
    p.src = reinterpret_cast<const char*>(src);
    p.dst = reinterpret_cast<char*>(dst);
    p.idx = idx; p.nnz_dev = nnz_dev; p.idx_kind = idx_kind;
    p.H = H; p.W = W; p.BH = BH; p.BW = BW;
    p.log_vpr = ilog2((int)(row_bytes / vb));
    p.sparse_batch_stride = sbs_bytes / vb;
    p.dense_row_pitch = pitch_bytes / vb;
    dim3 grid(nnz_bound, batch, 1);
    switch (vb) {
        case 16: hipLaunchKernelGGL((convert_kernel<vec16, GATHER>), grid, dim3(256), 0, st, p); break;
        case 8: hipLaunchKernelGGL((convert_kernel<uint64_t, GATHER>), grid, dim3(256), 0, st, p); break;
        case 4: hipLaunchKernelGGL((convert_kernel<uint32_t, GATHER>), grid, dim3(256), 0, st, p); break;
        case 2: hipLaunchKernelGGL((convert_kernel<uint16_t, GATHER>), grid, dim3(256), 0, st, p); break;
        default: hipLaunchKernelGGL((convert_kernel<uint8_t, GATHER>), grid, dim3(256), 0, st, p); break;
    }
    SPX_LAUNCH_CHECK("convert_kernel");
    return 0;
}

// ---- sums -------------------------------------------------------------------
struct SumParams {
    const void* sparse;
    float* result;  // fp32 accumulation buffer [batch, H] or [batch, W]
    const void* idx;
    int idx_kind;
    int nnz, H, W, BH, BW;
    int axis;
    int64_t sparse_batch_stride;
};

// One workgroup per (block row [axis 0] or block column [axis 1], batch): it scans the
// index 256 entries at a time, and adds the tiles of its row / column in index order
// (thread (o, s) owns output o and every per-th element along the reduced axis).  No
// atomics: the order of the additions is fixed by the index, so the sums are the same
// bits on every run, and every output is written exactly once (zero for an empty row).
template <typename T>
__global__ __launch_bounds__(256) void sum_kernel(SumParams p) {
    __shared__ float part[256];
    __shared__ unsigned long long s_match[4];
    const int mine = blockIdx.x;
    const int nout = p.axis == 0 ? p.BH : p.BW;   // <= 256
    const int nred = p.axis == 0 ? p.BW : p.BH;
    const int out_stride = p.axis == 0 ? p.BW : 1;
    const int red_stride = p.axis == 0 ? 1 : p.BW;
    const int per = 256 / nout;  // partial reducers per output
    const int o = threadIdx.x / per;
    const int s = threadIdx.x - o * per;
    const T* batch_base = reinterpret_cast<const T*>(p.sparse) + (int64_t)blockIdx.y * p.sparse_batch_stride;
    float acc = 0.f;
    for (int base = 0; base < p.nnz; base += 256) {
        const int i = base + threadIdx.x;
        bool match = false;
        if (i < p.nnz) {
            int br, bc;
            decode_block(p.idx, p.idx_kind, i, br, bc);
            match = (p.axis == 0 ? br : bc) == mine;
        }
        const unsigned long long bits = __ballot(match);
        if ((threadIdx.x & 63) == 0) s_match[threadIdx.x >> 6] = bits;
        __syncthreads();
        for (int w = 0; w < 4; ++w) {
            unsigned long long todo = s_match[w];
            while (todo) {
                const int j = __ffsll((long long)todo) - 1;
                todo &= todo - 1;
                const int slot = base + w * 64 + j;  // values follow the order of this index
                const T* tile = batch_base + (int64_t)slot * p.BH * p.BW;
                if (o < nout)
                    for (int k = s; k < nred; k += per)
                        acc += Elem<T>::to_float(tile[(int64_t)o * out_stride + (int64_t)k * red_stride]);
            }
        }
        __syncthreads();
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x < nout) {
        float t = 0.f;
        for (int k = 0; k < per; ++k) t += part[threadIdx.x * per + k];
        const int64_t pos = p.axis == 0 ? ((int64_t)blockIdx.y * p.H + (int64_t)mine * p.BH + threadIdx.x)
                                        : ((int64_t)blockIdx.y * p.W + (int64_t)mine * p.BW + threadIdx.x);
        p.result[pos] = t;
    }
}

}  // namespace spx

extern "C" int spx_bcs_gather(const void* dense, void* sparse, const void* idx, int idx_kind,
                              int nnz_bound, const int32_t* nnz_dev, int batch, int H, int W,
                              int BH, int BW, int elem_bytes, int64_t sparse_batch_stride,
                              spx_stream_t stream) {
    return spx::launch_convert<true>(dense, sparse, idx, idx_kind, nnz_bound, nnz_dev, batch, H, W,
                                     BH, BW, elem_bytes, sparse_batch_stride,
                                     reinterpret_cast<hipStream_t>(stream));
}

extern "C" int spx_bcs_scatter(const void* sparse, void* dense, const void* idx, int idx_kind,
                               int nnz_bound, const int32_t* nnz_dev, int batch, int H, int W,
                               int BH, int BW, int elem_bytes, int64_t sparse_batch_stride,
                               spx_stream_t stream) {
    return spx::launch_convert<false>(sparse, dense, idx, idx_kind, nnz_bound, nnz_dev, batch, H, W,
                                      BH, BW, elem_bytes, sparse_batch_stride,
                                      reinterpret_cast<hipStream_t>(stream));
}

extern "C" int spx_bcs_sum(const void* sparse, void* result, const void* idx, int idx_kind,
                           int nnz, int batch, int H, int W, int BH, int BW, int dtype, int axis,
                           int64_t sparse_batch_stride, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(result, SPX_E_NULL, "result buffer is NULL");
    SPX_REQUIRE(sparse || nnz == 0, SPX_E_NULL, "sparse buffer is NULL");
    SPX_REQUIRE(idx || nnz == 0, SPX_E_NULL, "index array is NULL");
    SPX_REQUIRE(idx_kind >= 0 && idx_kind <= 2, SPX_E_CONFIG, "unknown idx_kind %d", idx_kind);
    SPX_REQUIRE(valid_block_edge(BH) && valid_block_edge(BW), SPX_E_CONFIG,
                "block size (%d,%d) must be a power of two in [4,256]", BH, BW);
    SPX_REQUIRE(H > 0 && W > 0 && H % BH == 0 && W % BW == 0, SPX_E_SHAPE, "bad shape");
    SPX_REQUIRE(axis == 0 || axis == 1, SPX_E_CONFIG, "axis must be 0 (sum over W) or 1 (sum over H)");
    SPX_REQUIRE(dtype == SPX_F32 || dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE, "unknown dtype %d", dtype);
    SPX_REQUIRE(batch >= 0 && batch <= 65535 && nnz >= 0, SPX_E_SHAPE, "bad batch / nnz");
    if (batch == 0) return 0;
    // nnz == 0 is launched as well: every entry of `result` is written (zeros then), the
    // kernel reads neither `sparse` nor `idx`
    SumParams p;
    p.sparse = sparse; p.result = reinterpret_cast<float*>(result);
    p.idx = idx; p.idx_kind = idx_kind; p.nnz = nnz;
    p.H = H; p.W = W; p.BH = BH; p.BW = BW; p.axis = axis;
    p.sparse_batch_stride = sparse_batch_stride;
    const dim3 grid(axis == 0 ? H / BH : W / BW, batch, 1);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {   // the values are read in their own type; the result is fp32 in every case
        case SPX_F32: hipLaunchKernelGGL(sum_kernel<float>, grid, dim3(256), 0, st, p); break;
        case SPX_F16: hipLaunchKernelGGL(sum_kernel<_Float16>, grid, dim3(256), 0, st, p); break;
        default: hipLaunchKernelGGL(sum_kernel<bf16_t>, grid, dim3(256), 0, st, p); break;
    }
    SPX_LAUNCH_CHECK("sum_kernel");
    return 0;
}
