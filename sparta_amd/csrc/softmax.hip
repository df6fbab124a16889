// Masked block-sparse softmax, forward and backward.
//
// One wavefront owns one matrix row: its live blocks (row_ptr / BCSR_idx) form
// a list of nblk*BW candidate entries that the 64 lanes stride over.  The row is
// read from HBM once (values are cached in registers, up to 16 per lane, i.e.
// rows of up to 1024 live entries; longer rows re-read through L2), reduced with
// cross-lane shuffles and written once.  HBM-bound: one read and one write of
// the live entries plus one byte of mask per entry.
// Replaces sparta_sparse_softmax_{forward,backward}.cuh.j2 of the reference.
#include "common.hpp"

namespace spx {

struct SoftmaxParams {
    const void* x;       // forward: x;       backward: grad_y
    const void* y_in;    // forward: unused;  backward: y
    void* out;           // forward: y;       backward: grad_x
    const int32_t* row_ptr;
    const int32_t* bcsr_idx;
    const uint8_t* mask;
    float inv_t;
    int H, W, BH, BW, log_bh, log_bw;
    int compressed;
    int64_t batch_stride;
};

constexpr int SM_CACHE = 16;
constexpr int SM_ROWS = 4;  // rows (wavefronts) per workgroup

struct RowView {
    int first, nblk, n;   // first block position, live blocks, candidate entries
    int row, rr, br;
};

__device__ __forceinline__ int64_t entry_offset(const SoftmaxParams& p, const RowView& rv, int e) {
    const int bo = e >> p.log_bw;
    const int c = e & (p.BW - 1);
    if (p.compressed) return (((int64_t)(rv.first + bo) << p.log_bh) + rv.rr) * p.BW + c;
    const int bc = p.bcsr_idx[rv.first + bo] & 0xffff;
    return (int64_t)rv.row * p.W + (int64_t)bc * p.BW + c;
}

template <typename T, bool BACKWARD>
__global__ __launch_bounds__(64 * SM_ROWS) void softmax_kernel(SoftmaxParams p) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    RowView rv;
    rv.row = blockIdx.x * SM_ROWS + wave;
    if (rv.row >= p.H) return;
    rv.br = rv.row >> p.log_bh;
    rv.rr = rv.row & (p.BH - 1);
    rv.first = p.row_ptr[rv.br];
    rv.nblk = p.row_ptr[rv.br + 1] - rv.first;
    rv.n = rv.nblk << p.log_bw;
    if (rv.n == 0) return;

    const int64_t boff = (int64_t)blockIdx.y * p.batch_stride;
    const T* x = reinterpret_cast<const T*>(p.x) + boff;
    const T* yin = BACKWARD ? reinterpret_cast<const T*>(p.y_in) + boff : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + boff;

    float cache[SM_CACHE];
    unsigned live_bits = 0;  // bit t: cached entry t is unmasked

    if (!BACKWARD) {
        float vmax = -INFINITY;
#pragma unroll
        for (int t = 0; t < SM_CACHE; ++t) {
            const int e = lane + 64 * t;
            cache[t] = 0.f;
            if (e < rv.n) {
                const int64_t off = entry_offset(p, rv, e);
                if (p.mask[off]) {
                    cache[t] = Elem<T>::to_float(x[off]);
                    live_bits |= 1u << t;
                    vmax = fmaxf(vmax, cache[t]);
                }
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            if (p.mask[off]) vmax = fmaxf(vmax, Elem<T>::to_float(x[off]));
        }
        vmax = wave_reduce_max(vmax);
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < SM_CACHE; ++t) {
            if (live_bits & (1u << t)) {
                cache[t] = __expf((cache[t] - vmax) * p.inv_t);
                sum += cache[t];
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            if (p.mask[off]) sum += __expf((Elem<T>::to_float(x[off]) - vmax) * p.inv_t);
        }
        sum = wave_reduce_sum(sum);
        const float inv = sum > 0.f ? 1.f / sum : 0.f;
#pragma unroll
        for (int t = 0; t < SM_CACHE; ++t) {
            const int e = lane + 64 * t;
            if (e < rv.n) {
                const int64_t off = entry_offset(p, rv, e);
                out[off] = Elem<T>::from_float((live_bits & (1u << t)) ? cache[t] * inv : 0.f);
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            float v = 0.f;
            if (p.mask[off]) v = __expf((Elem<T>::to_float(x[off]) - vmax) * p.inv_t) * inv;
            out[off] = Elem<T>::from_float(v);
        }
    } else {
        // cache y*dy and y of the first entries
        float ycache[SM_CACHE];
        float dot = 0.f;
#pragma unroll
        for (int t = 0; t < SM_CACHE; ++t) {
            const int e = lane + 64 * t;
            cache[t] = 0.f;
            ycache[t] = 0.f;
            if (e < rv.n) {
                const int64_t off = entry_offset(p, rv, e);
                if (p.mask[off]) {
                    ycache[t] = Elem<T>::to_float(yin[off]);
                    cache[t] = ycache[t] * Elem<T>::to_float(x[off]);
                    dot += cache[t];
                }
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            if (p.mask[off]) dot += Elem<T>::to_float(yin[off]) * Elem<T>::to_float(x[off]);
        }
        dot = wave_reduce_sum(dot);
#pragma unroll
        for (int t = 0; t < SM_CACHE; ++t) {
            const int e = lane + 64 * t;
            if (e < rv.n) {
                const int64_t off = entry_offset(p, rv, e);
                out[off] = Elem<T>::from_float(p.inv_t * (cache[t] - ycache[t] * dot));
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            float v = 0.f;
            if (p.mask[off]) {
                const float yv = Elem<T>::to_float(yin[off]);
                v = p.inv_t * (yv * Elem<T>::to_float(x[off]) - yv * dot);
            }
            out[off] = Elem<T>::from_float(v);
        }
    }
}

template <bool BACKWARD>
static int launch_softmax(int dtype, int compressed, const void* x, const void* y_in, void* out,
                          const int32_t* row_ptr, const int32_t* bcsr_idx, const uint8_t* mask,
                          float inv_t, int batch, int H, int W, int BH, int BW,
                          int64_t batch_stride, hipStream_t st) {
    SPX_REQUIRE(x && out && row_ptr && bcsr_idx && mask, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(!BACKWARD || y_in, SPX_E_NULL, "y is required for the backward pass");
    SPX_REQUIRE(dtype == SPX_F32 || dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE, "unknown dtype %d", dtype);
    SPX_REQUIRE(valid_block_edge(BH) && valid_block_edge(BW), SPX_E_CONFIG,
                "block size (%d,%d) must be a power of two in [4,256]", BH, BW);
    SPX_REQUIRE(H > 0 && W > 0 && H % BH == 0 && W % BW == 0, SPX_E_SHAPE,
                "shape (%d,%d) is not a positive multiple of the block (%d,%d)", H, W, BH, BW);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    if (batch == 0) return 0;
    SoftmaxParams p;
    p.x = x; p.y_in = y_in; p.out = out;
    p.row_ptr = row_ptr; p.bcsr_idx = bcsr_idx; p.mask = mask;
    p.inv_t = inv_t;
    p.H = H; p.W = W; p.BH = BH; p.BW = BW; p.log_bh = ilog2(BH); p.log_bw = ilog2(BW);
    p.compressed = compressed; p.batch_stride = batch_stride;
    dim3 grid((H + SM_ROWS - 1) / SM_ROWS, batch, 1);
    dim3 block(64 * SM_ROWS);
    switch (dtype) {
        case SPX_F32: hipLaunchKernelGGL((softmax_kernel<float, BACKWARD>), grid, block, 0, st, p); break;
        case SPX_F16: hipLaunchKernelGGL((softmax_kernel<_Float16, BACKWARD>), grid, block, 0, st, p); break;
        default: hipLaunchKernelGGL((softmax_kernel<bf16_t, BACKWARD>), grid, block, 0, st, p); break;
    }
    SPX_LAUNCH_CHECK("softmax_kernel");
    return 0;
}

}  // namespace spx

extern "C" int spx_softmax_forward(int dtype, int compressed, const void* x, void* y,
                                   const int32_t* row_ptr, const int32_t* bcsr_idx,
                                   const uint8_t* mask, float inv_temperature,
                                   int batch, int H, int W, int BH, int BW,
                                   int64_t batch_stride, int tile_cfg, spx_stream_t stream) {
    (void)tile_cfg;
    return spx::launch_softmax<false>(dtype, compressed, x, nullptr, y, row_ptr, bcsr_idx, mask,
                                      inv_temperature, batch, H, W, BH, BW, batch_stride,
                                      reinterpret_cast<hipStream_t>(stream));
}

extern "C" int spx_softmax_backward(int dtype, int compressed, const void* grad_y, const void* y,
                                    void* grad_x, const int32_t* row_ptr, const int32_t* bcsr_idx,
                                    const uint8_t* mask, float inv_temperature,
                                    int batch, int H, int W, int BH, int BW,
                                    int64_t batch_stride, int tile_cfg, spx_stream_t stream) {
    (void)tile_cfg;
    return spx::launch_softmax<true>(dtype, compressed, grad_y, y, grad_x, row_ptr, bcsr_idx, mask,
                                     inv_temperature, batch, H, W, BH, BW, batch_stride,
                                     reinterpret_cast<hipStream_t>(stream));
}
