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
                if (!p.mask || p.mask[off]) {
                    cache[t] = Elem<T>::to_float(x[off]);
                    live_bits |= 1u << t;
                    vmax = fmaxf(vmax, cache[t]);
                }
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            if (!p.mask || p.mask[off]) vmax = fmaxf(vmax, Elem<T>::to_float(x[off]));
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
            if (!p.mask || p.mask[off]) sum += __expf((Elem<T>::to_float(x[off]) - vmax) * p.inv_t);
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
            if (!p.mask || p.mask[off]) v = __expf((Elem<T>::to_float(x[off]) - vmax) * p.inv_t) * inv;
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
                if (!p.mask || p.mask[off]) {
                    ycache[t] = Elem<T>::to_float(yin[off]);
                    cache[t] = ycache[t] * Elem<T>::to_float(x[off]);
                    dot += cache[t];
                }
            }
        }
        for (int e = lane + 64 * SM_CACHE; e < rv.n; e += 64) {
            const int64_t off = entry_offset(p, rv, e);
            if (!p.mask || p.mask[off]) dot += Elem<T>::to_float(yin[off]) * Elem<T>::to_float(x[off]);
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
            if (!p.mask || p.mask[off]) {
                const float yv = Elem<T>::to_float(yin[off]);
                v = p.inv_t * (yv * Elem<T>::to_float(x[off]) - yv * dot);
            }
            out[off] = Elem<T>::from_float(v);
        }
    }
}

// ---- vectorized variant -------------------------------------------------------------------
// Same row-per-wavefront scheme with 16-byte accesses: a lane owns whole vectors of VE
// consecutive entries of one live block row (VE = 8 for 16-bit types, 4 for fp32), reads
// the VE mask bytes as one word and keeps up to SMV_CACHE vectors in registers, so a row
// of up to 64 * SMV_CACHE * VE candidate entries moves through HBM once each way.  A NULL
// mask means that every entry of a live block takes part.  Needs BW % VE == 0.
constexpr int SMV_CACHE = 4;
constexpr int SMV_ROWS = 4;

template <typename T> struct SmVec;
template <> struct SmVec<float> {
    static constexpr int VE = 4;
    typedef uint32_t mask_t;
    __device__ static void unpack(const vec16& v, float* f) {
        f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
    }
    __device__ static vec16 pack(const float* f) {
        return vec16{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
    }
};
template <> struct SmVec<_Float16> {
    static constexpr int VE = 8;
    typedef uint64_t mask_t;
    __device__ static void unpack(const vec16& v, float* f) {
        union { vec16 q; _Float16 h[8]; } u; u.q = v;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)u.h[i];
    }
    __device__ static vec16 pack(const float* f) {
        union { vec16 q; _Float16 h[8]; } u;
#pragma unroll
        for (int i = 0; i < 8; ++i) u.h[i] = (_Float16)f[i];
        return u.q;
    }
};
template <> struct SmVec<bf16_t> {
    static constexpr int VE = 8;
    typedef uint64_t mask_t;
    __device__ static void unpack(const vec16& v, float* f) {
        f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
        f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
        f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
        f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    __device__ static vec16 pack(const float* f) {
        vec16 r;
        r.x = (uint32_t)float_to_bf16(f[0]) | ((uint32_t)float_to_bf16(f[1]) << 16);
        r.y = (uint32_t)float_to_bf16(f[2]) | ((uint32_t)float_to_bf16(f[3]) << 16);
        r.z = (uint32_t)float_to_bf16(f[4]) | ((uint32_t)float_to_bf16(f[5]) << 16);
        r.w = (uint32_t)float_to_bf16(f[6]) | ((uint32_t)float_to_bf16(f[7]) << 16);
        return r;
    }
};

// element offset of vector v (VE entries) of the row
template <int VE>
__device__ __forceinline__ int64_t vector_offset(const SoftmaxParams& p, const RowView& rv, int v, int log_vpb) {
    const int bo = v >> log_vpb;
    const int c = (v & ((1 << log_vpb) - 1)) * VE;
    if (p.compressed) return (((int64_t)(rv.first + bo) << p.log_bh) + rv.rr) * p.BW + c;
    const int bc = p.bcsr_idx[rv.first + bo] & 0xffff;
    return (int64_t)rv.row * p.W + (int64_t)bc * p.BW + c;
}

// LPR lanes share a row (16: four rows per wavefront, for rows of up to 16 * SMV_CACHE
// vectors; 64: one row per wavefront, any length).
template <int LPR> __device__ __forceinline__ float group_reduce_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror: 8 lanes
    if constexpr (LPR >= 16) v = fmaxf(v, dpp_move<0x140>(v));  // row_mirror: 16 lanes
    if constexpr (LPR >= 32) v = fmaxf(v, __shfl_xor(v, 16, 64));
    if constexpr (LPR == 64) v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
template <int LPR> __device__ __forceinline__ float group_reduce_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    if constexpr (LPR >= 16) v += dpp_move<0x140>(v);
    if constexpr (LPR >= 32) v += __shfl_xor(v, 16, 64);
    if constexpr (LPR == 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// Maximum of VE values as nested three-way maxima (one v_max3_f32 each).
template <int VE>
__device__ __forceinline__ float vec_max(const float* f) {
    float m = max3f(f[0], f[1], f[2]);
    if constexpr (VE == 8) {
        m = max3f(m, f[3], f[4]);
        m = max3f(m, f[5], f[6]);
        return fmaxf(m, f[7]);
    } else {
        return fmaxf(m, f[3]);
    }
}

// HAS_MASK = false: every entry of a live block takes part (p.mask is NULL) and no mask
// word is read or tested.
template <typename T, bool BACKWARD, int LPR, bool HAS_MASK>
__global__ __launch_bounds__(64 * SMV_ROWS) void softmax_vec_kernel(SoftmaxParams p) {
    constexpr int VE = SmVec<T>::VE;
    constexpr int RPW = 64 / LPR;
    typedef typename SmVec<T>::mask_t mask_t;
    const int lane = lane_id() % LPR;
    const int wave = threadIdx.x >> 6;
    RowView rv;
    rv.row = (blockIdx.x * SMV_ROWS + wave) * RPW + lane_id() / LPR;
    if (rv.row >= p.H) return;
    rv.br = rv.row >> p.log_bh;
    rv.rr = rv.row & (p.BH - 1);
    rv.first = p.row_ptr[rv.br];
    rv.nblk = p.row_ptr[rv.br + 1] - rv.first;
    const int log_vpb = p.log_bw - (VE == 8 ? 3 : 2);  // vectors per block row
    const int nvec = rv.nblk << log_vpb;
    rv.n = nvec;
    if (nvec == 0) return;

    const int64_t boff = (int64_t)blockIdx.y * p.batch_stride;
    const T* x = reinterpret_cast<const T*>(p.x) + boff;
    const T* yin = BACKWARD ? reinterpret_cast<const T*>(p.y_in) + boff : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + boff;
    auto on = [](mask_t m, int i) { return !HAS_MASK || ((m >> (8 * i)) & 0xff) != 0; };
    auto mask_at = [&](int64_t off) { return HAS_MASK ? *reinterpret_cast<const mask_t*>(p.mask + off) : ~(mask_t)0; };

    float cache[SMV_CACHE][VE];
    float ycache[BACKWARD ? SMV_CACHE : 1][VE];
    mask_t live[HAS_MASK ? SMV_CACHE : 1];
    int64_t offs[SMV_CACHE];
#pragma unroll
    for (int t = 0; t < SMV_CACHE; ++t) {
        const int v = lane + LPR * t;
        offs[t] = 0;
        if constexpr (HAS_MASK) live[t] = 0;
        if (v < nvec) {
            offs[t] = vector_offset<VE>(p, rv, v, log_vpb);
            if constexpr (HAS_MASK) live[t] = mask_at(offs[t]);
            SmVec<T>::unpack(load16_stream(x + offs[t]), cache[t]);
            if (BACKWARD) SmVec<T>::unpack(load16_stream(yin + offs[t]), ycache[t]);
        }
    }
    if (!BACKWARD) {
        // exp((x - max) / T) as exp2(x * c + nb): one fused multiply-add per entry
        const float c = p.inv_t * 1.4426950408889634f;
        float vmax = -INFINITY;
#pragma unroll
        for (int t = 0; t < SMV_CACHE; ++t) {
            if (lane + LPR * t < nvec) {
                if constexpr (HAS_MASK) {
#pragma unroll
                    for (int i = 0; i < VE; ++i)
                        if (on(live[t], i)) vmax = fmaxf(vmax, cache[t][i]);
                } else {
                    vmax = fmaxf(vmax, vec_max<VE>(cache[t]));
                }
            }
        }
        for (int v = lane + LPR * SMV_CACHE; v < nvec; v += LPR) {
            const int64_t off = vector_offset<VE>(p, rv, v, log_vpb);
            const mask_t m = mask_at(off);
            float f[VE];
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(x + off), f);
#pragma unroll
            for (int i = 0; i < VE; ++i)
                if (on(m, i)) vmax = fmaxf(vmax, f[i]);
        }
        vmax = group_reduce_max<LPR>(vmax);
        const float nb = vmax == -INFINITY ? 0.f : -vmax * c;   // a row without live entries sums to 0
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < SMV_CACHE; ++t) {
            if (lane + LPR * t < nvec) {
#pragma unroll
                for (int i = 0; i < VE; ++i) {
                    const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(cache[t][i], c, nb));
                    cache[t][i] = HAS_MASK ? (on(live[t], i) ? e : 0.f) : e;
                    sum += cache[t][i];
                }
            }
        }
        for (int v = lane + LPR * SMV_CACHE; v < nvec; v += LPR) {
            const int64_t off = vector_offset<VE>(p, rv, v, log_vpb);
            const mask_t m = mask_at(off);
            float f[VE];
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(x + off), f);
#pragma unroll
            for (int i = 0; i < VE; ++i)
                if (on(m, i)) sum += __builtin_amdgcn_exp2f(__builtin_fmaf(f[i], c, nb));
        }
        sum = group_reduce_sum<LPR>(sum);
        const float inv = sum > 0.f ? 1.f / sum : 0.f;
#pragma unroll
        for (int t = 0; t < SMV_CACHE; ++t) {
            if (lane + LPR * t < nvec) {
#pragma unroll
                for (int i = 0; i < VE; ++i) cache[t][i] *= inv;
                store16_stream(out + offs[t], SmVec<T>::pack(cache[t]));
            }
        }
        for (int v = lane + LPR * SMV_CACHE; v < nvec; v += LPR) {
            const int64_t off = vector_offset<VE>(p, rv, v, log_vpb);
            const mask_t m = mask_at(off);
            float f[VE];
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(x + off), f);
#pragma unroll
            for (int i = 0; i < VE; ++i)
                f[i] = on(m, i) ? __builtin_amdgcn_exp2f(__builtin_fmaf(f[i], c, nb)) * inv : 0.f;
            *reinterpret_cast<vec16*>(out + off) = SmVec<T>::pack(f);
        }
    } else {
        // cache holds grad_y, ycache holds y; grad_x = inv_t * y * (grad_y - sum(y * grad_y))
        float dot = 0.f;
#pragma unroll
        for (int t = 0; t < SMV_CACHE; ++t) {
            if (lane + LPR * t < nvec) {
#pragma unroll
                for (int i = 0; i < VE; ++i) {
                    if constexpr (HAS_MASK) ycache[t][i] = on(live[t], i) ? ycache[t][i] : 0.f;
                    cache[t][i] = ycache[t][i] * cache[t][i];
                    if constexpr (HAS_MASK) cache[t][i] = on(live[t], i) ? cache[t][i] : 0.f;
                    dot += cache[t][i];
                }
            }
        }
        for (int v = lane + LPR * SMV_CACHE; v < nvec; v += LPR) {
            const int64_t off = vector_offset<VE>(p, rv, v, log_vpb);
            const mask_t m = mask_at(off);
            float g[VE], yv[VE];
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(x + off), g);
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(yin + off), yv);
#pragma unroll
            for (int i = 0; i < VE; ++i)
                if (on(m, i)) dot += yv[i] * g[i];
        }
        dot = group_reduce_sum<LPR>(dot);
#pragma unroll
        for (int t = 0; t < SMV_CACHE; ++t) {
            if (lane + LPR * t < nvec) {
#pragma unroll
                for (int i = 0; i < VE; ++i) cache[t][i] = p.inv_t * (cache[t][i] - ycache[t][i] * dot);
                store16_stream(out + offs[t], SmVec<T>::pack(cache[t]));
            }
        }
        for (int v = lane + LPR * SMV_CACHE; v < nvec; v += LPR) {
            const int64_t off = vector_offset<VE>(p, rv, v, log_vpb);
            const mask_t m = mask_at(off);
            float g[VE], yv[VE];
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(x + off), g);
            SmVec<T>::unpack(*reinterpret_cast<const vec16*>(yin + off), yv);
#pragma unroll
            for (int i = 0; i < VE; ++i)
                g[i] = on(m, i) ? p.inv_t * (yv[i] * g[i] - yv[i] * dot) : 0.f;
            *reinterpret_cast<vec16*>(out + off) = SmVec<T>::pack(g);
        }
    }
}

template <bool BACKWARD>
static int launch_softmax(int dtype, int compressed, const void* x, const void* y_in, void* out,
                          const int32_t* row_ptr, const int32_t* bcsr_idx, const uint8_t* mask,
                          float inv_t, int batch, int H, int W, int BH, int BW,
                          int64_t batch_stride, int tile_cfg, hipStream_t st) {
    SPX_REQUIRE(x && out && row_ptr && bcsr_idx, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(tile_cfg >= 0 && tile_cfg <= 3, SPX_E_CONFIG, "unknown tile config %d", tile_cfg);
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
    // tile_cfg 0: pick; 1: one entry per access; 2: 16-byte accesses, a wavefront per row;
    // 3: 16-byte accesses, sixteen lanes per row (best when rows hold at most
    // 16 * SMV_CACHE vectors of live entries; longer rows stay correct).  The live length of
    // a row is only known on the device, so the default goes by the full width.
    const int ve = dtype == SPX_F32 ? 4 : 8;
    const bool vec_ok = BW % ve == 0 && aligned(x, 16) && aligned(out, 16) && (!y_in || aligned(y_in, 16)) &&
                        (!mask || aligned(mask, 8)) && batch_stride % ve == 0;
    // Few long rows (under 8192 in all, 256 vectors wide or more) also take a wavefront each:
    // sixteen-lane groups would leave most of the device without work (3072 rows of 4096:
    // 3.7 against 5.8 us forward, 3.8 against 6.7 us backward).
    const bool few_long_rows = (int64_t)H * batch < 8192 && W / ve >= 256;
    if (tile_cfg == 0) tile_cfg = vec_ok ? (W / ve <= 16 * SMV_CACHE && !few_long_rows ? 3 : 2) : 1;
    if (tile_cfg >= 2) {
        SPX_REQUIRE(vec_ok, SPX_E_CONFIG, "tile configs 2 and 3 need BW %% %d == 0 and 16-byte aligned tensors", ve);
        const bool narrow = tile_cfg == 3;
        const int rows_per_group = SMV_ROWS * (narrow ? 4 : 1);
        dim3 vgrid((H + rows_per_group - 1) / rows_per_group, batch, 1);
        dim3 vblock(64 * SMV_ROWS);
#define SPX_SMV(T) \
        if (narrow && mask) hipLaunchKernelGGL((softmax_vec_kernel<T, BACKWARD, 16, true>), vgrid, vblock, 0, st, p); \
        else if (narrow) hipLaunchKernelGGL((softmax_vec_kernel<T, BACKWARD, 16, false>), vgrid, vblock, 0, st, p); \
        else if (mask) hipLaunchKernelGGL((softmax_vec_kernel<T, BACKWARD, 64, true>), vgrid, vblock, 0, st, p); \
        else hipLaunchKernelGGL((softmax_vec_kernel<T, BACKWARD, 64, false>), vgrid, vblock, 0, st, p);
        switch (dtype) {
            case SPX_F32: SPX_SMV(float) break;
            case SPX_F16: SPX_SMV(_Float16) break;
            default: SPX_SMV(bf16_t) break;
        }
#undef SPX_SMV
        SPX_LAUNCH_CHECK("softmax_vec_kernel");
        return 0;
    }
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
    return spx::launch_softmax<false>(dtype, compressed, x, nullptr, y, row_ptr, bcsr_idx, mask,
                                      inv_temperature, batch, H, W, BH, BW, batch_stride, tile_cfg,
                                      reinterpret_cast<hipStream_t>(stream));
}

extern "C" int spx_softmax_backward(int dtype, int compressed, const void* grad_y, const void* y,
                                    void* grad_x, const int32_t* row_ptr, const int32_t* bcsr_idx,
                                    const uint8_t* mask, float inv_temperature,
                                    int batch, int H, int W, int BH, int BW,
                                    int64_t batch_stride, int tile_cfg, spx_stream_t stream) {
    return spx::launch_softmax<true>(dtype, compressed, grad_y, y, grad_x, row_ptr, bcsr_idx, mask,
                                     inv_temperature, batch, H, W, BH, BW, batch_stride, tile_cfg,
                                     reinterpret_cast<hipStream_t>(stream));
}
