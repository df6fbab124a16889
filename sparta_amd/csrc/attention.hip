// Fused block-sparse attention forward:
//   out = softmax_masked(q k^T * inv_temperature) v,  per batch*head,
// over the live (BH x BW) blocks of a BCSR index.  The score matrix never leaves
// the chip: for every live block of a block-row the workgroup computes the score
// tile, folds it into a running (max, sum) per query and accumulates P.V.
//
// Layout trick: scores are produced transposed, S^T = K Q^T, so that an MFMA
// accumulator lane (r = lane % 16, g = lane / 16) holds, for query r, the four
// consecutive keys g*4 .. g*4+3 of a 16-key tile.  That is exactly the B-operand
// layout of a 16x16x16 MFMA, so exp(S^T) feeds  O^T += V^T P^T  straight from
// registers, and every value a lane owns (scores, running max/sum, output
// accumulators) belongs to one query.  K tiles are staged in LDS as [key][e],
// V tiles transposed as [e][key]; each wavefront owns 16 queries.
//
// There is no counterpart kernel in the reference, whose SparseAttention.forward
// (sparta/specializer/operators/sparse_attention.py:76-80) runs three launches
// with two compressed intermediates in HBM; the result matches
// sparse_multi_head_attention_reference (sparta/testing/math.py:53-79).
#include "common.hpp"
#include "mma.hpp"

namespace spx {

struct AttnParams {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    const int32_t* row_ptr;
    const int32_t* bcsr_idx;
    const uint8_t* mask;  // [Nt, Ns] or NULL
    float inv_t;
    int Nt, Ns, BH;
};

template <typename T> struct AttnMma;
template <> struct AttnMma<_Float16> {
    typedef f16x4 pfrag;
    __device__ static pfrag pack(float a, float b, float c, float d) {
        return pfrag{(_Float16)a, (_Float16)b, (_Float16)c, (_Float16)d};
    }
};
template <> struct AttnMma<bf16_t> {
    typedef s16x4 pfrag;
    __device__ static pfrag pack(float a, float b, float c, float d) {
        return pfrag{(short)float_to_bf16(a), (short)float_to_bf16(b), (short)float_to_bf16(c),
                     (short)float_to_bf16(d)};
    }
};

// BW keys per block, E head dimension; BH = 16 * (waves per workgroup).
template <typename T, int BW, int E>
__global__ __launch_bounds__(512) void attention_kernel(AttnParams p) {
    constexpr int KT = BW / 16;     // key tiles per block
    constexpr int ET = E / 16;      // output (e) tiles
    constexpr int EC = E / 32;      // 32-wide chunks of the QK^T contraction
    constexpr int LDK = E + 8;      // K tile row pitch (elements): 16 bytes of padding
    constexpr int LDV = BW + 8;     // V^T tile row pitch
    typedef typename Mma32<T>::frag QFrag;
    typedef typename AttnMma<T>::pfrag PFrag;
    extern __shared__ __align__(16) char smem[];
    T* Ks = reinterpret_cast<T*>(smem);        // [BW][LDK]
    T* Vt = Ks + BW * LDK;                     // [E][LDV]

    const int br = blockIdx.x;
    const int64_t b = blockIdx.y;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int nthreads = blockDim.x;

    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E;
    T* O = reinterpret_cast<T*>(p.out) + b * (int64_t)p.Nt * E;

    const int qrow = br * p.BH + wave * 16 + r16;  // the query this lane belongs to
    // Q fragments (B operand of S^T = K Q^T): query r16, e = c*32 + g4*8 .. +7
    QFrag qf[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) qf[c] = Mma32<T>::load(Q + (int64_t)qrow * E + c * 32 + g4 * 8);

    f32x4 oacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -1e30f, l_run = 0.f;

    const int e_begin = p.row_ptr[br];
    const int e_end = p.row_ptr[br + 1];
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    for (int e = e_begin; e < e_end; ++e) {
        const int bc = p.bcsr_idx[e] & 0xffff;
        const int key0 = bc * BW;
        __syncthreads();  // previous block's fragments are consumed
        // ---- stage K [key][e] ----------------------------------------------------------
        for (int v = threadIdx.x; v < BW * (E / 8); v += nthreads) {
            const int key = v / (E / 8), c = v % (E / 8);
            *reinterpret_cast<u32x4*>(Ks + key * LDK + c * 8) =
                *reinterpret_cast<const u32x4*>(Kg + (int64_t)(key0 + key) * E + c * 8);
        }
        // ---- stage V transposed [e][key]: a thread moves a 2-key x 8-e patch --------------
        for (int v = threadIdx.x; v < (BW / 2) * (E / 8); v += nthreads) {
            const int kp = v / (E / 8), c = v % (E / 8);
            union { u32x4 v4; uint16_t h[8]; } a, bb;
            a.v4 = *reinterpret_cast<const u32x4*>(Vg + (int64_t)(key0 + 2 * kp) * E + c * 8);
            bb.v4 = *reinterpret_cast<const u32x4*>(Vg + (int64_t)(key0 + 2 * kp + 1) * E + c * 8);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                *reinterpret_cast<uint32_t*>(Vt + (c * 8 + i) * LDV + 2 * kp) = (uint32_t)a.h[i] | ((uint32_t)bb.h[i] << 16);
        }
        __syncthreads();

        // ---- S^T tiles: keys x this wave's 16 queries ------------------------------------
        f32x4 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const QFrag kf = Mma32<T>::load(Ks + (kt * 16 + r16) * LDK + c * 32 + g4 * 8);
                s[kt] = Mma32<T>::mma(kf, qf[c], s[kt]);
            }
        }
        // lane holds s[kt][q] = score(query r16, key kt*16 + g4*4 + q)
        unsigned live[KT];
        float tmax = -1e30f;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            unsigned bits = 0x01010101u;
            if (p.mask)
                bits = *reinterpret_cast<const uint32_t*>(p.mask + (int64_t)qrow * p.Ns + key0 + kt * 16 + g4 * 4);
            live[kt] = bits;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if ((bits >> (8 * q)) & 0xffu) tmax = fmaxf(tmax, s[kt][q]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __expf((m_run - m_new) * p.inv_t);
        float psum = 0.f;
        PFrag pf[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            float pv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                pv[q] = ((live[kt] >> (8 * q)) & 0xffu) ? __expf((s[kt][q] - m_new) * p.inv_t) : 0.f;
                psum += pv[q];
            }
            pf[kt] = AttnMma<T>::pack(pv[0], pv[1], pv[2], pv[3]);
        }
        psum += __shfl_xor(psum, 16, 64);
        psum += __shfl_xor(psum, 32, 64);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // ---- O^T[e][query] = alpha * O^T + V^T P^T ----------------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
            oacc[t] *= alpha;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const typename Mma16<T>::frag vf = Mma16<T>::load(Vt + (t * 16 + r16) * LDV + kt * 16 + g4 * 4);
                oacc[t] = Mma16<T>::mma(vf, pf[kt], oacc[t]);
            }
        }
    }

    // lane holds O^T[e = t*16 + g4*4 + q][query r16]; rows with no live entry give 0
    const float inv_l = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(oacc[t][q] * inv_l);
        *reinterpret_cast<uint64_t*>(O + (int64_t)qrow * E + t * 16 + g4 * 4) = *reinterpret_cast<const uint64_t*>(vals);
    }
}

template <typename T, int BW, int E>
static int launch_attention_inst(const AttnParams& p, int batch, hipStream_t st) {
    const int waves = p.BH / 16;
    const size_t smem = ((size_t)BW * (E + 8) + (size_t)E * (BW + 8)) * sizeof(T);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel<T, BW, E>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel)");
    }
    hipLaunchKernelGGL((attention_kernel<T, BW, E>), dim3(p.Nt / p.BH, batch, 1), dim3(64 * waves), smem, st, p);
    SPX_LAUNCH_CHECK("attention_kernel");
    return 0;
}

template <typename T>
static int launch_attention(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTN_CASE(bw, e) \
    if (BW == bw && E == e) return launch_attention_inst<T, bw, e>(p, batch, st);
    SPX_ATTN_CASE(16, 32) SPX_ATTN_CASE(16, 64) SPX_ATTN_CASE(16, 128)
    SPX_ATTN_CASE(32, 32) SPX_ATTN_CASE(32, 64) SPX_ATTN_CASE(32, 128)
    SPX_ATTN_CASE(64, 32) SPX_ATTN_CASE(64, 64) SPX_ATTN_CASE(64, 128)
    SPX_ATTN_CASE(128, 32) SPX_ATTN_CASE(128, 64) SPX_ATTN_CASE(128, 128)
#undef SPX_ATTN_CASE
    return fail(SPX_E_CONFIG, "fused attention supports key blocks of 16/32/64/128 and head dims 32/64/128 (got %d, %d)", BW, E);
}

}  // namespace spx

extern "C" int spx_attention_forward(int dtype, const void* q, const void* k, const void* v, void* out,
                                     const int32_t* row_ptr, const int32_t* bcsr_idx,
                                     const uint8_t* mask, float inv_temperature,
                                     int batch, int Nt, int Ns, int E, int BH, int BW,
                                     int tile_cfg, spx_stream_t stream) {
    using namespace spx;
    (void)tile_cfg;
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(q && k && v && out && row_ptr && bcsr_idx, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(BH == 16 || BH == 32 || BH == 64 || BH == 128, SPX_E_CONFIG, "query block %d not in {16,32,64,128}", BH);
    SPX_REQUIRE(Nt > 0 && Ns > 0 && Nt % BH == 0 && BW > 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out, 16), SPX_E_ALIGN,
                "q, k, v, out must be 16-byte aligned");
    SPX_REQUIRE(!mask || (Ns % 4 == 0 && aligned(mask, 4)), SPX_E_ALIGN, "mask rows must be 4-byte aligned");
    if (batch == 0) return 0;
    AttnParams p;
    p.q = q; p.k = k; p.v = v; p.out = out;
    p.row_ptr = row_ptr; p.bcsr_idx = bcsr_idx; p.mask = mask;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SPX_F16) return launch_attention<_Float16>(p, batch, BW, E, st);
    return launch_attention<bf16_t>(p, batch, BW, E, st);
}
