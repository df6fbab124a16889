// Sparse-output matmul (the reference's 'dds' mode): one workgroup per live
// (BM x BN) output block, full-K inner product of a dense A panel and a dense B
// panel.  K is walked in stages of KT elements staged through LDS as [row][k];
// the four wavefronts split the block's 16x16 MFMA tiles when it has at least
// four of them, otherwise they split each stage along k and the partial sums
// meet in LDS.  Dead blocks are never touched.
#pragma once
#include "common.hpp"
#include "mma.hpp"

namespace spx {

struct DdsParams {
    const void* A;
    const void* B;
    const void* bias;
    void* C;
    const int32_t* idx;      // BCSR_idx (row<<16 | col), one entry per live block
    const int32_t* nnz_dev;  // optional: blocks >= *nnz_dev are skipped
    int M, K, N;
    int a_kcontig;           // A[m*a_ld + k] if set, else A[k*a_ld + m]
    int64_t a_ld;
    int b_kcontig;           // B[n*b_ld + k] if set, else B[k*b_ld + n]
    int64_t b_ld;
    int compressed;          // C block i at i*BM*BN, else at its place in [M,N]
    int64_t a_batch, b_batch, c_batch, bias_batch;
};

template <int MT, int NT> struct DdsWaveGrid {
    static constexpr int TILES = MT * NT;
    static constexpr bool KSPLIT = TILES < 4;
    static constexpr int WGM = KSPLIT ? MT : (MT >= 2 && NT >= 2 ? 2 : (MT >= 4 ? 4 : 1));
    static constexpr int WGN = KSPLIT ? NT : 4 / WGM;
    static constexpr int KS = KSPLIT ? 4 / TILES : 1;  // k-split factor
    static constexpr int WTM = MT / WGM;               // tiles per wave along m
    static constexpr int WTN = NT / WGN;
};

template <typename T, int BM, int BN>
__global__ __launch_bounds__(256) void dds_kernel(DdsParams p) {
    constexpr int MT = BM / 16, NT = BN / 16;
    typedef DdsWaveGrid<MT, NT> G;
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int KT = sizeof(T) == 2 ? 128 : 64;  // k per stage
    constexpr int LOG_KT = sizeof(T) == 2 ? 7 : 6;
    constexpr int LDK = KT + VE;
    constexpr int KW = KT / G::KS;                  // k per wave per stage
    extern __shared__ __align__(16) char smem[];
    T* As = reinterpret_cast<T*>(smem);
    T* Bs = As + BM * LDK;

    const int i = blockIdx.x;
    if (p.nnz_dev && i >= p.nnz_dev[0]) return;
    const int code = p.idx[i];
    const int bi = (code >> 16) & 0xffff;
    const int bj = code & 0xffff;
    const int64_t b = blockIdx.y;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;

    // wave -> (tile row group, tile col group, k part)
    const int wt = wave % (G::WGM * G::WGN);
    const int kpart = wave / (G::WGM * G::WGN);
    const int wgm = wt / G::WGN;
    const int wgn = wt % G::WGN;

    const T* A = reinterpret_cast<const T*>(p.A) + b * p.a_batch;
    const T* B = reinterpret_cast<const T*>(p.B) + b * p.b_batch;

    f32x4 acc[G::WTM][G::WTN];
#pragma unroll
    for (int x = 0; x < G::WTM; ++x)
#pragma unroll
        for (int y = 0; y < G::WTN; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < p.K; k0 += KT) {
        // K is a multiple of 16; a short last stage is zero-filled.
        const int kvalid = p.K - k0 < KT ? p.K - k0 : KT;
        const T* asrc = p.a_kcontig ? A + (int64_t)bi * BM * p.a_ld + k0 : A + (int64_t)k0 * p.a_ld + (int64_t)bi * BM;
        const T* bsrc = p.b_kcontig ? B + (int64_t)bj * BN * p.b_ld + k0 : B + (int64_t)k0 * p.b_ld + (int64_t)bj * BN;
        if (kvalid == KT) {
            stage_tile<T, BM, 256>(As, LDK, KT, LOG_KT, asrc, p.a_ld, p.a_kcontig != 0, BM);
            stage_tile<T, BN, 256>(Bs, LDK, KT, LOG_KT, bsrc, p.b_ld, p.b_kcontig != 0, BN);
        } else {
            // tail: stage 16-wide k slices, zero the rest
            for (int v = threadIdx.x; v < (BM + BN) * (KT / VE); v += 256) {
                const int row = v / (KT / VE);
                const int cv = v - row * (KT / VE);
                if (cv * VE >= kvalid) *reinterpret_cast<vec16*>((row < BM ? As + row * LDK : Bs + (row - BM) * LDK) + cv * VE) = vec16{0u, 0u, 0u, 0u};
            }
            for (int ks = 0; ks < kvalid; ks += 16) {
                stage_tile<T, BM, 256>(As + ks, LDK, 16, 4, p.a_kcontig ? asrc + ks : asrc + (int64_t)ks * p.a_ld, p.a_ld, p.a_kcontig != 0, BM);
                stage_tile<T, BN, 256>(Bs + ks, LDK, 16, 4, p.b_kcontig ? bsrc + ks : bsrc + (int64_t)ks * p.b_ld, p.b_ld, p.b_kcontig != 0, BN);
            }
        }
        __syncthreads();
        const T* a_base = As + (wgm * G::WTM * 16 + r16) * LDK + kpart * KW;
        const T* b_base = Bs + (wgn * G::WTN * 16 + r16) * LDK + kpart * KW;
        if constexpr (HasMma32<T>::value) {
            for (int kc = 0; kc < KW; kc += 32) {
                typename Mma32<T>::frag af[G::WTM], bf[G::WTN];
#pragma unroll
                for (int x = 0; x < G::WTM; ++x) af[x] = Mma32<T>::load(a_base + x * 16 * LDK + kc + g4 * 8);
#pragma unroll
                for (int y = 0; y < G::WTN; ++y) bf[y] = Mma32<T>::load(b_base + y * 16 * LDK + kc + g4 * 8);
#pragma unroll
                for (int x = 0; x < G::WTM; ++x)
#pragma unroll
                    for (int y = 0; y < G::WTN; ++y) acc[x][y] = Mma32<T>::mma(af[x], bf[y], acc[x][y]);
            }
        } else {
            for (int kc = 0; kc < KW; kc += 16) {
                typename Mma16<T>::frag af[G::WTM], bf[G::WTN];
#pragma unroll
                for (int x = 0; x < G::WTM; ++x) af[x] = Mma16<T>::load(a_base + x * 16 * LDK + kc + g4 * 4);
#pragma unroll
                for (int y = 0; y < G::WTN; ++y) bf[y] = Mma16<T>::load(b_base + y * 16 * LDK + kc + g4 * 4);
#pragma unroll
                for (int x = 0; x < G::WTM; ++x)
#pragma unroll
                    for (int y = 0; y < G::WTN; ++y) acc[x][y] = Mma16<T>::mma(af[x], bf[y], acc[x][y]);
            }
        }
        __syncthreads();
    }

    // ---- epilogue: partial sums -> LDS fp32 -> sum over k parts, bias, store ----
    constexpr int LDE = BN + 1;
    float* Ef = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int x = 0; x < G::WTM; ++x)
#pragma unroll
        for (int y = 0; y < G::WTN; ++y)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = (wgm * G::WTM + x) * 16 + g4 * 4 + q;
                const int n = (wgn * G::WTN + y) * 16 + r16;
                Ef[(kpart * BM + m) * LDE + n] = acc[x][y][q];
            }
    __syncthreads();
    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* C = reinterpret_cast<T*>(p.C) + b * p.c_batch;
    for (int v = threadIdx.x; v < BM * BN; v += 256) {
        const int m = v / BN;
        const int n = v - m * BN;
        float s = 0.f;
#pragma unroll
        for (int kp = 0; kp < G::KS; ++kp) s += Ef[(kp * BM + m) * LDE + n];
        if (biasT) s += Elem<T>::to_float(biasT[bj * BN + n]);
        const int64_t off = p.compressed ? (int64_t)i * (BM * BN) + v
                                         : ((int64_t)bi * BM + m) * p.N + (int64_t)bj * BN + n;
        C[off] = Elem<T>::from_float(s);
    }
}

template <typename T, int BM, int BN>
static int launch_dds_inst(const DdsParams& p, int nnz_bound, int batch, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int KT = sizeof(T) == 2 ? 128 : 64;
    typedef DdsWaveGrid<BM / 16, BN / 16> G;
    size_t smem = (size_t)(BM + BN) * (KT + VE) * sizeof(T);
    size_t epi = (size_t)G::KS * BM * (BN + 1) * sizeof(float);
    if (epi > smem) smem = epi;
    hipLaunchKernelGGL((dds_kernel<T, BM, BN>), dim3(nnz_bound, batch, 1), dim3(256), smem, st, p);
    SPX_LAUNCH_CHECK("dds_kernel");
    return 0;
}

template <typename T>
int launch_dds_impl(const DdsParams& p, int BM, int BN, int nnz_bound, int batch, hipStream_t st) {
#define SPX_DDS_CASE(bm, bn) \
    if (BM == bm && BN == bn) return launch_dds_inst<T, bm, bn>(p, nnz_bound, batch, st);
    SPX_DDS_CASE(16, 16) SPX_DDS_CASE(16, 32) SPX_DDS_CASE(16, 64)
    SPX_DDS_CASE(32, 16) SPX_DDS_CASE(32, 32) SPX_DDS_CASE(32, 64)
    SPX_DDS_CASE(64, 16) SPX_DDS_CASE(64, 32) SPX_DDS_CASE(64, 64)
#undef SPX_DDS_CASE
    return fail(SPX_E_CONFIG, "output block (%d,%d) not in {16,32,64}^2", BM, BN);
}

template <typename T>
int launch_dds(const DdsParams& p, int BM, int BN, int nnz_bound, int batch, int tile_cfg, hipStream_t st);

}  // namespace spx
