// Sparse-operand matmul, register-direct variant for k-contiguous operands
// (dense operand stored [rows, K], sparse blocks stored [n, k]): the layouts of
// SparseLinear(weight_mask) ('dsd', B stored [N,K]) and of its 'sdd' mirror.
//
// Same canonical problem as matmul_spmm.hpp: out[m, n] = sum_k D[m,k] S[k,n].
// Every wavefront owns a (16*WM) x BN output tile and reads its MFMA fragments
// straight from global memory: a fragment is 8 (16-bit) or 4 (fp32) consecutive
// k of one row, i.e. one 16-byte load per lane, already in MFMA operand layout.
// Rows of the dense panel are private to a wavefront, so there is nothing to
// share through LDS and no barrier in the loop; the next (block, k-chunk) is
// prefetched into a second register set while the current one feeds the MFMAs.
//
// Workgroups are numbered so that all tiles of one row panel of D run on the
// same XCD (workgroup L lands on XCD L % 8): the panel is then fetched into that
// XCD's L2 once and every live block of the panel's block-columns hits it.
#pragma once
#include <type_traits>
#include "matmul_spmm.hpp"

namespace spx {

template <typename T, int BK> struct DirectMma {
    static constexpr bool WIDE = sizeof(T) == 2 && BK >= 32;
    typedef typename std::conditional<WIDE, Mma32<typename std::conditional<sizeof(T) == 2, T, _Float16>::type>,
                                      Mma16<T>>::type M;
    static constexpr int KC = WIDE ? 32 : 16;  // k per chunk
    static constexpr int LK = KC / 4;          // consecutive k per lane
    static constexpr int CH = BK / KC;         // chunks per block
};

constexpr int kNumXcd = 8;

template <typename T, int BN, int BK, int WM, bool SWAP>
__global__ __launch_bounds__(256) void spmm_direct_kernel(SpmmParams p, int n_mtiles) {
    typedef DirectMma<T, BK> DM;
    typedef typename DM::M MMA;
    typedef typename MMA::frag Frag;
    constexpr int NT = BN / 16;
    constexpr int TM = 64 * WM;
    constexpr int CH = DM::CH, KC = DM::KC, LK = DM::LK;

    // XCD-aware numbering: L -> (xcd, sequence); a row panel stays on one XCD.
    const int nb = p.Nc / BN;
    const int L = blockIdx.x;
    const int xcd = L % kNumXcd;
    const int seq = L / kNumXcd;
    const int mt = (seq / nb) * kNumXcd + xcd;
    const int j = p.sched ? p.sched[seq % nb] : seq % nb;
    if (mt >= n_mtiles) return;
    const int64_t b = blockIdx.y;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int m0 = mt * TM + wave * 16 * WM;  // first row of this wavefront
    if (m0 >= p.Mc) return;                   // no barriers below: a wave may leave

    const T* D = reinterpret_cast<const T*>(p.D) + b * p.d_batch;
    const T* S = reinterpret_cast<const T*>(p.S) + b * p.s_batch;

    // per-lane row pointers of the dense panel (rows past the end re-read the last row)
    const T* drow[WM];
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        int m = m0 + i * 16 + r16;
        if (m >= p.Mc) m = p.Mc - 1;
        drow[i] = D + (int64_t)m * p.d_ld + g4 * LK;
    }

    f32x4 acc[WM][NT];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int e_begin = p.ptr[j];
    const int n_it = (p.ptr[j + 1] - e_begin) * CH;

    auto fetch = [&](int it, Frag (&af)[WM], Frag (&bf)[NT]) {
        const int e = e_begin + it / CH;
        const int ch = it % CH;
        int kb;
        int64_t slot;
        if (p.idx_kind == SPX_IDX_BCSC_I64) {
            const long long v = reinterpret_cast<const long long*>(p.idx)[e];
            kb = (int)(v & 0xffff);
            slot = v >> 32;
        } else {
            kb = reinterpret_cast<const int32_t*>(p.idx)[e] & 0xffff;
            slot = e;
        }
        const int koff = kb * BK + ch * KC;
        const T* sblk = p.compressed ? S + slot * (int64_t)(BK * BN) + ch * KC
                                     : S + (int64_t)j * BN * p.s_ld + koff;
        const int64_t sld = p.compressed ? BK : p.s_ld;
#pragma unroll
        for (int i = 0; i < WM; ++i) af[i] = MMA::load(drow[i] + koff);
#pragma unroll
        for (int t = 0; t < NT; ++t) bf[t] = MMA::load(sblk + (int64_t)(t * 16 + r16) * sld + g4 * LK);
    };
    auto mma_all = [&](Frag (&af)[WM], Frag (&bf)[NT]) {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int t = 0; t < NT; ++t)
                acc[i][t] = SWAP ? MMA::mma(bf[t], af[i], acc[i][t]) : MMA::mma(af[i], bf[t], acc[i][t]);
    };

    Frag a0[WM], b0[NT], a1[WM], b1[NT];
    if (n_it > 0) fetch(0, a0, b0);
    int it = 0;
    for (; it + 1 < n_it; it += 2) {
        fetch(it + 1, a1, b1);
        mma_all(a0, b0);
        if (it + 2 < n_it) fetch(it + 2, a0, b0);
        mma_all(a1, b1);
    }
    if (it < n_it) mma_all(a0, b0);

    // ---- epilogue: each lane holds 4 memory-contiguous outputs per tile ------------
    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + b * p.o_batch;
    // The lane's bias values are fetched together, ahead of the stores: loaded where they are
    // used, every tile's values wait for their own round trip (the compiler cannot move a
    // load across the stores of the tile before).  bias_m[i][q] / bias_n[t][q]: q is the
    // position inside the lane's four contiguous outputs when the bias runs along them.
    float bias_m[WM][4], bias_n[NT][4];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) bias_m[i][q] = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) bias_n[t][q] = 0.f;
    if (biasT) {
        if (p.bias_on_m) {
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int m = m0 + i * 16 + (SWAP ? r16 : g4 * 4 + q);
                    bias_m[i][q] = Elem<T>::to_float(biasT[m < p.Mc ? m : 0]);
                }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q) bias_n[t][q] = Elem<T>::to_float(biasT[j * BN + t * 16 + (SWAP ? g4 * 4 + q : r16)]);
        }
    }
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            // SWAP: acc[q] = out[m = i*16 + r16][n = t*16 + g4*4 + q]   (n contiguous)
            // else: acc[q] = out[m = i*16 + g4*4 + q][n = t*16 + r16]   (m contiguous)
            const int m = m0 + i * 16 + (SWAP ? r16 : g4 * 4);
            const int n = j * BN + t * 16 + (SWAP ? g4 * 4 : r16);
            if (m >= p.Mc) continue;
            T vals[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float v = acc[i][t][q] + bias_m[i][q] + bias_n[t][q];
                vals[q] = Elem<T>::from_float(epilogue_act(v, p.relu));
            }
            T* dst = SWAP ? out + (int64_t)m * p.o_ld + n : out + (int64_t)n * p.o_ld + m;
            if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(vals);
            else *reinterpret_cast<vec16*>(dst) = *reinterpret_cast<const vec16*>(vals);
        }
}

template <typename T, int BN, int BK, int WM, bool SWAP>
static int launch_spmm_direct_inst(const SpmmParams& p, int batch, hipStream_t st) {
    constexpr int TM = 64 * WM;
    const int n_mtiles = (p.Mc + TM - 1) / TM;
    const int nb = p.Nc / BN;
    const int64_t groups = (n_mtiles + kNumXcd - 1) / kNumXcd;
    const int64_t nblocks = groups * kNumXcd * nb;
    if (nblocks > 0x7fffffffLL) return fail(SPX_E_SHAPE, "problem too large for one launch");
    hipLaunchKernelGGL((spmm_direct_kernel<T, BN, BK, WM, SWAP>), dim3((unsigned)nblocks, batch, 1), dim3(256), 0, st,
                       p, n_mtiles);
    SPX_LAUNCH_CHECK("spmm_direct_kernel");
    return 0;
}

template <typename T, int BN, int BK>
static int launch_spmm_direct_bnk(const SpmmParams& p, int batch, int wm, hipStream_t st) {
    const bool swap = p.out_ncontig != 0;
    if (wm == 4) {
        return swap ? launch_spmm_direct_inst<T, BN, BK, 4, true>(p, batch, st)
                    : launch_spmm_direct_inst<T, BN, BK, 4, false>(p, batch, st);
    }
    return swap ? launch_spmm_direct_inst<T, BN, BK, 1, true>(p, batch, st)
                : launch_spmm_direct_inst<T, BN, BK, 1, false>(p, batch, st);
}

// Requires p.d_kcontig && p.s_kcontig.  wm: 16-row tiles per wavefront (1 or 4).
template <typename T>
int launch_spmm_direct_impl(const SpmmParams& p, int BN, int batch, int wm, hipStream_t st) {
#define SPX_DIRECT_CASE(bn, bk) \
    if (BN == bn && p.BK == bk) return launch_spmm_direct_bnk<T, bn, bk>(p, batch, wm, st);
    SPX_DIRECT_CASE(16, 16) SPX_DIRECT_CASE(16, 32) SPX_DIRECT_CASE(16, 64)
    SPX_DIRECT_CASE(32, 16) SPX_DIRECT_CASE(32, 32) SPX_DIRECT_CASE(32, 64)
    SPX_DIRECT_CASE(64, 16) SPX_DIRECT_CASE(64, 32) SPX_DIRECT_CASE(64, 64)
#undef SPX_DIRECT_CASE
    return fail(SPX_E_CONFIG, "block (%d,%d) not in {16,32,64}^2", p.BK, BN);
}

template <typename T>
int launch_spmm_direct(const SpmmParams& p, int BN, int batch, int wm, hipStream_t st);

}  // namespace spx
