// Sparse-operand matmul for small dense operands (few rows): K-split panel kernel.
//
// Same canonical problem and per-step data path as matmul_spmm_panel.hpp
// (out[m,n] = sum_k D[m,k] S[k,n], k-contiguous operands, one step = 64 bytes of k of
// one live block, coalesced loads -> registers -> private swizzled LDS -> MFMA), but a
// workgroup owns ONE 64 x BN output tile and its four wavefronts split the live blocks of
// the block-column between them (wavefront w takes steps w, w+4, w+8, ...).  With few
// rows there are few tiles, so the walk over a long block-column is what bounds the
// time: splitting it four ways shortens that chain of dependent loads fourfold and
// gives the chip four times as many workgroups.  The partial sums meet in LDS.
#pragma once
#include "matmul_spmm_panel.hpp"

namespace spx {

template <typename T, int BN, int BK, bool SWAP>
__global__ __launch_bounds__(256) void spmm_ksplit_kernel(SpmmParams p, int n_mtiles) {
    typedef typename PanelMma<T>::M MMA;
    typedef typename MMA::frag Frag;
    constexpr int KC = PanelMma<T>::KC;
    constexpr int CH = BK / KC;          // steps per block
    constexpr int NT = BN / 16;
    constexpr int WL = BN / 16;          // 16-byte loads per lane for the S rows
    constexpr int ROWS = 64 + BN;        // private LDS rows (64 bytes each) per wave
    constexpr int E16 = 16 / (int)sizeof(T);
    constexpr int PB = BN + 4;           // pitch of a partial-sum row (floats)
    constexpr int STAGE_BYTES = 4 * ROWS * 64;
    constexpr int PART_BYTES = 4 * 64 * PB * 4;
    static_assert(BK % KC == 0, "block depth must be a multiple of the step");
    __shared__ __align__(16) char lds_all[STAGE_BYTES > PART_BYTES ? STAGE_BYTES : PART_BYTES];

    const int nb = p.Nc / BN;
    const int L = blockIdx.x;
    const int xcd = L % kPanelXcd;
    const int seq = L / kPanelXcd;
    const int mt = (seq / nb) * kPanelXcd + xcd;   // 64-row tile; neighbours in m share an XCD's L2
    const int j = p.sched ? p.sched[seq % nb] : seq % nb;
    if (mt >= n_mtiles) return;
    const int64_t b = blockIdx.y;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int m0 = mt * 64;
    char* lds = lds_all + wave * (ROWS * 64);

    const T* D = reinterpret_cast<const T*>(p.D) + b * p.d_batch;
    const T* S = reinterpret_cast<const T*>(p.S) + b * p.s_batch;

    const int lrow = lane >> 2;
    const int lchk = lane & 3;
    const T* dptr[4];
    int wofs[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int row = q * 16 + lrow;
        int m = m0 + row;
        if (m >= p.Mc) m = p.Mc - 1;  // rows past the end re-read the last row; never stored
        dptr[q] = D + (int64_t)m * p.d_ld + lchk * E16;
        wofs[q] = row * 64 + ((lchk ^ ((row >> 2) & 3)) << 4);
    }
    int sofs[WL];
#pragma unroll
    for (int q = 0; q < WL; ++q) {
        const int row = 64 + q * 16 + lrow;
        sofs[q] = row * 64 + ((lchk ^ ((row >> 2) & 3)) << 4);
    }
    int aofs[4], bofs[NT];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = i * 16 + r16;
        aofs[i] = row * 64 + ((g4 ^ ((row >> 2) & 3)) << 4);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int row = 64 + t * 16 + r16;
        bofs[t] = row * 64 + ((g4 ^ ((row >> 2) & 3)) << 4);
    }

    f32x4 acc[4][NT];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int e_begin = p.ptr[j];
    const int n_blk = p.ptr[j + 1] - e_begin;
    const int n_it = n_blk * CH;
    const int n_loc = n_it > wave ? (n_it - wave + 3) >> 2 : 0;   // steps of this wavefront
    const int64_t sld = p.compressed ? BK : p.s_ld;

    int kb_vec = 0, slot_vec = 0;   // index entries 0..63 of the block-column, one per lane
    if (lane < n_blk) {
        if (p.idx_kind == SPX_IDX_BCSC_I64) {
            const long long v = reinterpret_cast<const long long*>(p.idx)[e_begin + lane];
            kb_vec = (int)(v & 0xffff);
            slot_vec = (int)(v >> 32);
        } else {
            kb_vec = reinterpret_cast<const int32_t*>(p.idx)[e_begin + lane] & 0xffff;
            slot_vec = e_begin + lane;
        }
    }

    u32x4 d0[4], s0[WL], d1[4], s1[WL];

// LT: local step of this wavefront; the step of the block-column is wave + 4 * LT.
#define SPX_KS_ISSUE(LT, DREG, SREG)                                                               \
    do {                                                                                           \
        const int it_ = wave + 4 * (LT);                                                           \
        const int er_ = it_ / CH;                                                                  \
        const int ch_ = it_ % CH;                                                                  \
        int kb_;                                                                                   \
        int64_t slot_;                                                                             \
        if (er_ < 64) {                                                                            \
            kb_ = __builtin_amdgcn_readlane(kb_vec, er_);                                          \
            slot_ = __builtin_amdgcn_readlane(slot_vec, er_);                                      \
        } else if (p.idx_kind == SPX_IDX_BCSC_I64) {                                               \
            const long long v_ = reinterpret_cast<const long long*>(p.idx)[e_begin + er_];         \
            kb_ = (int)(v_ & 0xffff);                                                              \
            slot_ = v_ >> 32;                                                                      \
        } else {                                                                                   \
            kb_ = reinterpret_cast<const int32_t*>(p.idx)[e_begin + er_] & 0xffff;                 \
            slot_ = e_begin + er_;                                                                 \
        }                                                                                          \
        const int koff_ = kb_ * BK + ch_ * KC;                                                     \
        const T* sblk_ = p.compressed ? S + slot_ * (int64_t)(BK * BN) + ch_ * KC                  \
                                      : S + (int64_t)j * BN * p.s_ld + koff_;                      \
        _Pragma("unroll") for (int q = 0; q < 4; ++q)                                              \
            DREG[q] = *reinterpret_cast<const u32x4*>(dptr[q] + koff_);                            \
        _Pragma("unroll") for (int q = 0; q < WL; ++q)                                             \
            SREG[q] = *reinterpret_cast<const u32x4*>(sblk_ + (int64_t)(q * 16 + lrow) * sld + lchk * E16); \
    } while (0)

// Loads and LDS writes are unconditional (steps past the end re-load the last one and are
// not accumulated), so every wait covers the oldest stage only.
#define SPX_KS_STEP(LT, DREG, SREG)                                                                \
    do {                                                                                           \
        _Pragma("unroll") for (int q = 0; q < 4; ++q)                                              \
            *reinterpret_cast<u32x4*>(lds + wofs[q]) = DREG[q];                                    \
        _Pragma("unroll") for (int q = 0; q < WL; ++q)                                             \
            *reinterpret_cast<u32x4*>(lds + sofs[q]) = SREG[q];                                    \
        {                                                                                          \
            const int nx_ = (LT) + 2 < n_loc ? (LT) + 2 : n_loc - 1;                               \
            SPX_KS_ISSUE(nx_, DREG, SREG);                                                         \
        }                                                                                          \
        if ((LT) < n_loc) {                                                                        \
            Frag af_[4], bf_[NT];                                                                  \
            _Pragma("unroll") for (int i = 0; i < 4; ++i)                                          \
                af_[i] = *reinterpret_cast<const Frag*>(lds + aofs[i]);                            \
            _Pragma("unroll") for (int t = 0; t < NT; ++t)                                         \
                bf_[t] = *reinterpret_cast<const Frag*>(lds + bofs[t]);                            \
            _Pragma("unroll") for (int i = 0; i < 4; ++i)                                          \
                _Pragma("unroll") for (int t = 0; t < NT; ++t)                                     \
                    acc[i][t] = SWAP ? MMA::mma(bf_[t], af_[i], acc[i][t])                         \
                                     : MMA::mma(af_[i], bf_[t], acc[i][t]);                        \
        }                                                                                          \
    } while (0)

    if (n_loc > 0) {
        SPX_KS_ISSUE(0, d0, s0);
        SPX_KS_ISSUE((1 < n_loc ? 1 : n_loc - 1), d1, s1);
        for (int lt = 0; lt < n_loc; lt += 2) {
            SPX_KS_STEP(lt, d0, s0);
            SPX_KS_STEP(lt + 1, d1, s1);
        }
    }
#undef SPX_KS_ISSUE
#undef SPX_KS_STEP

    // ---- partial sums meet in LDS as P[wave][m][n] (fp32) ----------------------------------
    __syncthreads();   // every wavefront is done with its staging region
    float* P = reinterpret_cast<float*>(lds_all);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if constexpr (SWAP) {
                // lane holds out[m = i*16 + r16][n = t*16 + g4*4 + q]
                *reinterpret_cast<f32x4*>(P + (wave * 64 + i * 16 + r16) * PB + t * 16 + g4 * 4) = acc[i][t];
            } else {
                // lane holds out[m = i*16 + g4*4 + q][n = t*16 + r16]
#pragma unroll
                for (int q = 0; q < 4; ++q) P[(wave * 64 + i * 16 + g4 * 4 + q) * PB + t * 16 + r16] = acc[i][t][q];
            }
        }
    __syncthreads();

    // ---- wavefront w finishes rows 16w .. 16w+15 of the tile: sum, bias, store ------------
    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + b * p.o_batch;
    constexpr int EPL = 16 * BN / 64;   // elements per lane: 4, 8 or 16
    if constexpr (SWAP) {
        // out[m][n], n contiguous: a lane owns EPL consecutive n of one row
        const int row = wave * 16 + (lane * EPL) / BN;
        const int col = (lane * EPL) % BN;
        const int m = m0 + row;
        float v[EPL];
#pragma unroll
        for (int e = 0; e < EPL; e += 4) {
            f32x4 sum = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < 4; ++w) sum += *reinterpret_cast<const f32x4*>(P + (w * 64 + row) * PB + col + e);
            v[e] = sum[0]; v[e + 1] = sum[1]; v[e + 2] = sum[2]; v[e + 3] = sum[3];
        }
        if (m < p.Mc) {
            T vals[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                float x = v[e];
                if (biasT) x += Elem<T>::to_float(biasT[p.bias_on_m ? m : j * BN + col + e]);
                vals[e] = Elem<T>::from_float(epilogue_act(x, p.relu));
            }
            T* dst = out + (int64_t)m * p.o_ld + (int64_t)j * BN + col;
#pragma unroll
            for (int e = 0; e < EPL; e += 4) {
                if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst + e) = *reinterpret_cast<const uint64_t*>(vals + e);
                else *reinterpret_cast<u32x4*>(dst + e) = *reinterpret_cast<const u32x4*>(vals + e);
            }
        }
    } else {
        // out[n][m], m contiguous: a lane owns 4 consecutive m of one column, EPL / 4 columns
#pragma unroll
        for (int e = 0; e < EPL; e += 4) {
            const int item = lane * (EPL / 4) + e / 4;   // (column, group of 4 rows) of this wave's 16 rows
            const int n = item >> 2;
            const int row = wave * 16 + (item & 3) * 4;
            T vals[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float x = 0.f;
#pragma unroll
                for (int w = 0; w < 4; ++w) x += P[(w * 64 + row + q) * PB + n];
                const int m = m0 + row + q;
                if (biasT) x += Elem<T>::to_float(biasT[p.bias_on_m ? (m < p.Mc ? m : 0) : j * BN + n]);
                vals[q] = Elem<T>::from_float(epilogue_act(x, p.relu));
            }
            T* dst = out + ((int64_t)j * BN + n) * p.o_ld + m0 + row;
            if (m0 + row + 4 <= p.Mc) {
                if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(vals);
                else *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(vals);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (m0 + row + q < p.Mc) dst[q] = vals[q];
            }
        }
    }
}

template <typename T, int BN, int BK, bool SWAP>
static int launch_spmm_ksplit_inst(const SpmmParams& p, int batch, hipStream_t st) {
    const int n_mtiles = (p.Mc + 63) / 64;
    const int nb = p.Nc / BN;
    const int64_t groups = (n_mtiles + kPanelXcd - 1) / kPanelXcd;
    const int64_t nblocks = groups * kPanelXcd * nb;
    if (nblocks > 0x7fffffffLL) return fail(SPX_E_SHAPE, "problem too large for one launch");
    hipLaunchKernelGGL((spmm_ksplit_kernel<T, BN, BK, SWAP>), dim3((unsigned)nblocks, batch, 1), dim3(256), 0, st,
                       p, n_mtiles);
    SPX_LAUNCH_CHECK("spmm_ksplit_kernel");
    return 0;
}

// Supported: what the panel kernel supports with BN in {16, 32} (the partial sums of a
// 64-wide tile would not fit the static LDS budget).
template <typename T>
bool spmm_ksplit_supported(int BN, int BK) {
    return spmm_panel_supported<T>(BN, BK) && BN <= 32;
}

template <typename T>
int launch_spmm_ksplit_impl(const SpmmParams& p, int BN, int batch, hipStream_t st) {
    const bool swap = p.out_ncontig != 0;
#define SPX_KS_CASE(bn, bk)                                                                     \
    if (BN == bn && p.BK == bk) {                                                               \
        if constexpr (bk % (64 / (int)sizeof(T)) == 0) {                                        \
            return swap ? launch_spmm_ksplit_inst<T, bn, bk, true>(p, batch, st)                \
                        : launch_spmm_ksplit_inst<T, bn, bk, false>(p, batch, st);              \
        }                                                                                       \
    }
    SPX_KS_CASE(16, 16) SPX_KS_CASE(16, 32) SPX_KS_CASE(16, 64)
    SPX_KS_CASE(32, 16) SPX_KS_CASE(32, 32) SPX_KS_CASE(32, 64)
#undef SPX_KS_CASE
    return fail(SPX_E_CONFIG, "block (%d,%d) not supported by the K-split kernel", p.BK, BN);
}

template <typename T>
int launch_spmm_ksplit(const SpmmParams& p, int BN, int batch, hipStream_t st);

}  // namespace spx
