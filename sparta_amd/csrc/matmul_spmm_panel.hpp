// Sparse-operand matmul, panel variant for k-contiguous operands: the main kernel
// of SparseLinear(weight_mask) ('dsd', weight stored [N,K]) and of its 'sdd'
// mirror.  Canonical problem as in matmul_spmm.hpp: out[m,n] = sum_k D[m,k] S[k,n].
//
// Each wavefront owns a 64 x BN output tile and is fully independent (no
// workgroup barrier anywhere).  One pipeline step covers 64 bytes of k (32 x
// 16-bit or 16 x fp32) of one live block:
//   * global -> registers with a coalesced mapping: 4 consecutive lanes read the
//     64 contiguous bytes of one row, so a wave load touches 16 cache lines
//     instead of the 64 an MFMA-layout load would touch;
//   * registers -> private LDS (6 KB per wave) with an XOR swizzle, read back as
//     conflict-free 16-byte MFMA fragments (lane = row % 16, k group = lane / 16);
//   * NST register stages keep NST steps of loads in flight per wave.
// Workgroups are numbered so that all tiles of one 256-row panel of D run on
// one XCD and share its L2 (workgroup L is dispatched to XCD L % 8).
#pragma once
#include <type_traits>
#include "matmul_spmm.hpp"

namespace spx {

constexpr int kPanelXcd = 8;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct PanelMma {
    // one step = 64 bytes of k per row
    static constexpr bool WIDE = sizeof(T) == 2;
    typedef typename std::conditional<WIDE, Mma32<typename std::conditional<WIDE, T, _Float16>::type>,
                                      Mma16<typename std::conditional<WIDE, float, T>::type>>::type M;
    static constexpr int KC = 64 / (int)sizeof(T);  // k per step
};

// One MFMA fragment of the dense operand from the private LDS region: a plain 16-byte
// read of the [row][k] layout, or - for an operand kept as [k][m] - two transpose reads
// (16-bit: four k-rows each, 4 k-rows apart) / four 4-byte reads one k-row apart (fp32).
template <typename T, bool DT, typename Frag>
__device__ __forceinline__ Frag panel_dfrag(const char* at) {
    if constexpr (!DT) {
        return *reinterpret_cast<const Frag*>(at);
    } else if constexpr (sizeof(T) == 2) {
        typedef short s16x8_t __attribute__((ext_vector_type(8)));
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4_t;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(at));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(at + 4 * 128));
        return __builtin_bit_cast(Frag, (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    } else {
        Frag f;
#pragma unroll
        for (int j = 0; j < 4; ++j) f[j] = *reinterpret_cast<const float*>(at + j * 256);
        return f;
    }
}

// SHW: the S (sparse) block of a step is loaded once per workgroup - each of the four
// wavefronts fetches a quarter - into a double-buffered shared LDS tile, at the price
// of one workgroup barrier per step; otherwise every wavefront loads it privately.
// DT: the dense operand is stored with m contiguous (D[k * d_ld + m]).  A step then loads
// KC k-rows of 64 contiguous m per wavefront (fully coalesced), keeps them as [k][m] in
// the private LDS region and builds the k-contiguous MFMA fragments with the LDS transpose
// read of gfx950 (16-bit types) or 4-byte reads (fp32).
template <typename T, int BN, int BK, int NST, bool SWAP, bool SHW, bool DT = false>
__global__ __launch_bounds__(256, (BN <= 32 && NST == 2) ? 4 : 2) void spmm_panel_kernel(SpmmParams p, int n_mtiles) {
    typedef typename PanelMma<T>::M MMA;
    typedef typename MMA::frag Frag;
    constexpr int KC = PanelMma<T>::KC;
    constexpr int CH = BK / KC;          // steps per block
    constexpr int NT = BN / 16;
    constexpr int WL = SHW ? 1 : BN / 16;  // 16-byte loads per lane for the S rows
    constexpr int ROWS = SHW ? 80 : 64 + BN;  // private LDS rows (64 bytes each) per wave
    constexpr int SH_BYTES = SHW ? 2 * BN * 64 : 0;  // shared, double-buffered S tile
    constexpr int E16 = 16 / (int)sizeof(T);
    static_assert(BK % KC == 0, "block depth must be a multiple of the step");

    __shared__ __align__(16) char lds_all[4 * ROWS * 64 + SH_BYTES];

    const int nb = p.Nc / BN;
    const int L = blockIdx.x;
    const int xcd = L % kPanelXcd;
    const int seq = L / kPanelXcd;
    const int mt = (seq / nb) * kPanelXcd + xcd;
    const int j = p.sched ? p.sched[seq % nb] : seq % nb;
    if (mt >= n_mtiles) return;
    const int64_t b = blockIdx.y;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int m0 = mt * 256 + wave * 64;
    if (!SHW && m0 >= p.Mc) return;  // independent waves may leave early; with a shared S tile all four stay
    char* lds = lds_all + wave * (ROWS * 64);
    char* wsh = lds_all + 4 * ROWS * 64;

    const T* D = reinterpret_cast<const T*>(p.D) + b * p.d_batch;
    const T* S = reinterpret_cast<const T*>(p.S) + b * p.s_batch;

    // coalesced load mapping: lane -> (row within a 16-row group, 16-byte chunk)
    const int lrow = lane >> 2;
    const int lchk = lane & 3;
    const T* dptr[4];
    int wofs[4];  // LDS byte offsets of this lane's chunk for the 4 row groups of D
    constexpr int DT_CPR = 64 / E16;        // DT: 16-byte pieces per k-row of 64 m (8 or 16)
    constexpr int DT_RPL = 64 / DT_CPR;     // DT: k-rows covered by one wave load (8 or 4)
    constexpr int DT_PITCH = 64 * (int)sizeof(T);  // DT: bytes per k-row in LDS
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if constexpr (DT) {
            // lane -> (k-row lane / DT_CPR + DT_RPL q of the step, piece lane % DT_CPR of its 64 m)
            const int kr = lane / DT_CPR + DT_RPL * q;
            const int pc = lane % DT_CPR;
            int m = m0 + pc * E16;
            if (m >= p.Mc) m = 0;  // columns past the end re-read valid data; never stored
            dptr[q] = D + (int64_t)kr * p.d_ld + m;
            if constexpr (sizeof(T) == 2) {
                // 32-byte units (16 m) XOR-swizzled by bits 1 and 3 of the k-row
                const int f = ((kr >> 1) & 1) | (((kr >> 3) & 1) << 1);
                wofs[q] = kr * DT_PITCH + ((((pc >> 1) ^ f) & 3) << 5) + ((pc & 1) << 4);
            } else {
                // 64-byte units (16 m) XOR-swizzled by bits 2..3 of the k-row
                wofs[q] = kr * DT_PITCH + ((((pc >> 2) ^ (kr >> 2)) & 3) << 6) + ((pc & 3) << 4);
            }
        } else {
            const int row = q * 16 + lrow;
            int m = m0 + row;
            if (m >= p.Mc) m = p.Mc - 1;  // rows past the end re-read the last row; never stored
            dptr[q] = D + (int64_t)m * p.d_ld + lchk * E16;
            wofs[q] = row * 64 + ((lchk ^ ((row >> 2) & 3)) << 4);
        }
    }
    int sofs[WL];
    // shared S tile: this wave stages chunks wave*BN .. wave*BN+BN-1 of the BN*4 chunks.
    // k-contiguous S: chunk = (n row, 16-byte piece of its 64 bytes of k); otherwise S is
    // stored with n contiguous, a chunk is 16 bytes of n at one k and is transposed on
    // its way into LDS.
    const int sh_chunk = wave * BN + lane;
    const int sh_row = sh_chunk >> 2, sh_chk = sh_chunk & 3;
    const bool sh_active = lane < BN;
    const int sh_k = sh_chunk / (BN / E16), sh_n0 = (sh_chunk % (BN / E16)) * E16;
#pragma unroll
    for (int q = 0; q < WL; ++q) {
        if constexpr (SHW) {
            sofs[q] = sh_row * 64 + ((sh_chk ^ ((sh_row >> 2) & 3)) << 4);
        } else {
            const int row = 64 + q * 16 + lrow;
            sofs[q] = row * 64 + ((lchk ^ ((row >> 2) & 3)) << 4);
        }
    }
    // fragment read offsets (row = tile*16 + r16, chunk g4)
    int aofs[4], bofs[NT];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (DT && sizeof(T) == 2) {
            // transpose read: this lane addresses k-row g4*8 + r16/4 (and +4), m = i*16 + (r16%4)*4
            const int kr = g4 * 8 + (r16 >> 2);
            const int f = ((kr >> 1) & 1) | (((kr >> 3) & 1) << 1);
            aofs[i] = kr * DT_PITCH + (((i ^ f) & 3) << 5) + ((r16 & 3) << 3);
        } else if constexpr (DT) {
            // fp32: element (k = g4*4 + j, m = i*16 + r16); j adds DT_PITCH
            aofs[i] = (g4 * 4) * DT_PITCH + (((i ^ g4) & 3) << 6) + (r16 << 2);
        } else {
            const int row = i * 16 + r16;
            aofs[i] = row * 64 + ((g4 ^ ((row >> 2) & 3)) << 4);
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int row = (SHW ? 0 : 64) + t * 16 + r16;
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
    const int64_t sld = p.compressed ? (p.s_kcontig ? BK : BN) : p.s_ld;
    const int64_t sh_toff = p.s_kcontig ? (int64_t)sh_row * sld + sh_chk * E16 : (int64_t)sh_k * sld + sh_n0;

    // The first 64 index entries of the block-column live in one VGPR pair (lane l
    // holds entry l) and are broadcast with readlane, which keeps the index fetch
    // off the critical path of every step; longer columns fall back to scalar loads.
    int kb_vec = 0, slot_vec = 0;
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

    // Stage registers are separate named arrays (not an array of stages) so that
    // they stay in VGPRs.
    u32x4 d0[4], s0[WL], d1[4], s1[WL], d2[4], s2[WL];

#define SPX_PANEL_ISSUE(IT, LIVE, DREG, SREG)                                                          \
    do {                                                                                           \
        const int er_ = (IT) / CH;                                                                 \
        const int ch_ = (IT) % CH;                                                                 \
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
        const T* sblk_ = p.compressed ? S + slot_ * (int64_t)(BK * BN) + (p.s_kcontig ? ch_ * KC : ch_ * KC * BN) \
                                      : (p.s_kcontig ? S + (int64_t)j * BN * p.s_ld + koff_        \
                                                     : S + (int64_t)koff_ * p.s_ld + (int64_t)j * BN); \
        _Pragma("unroll") for (int q = 0; q < 4; ++q)                                              \
            DREG[q] = *reinterpret_cast<const u32x4*>((LIVE) ? dptr[q] + (DT ? (int64_t)koff_ * p.d_ld : (int64_t)koff_) : D); \
        if constexpr (SHW) {                                                                       \
            if (sh_active)                                                                         \
                SREG[0] = *reinterpret_cast<const u32x4*>((LIVE) ? sblk_ + sh_toff : S);           \
        } else {                                                                                   \
            _Pragma("unroll") for (int q = 0; q < WL; ++q)                                         \
                SREG[q] = *reinterpret_cast<const u32x4*>((LIVE) ? sblk_ + (int64_t)(q * 16 + lrow) * sld + lchk * E16 : S); \
        }                                                                                          \
    } while (0)

// All global loads and LDS writes of the pipeline are issued unconditionally (steps
// past the end load the first 16 bytes of each operand in every lane - one cache line
// per instruction - and are not accumulated): with no branch
// around a memory instruction the number of loads in flight is the same on every
// path, so each wait only covers the oldest stage and NST-1 stages stay in flight.
#define SPX_PANEL_STEP(IT, DREG, SREG)                                                             \
    do {                                                                                           \
        _Pragma("unroll") for (int q = 0; q < 4; ++q)                                              \
            *reinterpret_cast<u32x4*>(lds + wofs[q]) = DREG[q];                                    \
        char* sdst_ = SHW ? wsh + ((IT) & 1) * (BN * 64) : lds;                                     \
        if constexpr (SHW) {                                                                       \
            if (sh_active) {                                                                       \
                if (p.s_kcontig) {                                                                 \
                    *reinterpret_cast<u32x4*>(sdst_ + sofs[0]) = SREG[0];                          \
                } else {                                                                           \
                    union { u32x4 v4; T e[E16]; } u_;                                              \
                    u_.v4 = SREG[0];                                                               \
                    _Pragma("unroll") for (int i = 0; i < E16; ++i) {                              \
                        const int n_ = sh_n0 + i;                                                  \
                        *reinterpret_cast<T*>(sdst_ + n_ * 64 + (((sh_k / E16) ^ ((n_ >> 2) & 3)) << 4) + \
                                              (sh_k % E16) * (int)sizeof(T)) = u_.e[i];            \
                    }                                                                              \
                }                                                                                  \
            }                                                                                      \
        } else {                                                                                   \
            _Pragma("unroll") for (int q = 0; q < WL; ++q)                                         \
                *reinterpret_cast<u32x4*>(sdst_ + sofs[q]) = SREG[q];                              \
        }                                                                                          \
        {                                                                                          \
            const bool live_ = (IT) + NST < n_it;                                                  \
            const int nx_ = live_ ? (IT) + NST : n_it - 1;                                         \
            SPX_PANEL_ISSUE(nx_, live_, DREG, SREG);                                               \
        }                                                                                          \
        if constexpr (SHW) __syncthreads(); /* the S tile of this step is complete */             \
        if ((IT) < n_it) {                                                                         \
            Frag af_[4], bf_[NT];                                                                  \
            _Pragma("unroll") for (int i = 0; i < 4; ++i)                                          \
                af_[i] = panel_dfrag<T, DT, Frag>(lds + aofs[i]);                                  \
            _Pragma("unroll") for (int t = 0; t < NT; ++t)                                         \
                bf_[t] = *reinterpret_cast<const Frag*>(sdst_ + bofs[t]);                          \
            _Pragma("unroll") for (int i = 0; i < 4; ++i)                                          \
                _Pragma("unroll") for (int t = 0; t < NT; ++t)                                     \
                    acc[i][t] = SWAP ? MMA::mma(bf_[t], af_[i], acc[i][t])                         \
                                     : MMA::mma(af_[i], bf_[t], acc[i][t]);                        \
        }                                                                                          \
    } while (0)

    if (n_it > 0) {
        SPX_PANEL_ISSUE(0, true, d0, s0);
        SPX_PANEL_ISSUE((1 < n_it ? 1 : n_it - 1), 1 < n_it, d1, s1);
        if (NST > 2) SPX_PANEL_ISSUE((2 < n_it ? 2 : n_it - 1), 2 < n_it, d2, s2);
        for (int it = 0; it < n_it; it += NST) {
            SPX_PANEL_STEP(it, d0, s0);
            SPX_PANEL_STEP(it + 1, d1, s1);
            if (NST > 2) SPX_PANEL_STEP(it + 2, d2, s2);
        }
    }
#undef SPX_PANEL_ISSUE
#undef SPX_PANEL_STEP

    // ---- epilogue: registers -> private LDS -> 16-byte row-contiguous stores -----------
    // (LDS instructions of one wave execute in order, so the region can be reused
    // without a barrier once the last fragment reads have been issued.)
    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + b * p.o_batch;
    T* eT = reinterpret_cast<T*>(lds);
    if constexpr (SWAP) {
        // out[m][n], n contiguous.  One 16-row slab per pass: LDS [16][BN + pad].
        constexpr int LDE = BN + E16;
        constexpr int CPR = BN / E16;  // 16-byte chunks per row
        // The lane's bias values are fetched together, ahead of the LDS traffic below: loaded
        // where they are used, each one waits for its own round trip (the compiler cannot move
        // a load across the stores to the staging tile).
        float bias_n[NT][4], bias_m[4];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) bias_n[t][q] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) bias_m[i] = 0.f;
        if (biasT) {
            if (p.bias_on_m) {
#pragma unroll
                for (int i = 0; i < 4; ++i) bias_m[i] = Elem<T>::to_float(biasT[m0 + i * 16 + r16 < p.Mc ? m0 + i * 16 + r16 : 0]);
            } else {
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) bias_n[t][q] = Elem<T>::to_float(biasT[j * BN + t * 16 + g4 * 4 + q]);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                T vals[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float v = acc[i][t][q] + bias_n[t][q] + bias_m[i];
                    vals[q] = Elem<T>::from_float(epilogue_act(v, p.relu));
                }
                T* dst = eT + r16 * LDE + t * 16 + g4 * 4;
                if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(vals);
                else *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(vals);
            }
#pragma unroll
            for (int c0 = 0; c0 < 16 * CPR; c0 += 64) {
                const int c = c0 + lane;
                const int row = c / CPR;
                const int chunk = c % CPR;
                const int m = m0 + i * 16 + row;
                if (c < 16 * CPR && m < p.Mc)
                    __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(eT + row * LDE + chunk * E16),
                                                reinterpret_cast<u32x4*>(out + (int64_t)m * p.o_ld + (int64_t)j * BN + chunk * E16));
            }
        }
    } else {
        // out[n][m], m contiguous.  One 16-column slab per pass: LDS [16 n][64 m + pad].
        constexpr int LDE = 64 + E16;
        constexpr int CPR = 64 / E16;
        float bias_m[4][4], bias_n[NT];   // fetched together, as above
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) bias_m[i][q] = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t) bias_n[t] = 0.f;
        if (biasT) {
            if (p.bias_on_m) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int m = m0 + i * 16 + g4 * 4 + q;
                        bias_m[i][q] = Elem<T>::to_float(biasT[m < p.Mc ? m : 0]);
                    }
            } else {
#pragma unroll
                for (int t = 0; t < NT; ++t) bias_n[t] = Elem<T>::to_float(biasT[j * BN + t * 16 + r16]);
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                T vals[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float v = acc[i][t][q] + bias_m[i][q] + bias_n[t];
                    vals[q] = Elem<T>::from_float(epilogue_act(v, p.relu));
                }
                T* dst = eT + r16 * LDE + i * 16 + g4 * 4;
                if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(vals);
                else *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(vals);
            }
#pragma unroll
            for (int c0 = 0; c0 < 16 * CPR; c0 += 64) {
                const int c = c0 + lane;
                const int nrow = c / CPR;
                const int chunk = c % CPR;
                const int m = m0 + chunk * E16;
                if (m < p.Mc)
                    __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(eT + nrow * LDE + chunk * E16),
                                                reinterpret_cast<u32x4*>(out + ((int64_t)j * BN + t * 16 + nrow) * p.o_ld + m));
            }
        }
    }
}

template <typename T, int BN, int BK, int NST, bool SWAP, bool SHW, bool DT = false>
static int launch_spmm_panel_inst(const SpmmParams& p, int batch, hipStream_t st) {
    const int n_mtiles = (p.Mc + 255) / 256;
    const int nb = p.Nc / BN;
    const int64_t groups = (n_mtiles + kPanelXcd - 1) / kPanelXcd;
    const int64_t nblocks = groups * kPanelXcd * nb;
    if (nblocks > 0x7fffffffLL) return fail(SPX_E_SHAPE, "problem too large for one launch");
    hipLaunchKernelGGL((spmm_panel_kernel<T, BN, BK, NST, SWAP, SHW, DT>), dim3((unsigned)nblocks, batch, 1), dim3(256), 0, st,
                       p, n_mtiles);
    SPX_LAUNCH_CHECK("spmm_panel_kernel");
    return 0;
}

// Supported: 16-bit types with BK in {32,64}, fp32 with BK in {16,32,64}; BN in {16,32,64}.
template <typename T>
bool spmm_panel_supported(int BN, int BK) {
    const int kc = 64 / (int)sizeof(T);
    return BK % kc == 0 && (BN == 16 || BN == 32 || BN == 64);
}

template <typename T, int NST, bool SHW, bool DT = false>
int launch_spmm_panel_impl(const SpmmParams& p, int BN, int batch, hipStream_t st) {
    const bool swap = p.out_ncontig != 0;
#define SPX_PANEL_CASE(bn, bk)                                                                  \
    if (BN == bn && p.BK == bk) {                                                               \
        if constexpr (bk % (64 / (int)sizeof(T)) == 0) {                                        \
            return swap ? launch_spmm_panel_inst<T, bn, bk, NST, true, SHW, DT>(p, batch, st)   \
                        : launch_spmm_panel_inst<T, bn, bk, NST, false, SHW, DT>(p, batch, st); \
        }                                                                                       \
    }
    SPX_PANEL_CASE(16, 16) SPX_PANEL_CASE(16, 32) SPX_PANEL_CASE(16, 64)
    SPX_PANEL_CASE(32, 16) SPX_PANEL_CASE(32, 32) SPX_PANEL_CASE(32, 64)
    SPX_PANEL_CASE(64, 16) SPX_PANEL_CASE(64, 32) SPX_PANEL_CASE(64, 64)
#undef SPX_PANEL_CASE
    return fail(SPX_E_CONFIG, "block (%d,%d) not supported by the panel kernel", p.BK, BN);
}

template <typename T>
int launch_spmm_panel(const SpmmParams& p, int BN, int batch, int nst, hipStream_t st);

}  // namespace spx
