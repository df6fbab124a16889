// Sparse-operand matmul, variant for a thin dense operand stored with m contiguous:
// out[m, n] = sum_k D[m, k] S[k, n] with only 64 or 128 values of m, D given as
// D[k * d_ld + m], out as out[n * o_ld + m], S blocks in either storage order.
// This is probabilities x values of an attention layer run as separate operators
// ('sdd' with a [K, head_dim] second operand: m is the head dimension, n the queries,
// k the keys) and, with the sparse operand transposed, the gradient of the values.
//
// A workgroup owns one block-column (64 values of n) of one batch entry; wavefront w takes
// its 16 n (w = 0..3) and all of m.  Per live block the S block (k-contiguous rows of the
// 64 n, XOR-swizzled 16-byte chunks) and the D tile (BK k-rows of m, padded pitch) travel
// global -> registers -> one of two LDS buffers, one barrier per block; S fragments are
// plain 16-byte reads, D fragments come from the LDS transpose read of gfx950 (in a 16-lane
// group lane i addresses 4 consecutive m of k-row i / 4, lane j receives column j of the
// four rows).  The products are taken as  out^T-tile[m][n] += D-frag x S-frag, so a lane ends
// up with four consecutive m of one n and stores them as 8 bytes.  Workgroups are numbered so
// that all block-columns of one batch entry run on one XCD and find its D there.
#pragma once
#include "matmul_spmm.hpp"

namespace spx {

// ST: the sparse blocks are stored with n contiguous ([k][n], the layout a transposed sparse
// operand has); their fragments then come from transpose reads as well.
template <typename T, int MC, int BK, bool ST>
__global__ __launch_bounds__(256) void spmm_thin_kernel(SpmmParams p, int nb, int batch) {
    static_assert(sizeof(T) == 2, "16-bit element types only");
    constexpr int BN = 64;
    constexpr int MT = MC / 16;                 // 16-wide tiles of m
    constexpr int KS = BK / 32;                 // 32-deep MFMA steps per block
    constexpr int SP = ST ? BN * 2 + 32 : BK * 2;   // S row pitch in bytes ([k][n] rows are padded)
    constexpr int CPR = (ST ? BN : BK) * 2 / 16;    // 16-byte chunks per stored S row (4 or 8)
    constexpr int VP = MC * 2 + 32;             // D row pitch in bytes
    constexpr int S_BYTES = (ST ? BK : BN) * SP;
    constexpr int TILE = S_BYTES + BK * VP;
    constexpr int NVS = BN * BK / 8 / 256;      // vectors per thread: S block
    constexpr int DPR = MC / 8;                 // 16-byte chunks per D row
    constexpr int NVD = BK * DPR / 256;         // vectors per thread: D tile
    static_assert(NVS >= 1 && NVD >= 1, "tile does not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    __shared__ __align__(16) char smem[2 * TILE];

    // workgroup L runs on XCD L % 8: give each XCD whole batch entries
    const int L = blockIdx.x;
    const int slot_l = L >> 3;
    const int64_t b = (slot_l / nb) * 8 + (L & 7);
    const int j = slot_l % nb;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* D = reinterpret_cast<const T*>(p.D) + b * p.d_batch;
    const T* S = reinterpret_cast<const T*>(p.S) + b * p.s_batch;

    // staging maps
    int s_row[NVS], s_chunk[NVS], s_dst[NVS];
#pragma unroll
    for (int i = 0; i < NVS; ++i) {
        const int v = threadIdx.x + i * 256;
        s_row[i] = v / CPR;
        s_chunk[i] = v % CPR;
        const int swz = ST ? 0 : (CPR == 8 ? (s_row[i] & 7) : ((s_row[i] >> 2) & 3));
        s_dst[i] = s_row[i] * SP + ((s_chunk[i] ^ swz) << 4);
    }
    int d_row[NVD], d_chunk[NVD];
#pragma unroll
    for (int i = 0; i < NVD; ++i) {
        const int v = threadIdx.x + i * 256;
        d_row[i] = v / DPR;
        d_chunk[i] = v % DPR;
    }
    const int64_t sld = p.compressed ? (ST ? BN : BK) : p.s_ld;

    // fragment bases
    const int f_row = wave * 16 + r16;
    const int f_swz = CPR == 8 ? (f_row & 7) : ((f_row >> 2) & 3);
    const int v_src = S_BYTES + (g4 * 8 + (r16 >> 2)) * VP + (r16 & 3) * 8;
    const int st_src = (g4 * 8 + (r16 >> 2)) * SP + (wave * 16 + (r16 & 3) * 4) * 2;   // ST: transpose read of the S tile

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int e_begin = p.ptr[j];
    const int e_end = p.ptr[j + 1];
    auto entry = [&](int e, int& kb, int64_t& slot) {
        if (p.idx_kind == SPX_IDX_BCSC_I64) {
            const long long v = reinterpret_cast<const long long*>(p.idx)[e];
            kb = (int)(v & 0xffff);
            slot = v >> 32;
        } else {
            kb = reinterpret_cast<const int32_t*>(p.idx)[e] & 0xffff;
            slot = e;
        }
    };
    // Index entries of the block-column: lane l holds entry l (broadcast with readlane, so
    // no step waits for an index load); longer columns read the rest from the index.
    const int n_blk = e_end - e_begin;
    int kb_vec = 0, slot_vec = 0;
    if (lane < n_blk) {
        int kb0; int64_t slot0;
        entry(e_begin + lane, kb0, slot0);
        kb_vec = kb0; slot_vec = (int)slot0;
    }
    auto entry_at = [&](int i, int& kb, int64_t& slot) {
        const int ii = i < n_blk ? i : n_blk - 1;   // steps past the end re-read the last block; the copy is not used
        if (ii < 64) {
            kb = __builtin_amdgcn_readlane(kb_vec, ii);
            slot = __builtin_amdgcn_readlane(slot_vec, ii);
        } else {
            entry(e_begin + ii, kb, slot);
        }
    };
    // The loads of the two register stages are issued through inline assembly and waited for
    // with explicit counts: the compiler merges its own wait counts at the loop header and
    // then drains every outstanding load at each step, which is exactly the lead the second
    // stage is there to provide.  (S is read once: non-temporal, it must not displace the D
    // tiles from L2.)
    auto issue = [&](int i, u32x4 (&sr)[NVS], u32x4 (&dr)[NVD]) {
        int kb; int64_t slot;
        entry_at(i, kb, slot);
        const T* sblk = p.compressed ? S + slot * (int64_t)(BK * BN)
                      : ST           ? S + (int64_t)kb * BK * p.s_ld + (int64_t)j * BN
                                     : S + (int64_t)j * BN * p.s_ld + (int64_t)kb * BK;
#pragma unroll
        for (int i2 = 0; i2 < NVS; ++i2)
            asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(sr[i2]) : "v"(sblk + s_row[i2] * sld + s_chunk[i2] * 8) : "memory");
#pragma unroll
        for (int i2 = 0; i2 < NVD; ++i2)
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dr[i2]) : "v"(D + ((int64_t)kb * BK + d_row[i2]) * p.d_ld + d_chunk[i2] * 8) : "memory");
    };
    // wait until at most `newer` loads issued after this stage's are still outstanding; the
    // stage's registers pass through the statement so that no use is scheduled before it
    auto wait_stage = [&](u32x4 (&sr)[NVS], u32x4 (&dr)[NVD], bool other_in_flight) {
        if (other_in_flight) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NVS + NVD) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i2 = 0; i2 < NVS; ++i2) asm volatile("" : "+v"(sr[i2]));
#pragma unroll
        for (int i2 = 0; i2 < NVD; ++i2) asm volatile("" : "+v"(dr[i2]));
    };
    // Two register stages: the S block and D tile of step i + 2 are requested while step i is
    // staged and computed (a block is a dependent HBM round trip; one step of lead left
    // every step waiting for it).
    auto step = [&](int i, u32x4 (&sr)[NVS], u32x4 (&dr)[NVD]) {
        char* buf = smem + (i & 1) * TILE;
        wait_stage(sr, dr, i + 1 < n_blk);   // the other stage (step i + 1) may still be on its way
#pragma unroll
        for (int i2 = 0; i2 < NVS; ++i2) *reinterpret_cast<u32x4*>(buf + s_dst[i2]) = sr[i2];
#pragma unroll
        for (int i2 = 0; i2 < NVD; ++i2) *reinterpret_cast<u32x4*>(buf + S_BYTES + d_row[i2] * VP + d_chunk[i2] * 16) = dr[i2];
        if (i + 2 < n_blk) issue(i + 2, sr, dr);
        __syncthreads();   // the tile is complete; everyone is done with the buffer written next

#pragma unroll
        for (int c = 0; c < KS; ++c) {
            Frag sf;
            if constexpr (ST) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + st_src + (c * 32) * SP));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + st_src + (c * 32 + 4) * SP));
                sf = __builtin_bit_cast(Frag, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            } else {
                sf = *reinterpret_cast<const Frag*>(buf + f_row * SP + ((((c * 4 + g4) ^ f_swz) & (CPR - 1)) << 4));
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + v_src + (c * 32) * VP + t * 32));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + v_src + (c * 32 + 4) * VP + t * 32));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                acc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, both), sf, acc[t]);
            }
        }
    };
    u32x4 s0[NVS], d0[NVD], s1[NVS], d1[NVD];
    if (n_blk > 0) {
        issue(0, s0, d0);
        if (n_blk > 1) issue(1, s1, d1);
    }
    for (int i = 0; i < n_blk; i += 2) {
        step(i, s0, d0);
        if (i + 1 < n_blk) step(i + 1, s1, d1);
    }

    // lane holds out[m = t*16 + g4*4 + q][n = j*BN + wave*16 + r16]
    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + b * p.o_batch;
    const int n = j * BN + f_row;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            float v = acc[t][q];
            if (biasT) v += Elem<T>::to_float(biasT[p.bias_on_m ? t * 16 + g4 * 4 + q : n]);
            vals[q] = Elem<T>::from_float(epilogue_act(v, p.relu));
        }
        *reinterpret_cast<uint64_t*>(out + (int64_t)n * p.o_ld + t * 16 + g4 * 4) = *reinterpret_cast<const uint64_t*>(vals);
    }
}

// 16-bit types, 64 or 128 values of m stored contiguously (D[k * d_ld + m], out[n * o_ld + m]),
// 64-wide sparse blocks of depth 32 or 64 in either storage order.
template <typename T>
bool spmm_thin_ok(const SpmmParams& p, int BN) {
    if (sizeof(T) != 2) return false;
    return !p.d_kcontig && !p.out_ncontig && (p.Mc == 64 || p.Mc == 128) && BN == 64 &&
           (p.BK == 32 || p.BK == 64) && p.d_ld % 8 == 0 && p.o_ld % 4 == 0 && (p.compressed || p.s_ld % 8 == 0) &&
           p.d_batch % 8 == 0 && p.s_batch % 8 == 0 && p.o_batch % 4 == 0;
}

template <typename T>
int launch_spmm_thin_impl(const SpmmParams& p, int batch, hipStream_t st) {
    if constexpr (sizeof(T) == 2) {
        const int nb = p.Nc / 64;
        const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nb;
        if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
#define SPX_THIN_CASE(mc, bk)                                                                                     \
        if (p.Mc == mc && p.BK == bk) {                                                                           \
            if (p.s_kcontig)                                                                                      \
                hipLaunchKernelGGL((spmm_thin_kernel<T, mc, bk, false>), dim3((unsigned)groups), dim3(256), 0, st, p, nb, batch); \
            else                                                                                                  \
                hipLaunchKernelGGL((spmm_thin_kernel<T, mc, bk, true>), dim3((unsigned)groups), dim3(256), 0, st, p, nb, batch); \
            SPX_LAUNCH_CHECK("spmm_thin_kernel");                                                                 \
            return 0;                                                                                             \
        }
        SPX_THIN_CASE(64, 32) SPX_THIN_CASE(64, 64) SPX_THIN_CASE(128, 32) SPX_THIN_CASE(128, 64)
#undef SPX_THIN_CASE
    }
    return fail(SPX_E_CONFIG, "the thin-operand kernel takes 16-bit types, 64 or 128 contiguous m and 64-wide blocks of depth 32 / 64");
}

}  // namespace spx
