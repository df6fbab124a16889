// Sparse-operand matmul, persistent variant of the panel kernel (matmul_spmm_panel.hpp)
// for a k-contiguous dense operand with many 256-row tiles: out[m,n] = sum_k D[m,k] S[k,n].
//
// The panel kernel launches one workgroup per (256-row tile, block-column).  Every such
// workgroup pays a chain of dependent loads before its first MFMA (launch order -> column
// pointer -> index entries -> first blocks of D) and an epilogue during which it loads
// nothing, and the workgroups of a launch generation go through these phases together,
// so HBM, the L2 -> L1 gathers and the stores take turns instead of overlapping.  Here a
// workgroup is a slot that stays: slot (xcd, pos) walks the tiles (m-tile 8 g + xcd,
// block-column order[g odd ? nb-1-pos : pos]) for g = 0, 1, ... as ONE stream of steps.
// The index entries of tile g+1 are fetched while tile g runs, the loads of its first two
// steps are issued during the last two steps of tile g, and the stores of tile g are in
// flight while tile g+1 gathers.  Alternating the walk direction over the launch order
// (longest block-column first) pairs long columns with short ones, so the slots of an XCD
// finish together.  All m-tiles of one XCD share its L2, as in the panel kernel.
//
// Step, LDS layout, fragment mapping and epilogue are those of the panel kernel with the
// sparse block shared by the four wavefronts (one barrier per step).
#pragma once
#include <type_traits>
#include "matmul_spmm_panel.hpp"

namespace spx {

template <typename T, int BN, int BK, bool SWAP>
__global__ __launch_bounds__(256, BN <= 32 ? 4 : 2) void spmm_stream_kernel(SpmmParams p, int n_mtiles) {
    typedef typename PanelMma<T>::M MMA;
    typedef typename MMA::frag Frag;
    constexpr int KC = PanelMma<T>::KC;
    constexpr int CH = BK / KC;          // steps per block
    constexpr int NT = BN / 16;
    constexpr int ROWS = 80;             // private LDS rows (64 bytes each) per wave
    constexpr int SH_BYTES = 2 * BN * 64;  // shared, double-buffered S tile
    constexpr int E16 = 16 / (int)sizeof(T);
    static_assert(BK % KC == 0, "block depth must be a multiple of the step");

    __shared__ __align__(16) char lds_all[4 * ROWS * 64 + SH_BYTES];

    const int nb = p.Nc / BN;
    const int xcd = (int)blockIdx.x % kPanelXcd;
    const int pos = (int)blockIdx.x / kPanelXcd;  // [0, nb)
    if (xcd >= n_mtiles) return;
    const int n_tiles = (n_mtiles - xcd + kPanelXcd - 1) / kPanelXcd;
    const int64_t b = blockIdx.y;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    char* lds = lds_all + wave * (ROWS * 64);
    char* wsh = lds_all + 4 * ROWS * 64;

    const T* D = reinterpret_cast<const T*>(p.D) + b * p.d_batch;
    const T* S = reinterpret_cast<const T*>(p.S) + b * p.s_batch;

    // coalesced load mapping: lane -> (row within a 16-row group, 16-byte chunk).  Element
    // offsets from the first row of a tile fit 32 bits (checked on the host); the last
    // m-tile may be partial: its rows past the end re-read the last row and are never stored.
    const int lrow = lane >> 2;
    const int lchk = lane & 3;
    const int last_rows = p.Mc - (n_mtiles - 1) * 256;  // rows of the last m-tile (1..256)
    int roff[4];  // byte offset of this lane's chunk from the start of a tile's first row
    int wofs[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int row = wave * 64 + q * 16 + lrow;
        roff[q] = (row * (int)p.d_ld + lchk * E16) * (int)sizeof(T);
        const int lr = q * 16 + lrow;
        wofs[q] = lr * 64 + ((lchk ^ ((lr >> 2) & 3)) << 4);
    }
    // shared S tile: this wave stages chunks wave*BN .. wave*BN+BN-1 of the BN*4 chunks
    // (k-contiguous S: chunk = (n row, 16-byte piece of its 64 bytes of k); otherwise a chunk
    // is 16 bytes of n at one k and is transposed on its way into LDS)
    // (lanes past BN fetch the chunk of lane % BN once more - the same cache lines - and do not
    // write it to LDS: every load instruction below is then issued by every wavefront on every
    // path, which the explicit wait counts rely on)
    const int sh_chunk = wave * BN + (lane & (BN - 1));
    const int sh_row = sh_chunk >> 2, sh_chk = sh_chunk & 3;
    const bool sh_active = lane < BN;
    const int sh_k = sh_chunk / (BN / E16), sh_n0 = (sh_chunk % (BN / E16)) * E16;
    const int sofs = sh_row * 64 + ((sh_chk ^ ((sh_row >> 2) & 3)) << 4);
    int aofs[4], bofs[NT];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = i * 16 + r16;
        aofs[i] = row * 64 + ((g4 ^ ((row >> 2) & 3)) << 4);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int row = t * 16 + r16;
        bofs[t] = row * 64 + ((g4 ^ ((row >> 2) & 3)) << 4);
    }
    const int64_t sld = p.compressed ? (p.s_kcontig ? BK : BN) : p.s_ld;
    const int sh_boff = (int)((p.s_kcontig ? (int64_t)sh_row * sld + sh_chk * E16 : (int64_t)sh_k * sld + sh_n0) * (int64_t)sizeof(T));

    // ---- per-tile state: the tile being computed and the one after it -------------------
    struct Tile {
        int mt, j, e_begin, n_it;   // uniform
        int kb_vec, slot_vec;       // lane l: k-block and value slot of index entry l (first 64)
    };
    // Up to 128 block-columns: the launch order and the column pointers sit in lane vectors,
    // fetched by one round of independent loads at kernel start, so that a tile's look-up
    // (order -> pointer pair) costs no memory round trip; the chain ahead of a slot's first
    // operand loads is then two trips (these vectors, the index entries) instead of three.
    const bool small_nb = nb <= 128;
    int sv0 = 0, sv1 = 0, pv0 = 0, pv1 = 0, pv2 = 0;
    if (small_nb) {
        if (p.sched) {
            if (lane < nb) sv0 = p.sched[lane];
            if (64 + lane < nb) sv1 = p.sched[64 + lane];
        }
        if (lane <= nb) pv0 = p.ptr[lane];
        if (64 + lane <= nb) pv1 = p.ptr[64 + lane];
        if (nb == 128) pv2 = p.ptr[128];
    }
    auto ptr_at = [&](int i) {
        return i < 64 ? __builtin_amdgcn_readlane(pv0, i) : (i < 128 ? __builtin_amdgcn_readlane(pv1, i - 64) : __builtin_amdgcn_readfirstlane(pv2));
    };
    // (The lane vectors serve the two tiles that are looked up at kernel start, where the round
    // trip matters.  Later tiles are looked up a whole tile ahead and read the two arrays
    // directly: the vectors do not have to stay in registers - or, as it turned out in one of
    // the two output layouts, in scratch memory, each load waited for so that it could be
    // spilled - for the rest of the kernel.)
    auto load_tile = [&](int g, Tile& t, bool from_vectors) {
        t.mt = g * kPanelXcd + xcd;
        const int o = (g & 1) ? nb - 1 - pos : pos;
        if (from_vectors) {
            t.j = p.sched ? (o < 64 ? __builtin_amdgcn_readlane(sv0, o) : __builtin_amdgcn_readlane(sv1, o - 64)) : o;
            t.e_begin = ptr_at(t.j);
        } else {
            t.j = p.sched ? p.sched[o] : o;
            t.e_begin = p.ptr[t.j];
        }
        const int n_blk = (from_vectors ? ptr_at(t.j + 1) : p.ptr[t.j + 1]) - t.e_begin;
        t.n_it = n_blk * CH;
        t.kb_vec = 0;
        t.slot_vec = 0;
        if (lane < n_blk) {
            if (p.idx_kind == SPX_IDX_BCSC_I64) {
                const long long v = reinterpret_cast<const long long*>(p.idx)[t.e_begin + lane];
                t.kb_vec = (int)(v & 0xffff);
                t.slot_vec = (int)(v >> 32);
            } else {
                t.kb_vec = reinterpret_cast<const int32_t*>(p.idx)[t.e_begin + lane] & 0xffff;
                t.slot_vec = t.e_begin + lane;
            }
        }
    };
    Tile cur, nxt;
    load_tile(0, cur, small_nb);
    if (n_tiles > 1) load_tile(1, nxt, small_nb); else nxt = cur;

    // Loads of one step of tile t into a stage (dreg: 4 x 16 bytes of D per lane, sreg: this
    // lane's piece of the shared S block).  A step past the end (live == false) loads one
    // fixed line per instruction and is never accumulated: every call issues exactly
    // kStageLoads load instructions, on every path.
    //
    // The loads go out through inline assembly and are waited for with explicit counts.  Left to
    // the compiler, the wait counts of the two stages are merged at the loop header and every
    // second step drains ALL loads in flight - the lead of the second stage, which is there to
    // cover a load that takes longer than one step, is lost.  Each load takes a scalar base (the
    // tile's first row plus the k offset, or the S block) and a 32-bit lane offset.
    constexpr int kStageLoads = 5;
    // (marker for the build's check of the assembly: this kernel's waits are to be verified along
    // every path of its control flow, not only in text order)
    asm volatile("; spx-uniform-waits");
    auto uniform_base = [](const void* ptr) {
        const uint64_t v = (uint64_t)ptr;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return ((uint64_t)hi << 32) | lo;
    };
    auto issue = [&](const Tile& t, int it, bool live, u32x4 (&dreg)[4], u32x4& sreg) {
        const int er = it / CH;
        const int ch = it % CH;
        int kb;
        int64_t slot;
        if (er < 64) {
            kb = __builtin_amdgcn_readlane(t.kb_vec, er);
            slot = __builtin_amdgcn_readlane(t.slot_vec, er);
        } else if (p.idx_kind == SPX_IDX_BCSC_I64) {
            const long long v = reinterpret_cast<const long long*>(p.idx)[t.e_begin + er];
            kb = (int)(v & 0xffff);
            slot = v >> 32;
        } else {
            kb = reinterpret_cast<const int32_t*>(p.idx)[t.e_begin + er] & 0xffff;
            slot = t.e_begin + er;
        }
        const int koff = kb * BK + ch * KC;
        // A step that is not live reads the first bytes of the dense operand.
        const uint64_t dbase = uniform_base(live ? D + (int64_t)t.mt * 256 * p.d_ld + koff : D);
        int voff[4];
        if (live && t.mt == n_mtiles - 1 && last_rows < 256) {
            // partial last m-tile: rows past the end re-read its last row
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int row = wave * 64 + q * 16 + lrow;
                voff[q] = ((row < last_rows ? row : last_rows - 1) * (int)p.d_ld + lchk * E16) * (int)sizeof(T);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) voff[q] = live ? roff[q] : 0;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dreg[q]) : "v"(voff[q]), "s"(dbase) : "memory");
        const T* sblk = p.compressed ? S + slot * (int64_t)(BK * BN) + (p.s_kcontig ? ch * KC : ch * KC * BN)
                                     : (p.s_kcontig ? S + (int64_t)t.j * BN * p.s_ld + koff
                                                    : S + (int64_t)koff * p.s_ld + (int64_t)t.j * BN);
        // an idle step reads the first bytes of the dense operand: the sparse operand may be NULL
        // when no block is live (every step of every tile is idle then)
        const uint64_t sbase = uniform_base(live ? (const void*)sblk : (const void*)D);
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sreg) : "v"(live ? sh_boff : 0), "s"(sbase) : "memory");
    };
    // Wait until at most NEWER vector-memory instructions issued after this stage's loads are
    // still outstanding (they retire in order); the stage's registers pass through the statement
    // so that no use is scheduled ahead of it.  NEWER may undercount (a stricter wait), never
    // overcount.  The count is a compile-time property of the call site - a run-time choice
    // between two counts would put them on two paths of which a reader of the code (and the
    // build's check of the assembly) cannot tell which one ran.
    auto wait_stage = [&](auto newer, u32x4 (&dreg)[4], u32x4& sreg) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(decltype(newer)::value) : "memory");
#pragma unroll
        for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(dreg[q]));
        asm volatile("" : "+v"(sreg));
    };

    f32x4 acc[4][NT];
    u32x4 d0[4], d1[4], s0, s1;
    s0 = s1 = u32x4{0u, 0u, 0u, 0u};

    // One step: stage -> LDS, refill the stage with the step two ahead (which may belong to
    // the next tile), barrier for the shared S tile, MFMAs.
    auto step = [&](auto newer, int it, int n_pad, bool have_next, u32x4 (&dreg)[4], u32x4& sreg) {
        wait_stage(newer, dreg, sreg);
#pragma unroll
        for (int q = 0; q < 4; ++q) *reinterpret_cast<u32x4*>(lds + wofs[q]) = dreg[q];
        char* sdst = wsh + (it & 1) * (BN * 64);
        if (sh_active) {
            if (p.s_kcontig) {
                *reinterpret_cast<u32x4*>(sdst + sofs) = sreg;
            } else {
                union { u32x4 v4; T e[E16]; } u;
                u.v4 = sreg;
#pragma unroll
                for (int i = 0; i < E16; ++i) {
                    const int n = sh_n0 + i;
                    *reinterpret_cast<T*>(sdst + n * 64 + (((sh_k / E16) ^ ((n >> 2) & 3)) << 4) +
                                          (sh_k % E16) * (int)sizeof(T)) = u.e[i];
                }
            }
        }
        {
            // one call site: the compiler must not end up with two copies of the loads on
            // different paths, so the tile is selected first
            const int ahead = it + 2;
            const bool in_cur = ahead < n_pad;
            const int ait = in_cur ? ahead : ahead - n_pad;
            Tile t;
            t.mt = in_cur ? cur.mt : nxt.mt;
            t.j = in_cur ? cur.j : nxt.j;
            t.e_begin = in_cur ? cur.e_begin : nxt.e_begin;
            t.n_it = in_cur ? cur.n_it : nxt.n_it;
            t.kb_vec = in_cur ? cur.kb_vec : nxt.kb_vec;
            t.slot_vec = in_cur ? cur.slot_vec : nxt.slot_vec;
            const bool live = (in_cur || have_next) && ait < t.n_it;
            issue(t, live ? ait : 0, live, dreg, sreg);
        }
        __syncthreads();  // the S tile of this step is complete
        if (it < cur.n_it) {
            Frag af[4], bf[NT];
#pragma unroll
            for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const Frag*>(lds + aofs[i]);
#pragma unroll
            for (int t = 0; t < NT; ++t) bf[t] = *reinterpret_cast<const Frag*>(sdst + bofs[t]);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    acc[i][t] = SWAP ? MMA::mma(bf[t], af[i], acc[i][t]) : MMA::mma(af[i], bf[t], acc[i][t]);
        }
    };

    issue(cur, 0, 0 < cur.n_it, d0, s0);
    issue(cur, cur.n_it > 1 ? 1 : 0, 1 < cur.n_it, d1, s1);

    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + b * p.o_batch;
    T* eT = reinterpret_cast<T*>(lds);

    // The other stage's kStageLoads loads are newer than the ones a step waits for.  In the first
    // two steps of a tile so are the stores of the tile before it, a number that varies (a
    // partial last m-tile stores from some of its wavefronts only): the count leaves them out,
    // which only makes those two waits stricter.
    typedef std::integral_constant<int, kStageLoads> InTile;
    for (int g = 0; g < n_tiles; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        // every tile runs an even number of steps, at least two (the surplus ones are idle),
        // so that the stage a step uses is fixed by its position in its tile
        const int n_pad = cur.n_it < 2 ? 2 : (cur.n_it + 1) & ~1;
        const bool have_next = g + 1 < n_tiles;
        for (int it = 0; it < n_pad; it += 2) {
            step(InTile{}, it, n_pad, have_next, d0, s0);
            step(InTile{}, it + 1, n_pad, have_next, d1, s1);
        }

        // ---- epilogue of tile g: registers -> private LDS -> 16-byte row-contiguous stores
        // (LDS instructions of one wave execute in order, so the region can be reused
        // without a barrier once the last fragment reads have been issued)
        const int m0 = cur.mt * 256 + wave * 64;
        const int j = cur.j;
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

        // ---- move on: tile g+1 becomes current, the index entries of tile g+2 are fetched --
        cur = nxt;
        if (g + 2 < n_tiles) load_tile(g + 2, nxt, false);
    }
}

template <typename T>
bool spmm_stream_supported(const SpmmParams& p, int BN) {
    const int kc = 64 / (int)sizeof(T);
    // element offsets inside a 256-row tile are kept in 32 bits
    // (and so is a lane's byte offset inside the rows of an uncompressed sparse operand)
    return p.d_kcontig && p.BK % kc == 0 && (BN == 16 || BN == 32 || BN == 64) &&
           p.d_ld * 256 + 64 < (int64_t)0x7fffffff / (int)sizeof(T) &&
           (p.compressed || p.s_ld * 64 + 64 < (int64_t)0x7fffffff / (int)sizeof(T));
}

// 256-row tiles of the dense operand per launch.  The slots of an XCD drift apart as they walk
// their tiles (block columns differ in length), and once they are spread over more than two row
// panels of 2 MB the panels no longer share the XCD's 4 MB L2 with the sparse operand: measured
// on the 4096 x 4096 weight of the headline shape, 4 tiles per slot cost 12.7 us each, 8 tiles
// 16.3 and 16 tiles 21.6.  Longer operands are therefore walked in several launches.
constexpr int kStreamTilesPerLaunch = 4 * kPanelXcd;

template <typename T, int BN, int BK, bool SWAP>
static int launch_spmm_stream_inst(const SpmmParams& p0, int batch, hipStream_t st) {
    const int64_t nblocks = (int64_t)kPanelXcd * (p0.Nc / BN);
    if (nblocks > 0x7fffffffLL) return fail(SPX_E_SHAPE, "problem too large for one launch");
    const int total_tiles = (p0.Mc + 255) / 256;
    for (int t0 = 0; t0 < total_tiles || t0 == 0; t0 += kStreamTilesPerLaunch) {
        SpmmParams p = p0;
        const int64_t m_begin = (int64_t)t0 * 256;
        p.Mc = (int)(p0.Mc - m_begin < (int64_t)kStreamTilesPerLaunch * 256 ? p0.Mc - m_begin : (int64_t)kStreamTilesPerLaunch * 256);
        // the chunk's first row of the dense operand, of the result, and of a bias along m
        p.D = reinterpret_cast<const T*>(p0.D) + m_begin * p0.d_ld;
        p.out = reinterpret_cast<T*>(p0.out) + (p0.out_ncontig ? m_begin * p0.o_ld : m_begin);
        if (p0.bias && p0.bias_on_m) p.bias = reinterpret_cast<const T*>(p0.bias) + m_begin;
        const int n_mtiles = (p.Mc + 255) / 256;
        hipLaunchKernelGGL((spmm_stream_kernel<T, BN, BK, SWAP>), dim3((unsigned)nblocks, batch, 1), dim3(256), 0, st, p, n_mtiles);
        SPX_LAUNCH_CHECK("spmm_stream_kernel");
    }
    return 0;
}

template <typename T>
int launch_spmm_stream_impl(const SpmmParams& p, int BN, int batch, hipStream_t st) {
    const bool swap = p.out_ncontig != 0;
#define SPX_STREAM_CASE(bn, bk)                                                              \
    if (BN == bn && p.BK == bk) {                                                            \
        if constexpr (bk % (64 / (int)sizeof(T)) == 0) {                                     \
            return swap ? launch_spmm_stream_inst<T, bn, bk, true>(p, batch, st)             \
                        : launch_spmm_stream_inst<T, bn, bk, false>(p, batch, st);           \
        }                                                                                    \
    }
    SPX_STREAM_CASE(16, 16) SPX_STREAM_CASE(16, 32) SPX_STREAM_CASE(16, 64)
    SPX_STREAM_CASE(32, 16) SPX_STREAM_CASE(32, 32) SPX_STREAM_CASE(32, 64)
    SPX_STREAM_CASE(64, 16) SPX_STREAM_CASE(64, 32) SPX_STREAM_CASE(64, 64)
#undef SPX_STREAM_CASE
    return fail(SPX_E_CONFIG, "block (%d,%d) not supported by the persistent panel kernel", p.BK, BN);
}

template <typename T>
int launch_spmm_stream(const SpmmParams& p, int BN, int batch, hipStream_t st);

}  // namespace spx
