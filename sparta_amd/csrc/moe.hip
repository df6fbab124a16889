// MoE sparse forward: out[t,:] = tokens[t,:] . W[exp_ids[t]].
//
//  spx_moe_index   stable counting sort of the tokens by expert, no atomics on
//                  global memory, no per-expert capacity, no host round trip:
//                  (1) per-chunk histograms, (2) an exclusive scan of them in
//                  (expert, chunk) order, (3) every chunk places its tokens in
//                  ascending order behind its scanned base.  A table of at most
//                  1024 (chunk, expert) counts is scanned by every placement
//                  workgroup itself (two launches); larger ones get a scan
//                  launch of their own.
//  spx_moe_forward one gathered GEMM over a flattened (expert, 128-row tile) list:
//                  a workgroup looks its tile up in the prefix of per-expert tile
//                  counts, gathers its token rows through token_perm, and walks
//                  K in 64-wide stages through LDS ([row][k], XOR-swizzled 16-byte
//                  chunks) into 16x16 MFMAs; rows are scattered back on store.
// Replaces convert_sparse_index / BATCH_BLOCK_SPARSE_MATMUL[_FP16] of the
// reference (csrc/moe_sparse_forward_kernel.cu.j2:58-71,120-325,363-483), whose
// grid is sized by the largest expert and whose fp16 path accumulates in fp16.
#include <type_traits>
#include "common.hpp"
#include "mma.hpp"

namespace spx {

constexpr int MOE_CHUNK = 1024;   // most tokens per workgroup in the index kernels (a multiple of 256)
constexpr int MOE_FUSED_TABLE = 1024;  // (chunk, expert) counts a placement workgroup scans itself
constexpr int MOE_MAX_EXP = 2048; // LDS table capacity of the placement kernel

// ---- index -------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_hist_kernel(const int32_t* exp_ids, int n_tok, int n_exp, int chunk,
                                                       int32_t* partial /* [n_chunk][n_exp] */) {
    // n_exp here counts the pseudo expert that collects the tokens whose id is out of range
    extern __shared__ int hist[];
    for (int e = threadIdx.x; e < n_exp; e += 256) hist[e] = 0;
    __syncthreads();
    const int base = blockIdx.x * chunk;
    for (int i = threadIdx.x; i < chunk; i += 256) {
        const int t = base + i;
        if (t < n_tok) {
            int e = exp_ids[t];
            if (e < 0 || e >= n_exp - 1) e = n_exp - 1;
            atomicAdd(&hist[e], 1);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_exp; e += 256) partial[(int64_t)blockIdx.x * n_exp + e] = hist[e];
}

// Wavefront e: exclusive prefix of expert e's counts over the chunks, in place, and the
// expert's total.  Every lane takes a run of consecutive chunks (sums it, then rewrites it
// from the lane's offset), so the serial part is 1/64 of the chunks.  n_exp counts the
// pseudo expert of out-of-range ids.
__global__ __launch_bounds__(256) void moe_colscan_kernel(int32_t* partial, int n_chunk, int n_exp, int32_t* totals) {
    const int lane = lane_id();
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= n_exp) return;
    const int per = (n_chunk + 63) / 64;
    const int c0 = lane * per < n_chunk ? lane * per : n_chunk;
    const int c1 = c0 + per < n_chunk ? c0 + per : n_chunk;
    int sum = 0;
    for (int c = c0; c < c1; ++c) sum += partial[(int64_t)c * n_exp + e];
    const int inc = wave_inclusive_scan(sum);
    int run = inc - sum;
    for (int c = c0; c < c1; ++c) {
        const int v = partial[(int64_t)c * n_exp + e];
        partial[(int64_t)c * n_exp + e] = run;
        run += v;
    }
    if (lane == 63) totals[e] = inc;
}

__global__ __launch_bounds__(256) void moe_zero_index_kernel(int n_exp, int32_t* expert_count, int32_t* expert_offset) {
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e < n_exp) expert_count[e] = 0;
    if (e <= n_exp) expert_offset[e] = 0;
}

// Stable placement of one chunk.  Waves take 64 tokens at a time; inside a wave the
// rank among equal experts comes from ballots, between waves from a small table.
// FUSED: `counts` holds the raw per-chunk histograms (at most MOE_FUSED_TABLE of them);
// every workgroup scans them in (expert, chunk) order itself and workgroup 0 also writes
// expert_offset and expert_count.  Otherwise `counts` holds every expert's prefix over the
// chunks (moe_colscan_kernel) and `totals` the experts' token counts, which every workgroup
// turns into the experts' offsets itself (at most MOE_MAX_EXP + 1 of them).
template <bool FUSED>
__global__ __launch_bounds__(256) void moe_place_kernel(const int32_t* exp_ids, int n_tok, int n_exp, int chunk,
                                                        const int32_t* counts, const int32_t* totals, int32_t* token_perm,
                                                        int32_t* expert_count, int32_t* expert_offset) {
    extern __shared__ int sm[];
    int* running = sm;               // [n_exp] tokens of expert e already placed by this chunk
    int* wavecnt = sm + n_exp;       // [4][n_exp] tokens of expert e in the current pass, per wave
    int* ebase = sm + 5 * n_exp;     // [n_exp] first position of expert e (not FUSED)
    __shared__ int tab[FUSED ? MOE_FUSED_TABLE : 1];
    __shared__ int wave_total[4];
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 5 * n_exp; i += 256) sm[i] = 0;
    if constexpr (FUSED) {
        // entries 4 tid .. 4 tid + 3 of the (expert, chunk) order
        const int n_chunk = gridDim.x;
        const int n = n_chunk * n_exp;
        int v[4], sum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = threadIdx.x * 4 + j;
            v[j] = 0;
            if (i < n) {
                const int e = i / n_chunk, c = i - e * n_chunk;
                v[j] = counts[c * n_exp + e];
            }
            sum += v[j];
        }
        const int inc = wave_inclusive_scan(sum);
        if (lane == 63) wave_total[wave] = inc;
        __syncthreads();
        int excl = inc - sum;
        for (int w = 0; w < wave; ++w) excl += wave_total[w];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = threadIdx.x * 4 + j;
            if (i < n) tab[i] = excl;
            excl += v[j];
        }
        __syncthreads();
        if (blockIdx.x == 0) {
            for (int e = threadIdx.x; e < n_exp; e += 256) {
                expert_offset[e] = tab[e * n_chunk];
                if (e + 1 < n_exp) expert_count[e] = tab[(e + 1) * n_chunk] - tab[e * n_chunk];
            }
        }
    }
    if constexpr (!FUSED) {
        // experts per * tid .. per * tid + per - 1: exclusive scan of their totals
        const int per = (n_exp + 255) / 256;
        int sum = 0;
        for (int j = 0; j < per; ++j) {
            const int e = threadIdx.x * per + j;
            if (e < n_exp) sum += totals[e];
        }
        const int inc = wave_inclusive_scan(sum);
        if (lane == 63) wave_total[wave] = inc;
        __syncthreads();
        int excl = inc - sum;
        for (int w = 0; w < wave; ++w) excl += wave_total[w];
        for (int j = 0; j < per; ++j) {
            const int e = threadIdx.x * per + j;
            if (e < n_exp) {
                const int t = totals[e];
                ebase[e] = excl;
                if (blockIdx.x == 0) {
                    expert_offset[e] = excl;
                    if (e + 1 < n_exp) expert_count[e] = t;
                }
                excl += t;
            }
        }
    }
    __syncthreads();
    const int chunk0 = blockIdx.x * chunk;
    const unsigned long long lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int pass = 0; pass < chunk; pass += 256) {
        const int t = chunk0 + pass + threadIdx.x;
        int e = -1;
        if (t < n_tok) {
            e = exp_ids[t];
            if (e < 0 || e >= n_exp - 1) e = n_exp - 1;  // out of range: the pseudo expert
        }
        // intra-wave rank and per-wave count of my expert
        int rank = 0, cnt = 0;
        bool leader = false;
        unsigned long long todo = __ballot(e >= 0);
        while (todo) {
            const int src = __ffsll((long long)todo) - 1;
            const int e0 = __shfl(e, src, 64);
            const unsigned long long same = __ballot(e == e0);
            if (e == e0) {
                rank = __popcll(same & lt_mask);
                cnt = __popcll(same);
                leader = lane == src;
            }
            todo &= ~same;
        }
        if (leader) wavecnt[wave * n_exp + e] = cnt;
        __syncthreads();
        if (e >= 0) {
            int before = running[e];
            for (int w = 0; w < wave; ++w) before += wavecnt[w * n_exp + e];
            const int base = FUSED ? tab[e * gridDim.x + blockIdx.x] : ebase[e] + counts[(int64_t)blockIdx.x * n_exp + e];
            token_perm[base + before + rank] = t;
        }
        __syncthreads();
        if (leader) {
            atomicAdd(&running[e], cnt);
            wavecnt[wave * n_exp + e] = 0;
        }
        __syncthreads();
    }
}

// ---- gathered GEMM -------------------------------------------------------------
struct MoeParams {
    const void* tokens;
    const void* weight;
    void* out;
    const int32_t* expert_offset;
    const int32_t* token_perm;
    int n_tok, K, N, n_exp;
    int w_kcontig;  // weight [E, N, K] if set, else [E, K, N]
    int split;      // 0: one launch; 1 / 2: first / second launch of a split (see moe_find_tile)
    int round_rows; // split: 256-row tiles that one round of the big-tile launch covers
};

// Which (expert, row tile) belongs to tile index y: one wavefront scans the per-expert
// tile counts.  Expert n_exp is the pseudo expert of the tokens whose id was out of
// range (token_perm[expert_offset[n_exp] .. n_tok)): its tiles are zero-filled instead
// of multiplied.  found_e = -1 when y is past the last tile.
//
// split (MoeParams::split): a launch of big (256-row) tiles leaves most CUs idle during
// its last round when the number of row tiles is a little over a multiple of the row
// tiles one round takes (round_rows).  The work can therefore go out as two launches:
// split 1 = the 256-row tiles below the last multiple of round_rows (whole rounds),
// split 2 = the remaining row tiles cut into 128-row halves for the small-tile kernel,
// which fills the device with them.  Both launches derive the same boundary from the
// device-side expert counts.
// Single launch (split == 0): the row tiles are numbered with every expert's full tiles first
// and the partly filled last tiles of the experts behind them (longest first).  Workgroups start in the order
// of their tile numbers, so the short tiles (a partly filled tile skips the work of its empty
// 64-row groups) fill the end of the launch, where the long ones would leave most CUs idle.
template <int TM>
__device__ __forceinline__ void moe_find_tile_sorted(const MoeParams& p, int y, int lane,
                                                     int& found_e, int& found_row0, int& found_rows) {
    int total_full = 0;
    for (int e0 = 0; e0 <= p.n_exp; e0 += 64) {
        const int e = e0 + lane;
        int cnt = 0;
        if (e <= p.n_exp) cnt = (e < p.n_exp ? p.expert_offset[e + 1] : p.n_tok) - p.expert_offset[e];
        total_full += __shfl(wave_inclusive_scan(cnt / TM), 63, 64);
    }
    const bool part = y >= total_full;   // looking for a partly filled tile
    const int want = part ? y - total_full : y;
    int before = 0;
    found_e = -1; found_row0 = 0; found_rows = 0;
    if (part && p.n_exp < 64) {
        // at most 64 candidates: the partly filled tiles go out longest first (rank = number of
        // experts whose last tile holds more rows, ties in expert order)
        int cnt = 0, off = 0;
        if (lane <= p.n_exp) {
            off = p.expert_offset[lane];
            cnt = (lane < p.n_exp ? p.expert_offset[lane + 1] : p.n_tok) - off;
        }
        const int full = cnt / TM, rest = cnt - full * TM;
        int rank = 0;
        for (int o = 0; o <= p.n_exp; ++o) {
            const int r = __shfl(rest, o, 64);
            rank += (r > rest || (r == rest && o < lane)) ? 1 : 0;
        }
        const unsigned long long hit = __ballot(rest > 0 && rank == want);
        if (hit) {
            const int src = __ffsll((long long)hit) - 1;
            found_e = src;
            found_row0 = __shfl(off, src, 64) + __shfl(full, src, 64) * TM;
            found_rows = __shfl(rest, src, 64);
        }
        return;
    }
    for (int e0 = 0; e0 <= p.n_exp; e0 += 64) {
        const int e = e0 + lane;
        int cnt = 0, off = 0;
        if (e <= p.n_exp) {
            off = p.expert_offset[e];
            cnt = (e < p.n_exp ? p.expert_offset[e + 1] : p.n_tok) - off;
        }
        const int full = cnt / TM, rest = cnt - full * TM;
        const int tiles = part ? (rest ? 1 : 0) : full;
        const int inc = wave_inclusive_scan(tiles);
        const int excl = before + inc - tiles;
        const unsigned long long hit = __ballot(want >= excl && want < excl + tiles);
        if (hit) {
            const int src = __ffsll((long long)hit) - 1;
            const int lt = want - __shfl(excl, src, 64);
            found_e = e0 + src;
            found_row0 = __shfl(off, src, 64) + (part ? __shfl(full, src, 64) : lt) * TM;
            found_rows = part ? __shfl(rest, src, 64) : TM;
            return;
        }
        before += __shfl(inc, 63, 64);
    }
}

template <int TM>
__device__ __forceinline__ void moe_find_tile(const MoeParams& p, int y, int lane,
                                              int& found_e, int& found_row0, int& found_rows) {
    if (p.split == 0) {
        moe_find_tile_sorted<TM>(p, y, lane, found_e, found_row0, found_rows);
        return;
    }
    const int TS = p.split ? 256 : TM;      // tile height the row tiles are counted in
    int half = 0;
    if (p.split == 2) { half = y & 1; y >>= 1; }
    int tiles_before = 0;
    int fe = -1, frow0 = 0, frows = 0, fy = -1;
    for (int e0 = 0; e0 <= p.n_exp && (fe < 0 || p.split); e0 += 64) {
        const int e = e0 + lane;
        int cnt = 0, off = 0;
        if (e <= p.n_exp) {
            off = p.expert_offset[e];
            cnt = (e < p.n_exp ? p.expert_offset[e + 1] : p.n_tok) - off;
        }
        const int tiles = (cnt + TS - 1) / TS;
        const int inc = wave_inclusive_scan(tiles);
        const int excl = tiles_before + inc - tiles;
        // split 2 counts y from the boundary, which is only known after the whole scan:
        // remember every expert's range and pick afterwards (n_exp <= 64 in one pass)
        if (p.split != 2) {
            const bool mine = y >= excl && y < excl + tiles;
            const unsigned long long hit = __ballot(mine);
            if (hit && fe < 0) {
                const int src = __ffsll((long long)hit) - 1;
                const int lt = y - __shfl(excl, src, 64);
                fe = e0 + src; fy = y;
                frow0 = __shfl(off, src, 64) + lt * TS;
                frows = min(TS, __shfl(cnt, src, 64) - lt * TS);
            }
        }
        tiles_before += __shfl(inc, 63, 64);
    }
    int boundary = tiles_before;  // first row tile of the second launch
    if (p.split) {
        const int rem = tiles_before % p.round_rows;
        // a last round that is mostly full stays with the big tiles
        if (rem * 10 <= p.round_rows * 6) boundary = tiles_before - rem;
    }
    if (p.split == 1 && fy >= boundary) fe = -1;
    if (p.split == 2) {
        const int yb = boundary + y;
        fe = -1;
        int before = 0;
        for (int e0 = 0; e0 <= p.n_exp && fe < 0 && yb < tiles_before; e0 += 64) {
            const int e = e0 + lane;
            int cnt = 0, off = 0;
            if (e <= p.n_exp) {
                off = p.expert_offset[e];
                cnt = (e < p.n_exp ? p.expert_offset[e + 1] : p.n_tok) - off;
            }
            const int tiles = (cnt + 255) / 256;
            const int inc = wave_inclusive_scan(tiles);
            const int excl = before + inc - tiles;
            const unsigned long long hit = __ballot(yb >= excl && yb < excl + tiles);
            if (hit) {
                const int src = __ffsll((long long)hit) - 1;
                const int lt = yb - __shfl(excl, src, 64);
                const int r0 = lt * 256 + half * 128;
                const int left = __shfl(cnt, src, 64) - r0;
                if (left > 0) {
                    fe = e0 + src;
                    frow0 = __shfl(off, src, 64) + r0;
                    frows = min(128, left);
                } else {
                    break;  // the upper half of a row tile with at most 128 rows
                }
            }
            before += __shfl(inc, 63, 64);
        }
    }
    found_e = fe; found_row0 = frow0; found_rows = frows;
}

// Zero rows token_perm[row0 .. row0 + rows) of `out`, columns n0 .. n0 + TN (16-byte stores).
template <typename T>
__device__ __forceinline__ void moe_zero_tile(const MoeParams& p, int row0, int rows, int n0, int TN, int nthreads) {
    constexpr int VE = 16 / (int)sizeof(T);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    T* out = reinterpret_cast<T*>(p.out);
    const int ncol = (min(n0 + TN, p.N) - n0) / VE;  // N is a multiple of VE
    for (int v = threadIdx.x; v < rows * ncol; v += nthreads) {
        const int r = v / ncol, c = v - r * ncol;
        const int tok = p.token_perm[row0 + r];
        *reinterpret_cast<u32x4*>(out + (int64_t)tok * p.N + n0 + c * VE) = u32x4{0u, 0u, 0u, 0u};
    }
}

constexpr int MOE_TM = 128, MOE_TN = 128;
// k per LDS stage: 128 bytes per row for every element type
template <typename T> struct MoeKt { static constexpr int value = 128 / (int)sizeof(T); };

// LDS tile: rows of 128 bytes = 8 chunks of 16 bytes; chunk c of row r is stored at
// chunk position c ^ (r & 7).
template <typename T>
__device__ __forceinline__ int moe_lds_off(int row, int chunk) {
    return (row * 8 + (chunk ^ (row & 7))) * 16;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_gemm_kernel(MoeParams p) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int MOE_KT = MoeKt<T>::value;
    constexpr int CPR = MOE_KT / VE;                 // 16-byte chunks per LDS row (8)
    constexpr int TILE_BYTES = MOE_TM * MOE_KT * (int)sizeof(T);
    extern __shared__ __align__(16) char smem[];
    char* As = smem;
    char* Bs = smem + TILE_BYTES;
    __shared__ int s_expert, s_row0, s_rows;

    // ---- which (expert, row tile) is mine ------------------------------------------
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        int found_e, found_row0, found_rows;
        moe_find_tile<MOE_TM>(p, blockIdx.y, lane, found_e, found_row0, found_rows);
        if (lane == 0) { s_expert = found_e; s_row0 = found_row0; s_rows = found_rows; }
    }
    __syncthreads();
    const int expert = s_expert;
    if (expert < 0) return;  // uniform: this tile index is past the last tile
    const int row0 = s_row0, rows = s_rows;
    const int n0 = blockIdx.x * MOE_TN;
    if (expert == p.n_exp) {  // tokens without a valid expert id: zero rows
        moe_zero_tile<T>(p, row0, rows, n0, MOE_TN, 256);
        return;
    }

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 waves, each 64 x 64

    const T* X = reinterpret_cast<const T*>(p.tokens);
    const T* W = reinterpret_cast<const T*>(p.weight) + (int64_t)expert * p.K * p.N;

    // staging map: thread -> (row, 16-byte chunk) pairs; 128 rows x CPR chunks per tile
    constexpr int LOADS = MOE_TM * CPR / 256;
    int a_tok[LOADS];
#pragma unroll
    for (int q = 0; q < LOADS; ++q) {
        const int v = q * 256 + threadIdx.x;
        const int r = v / CPR;
        a_tok[q] = p.token_perm[row0 + (r < rows ? r : rows - 1)];
    }

    // 2-byte types: 2 x 2 tiles of 32 x 32 (accw); fp32: 4 x 4 tiles of 16 x 16 (acc)
    constexpr bool WIDE = HasMma32<T>::value;
    f32x4 acc[WIDE ? 1 : 4][WIDE ? 1 : 4];
    f32x16 accw[WIDE ? 2 : 1][WIDE ? 2 : 1];
#pragma unroll
    for (int i = 0; i < (WIDE ? 1 : 4); ++i)
#pragma unroll
        for (int t = 0; t < (WIDE ? 1 : 4); ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < (WIDE ? 2 : 1); ++i)
#pragma unroll
        for (int t = 0; t < (WIDE ? 2 : 1); ++t)
#pragma unroll
            for (int j = 0; j < 16; ++j) accw[i][t][j] = 0.f;
    const int l32 = lane & 31, h2 = lane >> 5;

    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    for (int k0 = 0; k0 < p.K; k0 += MOE_KT) {
        // ---- stage A (gathered token rows) and B (weight rows n0..n0+127) ---------------
#pragma unroll
        for (int q = 0; q < LOADS; ++q) {
            const int v = q * 256 + threadIdx.x;
            const int r = v / CPR, c = v % CPR;
            const u32x4 val = *reinterpret_cast<const u32x4*>(X + (int64_t)a_tok[q] * p.K + k0 + c * VE);
            *reinterpret_cast<u32x4*>(As + moe_lds_off<T>(r, c)) = val;
        }
        if (p.w_kcontig) {
#pragma unroll
            for (int q = 0; q < LOADS; ++q) {
                const int v = q * 256 + threadIdx.x;
                const int r = v / CPR, c = v % CPR;
                const int n = n0 + r < p.N ? n0 + r : p.N - 1;
                const u32x4 val = *reinterpret_cast<const u32x4*>(W + (int64_t)n * p.K + k0 + c * VE);
                *reinterpret_cast<u32x4*>(Bs + moe_lds_off<T>(r, c)) = val;
            }
        } else {
            // weight stored [K, N]: 16-byte loads along n, transposed into [n][k]
            constexpr int NV = MOE_TN / VE;  // vectors per k row
            for (int v = threadIdx.x; v < MOE_KT * NV; v += 256) {
                const int k = v / NV, nv = v % NV;
                union { u32x4 v4; T e[VE]; } u;
                const int n = n0 + nv * VE;
                if (n + VE <= p.N) {
                    u.v4 = *reinterpret_cast<const u32x4*>(W + (int64_t)(k0 + k) * p.N + n);
                } else {
#pragma unroll
                    for (int i = 0; i < VE; ++i) u.e[i] = W[(int64_t)(k0 + k) * p.N + (n + i < p.N ? n + i : p.N - 1)];
                }
#pragma unroll
                for (int i = 0; i < VE; ++i) {
                    const int r = nv * VE + i;
                    reinterpret_cast<T*>(Bs + moe_lds_off<T>(r, k / VE))[k % VE] = u.e[i];
                }
            }
        }
        __syncthreads();
        // ---- MFMA over the stage -----------------------------------------------------------
        if constexpr (WIDE) {
#pragma unroll
            for (int kc = 0; kc < MOE_KT; kc += 16) {
                typename MmaW<T>::frag af[2], bf[2];
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    af[i] = *reinterpret_cast<const typename MmaW<T>::frag*>(As + moe_lds_off<T>(wm * 64 + i * 32 + l32, kc / VE + h2));
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    bf[t] = *reinterpret_cast<const typename MmaW<T>::frag*>(Bs + moe_lds_off<T>(wn * 64 + t * 32 + l32, kc / VE + h2));
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int t = 0; t < 2; ++t) accw[i][t] = MmaW<T>::mma(bf[t], af[i], accw[i][t]);
            }
        } else {
#pragma unroll
            for (int kc = 0; kc < MOE_KT; kc += 16) {
                typename Mma16<T>::frag af[4], bf[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    af[i] = *reinterpret_cast<const typename Mma16<T>::frag*>(As + moe_lds_off<T>(wm * 64 + i * 16 + r16, kc / VE + g4));
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    bf[t] = *reinterpret_cast<const typename Mma16<T>::frag*>(Bs + moe_lds_off<T>(wn * 64 + t * 16 + r16, kc / VE + g4));
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[i][t] = Mma16<T>::mma(bf[t], af[i], acc[i][t]);
            }
        }
        __syncthreads();
    }

    // ---- scatter the rows back (fp32: lane holds out[m = i*16 + r16][n = t*16 + g4*4 .. +3]) ----
    T* out = reinterpret_cast<T*>(p.out);
    if constexpr (sizeof(T) == 2) {
        // 16-bit outputs leave through LDS (free after the last barrier): the wavefront's
        // 64 x 64 tile is laid out as 64 rows of 128 bytes (chunks XOR-swizzled by the
        // row), then every store instruction writes eight complete 128-byte row segments
        // instead of sixteen 32-byte pieces.
        // lane holds out[m = i*32 + lane%32][n = t*32 + 8*jj + 4*(lane/32) + q] in accw[i][t][4*jj + q]
        char* ep = smem + wave * (64 * 128);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    T vals[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(accw[i][t][4 * jj + q]);
                    const int row = i * 32 + l32;
                    const int chunk = t * 4 + jj;
                    *reinterpret_cast<uint64_t*>(ep + row * 128 + ((chunk ^ (row & 7)) << 4) + h2 * 8) =
                        *reinterpret_cast<const uint64_t*>(vals);
                }
        // LDS operations of one wavefront complete in order: no barrier needed
        const int c = lane & 7;
        const int n = n0 + wn * 64 + c * 8;
        // the tokens of the lane's rows, fetched together ahead of the stores (a load between
        // two stores waits for the store before it as well)
        int toks[8];
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) {
            const int r = wm * 64 + pass * 8 + (lane >> 3);
            toks[pass] = r < rows ? p.token_perm[row0 + r] : -1;
        }
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) {
            const int row = pass * 8 + (lane >> 3);
            const u32x4 v = *reinterpret_cast<const u32x4*>(ep + row * 128 + ((c ^ (row & 7)) << 4));
            if (toks[pass] >= 0 && n < p.N) *reinterpret_cast<u32x4*>(out + (int64_t)toks[pass] * p.N + n) = v;
        }
    } else {
    int toks[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = wm * 64 + i * 16 + r16;
        toks[i] = r < rows ? p.token_perm[row0 + r] : -1;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (toks[i] < 0) continue;
        const int tok = toks[i];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int n = n0 + wn * 64 + t * 16 + g4 * 4;
            T vals[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(acc[i][t][q]);
            T* dst = out + (int64_t)tok * p.N + n;
            if (n + 4 <= p.N) {
                if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(vals);
                else *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(vals);
            } else {
                for (int q = 0; q < 4; ++q)
                    if (n + q < p.N) dst[q] = vals[q];
            }
        }
    }
    }
}

// ---- gathered GEMM with LDS-direct loads ------------------------------------------------
// Same tile lookup and LDS layout as moe_gemm_kernel (k-contiguous weights only); the
// workgroup tile is TM x TN with WAVES wavefronts (WGM of them along the rows), and the
// operands go from global memory straight into LDS (global_load_lds_dwordx4: each
// wavefront instruction writes 64 x 16 bytes to consecutive LDS addresses starting at
// M0), so no registers or LDS-store instructions are spent on staging.  NBUF LDS buffers hold stages s .. s + NBUF - 1; one barrier per
// stage.  The loads are issued through inline assembly, which keeps the compiler from
// serialising them against the fragment reads of the other buffers.

template <typename T, int TM, int TN, int WAVES, int WGM, int NBUF, int KTB, bool BKN, bool XS>
__global__ __launch_bounds__(64 * WAVES, (TM + TN) * NBUF * KTB > 80 * 1024 ? 1 : 2) void moe_gemm_direct_kernel(MoeParams p) {
    static_assert(!BKN || sizeof(T) == 2, "the [K, N] weight layout is read with 16-bit LDS transpose loads");
    static_assert(!XS || (HasMma32<T>::value && NBUF >= 3 && NBUF <= 4 && (KTB / (int)sizeof(T) / 16) % 2 == 0),
                  "the cross-stage pipeline needs 32x32 MFMAs, three or four buffers and an even number of k-steps per stage");
    constexpr int NTH = 64 * WAVES;
    constexpr int WGN = WAVES / WGM;
    constexpr int MT = TM / WGM / 16;   // 16-row tiles per wave
    constexpr int NTT = TN / WGN / 16;  // 16-column tiles per wave
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int KT = KTB / (int)sizeof(T);  // k per row and stage (KTB = 64 or 128 bytes)
    constexpr int CPR = KTB / 16;             // 16-byte chunks per LDS row
    constexpr int A_LOADS = TM * CPR / NTH;
    constexpr int B_LOADS = TN * CPR / NTH;
    constexpr int RSTEP = NTH / CPR;          // tile rows between a thread's vectors
    constexpr int A_BYTES = TM * KTB;
    constexpr int BUF = (TM + TN) * KTB;
    // chunk c of row r sits at position c ^ swz(r): rows of 128 bytes use the low three bits
    // of the row, rows of 64 bytes bits 2..3 (sixteen lanes of a 16-byte read then touch
    // sixteen different 16-byte bank groups)
    auto swz = [](int row) { return KTB == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3); };
    auto lds_off = [&](int row, int chunk) { return (row * CPR + (chunk ^ swz(row))) * 16; };
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) char smem[];
    __shared__ int s_expert, s_row0, s_rows;

    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        int found_e, found_row0, found_rows;
        moe_find_tile<TM>(p, blockIdx.y, lane, found_e, found_row0, found_rows);
        if (lane == 0) { s_expert = found_e; s_row0 = found_row0; s_rows = found_rows; }
    }
    __syncthreads();
    const int expert = s_expert;
    if (expert < 0) return;
    const int row0 = s_row0, rows = s_rows;
    const int n0 = blockIdx.x * TN;
    if (expert == p.n_exp) {  // tokens without a valid expert id: zero rows
        moe_zero_tile<T>(p, row0, rows, n0, TN, NTH);
        return;
    }

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int wm = wave / WGN, wn = wave % WGN;
    const int wrow = wm * (TM / WGM), wcol = wn * (TN / WGN);
    // a partly filled tile: wavefronts whose rows are all past its end load their share of the
    // stages and meet the barriers, but read no fragments, issue no MFMAs and store nothing
    const bool active = __builtin_amdgcn_readfirstlane(wrow) < rows;

    const T* X = reinterpret_cast<const T*>(p.tokens);
    const T* W = reinterpret_cast<const T*>(p.weight) + (int64_t)expert * p.K * p.N;

    // staging map: every wavefront instruction fills 1 KB of consecutive LDS rows (8 or 16);
    // lane l lands at position l % CPR of row l / CPR, so it fetches the chunk that the
    // swizzle keeps at that position
    const int srow = threadIdx.x / CPR;
    const int chunk = (threadIdx.x % CPR) ^ swz(srow);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const uint32_t st_dst = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
    const T* a_src[A_LOADS];
#pragma unroll
    for (int q = 0; q < A_LOADS; ++q) {
        const int r = srow + RSTEP * q;
        const int tok = p.token_perm[row0 + (r < rows ? r : rows - 1)];
        a_src[q] = X + (int64_t)tok * p.K + chunk * VE;
    }
    // Weight tile.  [N, K] storage (k contiguous): rows of KTB bytes like the token tile.
    // [K, N] storage (BKN, the stacked weight.T of the reference): the stage is kept as
    // KT k-rows of TN * 2 bytes; a wavefront instruction fills 1 KB of them linearly, the
    // 32-byte units of a k-row are XOR-swizzled by twice its low two bits (the source
    // address carries the swizzle; the two 16-lane groups that read neighbouring units of
    // the same four k-rows then cover eight different units), and the k-contiguous MFMA fragments come out of LDS transpose
    // reads, sixteen lanes fetching four k-rows of sixteen columns at a time.
    constexpr int RB = TN * (int)sizeof(T);   // BKN: bytes of a k-row in LDS
    constexpr int CB = RB / 16;               // BKN: 16-byte slots of a k-row
    const T* b_src[B_LOADS];
#pragma unroll
    for (int q = 0; q < B_LOADS; ++q) {
        if constexpr (BKN) {
            const int slot = q * NTH + (int)threadIdx.x;
            const int kr = slot / CB, c = slot % CB;
            int n = n0 + ((((c >> 1) ^ ((kr & 3) << 1)) << 1) | (c & 1)) * VE;
            if (n + VE > p.N) n = p.N - VE;   // columns past the end re-read valid data; never stored
            b_src[q] = W + (int64_t)kr * p.N + n;
        } else {
            const int r = srow + RSTEP * q;
            const int n = n0 + r < p.N ? n0 + r : p.N - 1;
            b_src[q] = W + (int64_t)n * p.K + chunk * VE;
        }
    }
    // load q of stage s (q < A_LOADS: token rows, else weight rows)
    auto issue_one = [&](int s, int q) {
        const uint32_t dst = st_dst + (uint32_t)((s % NBUF) * BUF);
        const int k = s * KT;
        if (q < A_LOADS) lds_direct_load16(a_src[q] + k, dst + q * RSTEP * KTB);
        else if constexpr (BKN) lds_direct_load16(b_src[q - A_LOADS] + (int64_t)k * p.N, dst + A_BYTES + (q - A_LOADS) * NTH * 16);
        else lds_direct_load16(b_src[q - A_LOADS] + k, dst + A_BYTES + (q - A_LOADS) * RSTEP * KTB);
    };
    auto issue_stage = [&](int s) {
#pragma unroll
        for (int q = 0; q < A_LOADS + B_LOADS; ++q) issue_one(s, q);
    };

    // 2-byte types: 32 x 32 x 16 MFMAs (twice the sustained rate of the 16 x 16 x 32 ones)
    constexpr bool WIDE = HasMma32<T>::value;
    constexpr int MTW = TM / WGM / 32, NTW = TN / WGN / 32;
    const int l32 = lane & 31, h2 = lane >> 5;
    f32x4 acc[WIDE ? 1 : MT][WIDE ? 1 : NTT];
    f32x16 accw[WIDE ? MTW : 1][WIDE ? NTW : 1];
#pragma unroll
    for (int i = 0; i < (WIDE ? 1 : MT); ++i)
#pragma unroll
        for (int t = 0; t < (WIDE ? 1 : NTT); ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < (WIDE ? MTW : 1); ++i)
#pragma unroll
        for (int t = 0; t < (WIDE ? NTW : 1); ++t)
#pragma unroll
            for (int j = 0; j < 16; ++j) accw[i][t][j] = 0.f;

    const int n_st = p.K / KT;
    constexpr int L = A_LOADS + B_LOADS;   // loads per thread and stage
#pragma unroll
    for (int s0 = 0; s0 < NBUF - 1; ++s0)
        if (s0 < n_st) issue_stage(s0);

    // wait until at most `newer` stages of this thread's loads are still in flight
    auto wait_stages = [&](int newer) {
        if (NBUF > 3 && newer >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L) : "memory");
        else if (NBUF > 2 && newer == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(L) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    if constexpr (XS) {
        // Cross-stage pipeline: shallow stages (KTB bytes of k) in a ring of NBUF buffers, and the
        // barrier that publishes stage s + 1 sits ahead of the LAST k-step of stage s, whose MFMAs
        // then run over the first fragment reads of stage s + 1.  The wait for the loads, the
        // barrier and the LDS latency of a stage's first fragments - about 800 clocks that a
        // barrier at the top of the stage leaves the matrix cores idle - are covered by MFMAs
        // that are already queued.  Loads run NBUF - 1 stages ahead, so the wait is short.
        constexpr int KSTEPS = KT / 16;
        typename MmaW<T>::frag af[2][MTW], bf[2][NTW];
        auto read_frags = [&](const char* As, const char* Bs, int c, int slot) {
#pragma unroll
            for (int i = 0; i < MTW; ++i)
                af[slot][i] = *reinterpret_cast<const typename MmaW<T>::frag*>(As + lds_off(wrow + i * 32 + l32, c * 2 + h2));
#pragma unroll
            for (int t = 0; t < NTW; ++t) {
                if constexpr (BKN) {
                    typedef short s16x8_t __attribute__((ext_vector_type(8)));
                    typedef __attribute__((address_space(3))) s16x4 lds_s16x4_t;
                    const int kr = c * 16 + 8 * h2 + (r16 >> 2);             // and kr + 4
                    const int unit = (wcol + t * 32 + 16 * ((lane >> 4) & 1)) >> 4;
                    const char* at = Bs + kr * RB + ((unit ^ ((kr & 3) << 1)) << 5) + ((r16 & 3) << 3);
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(at));
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(at + 4 * RB));
                    bf[slot][t] = __builtin_bit_cast(typename MmaW<T>::frag,
                                                     (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                } else {
                    bf[slot][t] = *reinterpret_cast<const typename MmaW<T>::frag*>(Bs + lds_off(wcol + t * 32 + l32, c * 2 + h2));
                }
            }
        };
        // The walk exists twice, with and without the fragment reads and MFMAs, chosen once per
        // wavefront: a test of `active` inside the k-steps splits them into basic blocks, and the
        // compiler then waits for ALL fragment reads in flight ahead of a step's MFMAs instead of
        // the older ones only - the reads of step c + 1 no longer run under the MFMAs of step c.
        auto walk = [&](auto act) {
        constexpr bool ACT = decltype(act)::value;
        wait_stages(n_st - 1 < NBUF - 2 ? n_st - 1 : NBUF - 2);
        __syncthreads();
        if constexpr (ACT) read_frags(smem, smem + A_BYTES, 0, 0);
        for (int s = 0; s < n_st; ++s) {
            const char* cur = smem + (s % NBUF) * BUF;
            const char* nxt = smem + ((s + 1) % NBUF) * BUF;
            const bool more = s + NBUF - 1 < n_st;
#pragma unroll
            for (int c = 0; c < KSTEPS; ++c) {
                if (c + 1 < KSTEPS) {
                    if constexpr (ACT) read_frags(cur, cur + A_BYTES, c + 1, (c + 1) & 1);
                } else if (s + 1 < n_st) {
                    // stage s + 1 has landed once only the stages after it are in flight; every
                    // fragment read of stage s has been issued by now, and is complete before
                    // the barrier lets anyone's loads into that buffer
                    const int last = s + NBUF - 1 < n_st - 1 ? s + NBUF - 1 : n_st - 1;
                    wait_stages(last - (s + 1));
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    __syncthreads();
                    if constexpr (ACT) read_frags(nxt, nxt + A_BYTES, 0, 0);
                }
                // the loads of stage s + NBUF - 1 reuse the buffer of stage s - 1, which the
                // barrier inside stage s - 1 has freed
                // (all of them in the first k-step, so that the wait above counts whole stages)
                if (more && c == 0) issue_stage(s + NBUF - 1);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (ACT) {
#pragma unroll
                    for (int i = 0; i < MTW; ++i)
#pragma unroll
                        for (int t = 0; t < NTW; ++t) accw[i][t] = MmaW<T>::mma(bf[c & 1][t], af[c & 1][i], accw[i][t]);
                }
            }
        }
        };
        if (active) walk(std::true_type{}); else walk(std::false_type{});
    } else {
    // (two copies of the walk, as above)
    auto walk = [&](auto act) {
    constexpr bool ACT = decltype(act)::value;
    for (int s = 0; s < n_st; ++s) {
        // stage s has landed once at most the loads of the stages after it are outstanding
        // (NBUF - 2 of them, fewer at the end of the walk)
        const int newer = n_st - 1 - s < NBUF - 2 ? n_st - 1 - s : NBUF - 2;
        if (NBUF > 3 && newer == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L) : "memory");
        else if (NBUF > 2 && newer == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(L) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();   // everyone's part of stage s is in LDS; the buffer of stage s - 1 is free
        // The loads of stage s + NBUF - 1 go out a few at a time between the MFMA groups of
        // this stage (16-bit types): issued in one burst right after the barrier, the
        // sixteen wavefronts queue up behind the address unit (one 1 KB instruction per 16
        // clocks) with the matrix cores idle.
        const bool more = s + NBUF - 1 < n_st;
        if (!WIDE && more) issue_stage(s + NBUF - 1);
        const char* cur = smem + (s % NBUF) * BUF;
        const char* As = cur;
        const char* Bs = cur + A_BYTES;
        if constexpr (WIDE) {
            // fragments of k-step c + 1 are read while the MFMAs of step c run
            constexpr int KSTEPS = KT / 16;
            typename MmaW<T>::frag af[2][MTW], bf[2][NTW];
            auto read_frags = [&](int c, int slot) {
#pragma unroll
                for (int i = 0; i < MTW; ++i)
                    af[slot][i] = *reinterpret_cast<const typename MmaW<T>::frag*>(As + lds_off(wrow + i * 32 + l32, c * 2 + h2));
#pragma unroll
                for (int t = 0; t < NTW; ++t) {
                    if constexpr (BKN) {
                        typedef short s16x8_t __attribute__((ext_vector_type(8)));
                        typedef __attribute__((address_space(3))) s16x4 lds_s16x4_t;
                        const int kr = c * 16 + 8 * h2 + (r16 >> 2);             // and kr + 4
                        const int unit = (wcol + t * 32 + 16 * ((lane >> 4) & 1)) >> 4;
                        const char* at = Bs + kr * RB + ((unit ^ ((kr & 3) << 1)) << 5) + ((r16 & 3) << 3);
                        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(at));
                        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(at + 4 * RB));
                        bf[slot][t] = __builtin_bit_cast(typename MmaW<T>::frag,
                                                         (s16x8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                    } else {
                        bf[slot][t] = *reinterpret_cast<const typename MmaW<T>::frag*>(Bs + lds_off(wcol + t * 32 + l32, c * 2 + h2));
                    }
                }
            };
            constexpr int LPS = (L + KSTEPS - 1) / KSTEPS;  // loads per k-step
            if constexpr (ACT) read_frags(0, 0);
#pragma unroll
            for (int c = 0; c < KSTEPS; ++c) {
                if constexpr (ACT) if (c + 1 < KSTEPS) read_frags(c + 1, (c + 1) & 1);
                if (more) {
#pragma unroll
                    for (int q = c * LPS; q < (c + 1) * LPS && q < L; ++q) issue_one(s + NBUF - 1, q);
                }
                __builtin_amdgcn_sched_barrier(0);   // the reads stay ahead of this step's MFMAs
                if constexpr (ACT) {
#pragma unroll
                    for (int i = 0; i < MTW; ++i)
#pragma unroll
                        for (int t = 0; t < NTW; ++t) accw[i][t] = MmaW<T>::mma(bf[c & 1][t], af[c & 1][i], accw[i][t]);
                }
            }
        } else if constexpr (ACT) {
#pragma unroll
            for (int kc = 0; kc < KT; kc += 16) {
                typename Mma16<T>::frag af[MT], bf[NTT];
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    af[i] = *reinterpret_cast<const typename Mma16<T>::frag*>(As + lds_off(wrow + i * 16 + r16, kc / VE + g4));
#pragma unroll
                for (int t = 0; t < NTT; ++t)
                    bf[t] = *reinterpret_cast<const typename Mma16<T>::frag*>(Bs + lds_off(wcol + t * 16 + r16, kc / VE + g4));
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int t = 0; t < NTT; ++t) acc[i][t] = Mma16<T>::mma(bf[t], af[i], acc[i][t]);
            }
        }
    }
    };
    if (active) walk(std::true_type{}); else walk(std::false_type{});
    }
    __syncthreads();   // the epilogue reuses the LDS buffers
    if (!active) return;   // no barrier follows

    T* out = reinterpret_cast<T*>(p.out);
    if constexpr (WIDE) {
        // the wavefront's (TM / WGM) x 64 tile leaves through LDS (free after the last
        // barrier) as rows of 128 bytes, chunks XOR-swizzled by the row; every store
        // instruction then writes eight complete 128-byte row segments.
        // lane holds out[m = i*32 + lane%32][n = t*32 + 8*jj + 4*(lane/32) + q] in accw[i][t][4*jj + q]
        static_assert(!WIDE || TN / WGN == 64, "epilogue assumes 64 output columns per wavefront");
        constexpr int WR = TM / WGM;
        char* ep = smem + wave * (WR * 128);
#pragma unroll
        for (int i = 0; i < MTW; ++i)
#pragma unroll
            for (int t = 0; t < NTW; ++t)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    T vals[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(accw[i][t][4 * jj + q]);
                    const int row = i * 32 + l32;
                    const int ch = t * 4 + jj;
                    *reinterpret_cast<uint64_t*>(ep + row * 128 + ((ch ^ (row & 7)) << 4) + h2 * 8) =
                        *reinterpret_cast<const uint64_t*>(vals);
                }
        const int c = lane & 7;
        const int n = n0 + wcol + c * 8;
        // The token of every row this lane stores, fetched together ahead of the stores: a
        // load placed between the stores waits for the store before it as well (one counter,
        // in order), i.e. for a write to memory and a read from it per pass.
        int toks[WR / 8];
#pragma unroll
        for (int pass = 0; pass < WR / 8; ++pass) {
            const int r = wrow + pass * 8 + (lane >> 3);
            toks[pass] = r < rows ? p.token_perm[row0 + r] : -1;
        }
#pragma unroll
        for (int pass = 0; pass < WR / 8; ++pass) {
            const int row = pass * 8 + (lane >> 3);
            const u32x4 v = *reinterpret_cast<const u32x4*>(ep + row * 128 + ((c ^ (row & 7)) << 4));
            if (toks[pass] >= 0 && n < p.N) *reinterpret_cast<u32x4*>(out + (int64_t)toks[pass] * p.N + n) = v;
        }
    } else {
    int toks[MT];   // fetched together ahead of the stores, as above
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int r = wrow + i * 16 + r16;
        toks[i] = r < rows ? p.token_perm[row0 + r] : -1;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        if (toks[i] < 0) continue;
        const int tok = toks[i];
#pragma unroll
        for (int t = 0; t < NTT; ++t) {
            const int n = n0 + wcol + t * 16 + g4 * 4;
            T vals[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(acc[i][t][q]);
            T* dst = out + (int64_t)tok * p.N + n;
            if (n + 4 <= p.N) {
                *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(vals);
            } else {
                for (int q = 0; q < 4; ++q)
                    if (n + q < p.N) dst[q] = vals[q];
            }
        }
    }
    }
}

template <typename T, int TM, int TN, int WAVES, int WGM, int NBUF, int KTB, bool BKN, bool XS>
static int launch_moe_direct_inst(const MoeParams& p, hipStream_t st) {
    // split 2 covers at most one round of 256-row tiles, as 128-row halves
    const int tiles = p.split == 2 ? 2 * p.round_rows : (p.n_tok + TM - 1) / TM + p.n_exp + 1;
    if (tiles > 65535) return fail(SPX_E_SHAPE, "too many row tiles for one launch");
    // the epilogue stages every wavefront's (TM / WGM) x 64 output tile as rows of 128 bytes
    const int epi = sizeof(T) == 2 ? WAVES * (TM / WGM) * 128 : 0;
    const int smem = NBUF * (TM + TN) * KTB > epi ? NBUF * (TM + TN) * KTB : epi;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_direct_kernel<T, TM, TN, WAVES, WGM, NBUF, KTB, BKN, XS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(moe_gemm_direct_kernel)");
    hipLaunchKernelGGL((moe_gemm_direct_kernel<T, TM, TN, WAVES, WGM, NBUF, KTB, BKN, XS>), dim3((p.N + TN - 1) / TN, tiles, 1), dim3(64 * WAVES), smem, st, p);
    SPX_LAUNCH_CHECK("moe_gemm_direct_kernel");
    return 0;
}

template <typename T, int TM, int TN, int WAVES, int WGM, int NBUF, int KTB, bool XS = false>
static int launch_moe_direct(const MoeParams& p, hipStream_t st) {
    if constexpr (XS && sizeof(T) != 2) {
        return fail(SPX_E_CONFIG, "the cross-stage pipelined tile configurations take 16-bit types");
    } else {
        if (p.w_kcontig) return launch_moe_direct_inst<T, TM, TN, WAVES, WGM, NBUF, KTB, false, XS>(p, st);
        if constexpr (sizeof(T) == 2) return launch_moe_direct_inst<T, TM, TN, WAVES, WGM, NBUF, KTB, true, XS>(p, st);
        else return fail(SPX_E_CONFIG, "fp32 weights stored [E, in, out] run through tile config 1");
    }
}

// Tokens per workgroup of the index kernels: the smallest multiple of 256 (up to MOE_CHUNK)
// whose table of (chunk, expert) counts the placement workgroups can scan themselves;
// else 256 (more beyond 262144 tokens, so that a launch has at most 1024 chunks)
// with a launch in between that scans every expert's column of the table.
static int moe_index_chunk(int n_tok, int n_exp, bool* fused) {
    for (int chunk = 256; chunk <= MOE_CHUNK; chunk += 256) {
        const int64_t n_chunk = (n_tok + chunk - 1) / chunk;
        if (n_chunk * (n_exp + 1) <= MOE_FUSED_TABLE) { *fused = true; return chunk; }
    }
    *fused = false;
    int chunk = 256;
    while ((n_tok + chunk - 1) / chunk > 1024) chunk += 256;
    return chunk;
}

// [n_chunk][n_exp + 1] counts, then the n_exp + 1 totals of the experts
static size_t moe_index_table_bytes(int n_tok, int n_exp) {
    bool fused;
    const int chunk = moe_index_chunk(n_tok, n_exp, &fused);
    const int n_chunk = (n_tok + chunk - 1) / chunk;
    return round_up((size_t)(n_chunk > 0 ? n_chunk : 1) * (n_exp + 1) * sizeof(int32_t), 256);
}

static size_t moe_index_ws(int n_tok, int n_exp) {
    return moe_index_table_bytes(n_tok, n_exp) + round_up((size_t)(n_exp + 1) * sizeof(int32_t), 256);
}

}  // namespace spx

extern "C" size_t spx_moe_index_workspace_bytes(int n_tok, int n_exp) {
    if (n_tok < 0 || n_exp <= 0 || n_exp > spx::MOE_MAX_EXP) return 0;
    return spx::moe_index_ws(n_tok, n_exp);
}

extern "C" int spx_moe_index(const int32_t* exp_ids, int n_tok, int n_exp,
                             int32_t* expert_count, int32_t* expert_offset, int32_t* token_perm,
                             void* workspace, size_t workspace_bytes, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(n_tok >= 0, SPX_E_SHAPE, "negative token count");
    SPX_REQUIRE(n_exp > 0 && n_exp <= MOE_MAX_EXP, SPX_E_SHAPE, "n_exp=%d must be in [1,%d]", n_exp, MOE_MAX_EXP);
    SPX_REQUIRE(expert_count && expert_offset && workspace, SPX_E_NULL, "expert_count, expert_offset and workspace are required");
    SPX_REQUIRE((exp_ids && token_perm) || n_tok == 0, SPX_E_NULL, "exp_ids and token_perm are required");
    SPX_REQUIRE(workspace_bytes >= moe_index_ws(n_tok, n_exp), SPX_E_WORKSPACE,
                "workspace of %zu bytes is smaller than the %zu required", workspace_bytes, moe_index_ws(n_tok, n_exp));
    SPX_REQUIRE(aligned(workspace, 256), SPX_E_ALIGN, "workspace must be 256-byte aligned");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    int32_t* partial = reinterpret_cast<int32_t*>(workspace);
    bool fused;
    const int chunk = moe_index_chunk(n_tok, n_exp, &fused);
    const int n_chunk = (n_tok + chunk - 1) / chunk;
    if (n_chunk > 0) {
        hipLaunchKernelGGL(moe_hist_kernel, dim3(n_chunk), dim3(256), (n_exp + 1) * sizeof(int), st, exp_ids, n_tok, n_exp + 1, chunk, partial);
        SPX_LAUNCH_CHECK("moe_hist_kernel");
    }
    int32_t* totals = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + moe_index_table_bytes(n_tok, n_exp));
    if (n_chunk == 0) {   // no tokens: all offsets and counts are zero (a kernel, so that the call can be captured)
        hipLaunchKernelGGL(moe_zero_index_kernel, dim3((n_exp + 1 + 255) / 256), dim3(256), 0, st, n_exp, expert_count, expert_offset);
        SPX_LAUNCH_CHECK("moe_zero_index_kernel");
        return 0;
    }
    if (!fused) {
        hipLaunchKernelGGL(moe_colscan_kernel, dim3((n_exp + 1 + 3) / 4), dim3(256), 0, st, partial, n_chunk, n_exp + 1, totals);
        SPX_LAUNCH_CHECK("moe_colscan_kernel");
    }
    const size_t smem = 6 * (n_exp + 1) * sizeof(int);
    if (fused)
        hipLaunchKernelGGL(moe_place_kernel<true>, dim3(n_chunk), dim3(256), smem, st, exp_ids, n_tok, n_exp + 1, chunk, partial,
                           totals, token_perm, expert_count, expert_offset);
    else
        hipLaunchKernelGGL(moe_place_kernel<false>, dim3(n_chunk), dim3(256), smem, st, exp_ids, n_tok, n_exp + 1, chunk, partial,
                           totals, token_perm, expert_count, expert_offset);
    SPX_LAUNCH_CHECK("moe_place_kernel");
    return 0;
}

extern "C" int spx_moe_forward(int dtype, const void* tokens, const void* weight, int weight_layout, void* out,
                               const int32_t* expert_offset, const int32_t* token_perm,
                               int n_tok, int in_dim, int out_dim, int n_exp,
                               int tile_cfg, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(tile_cfg >= 0 && tile_cfg <= 6, SPX_E_CONFIG, "unknown tile config %d", tile_cfg);
    SPX_REQUIRE(dtype == SPX_F32 || dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE, "unknown dtype %d", dtype);
    SPX_REQUIRE(n_tok >= 0 && in_dim > 0 && out_dim > 0 && n_exp > 0, SPX_E_SHAPE, "bad sizes");
    SPX_REQUIRE(weight_layout == 0 || weight_layout == 1, SPX_E_CONFIG, "weight_layout must be 0 ([E,in,out]) or 1 ([E,out,in])");
    const int es = dtype_bytes(dtype);
    SPX_REQUIRE(in_dim % (128 / es) == 0, SPX_E_SHAPE, "in_dim=%d must be a multiple of %d", in_dim, 128 / es);
    SPX_REQUIRE(out_dim % (16 / es) == 0, SPX_E_SHAPE, "out_dim=%d must be a multiple of %d", out_dim, 16 / es);
    if (n_tok == 0) return 0;
    SPX_REQUIRE(tokens && weight && out && expert_offset && token_perm, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(aligned(tokens, 16) && aligned(weight, 16) && aligned(out, 16), SPX_E_ALIGN, "buffers must be 16-byte aligned");
    MoeParams p;
    p.tokens = tokens; p.weight = weight; p.out = out;
    p.expert_offset = expert_offset; p.token_perm = token_perm;
    p.n_tok = n_tok; p.K = in_dim; p.N = out_dim; p.n_exp = n_exp;
    p.w_kcontig = weight_layout == 1;
    p.split = 0; p.round_rows = 1;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // tile_cfg 1: 128x128 tiles staged through registers (any dtype and weight layout);
    // 2 / 3 / 4: tiles filled by LDS-direct loads - 128x128 with four wavefronts (two
    // workgroups per CU), 256x256 with eight wavefronts of 128x64, 256x256 with sixteen
    // wavefronts of 64x64 - for 16-bit types in either weight layout and fp32 with
    // k-contiguous weights.  256x256 tiles move half the bytes from L2 to the CUs, which is
    // what bounds the 128x128 kernel.  5 = 4 for the whole rounds of 256-row tiles plus 2 for
    // the row tiles of a thinly filled last round (two launches, see moe_find_tile).  0 picks
    // between 5, 4 and 2 by the number of 256x256 tiles (below); fp32 [E, in, out] weights take 1.
    const bool direct_ok = p.w_kcontig || es == 2;
    static int n_cu = 0;
    if (n_cu == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) n_cu = prop.multiProcessorCount;
        if (n_cu <= 0) n_cu = 256;
    }
    if (tile_cfg == 0) {
        // 16-bit types: 256x256 tiles from 256 of them on (split launch, 5); from 128 on when
        // all of them, the partly filled ones at the expert boundaries included, run in a
        // single round (4: ten mid-size problems measured 10 - 25 % ahead of the 128x128
        // tiles there, and behind them as soon as a second round starts); else 128x128
        const int64_t row_tiles = (n_tok + 255) / 256, col_tiles = (out_dim + 255) / 256;
        const int64_t big_tiles = row_tiles * col_tiles;
        if (!direct_ok) tile_cfg = 1;
        else if (es == 2 && big_tiles >= 256) tile_cfg = 5;
        else if (es == 2 && big_tiles >= 128 && (row_tiles + n_exp) * col_tiles <= n_cu) tile_cfg = 4;
        else tile_cfg = 2;
    }
    if (tile_cfg >= 2) {
        SPX_REQUIRE(direct_ok, SPX_E_CONFIG, "tile config %d takes fp32 weights in layout 1 only", tile_cfg);
        if (tile_cfg == 5) {
            const int ntn = (out_dim + 255) / 256;
            p.round_rows = n_cu / ntn > 0 ? n_cu / ntn : 1;
        }
#define SPX_MOE_DIRECT(T)                                                                  \
        if (tile_cfg == 5) {                                                               \
            p.split = 1;                                                                   \
            const int rc = launch_moe_direct<T, 256, 256, 16, 4, 2, 128>(p, st);           \
            if (rc) return rc;                                                             \
            p.split = 2;                                                                   \
            return launch_moe_direct<T, 128, 128, 4, 2, 2, 128>(p, st);                    \
        }                                                                                  \
        if (tile_cfg == 6) return launch_moe_direct<T, 256, 256, 16, 4, 4, 64, true>(p, st); \
        if (tile_cfg == 2) return launch_moe_direct<T, 128, 128, 4, 2, 2, 128>(p, st);     \
        if (tile_cfg == 3) return launch_moe_direct<T, 256, 256, 8, 2, 2, 128>(p, st);     \
        return launch_moe_direct<T, 256, 256, 16, 4, 2, 128>(p, st);
        switch (dtype) {
            case SPX_F32: SPX_MOE_DIRECT(float)
            case SPX_F16: SPX_MOE_DIRECT(_Float16)
            default: SPX_MOE_DIRECT(bf16_t)
        }
#undef SPX_MOE_DIRECT
    }
    const int max_tiles = (n_tok + MOE_TM - 1) / MOE_TM + n_exp + 1;
    SPX_REQUIRE(max_tiles <= 65535, SPX_E_SHAPE, "too many row tiles for one launch");
    dim3 grid((out_dim + MOE_TN - 1) / MOE_TN, max_tiles, 1);
    const size_t smem = 2 * (size_t)MOE_TM * 128;
    switch (dtype) {
        case SPX_F32: hipLaunchKernelGGL(moe_gemm_kernel<float>, grid, dim3(256), smem, st, p); break;
        case SPX_F16: hipLaunchKernelGGL(moe_gemm_kernel<_Float16>, grid, dim3(256), smem, st, p); break;
        default: hipLaunchKernelGGL(moe_gemm_kernel<bf16_t>, grid, dim3(256), smem, st, p); break;
    }
    SPX_LAUNCH_CHECK("moe_gemm_kernel");
    return 0;
}
