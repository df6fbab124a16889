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
    const int32_t* row_ptr;  // optional: enables the XCD-aware assignment of blocks to workgroups
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

// Which live block a workgroup computes.  Workgroup L of a launch runs on XCD L % 8, each
// with its own L2.  With row_ptr at hand, XCD x takes the blocks of the x-th band of
// block rows (a contiguous range of the BCSR order) one after the other, so an A panel is
// fetched into one L2 only and consecutive workgroups of an XCD reuse it; B panels are
// shared by the blocks of the band.  Every XCD still gets the same number of workgroups:
// those left over in short bands take the surplus of long ones.  Returns -1 for none.
template <int BM>
__device__ __forceinline__ int dds_block_of_workgroup(const DdsParams& p) {
    const int L = blockIdx.x;
    if (!p.row_ptr) return (p.nnz_dev && L >= p.nnz_dev[0]) ? -1 : L;
    const int R = p.M / BM;
    const int n_pos = gridDim.x;
    const int x = L & 7, t = L >> 3;
    int start[9];
#pragma unroll
    for (int y = 0; y <= 8; ++y) start[y] = p.row_ptr[(int)((int64_t)y * R / 8)];
    if (t < start[x + 1] - start[x]) return start[x] + t;
    int q = t - (start[x + 1] - start[x]);  // rank among the workgroups without a band block
#pragma unroll
    for (int y = 0; y < 8; ++y) {
        const int idle = (n_pos - y + 7) / 8 - (start[y + 1] - start[y]);
        if (y < x && idle > 0) q += idle;
    }
#pragma unroll
    for (int y = 0; y < 8; ++y) {
        const int slots = (n_pos - y + 7) / 8;
        const int surplus = start[y + 1] - start[y] - slots;
        if (surplus > 0) {
            if (q < surplus) return start[y] + slots + q;
            q -= surplus;
        }
    }
    return -1;
}

// Epilogue shared by both kernels: the accumulators meet in LDS as fp32 (one copy per
// k part), each thread then sums, adds the bias and stores 16 bytes of one output row.
template <typename T, int BM, int BN, typename Acc>
__device__ __forceinline__ void dds_epilogue(const DdsParams& p, const Acc& acc, float* Ef, int i, int bi, int bj,
                                             int64_t b, int wgm, int wgn, int kpart, int r16, int g4) {
    typedef DdsWaveGrid<BM / 16, BN / 16> G;
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int LDE = BN + 4;  // keeps 16-byte alignment of a row, shifts rows by four banks
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
    constexpr int VPR = BN / VE;  // 16-byte vectors per output row
    for (int v = threadIdx.x; v < BM * VPR; v += 256) {
        const int m = v / VPR;
        const int n = (v - m * VPR) * VE;
        float s[VE];
#pragma unroll
        for (int e = 0; e < VE; ++e) s[e] = 0.f;
#pragma unroll
        for (int kp = 0; kp < G::KS; ++kp) {
#pragma unroll
            for (int e = 0; e < VE; e += 4) {
                const f32x4 part = *reinterpret_cast<const f32x4*>(Ef + (kp * BM + m) * LDE + n + e);
                s[e] += part[0]; s[e + 1] += part[1]; s[e + 2] += part[2]; s[e + 3] += part[3];
            }
        }
        if (biasT) {
#pragma unroll
            for (int e = 0; e < VE; ++e) s[e] += Elem<T>::to_float(biasT[bj * BN + n + e]);
        }
        union { vec16 q; T t[VE]; } u;
#pragma unroll
        for (int e = 0; e < VE; ++e) u.t[e] = Elem<T>::from_float(s[e]);
        const int64_t off = p.compressed ? (int64_t)i * (BM * BN) + m * BN + n
                                         : ((int64_t)bi * BM + m) * p.N + (int64_t)bj * BN + n;
        store16_stream(C + off, u.q);   // written once: leave the operand panels in L2
    }
}

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

    const int i = dds_block_of_workgroup<BM>(p);
    if (i < 0) return;
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

    dds_epilogue<T, BM, BN>(p, acc, reinterpret_cast<float*>(smem), i, bi, bj, b, wgm, wgn, kpart, r16, g4);
}

// ---- pipelined variant -----------------------------------------------------------------
// A live block is a skinny product (BM x K by K x BN): almost no arithmetic per byte, so
// the kernel is a data mover and wants many bytes in flight.  Each thread keeps NST
// stages of its 16-byte pieces of the A and B panels in registers (issued NST steps
// ahead, unconditionally, so the compiler keeps them asynchronous), drops the oldest
// into one of two LDS buffers and the MFMAs read it after a single barrier per stage.
// Needs k-contiguous A and B and K a multiple of the stage depth.
template <int BM, int BN> struct DdsPipeCfg {
    static constexpr int STAGE_BYTES = BM + BN == 128 ? 128 : 256;
    static constexpr int NST = BM + BN <= 32 ? 4 : (BM + BN == 64 || BM + BN == 128 ? 3 : 2);
};

template <typename T, int BM, int BN, int NST>
__global__ __launch_bounds__(256) void dds_pipe_kernel(DdsParams p) {
    constexpr int MT = BM / 16, NT = BN / 16;
    typedef DdsWaveGrid<MT, NT> G;
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int SB = DdsPipeCfg<BM, BN>::STAGE_BYTES;  // bytes of k per row and stage
    constexpr int KT = SB / (int)sizeof(T);
    constexpr int LDK = KT + VE;
    constexpr int KW = KT / G::KS;
    constexpr int CH = SB / 16;                     // 16-byte chunks per row and stage
    constexpr int RP = 256 / CH;                    // panel rows per pass of the workgroup
    constexpr int NV = (BM + BN) / RP;              // 16-byte vectors per thread and stage
    static_assert((BM + BN) % RP == 0, "panel rows do not split over the workgroup");
    constexpr int BUF = (BM + BN) * LDK * (int)sizeof(T);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) char smem[];

    const int i = dds_block_of_workgroup<BM>(p);
    if (i < 0) return;
    const int code = p.idx[i];
    const int bi = (code >> 16) & 0xffff;
    const int bj = code & 0xffff;
    const int64_t b = blockIdx.y;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int wt = wave % (G::WGM * G::WGN);
    const int kpart = wave / (G::WGM * G::WGN);
    const int wgm = wt / G::WGN;
    const int wgn = wt % G::WGN;

    const T* A = reinterpret_cast<const T*>(p.A) + b * p.a_batch;
    const T* B = reinterpret_cast<const T*>(p.B) + b * p.b_batch;

    // staging map: vector v = tid + 256 u covers panel row tid / CH + RP u, bytes (tid % CH) * 16;
    // panel rows 0 .. BM-1 are A rows, the rest B rows
    const int st_row = threadIdx.x / CH, st_chunk = threadIdx.x % CH;
    const T* src[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int row = st_row + RP * u;
        src[u] = (row < BM ? A + ((int64_t)bi * BM + row) * p.a_ld : B + ((int64_t)bj * BN + row - BM) * p.b_ld) + st_chunk * VE;
    }
    const int st_dst = (st_row * LDK + st_chunk * VE) * (int)sizeof(T);

    f32x4 acc[G::WTM][G::WTN];
#pragma unroll
    for (int x = 0; x < G::WTM; ++x)
#pragma unroll
        for (int y = 0; y < G::WTN; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int n_st = p.K / KT;
    // The workgroups of one XCD walk k in step (they share panels through its L2); the
    // XCDs start at staggered depths, so that at any time the chip reads eight different
    // column ranges of the row-major operands rather than one (rows are a power of two
    // apart, which would keep hitting the same memory channels).
    const int rot = (int)(((int64_t)(blockIdx.x & 7) * n_st) >> 3);
    u32x4 ring[NST][NV];
#pragma unroll
    for (int r = 0; r < NST; ++r) {
        int st0 = (r < n_st ? r : n_st - 1) + rot;
        st0 = st0 >= n_st ? st0 - n_st : st0;
        const int k0 = st0 * KT;
#pragma unroll
        for (int u = 0; u < NV; ++u) ring[r][u] = *reinterpret_cast<const u32x4*>(src[u] + k0);
    }
    for (int it = 0; it < n_st; it += NST) {
#pragma unroll
        for (int r = 0; r < NST; ++r) {
            const int s = it + r;
            char* buf = smem + (s & 1) * BUF;
            if (s < n_st) {
#pragma unroll
                for (int u = 0; u < NV; ++u)
                    *reinterpret_cast<u32x4*>(buf + st_dst + u * RP * LDK * (int)sizeof(T)) = ring[r][u];
            }
            {   // refill the slot NST stages ahead (clamped: the extra copies are never used)
                int st1 = (s + NST < n_st ? s + NST : n_st - 1) + rot;
                st1 = st1 >= n_st ? st1 - n_st : st1;
                const int k0 = st1 * KT;
#pragma unroll
                for (int u = 0; u < NV; ++u) ring[r][u] = *reinterpret_cast<const u32x4*>(src[u] + k0);
            }
            if (s < n_st) {
                __syncthreads();
                const T* a_base = reinterpret_cast<const T*>(buf) + (wgm * G::WTM * 16 + r16) * LDK + kpart * KW;
                const T* b_base = reinterpret_cast<const T*>(buf) + (BM + wgn * G::WTN * 16 + r16) * LDK + kpart * KW;
                if constexpr (HasMma32<T>::value) {
#pragma unroll
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
#pragma unroll
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
            }
        }
    }
    __syncthreads();  // all fragments are consumed before the buffers are reused

    dds_epilogue<T, BM, BN>(p, acc, reinterpret_cast<float*>(smem), i, bi, bj, b, wgm, wgn, kpart, r16, g4);
}

template <typename T, int BM, int BN>
static int launch_dds_pipe_inst(const DdsParams& p, int nnz_bound, int batch, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int KT = DdsPipeCfg<BM, BN>::STAGE_BYTES / (int)sizeof(T);
    constexpr int NST = DdsPipeCfg<BM, BN>::NST;
    typedef DdsWaveGrid<BM / 16, BN / 16> G;
    size_t smem = 2 * (size_t)(BM + BN) * (KT + VE) * sizeof(T);
    size_t epi = (size_t)G::KS * BM * (BN + 4) * sizeof(float);
    if (epi > smem) smem = epi;
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dds_pipe_kernel<T, BM, BN, NST>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(dds_pipe_kernel)");
    }
    hipLaunchKernelGGL((dds_pipe_kernel<T, BM, BN, NST>), dim3(nnz_bound, batch, 1), dim3(256), smem, st, p);
    SPX_LAUNCH_CHECK("dds_pipe_kernel");
    return 0;
}

// ---- pipelined variant for operands stored the other way round ---------------------------
// A is [K, M] and B is [K, N] (m / n contiguous): the layout of the weight gradient
// grad_W = grad_y^T x.  Same register ring and two LDS buffers; a stage keeps KT k-rows
// of the A and of the B panel as they are in memory ([k][m], [k][n]), and the
// k-contiguous MFMA fragments come from the LDS transpose read of gfx950 for the 16-bit
// types (lane i of a 16-lane group addresses 4 entries of k-row i/4, lane j receives
// column j of the four rows) or from four 4-byte reads for fp32.
// AT / BT say which of the two is stored that way; an operand with the flag off is
// k-contiguous ([M, K] / [N, K]), kept as [m][k] rows in its part of the stage and read
// with plain 16-byte fragment loads as in dds_pipe_kernel - the mixed layouts of a plain
// C = A B (A [M, K], B [K, N]) and of C = A^T B^T.
template <typename T, int BM, int BN, int NST, bool AT = true, bool BT = true>
__global__ __launch_bounds__(256) void dds_pipe_t_kernel(DdsParams p) {
    constexpr int MT = BM / 16, NT = BN / 16;
    typedef DdsWaveGrid<MT, NT> G;
    constexpr int ES = (int)sizeof(T);
    constexpr int VE = 16 / ES;
    constexpr int KT = DdsPipeCfg<BM, BN>::STAGE_BYTES / ES;   // k per stage
    constexpr int KW = KT / G::KS;
    constexpr int LDA = (AT ? BM : KT) + VE, LDB = (BT ? BN : KT) + VE;   // row pitches (elements)
    constexpr int A_ROWS = AT ? KT : BM, B_ROWS = BT ? KT : BN;           // LDS rows of the two parts
    constexpr int A_BYTES = A_ROWS * LDA * ES;
    constexpr int BUF = A_BYTES + B_ROWS * LDB * ES;
    constexpr int CA = (AT ? BM : KT) / VE, CB = (BT ? BN : KT) / VE;     // 16-byte chunks per row
    constexpr int NA = A_ROWS * CA;                            // chunks of the A part
    constexpr int NV = (NA + B_ROWS * CB) / 256;
    static_assert((NA + B_ROWS * CB) % 256 == 0, "stage does not split over the workgroup");
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    const int i = dds_block_of_workgroup<BM>(p);
    if (i < 0) return;
    const int code = p.idx[i];
    const int bi = (code >> 16) & 0xffff;
    const int bj = code & 0xffff;
    const int64_t b = blockIdx.y;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int wt = wave % (G::WGM * G::WGN);
    const int kpart = wave / (G::WGM * G::WGN);
    const int wgm = wt / G::WGN;
    const int wgn = wt % G::WGN;

    const T* A = reinterpret_cast<const T*>(p.A) + b * p.a_batch + (int64_t)bi * BM * (AT ? 1 : p.a_ld);
    const T* B = reinterpret_cast<const T*>(p.B) + b * p.b_batch + (int64_t)bj * BN * (BT ? 1 : p.b_ld);

    // staging map: chunk v = tid + 256 u; the first NA chunks are (row, piece) of the A part
    // (k-rows, or rows of the block with the stage's k range), the rest of the B part
    const T* src[NV];
    int64_t sstep[NV];
    int dst[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int v = threadIdx.x + 256 * u;
        if (v < NA) {
            const int r = v / CA, c = v % CA;
            src[u] = A + (int64_t)r * p.a_ld + c * VE;
            sstep[u] = AT ? (int64_t)KT * p.a_ld : (int64_t)KT;
            dst[u] = (r * LDA + c * VE) * ES;
        } else {
            const int w = v - NA;
            const int r = w / CB, c = w % CB;
            src[u] = B + (int64_t)r * p.b_ld + c * VE;
            sstep[u] = BT ? (int64_t)KT * p.b_ld : (int64_t)KT;
            dst[u] = A_BYTES + (r * LDB + c * VE) * ES;
        }
    }

    f32x4 acc[G::WTM][G::WTN];
#pragma unroll
    for (int x = 0; x < G::WTM; ++x)
#pragma unroll
        for (int y = 0; y < G::WTN; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int n_st = p.K / KT;
    const int rot = (int)(((int64_t)(blockIdx.x & 7) * n_st) >> 3);  // XCDs start at staggered depths
    u32x4 ring[NST][NV];
#pragma unroll
    for (int r = 0; r < NST; ++r) {
        int st0 = (r < n_st ? r : n_st - 1) + rot;
        st0 = st0 >= n_st ? st0 - n_st : st0;
#pragma unroll
        for (int u = 0; u < NV; ++u) ring[r][u] = *reinterpret_cast<const u32x4*>(src[u] + st0 * sstep[u]);
    }
    // fragment bases inside a buffer (bytes)
    const int a_tr = ((g4 * 8 + (r16 >> 2)) * LDA + (wgm * G::WTM * 16 + (r16 & 3) * 4)) * ES;
    const int b_tr = A_BYTES + ((g4 * 8 + (r16 >> 2)) * LDB + (wgn * G::WTN * 16 + (r16 & 3) * 4)) * ES;
    const int a_f32 = ((g4 * 4) * LDA + wgm * G::WTM * 16 + r16) * ES;
    const int b_f32 = A_BYTES + ((g4 * 4) * LDB + wgn * G::WTN * 16 + r16) * ES;
    // k-contiguous parts: row r16 of the wavefront's first tile, element 0 of the row
    const int a_row = ((wgm * G::WTM * 16 + r16) * LDA) * ES;
    const int b_row = A_BYTES + ((wgn * G::WTN * 16 + r16) * LDB) * ES;
    for (int it = 0; it < n_st; it += NST) {
#pragma unroll
        for (int r = 0; r < NST; ++r) {
            const int s = it + r;
            char* buf = smem + (s & 1) * BUF;
            if (s < n_st) {
#pragma unroll
                for (int u = 0; u < NV; ++u) *reinterpret_cast<u32x4*>(buf + dst[u]) = ring[r][u];
            }
            {   // refill the slot NST stages ahead (clamped: the extra copies are never used)
                int st1 = (s + NST < n_st ? s + NST : n_st - 1) + rot;
                st1 = st1 >= n_st ? st1 - n_st : st1;
#pragma unroll
                for (int u = 0; u < NV; ++u) ring[r][u] = *reinterpret_cast<const u32x4*>(src[u] + st1 * sstep[u]);
            }
            if (s < n_st) {
                __syncthreads();
                if constexpr (HasMma32<T>::value) {
                    typedef typename Mma32<T>::frag Frag;
#pragma unroll
                    for (int kc = 0; kc < KW; kc += 32) {
                        const int kb = kpart * KW + kc;
                        Frag af[G::WTM], bf[G::WTN];
#pragma unroll
                        for (int x = 0; x < G::WTM; ++x) {
                            if constexpr (AT) {
                                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + a_tr + (kb * LDA + x * 16) * ES));
                                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + a_tr + ((kb + 4) * LDA + x * 16) * ES));
                                af[x] = __builtin_bit_cast(Frag, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                            } else {
                                af[x] = Mma32<T>::load(reinterpret_cast<const T*>(buf + a_row) + x * 16 * LDA + kb + g4 * 8);
                            }
                        }
#pragma unroll
                        for (int y = 0; y < G::WTN; ++y) {
                            if constexpr (BT) {
                                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + b_tr + (kb * LDB + y * 16) * ES));
                                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(buf + b_tr + ((kb + 4) * LDB + y * 16) * ES));
                                bf[y] = __builtin_bit_cast(Frag, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                            } else {
                                bf[y] = Mma32<T>::load(reinterpret_cast<const T*>(buf + b_row) + y * 16 * LDB + kb + g4 * 8);
                            }
                        }
#pragma unroll
                        for (int x = 0; x < G::WTM; ++x)
#pragma unroll
                            for (int y = 0; y < G::WTN; ++y) acc[x][y] = Mma32<T>::mma(af[x], bf[y], acc[x][y]);
                    }
                } else {
#pragma unroll
                    for (int kc = 0; kc < KW; kc += 16) {
                        const int kb = kpart * KW + kc;
                        typename Mma16<T>::frag af[G::WTM], bf[G::WTN];
#pragma unroll
                        for (int x = 0; x < G::WTM; ++x) {
                            if constexpr (AT) {
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    af[x][j] = *reinterpret_cast<const float*>(buf + a_f32 + ((kb + j) * LDA + x * 16) * ES);
                            } else {
                                af[x] = Mma16<T>::load(reinterpret_cast<const T*>(buf + a_row) + x * 16 * LDA + kb + g4 * 4);
                            }
                        }
#pragma unroll
                        for (int y = 0; y < G::WTN; ++y) {
                            if constexpr (BT) {
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    bf[y][j] = *reinterpret_cast<const float*>(buf + b_f32 + ((kb + j) * LDB + y * 16) * ES);
                            } else {
                                bf[y] = Mma16<T>::load(reinterpret_cast<const T*>(buf + b_row) + y * 16 * LDB + kb + g4 * 4);
                            }
                        }
#pragma unroll
                        for (int x = 0; x < G::WTM; ++x)
#pragma unroll
                            for (int y = 0; y < G::WTN; ++y) acc[x][y] = Mma16<T>::mma(af[x], bf[y], acc[x][y]);
                    }
                }
            }
        }
    }
    __syncthreads();  // all fragments are consumed before the buffers are reused
    dds_epilogue<T, BM, BN>(p, acc, reinterpret_cast<float*>(smem), i, bi, bj, b, wgm, wgn, kpart, r16, g4);
}

template <typename T, int BM, int BN, bool AT = true, bool BT = true>
static int launch_dds_pipe_t_inst(const DdsParams& p, int nnz_bound, int batch, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int KT = DdsPipeCfg<BM, BN>::STAGE_BYTES / (int)sizeof(T);
    constexpr int NST = DdsPipeCfg<BM, BN>::NST;
    typedef DdsWaveGrid<BM / 16, BN / 16> G;
    constexpr size_t a_part = AT ? (size_t)KT * (BM + VE) : (size_t)BM * (KT + VE);
    constexpr size_t b_part = BT ? (size_t)KT * (BN + VE) : (size_t)BN * (KT + VE);
    size_t smem = 2 * (a_part + b_part) * sizeof(T);
    size_t epi = (size_t)G::KS * BM * (BN + 4) * sizeof(float);
    if (epi > smem) smem = epi;
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dds_pipe_t_kernel<T, BM, BN, NST, AT, BT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(dds_pipe_t_kernel)");
    }
    hipLaunchKernelGGL((dds_pipe_t_kernel<T, BM, BN, NST, AT, BT>), dim3(nnz_bound, batch, 1), dim3(256), smem, st, p);
    SPX_LAUNCH_CHECK("dds_pipe_t_kernel");
    return 0;
}

// ---- short-K variant: one workgroup per block row ------------------------------------------
// When the whole K fits one or two stages (attention scores: K = head dimension) a block
// is a single load -> MFMA -> store chain and the one-block-per-workgroup kernels are
// bound by that latency.  Here a workgroup owns a block row: its A panel is staged once,
// the B panel of the next live block travels in registers while the current one is
// computed from one of two LDS buffers, and every block leaves through the shared
// epilogue.  Needs row_ptr, k-contiguous operands and K * sizeof(T) of 128 or 256 bytes.
template <typename T, int BM, int BN, int KB>
__global__ __launch_bounds__(256) void dds_row_kernel(DdsParams p) {
    constexpr int MT = BM / 16, NT = BN / 16;
    typedef DdsWaveGrid<MT, NT> G;
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int K = KB / (int)sizeof(T);
    constexpr int LDK = K + VE;
    constexpr int KW = K / G::KS;
    constexpr int CH = KB / 16;                     // 16-byte chunks per row
    constexpr int RP = 256 / CH;                    // panel rows per pass of the workgroup
    constexpr int NVA = BM / RP, NVB = BN / RP;     // vectors per thread for an A / a B panel
    static_assert(BM % RP == 0 && BN % RP == 0 && KW % 16 == 0 && G::KS == 1, "panel does not split over the workgroup");
    constexpr int PANEL_A = BM * LDK * (int)sizeof(T), PANEL_B = BN * LDK * (int)sizeof(T);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) char smem[];
    T* As = reinterpret_cast<T*>(smem);
    float* Ef = reinterpret_cast<float*>(smem + PANEL_A + 2 * PANEL_B);

    const int bi = blockIdx.x;
    const int e_begin = p.row_ptr[bi], e_end = p.row_ptr[bi + 1];
    if (e_begin >= e_end) return;
    const int64_t b = blockIdx.y;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;
    const int wt = wave % (G::WGM * G::WGN);
    const int kpart = wave / (G::WGM * G::WGN);
    const int wgm = wt / G::WGN;
    const int wgn = wt % G::WGN;

    const T* A = reinterpret_cast<const T*>(p.A) + b * p.a_batch;
    const T* B = reinterpret_cast<const T*>(p.B) + b * p.b_batch;

    const int st_row = threadIdx.x / CH, st_chunk = threadIdx.x % CH;
    const int st_dst = (st_row * LDK + st_chunk * VE) * (int)sizeof(T);
#pragma unroll
    for (int u = 0; u < NVA; ++u)
        *reinterpret_cast<u32x4*>(smem + st_dst + u * RP * LDK * (int)sizeof(T)) =
            *reinterpret_cast<const u32x4*>(A + ((int64_t)bi * BM + st_row + RP * u) * p.a_ld + st_chunk * VE);

    u32x4 rb[NVB];
    int bj = p.idx[e_begin] & 0xffff;
    int bj_next = p.idx[e_begin + 1 < e_end ? e_begin + 1 : e_begin] & 0xffff;
#pragma unroll
    for (int u = 0; u < NVB; ++u)
        rb[u] = *reinterpret_cast<const u32x4*>(B + ((int64_t)bj * BN + st_row + RP * u) * p.b_ld + st_chunk * VE);

    for (int e = e_begin; e < e_end; ++e) {
        char* bbuf = smem + PANEL_A + ((e - e_begin) & 1) * PANEL_B;
#pragma unroll
        for (int u = 0; u < NVB; ++u) *reinterpret_cast<u32x4*>(bbuf + st_dst + u * RP * LDK * (int)sizeof(T)) = rb[u];
        const int bj_cur = bj;
        // next live block of the row (the last step re-reads its own panel; the copy is not used)
        bj = bj_next;
        bj_next = p.idx[e + 2 < e_end ? e + 2 : e_end - 1] & 0xffff;
#pragma unroll
        for (int u = 0; u < NVB; ++u)
            rb[u] = *reinterpret_cast<const u32x4*>(B + ((int64_t)bj * BN + st_row + RP * u) * p.b_ld + st_chunk * VE);
        __syncthreads();   // panels complete; the previous block's epilogue reads are done

        f32x4 acc[G::WTM][G::WTN];
#pragma unroll
        for (int x = 0; x < G::WTM; ++x)
#pragma unroll
            for (int y = 0; y < G::WTN; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};
        const T* a_base = As + (wgm * G::WTM * 16 + r16) * LDK + kpart * KW;
        const T* b_base = reinterpret_cast<const T*>(bbuf) + (wgn * G::WTN * 16 + r16) * LDK + kpart * KW;
        if constexpr (HasMma32<T>::value && KW % 32 == 0) {
#pragma unroll
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
#pragma unroll
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
        // 16-byte stores of complete output rows through the shared epilogue (direct 8-byte
        // stores from the accumulators were 15 % slower)
        dds_epilogue<T, BM, BN>(p, acc, Ef, e, bi, bj_cur, b, wgm, wgn, kpart, r16, g4);
    }
}

template <typename T, int BM, int BN, int KB>
static int launch_dds_row_inst(const DdsParams& p, int batch, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int K = KB / (int)sizeof(T);
    typedef DdsWaveGrid<BM / 16, BN / 16> G;
    const size_t smem = (size_t)(BM + 2 * BN) * (K + VE) * sizeof(T) + (size_t)G::KS * BM * (BN + 4) * sizeof(float);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dds_row_kernel<T, BM, BN, KB>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(dds_row_kernel)");
    }
    hipLaunchKernelGGL((dds_row_kernel<T, BM, BN, KB>), dim3(p.M / BM, batch, 1), dim3(256), smem, st, p);
    SPX_LAUNCH_CHECK("dds_row_kernel");
    return 0;
}

// ---- short-K variant for 16-bit types and compressed output: a wavefront per 16 rows --------
// The workgroup-wide kernel above spends a block step in two barriers and an fp32 round
// trip through LDS, and - like every kernel here that loads and stores in the same loop -
// it pays for the fact that loads and stores share one in-order completion counter
// (vmcnt) on this chip: waiting for a prefetched panel also waits for the output stores
// issued before it, so the 308 MB of scores of the attention shape and the work that
// produces them ran one after the other (90 us = 48 us with the stores removed + the 45 us
// a plain fill of the same size takes).  This kernel separates the two streams by
// wavefront:
//   * WAVES compute wavefronts own 16 rows of the block row each for the whole walk: A
//     fragments in registers (loaded once), products taken transposed (B rows as the first
//     MFMA operand) so that a lane ends up with four consecutive n of one output row; the
//     wave passes its 16 x BN tile through a private LDS tile and stores whole 16-byte
//     vectors - 16 complete, contiguous rows of the compressed block.  They never wait on
//     vmcnt inside the loop.
//   * one more wavefront only loads: the B panel of step i + 2 goes global -> LDS
//     (global_load_lds_dwordx4, the XOR swizzle applied to the source address) into one of
//     three buffers while steps i and i + 1 are computed; its waits see loads only.
//   * one barrier per step hands a panel over; workgroup L runs on XCD L % 8 and every
//     batch entry (whose B operand all of its block rows share) stays within one XCD's L2.
// Needs row_ptr, k-contiguous operands, K of 64 or 128 and the compressed output layout.
template <typename T, int BN, int K, int WAVES, bool HAS_BIAS>
__global__ __launch_bounds__(64 * (WAVES + 1)) void dds_rowq_kernel(DdsParams p, int batch) {
    static_assert(sizeof(T) == 2, "16-bit types only");
    constexpr int BM = 16 * WAVES;
    constexpr int KT = BN / 16, EC = K / 32;
    constexpr int KP = K * 2;                 // bytes per staged B row
    constexpr int PANEL = BN * KP;
    constexpr int CPR = KP / 16;              // 16-byte chunks per B row
    constexpr int NVL = PANEL / 1024;         // loader instructions per panel (1 KB each)
    constexpr int RPI = 1024 / KP;            // panel rows per loader instruction
    constexpr int NBUF = 3;
    constexpr int OT = 16 * (BN * 2 + 16);    // a wavefront's output tile
    static_assert(PANEL % 1024 == 0 && RPI >= 1, "panel is not a whole number of loader instructions");
    typedef typename Mma32<T>::frag Frag;
    extern __shared__ __align__(16) char smem[];

    const int nbr = p.M / BM;
    const int L = blockIdx.x;
    const int slot = L >> 3;
    const int64_t b = (int64_t)(slot / nbr) * 8 + (L & 7);
    const int bi = slot % nbr;
    if (b >= batch) return;
    const int e_begin = p.row_ptr[bi];
    const int n_blk = p.row_ptr[bi + 1] - e_begin;
    if (n_blk <= 0) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    // block columns of the row: lane l holds entry l; longer rows read the rest from the index
    int bj_vec = 0;
    if (lane < n_blk) bj_vec = p.idx[e_begin + lane] & 0xffff;
    auto column = [&](int i) {
        return i < 64 ? __builtin_amdgcn_readlane(bj_vec, i) : (p.idx[e_begin + i] & 0xffff);
    };

    if (wave == WAVES) {
        // ---- loader ---------------------------------------------------------------------------
        const T* B = reinterpret_cast<const T*>(p.B) + b * p.b_batch;
        const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
        // lane l of instruction q lands at byte q * 1024 + l * 16 of the panel: row q * RPI + l / CPR,
        // position l % CPR, which holds chunk position ^ (row & 7)
        const int lrow = lane / CPR;
        const int lchunk = (lane % CPR) ^ (lrow & 7);   // RPI is 8 or 4 and q * RPI keeps row & 7 only if RPI == 8
        auto issue_panel = [&](int i) {
            const int bj = column(i);
            const uint32_t dst = lds_base + (uint32_t)((i % NBUF) * PANEL);
#pragma unroll
            for (int q = 0; q < NVL; ++q) {
                const int row = q * RPI + lrow;
                const int chunk = RPI == 8 ? lchunk : ((lane % CPR) ^ (row & 7));
                lds_direct_load16(B + ((int64_t)bj * BN + row) * p.b_ld + chunk * 8, dst + q * 1024);
            }
        };
        issue_panel(0);
        if (n_blk > 1) issue_panel(1);
        for (int i = 0; i < n_blk; ++i) {
            // panel i must have landed; panel i + 1 may still be on its way
            if (i + 1 < n_blk) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NVL) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (i + 2 < n_blk) issue_panel(i + 2);   // its buffer was read in step i - 1
        }
        return;
    }

    // ---- compute wavefronts -----------------------------------------------------------------
    const T* A = reinterpret_cast<const T*>(p.A) + b * p.a_batch;
    const T* biasT = HAS_BIAS ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* C = reinterpret_cast<T*>(p.C) + b * p.c_batch;
    Frag af[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) af[c] = Mma32<T>::load(A + ((int64_t)bi * BM + wave * 16 + r16) * p.a_ld + c * 32 + g4 * 8);
    const int k_src = r16 * KP, k_sw = r16 & 7;
    char* const otile = smem + NBUF * PANEL + wave * OT;
    for (int i = 0; i < n_blk; ++i) {
        const char* buf = smem + (i % NBUF) * PANEL;
        __syncthreads();   // panel i is complete
        uint64_t pieces[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag bf = *reinterpret_cast<const Frag*>(buf + k_src + kt * 16 * KP + (((c * 4 + g4) ^ k_sw) << 4));
                acc = Mma32<T>::mma(bf, af[c], acc);   // lane: row r16, columns kt * 16 + g4 * 4 .. + 3
            }
            if constexpr (HAS_BIAS) {
                // the lane's four bias entries are 8 contiguous bytes
                union { uint64_t u; T t[4]; } bv;
                bv.u = *reinterpret_cast<const uint64_t*>(biasT + column(i) * BN + kt * 16 + g4 * 4);
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[q] += Elem<T>::to_float(bv.t[q]);
            }
            T vals[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(acc[q]);
            pieces[kt] = *reinterpret_cast<const uint64_t*>(vals);
        }
        wave_rows_store<BN>(otile, C + (int64_t)(e_begin + i) * (BM * BN) + wave * 16 * BN, pieces);
    }
}

template <typename T, int BN, int K, int WAVES>
static int launch_dds_rowq_inst(const DdsParams& p, int batch, hipStream_t st) {
    const size_t smem = (size_t)3 * BN * K * 2 + (size_t)WAVES * 16 * (BN * 2 + 16);
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * (p.M / (16 * WAVES));
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dds_rowq_kernel<T, BN, K, WAVES, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dds_rowq_kernel<T, BN, K, WAVES, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(dds_rowq_kernel)");
    }
    if (p.bias) hipLaunchKernelGGL((dds_rowq_kernel<T, BN, K, WAVES, true>), dim3((unsigned)groups), dim3(64 * (WAVES + 1)), smem, st, p, batch);
    else hipLaunchKernelGGL((dds_rowq_kernel<T, BN, K, WAVES, false>), dim3((unsigned)groups), dim3(64 * (WAVES + 1)), smem, st, p, batch);
    SPX_LAUNCH_CHECK("dds_rowq_kernel");
    return 0;
}

template <typename T>
static bool dds_rowq_ok(const DdsParams& p, int BM, int BN) {
    if constexpr (sizeof(T) != 2) return false;
    return p.row_ptr && p.a_kcontig && p.b_kcontig && p.compressed && (p.K == 64 || p.K == 128) &&
           (BM == 32 || BM == 64) && (BN == 32 || BN == 64) && p.a_ld % 8 == 0 && p.b_ld % 8 == 0 &&
           (!p.bias || (aligned(p.bias, 8) && p.bias_batch % 4 == 0));
}

template <typename T>
static int launch_dds_rowq(const DdsParams& p, int BM, int BN, int batch, hipStream_t st) {
    if constexpr (sizeof(T) == 2) {
#define SPX_DDS_ROWQ_CASE(bm, bn) \
        if (BM == bm && BN == bn) return p.K == 64 ? launch_dds_rowq_inst<T, bn, 64, bm / 16>(p, batch, st) \
                                                   : launch_dds_rowq_inst<T, bn, 128, bm / 16>(p, batch, st);
        SPX_DDS_ROWQ_CASE(32, 32) SPX_DDS_ROWQ_CASE(32, 64) SPX_DDS_ROWQ_CASE(64, 32) SPX_DDS_ROWQ_CASE(64, 64)
#undef SPX_DDS_ROWQ_CASE
    }
    return fail(SPX_E_CONFIG, "the wavefront-per-16-rows kernel takes 16-bit types and 32 / 64-wide blocks");
}

// The block-row kernel covers 32 / 64-wide blocks with K * sizeof(T) of 128 or 256 bytes.
template <typename T>
static bool dds_row_ok(const DdsParams& p, int BM, int BN) {
    const int kb = p.K * (int)sizeof(T);
    return p.row_ptr && p.a_kcontig && p.b_kcontig && (kb == 128 || kb == 256) && (BM == 32 || BM == 64) &&
           (BN == 32 || BN == 64) && p.M / BM <= 65535;
}

template <typename T>
static int launch_dds_row(const DdsParams& p, int BM, int BN, int batch, hipStream_t st) {
    const int kb = p.K * (int)sizeof(T);
#define SPX_DDS_ROW_CASE(bm, bn) \
    if (BM == bm && BN == bn) return kb == 128 ? launch_dds_row_inst<T, bm, bn, 128>(p, batch, st) \
                                               : launch_dds_row_inst<T, bm, bn, 256>(p, batch, st);
    SPX_DDS_ROW_CASE(32, 32) SPX_DDS_ROW_CASE(32, 64) SPX_DDS_ROW_CASE(64, 32) SPX_DDS_ROW_CASE(64, 64)
#undef SPX_DDS_ROW_CASE
    return fail(SPX_E_CONFIG, "the block-row kernel takes 32 / 64-wide blocks");
}

// The pipelined kernels need K to be a multiple of the stage depth (256 bytes of k per row;
// 128 bytes for 64 x 64 blocks).  Returns 0 (no), 1 (both operands k-contiguous), 2 (A as
// [K, M] and B as [K, N]), 3 or 4 (one of each).
template <typename T>
static int dds_pipe_ok(const DdsParams& p, int BM, int BN) {
    const int stage = (BM + BN == 128 ? 128 : 256) / (int)sizeof(T);
    if (p.K % stage != 0) return 0;
    if (p.a_kcontig && p.b_kcontig) return 1;
    if (!p.a_kcontig && !p.b_kcontig) return 2;
    return p.a_kcontig ? 3 : 4;   // mixed: A k-contiguous and B [K, N], or A [K, M] and B k-contiguous
}

template <typename T, int BM, int BN>
static int launch_dds_inst(const DdsParams& p, int nnz_bound, int batch, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int KT = sizeof(T) == 2 ? 128 : 64;
    typedef DdsWaveGrid<BM / 16, BN / 16> G;
    size_t smem = (size_t)(BM + BN) * (KT + VE) * sizeof(T);
    size_t epi = (size_t)G::KS * BM * (BN + 4) * sizeof(float);
    if (epi > smem) smem = epi;
    hipLaunchKernelGGL((dds_kernel<T, BM, BN>), dim3(nnz_bound, batch, 1), dim3(256), smem, st, p);
    SPX_LAUNCH_CHECK("dds_kernel");
    return 0;
}

// tile_cfg: 0 = the pipelined kernel where it applies; 1 = one LDS buffer, no prefetch;
//           2 = pipelined (register ring + two LDS buffers).
template <typename T>
int launch_dds_impl(const DdsParams& p, int BM, int BN, int nnz_bound, int batch, int tile_cfg, hipStream_t st) {
    if (tile_cfg < 0 || tile_cfg > 4) return fail(SPX_E_CONFIG, "unknown tile config %d", tile_cfg);
    const int pipe = dds_pipe_ok<T>(p, BM, BN);
    const bool row = dds_row_ok<T>(p, BM, BN);
    const bool rowq = dds_rowq_ok<T>(p, BM, BN);
    if (tile_cfg == 0) tile_cfg = rowq ? 4 : (row ? 3 : (pipe ? 2 : 1));
    if (tile_cfg == 4) {
        if (!rowq) return fail(SPX_E_CONFIG, "tile config 4 needs a 16-bit type, row_ptr, k-contiguous operands, compressed output, 32/64-wide blocks and K of 64 or 128");
        return launch_dds_rowq<T>(p, BM, BN, batch, st);
    }
    if (tile_cfg == 3) {
        if (!row) return fail(SPX_E_CONFIG, "tile config 3 needs row_ptr, k-contiguous operands, 32/64-wide blocks and K of 128 or 256 bytes");
        return launch_dds_row<T>(p, BM, BN, batch, st);
    }
    if (tile_cfg == 2 && !pipe)
        return fail(SPX_E_CONFIG, "tile config 2 needs K to be a multiple of the stage depth");
#define SPX_DDS_CASE(bm, bn) \
    if (BM == bm && BN == bn) \
        return tile_cfg != 2 ? launch_dds_inst<T, bm, bn>(p, nnz_bound, batch, st) \
             : pipe == 1 ? launch_dds_pipe_inst<T, bm, bn>(p, nnz_bound, batch, st) \
             : pipe == 2 ? launch_dds_pipe_t_inst<T, bm, bn>(p, nnz_bound, batch, st) \
             : pipe == 3 ? launch_dds_pipe_t_inst<T, bm, bn, false, true>(p, nnz_bound, batch, st) \
                         : launch_dds_pipe_t_inst<T, bm, bn, true, false>(p, nnz_bound, batch, st);
    SPX_DDS_CASE(16, 16) SPX_DDS_CASE(16, 32) SPX_DDS_CASE(16, 64)
    SPX_DDS_CASE(32, 16) SPX_DDS_CASE(32, 32) SPX_DDS_CASE(32, 64)
    SPX_DDS_CASE(64, 16) SPX_DDS_CASE(64, 32) SPX_DDS_CASE(64, 64)
#undef SPX_DDS_CASE
    return fail(SPX_E_CONFIG, "output block (%d,%d) not in {16,32,64}^2", BM, BN);
}

template <typename T>
int launch_dds(const DdsParams& p, int BM, int BN, int nnz_bound, int batch, int tile_cfg, hipStream_t st);

}  // namespace spx
