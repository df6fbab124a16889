// Sparse-operand matmul (the reference's 'sdd' and 'dsd' modes) in one canonical
// form:   out[m, n] = sum_k D[m, k] * S[k, n] (+ bias)
// where S is block-sparse with (BK x BN) blocks listed per block-column n, and D,
// out are dense with arbitrary (row- or column-major) layout.  'dsd' maps
// directly (D = A, S = B); 'sdd' is the transposed problem (D = B^T, S = A^T,
// out = C^T), so both modes, every transpose flag and the compressed /
// uncompressed storage of S differ only in strides.
//
// One workgroup (4 wavefronts) owns a (64*WM) x BN output tile and walks the
// live blocks of its block-column: each live block stages the D panel and the S
// block through LDS as [row][k] and feeds 16x16 MFMAs; the tile leaves through
// LDS so HBM sees full-width row segments.
#pragma once
#include "common.hpp"
#include "mma.hpp"

namespace spx {

struct SpmmParams {
    const void* D;
    const void* S;
    const void* bias;
    void* out;
    const int32_t* ptr;
    const void* idx;
    const int32_t* sched;  // optional launch order of the block-columns (longest first)
    int idx_kind;
    int Mc, K, Nc;       // canonical sizes (Mc: dense rows, Nc: sparse-side cols)
    int BK, log_bk;
    int d_kcontig;       // D[m*d_ld + k] if set, else D[k*d_ld + m]
    int64_t d_ld;
    int s_kcontig;       // block element (k, n): n*s_ld + k if set, else k*s_ld + n
    int compressed;      // S blocks at slot*BK*BN, else inside the dense matrix
    int64_t s_ld;        // leading dimension of the stored S (block-local if compressed)
    int out_ncontig;     // out[m*o_ld + n] if set, else out[n*o_ld + m]
    int64_t o_ld;
    int bias_on_m;       // bias indexed by canonical m instead of n
    int64_t d_batch, s_batch, o_batch, bias_batch;
    int relu;           // epilogue: negative results (after the bias) become zero
};

// Optional activation of the epilogue; NaN stays NaN (as torch.relu keeps it).
__device__ __forceinline__ float epilogue_act(float v, int relu) { return (relu && v < 0.f) ? 0.f : v; }

template <typename T, int BN, int WM>
__global__ __launch_bounds__(256) void spmm_kernel(SpmmParams p) {
    constexpr int TM = 64 * WM;
    constexpr int NT = BN / 16;
    constexpr int VE = 16 / (int)sizeof(T);
    extern __shared__ __align__(16) char smem[];

    const int ldk = p.BK + VE;  // 16 bytes of padding per row
    T* Ds = reinterpret_cast<T*>(smem);
    T* Ss = Ds + TM * ldk;

    const int j = blockIdx.x;
    const int m0 = blockIdx.y * TM;
    const int64_t b = blockIdx.z;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g4 = lane >> 4;

    const T* D = reinterpret_cast<const T*>(p.D) + b * p.d_batch;
    const T* S = reinterpret_cast<const T*>(p.S) + b * p.s_batch;
    const int rows_valid = p.Mc - m0;  // > 0 by grid construction

    f32x4 acc[WM][NT];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int e_begin = p.ptr[j];
    const int e_end = p.ptr[j + 1];
    for (int e = e_begin; e < e_end; ++e) {
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
        const int64_t k0 = (int64_t)kb * p.BK;
        const T* dsrc = p.d_kcontig ? D + (int64_t)m0 * p.d_ld + k0 : D + k0 * p.d_ld + m0;
        const T* ssrc;
        if (p.compressed) ssrc = S + slot * (int64_t)(p.BK * BN);
        else ssrc = p.s_kcontig ? S + (int64_t)j * BN * p.s_ld + k0 : S + k0 * p.s_ld + (int64_t)j * BN;

        stage_tile<T, TM, 256>(Ds, ldk, p.BK, p.log_bk, dsrc, p.d_ld, p.d_kcontig != 0, rows_valid);
        stage_tile<T, BN, 256>(Ss, ldk, p.BK, p.log_bk, ssrc, p.s_ld, p.s_kcontig != 0, BN);
        __syncthreads();

        const T* a_base = Ds + (wave * 16 * WM + r16) * ldk;
        const T* b_base = Ss + r16 * ldk;
        bool done = false;
        if constexpr (HasMma32<T>::value) {
            if ((p.BK & 31) == 0) {
                for (int kc = 0; kc < p.BK; kc += 32) {
                    typename Mma32<T>::frag af[WM], bf[NT];
#pragma unroll
                    for (int i = 0; i < WM; ++i) af[i] = Mma32<T>::load(a_base + i * 16 * ldk + kc + g4 * 8);
#pragma unroll
                    for (int t = 0; t < NT; ++t) bf[t] = Mma32<T>::load(b_base + t * 16 * ldk + kc + g4 * 8);
#pragma unroll
                    for (int i = 0; i < WM; ++i)
#pragma unroll
                        for (int t = 0; t < NT; ++t) acc[i][t] = Mma32<T>::mma(af[i], bf[t], acc[i][t]);
                }
                done = true;
            }
        }
        if (!done) {
            for (int kc = 0; kc < p.BK; kc += 16) {
                typename Mma16<T>::frag af[WM], bf[NT];
#pragma unroll
                for (int i = 0; i < WM; ++i) af[i] = Mma16<T>::load(a_base + i * 16 * ldk + kc + g4 * 4);
#pragma unroll
                for (int t = 0; t < NT; ++t) bf[t] = Mma16<T>::load(b_base + t * 16 * ldk + kc + g4 * 4);
#pragma unroll
                for (int i = 0; i < WM; ++i)
#pragma unroll
                    for (int t = 0; t < NT; ++t) acc[i][t] = Mma16<T>::mma(af[i], bf[t], acc[i][t]);
            }
        }
        __syncthreads();
    }

    // ---- epilogue: registers -> LDS (output orientation) -> HBM -----------------
    T* Es = reinterpret_cast<T*>(smem);
    const T* biasT = p.bias ? reinterpret_cast<const T*>(p.bias) + b * p.bias_batch : nullptr;
    T* out = reinterpret_cast<T*>(p.out) + b * p.o_batch;
    if (p.out_ncontig) {
        constexpr int LDE = BN + VE;
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int m = wave * 16 * WM + i * 16 + g4 * 4 + q;
                    const int n = t * 16 + r16;
                    float v = acc[i][t][q];
                    if (biasT) {
                        const int bi = p.bias_on_m ? (m0 + m < p.Mc ? m0 + m : 0) : j * BN + n;
                        v += Elem<T>::to_float(biasT[bi]);
                    }
                    Es[m * LDE + n] = Elem<T>::from_float(epilogue_act(v, p.relu));
                }
        __syncthreads();
        constexpr int VPR = BN / VE;
        for (int v = threadIdx.x; v < TM * VPR; v += 256) {
            const int m = v / VPR;
            const int nv = v - m * VPR;
            if (m < rows_valid)
                *reinterpret_cast<vec16*>(out + (int64_t)(m0 + m) * p.o_ld + (int64_t)j * BN + nv * VE) =
                    *reinterpret_cast<const vec16*>(Es + m * LDE + nv * VE);
        }
    } else {
        constexpr int LDE = TM + VE;
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int m = wave * 16 * WM + i * 16 + g4 * 4 + q;
                    const int n = t * 16 + r16;
                    float v = acc[i][t][q];
                    if (biasT) {
                        const int bi = p.bias_on_m ? (m0 + m < p.Mc ? m0 + m : 0) : j * BN + n;
                        v += Elem<T>::to_float(biasT[bi]);
                    }
                    Es[n * LDE + m] = Elem<T>::from_float(epilogue_act(v, p.relu));
                }
        __syncthreads();
        constexpr int VPR = TM / VE;
        for (int v = threadIdx.x; v < BN * VPR; v += 256) {
            const int n = v / VPR;
            const int mv = v - n * VPR;
            if (mv * VE < rows_valid)
                *reinterpret_cast<vec16*>(out + ((int64_t)j * BN + n) * p.o_ld + m0 + mv * VE) =
                    *reinterpret_cast<const vec16*>(Es + n * LDE + mv * VE);
        }
    }
}

template <typename T>
int launch_spmm(const SpmmParams& p, int BN, int batch, int tile_cfg, hipStream_t st);

template <typename T, int BN, int WM>
static int launch_spmm_inst(const SpmmParams& p, int batch, hipStream_t st) {
    constexpr int TM = 64 * WM;
    constexpr int VE = 16 / (int)sizeof(T);
    const int ldk = p.BK + VE;
    size_t main_bytes = (size_t)(TM + BN) * ldk * sizeof(T);
    size_t epi_a = (size_t)TM * (BN + VE) * sizeof(T);
    size_t epi_b = (size_t)BN * (TM + VE) * sizeof(T);
    size_t smem = main_bytes;
    if (epi_a > smem) smem = epi_a;
    if (epi_b > smem) smem = epi_b;
    dim3 grid(p.Nc / BN, (p.Mc + TM - 1) / TM, batch);
    hipLaunchKernelGGL((spmm_kernel<T, BN, WM>), grid, dim3(256), smem, st, p);
    SPX_LAUNCH_CHECK("spmm_kernel");
    return 0;
}

template <typename T>
int launch_spmm_direct(const SpmmParams& p, int BN, int batch, int wm, hipStream_t st);
template <typename T>
int launch_spmm_panel(const SpmmParams& p, int BN, int batch, int nst, hipStream_t st);
template <typename T>
int launch_spmm_stream(const SpmmParams& p, int BN, int batch, hipStream_t st);
template <typename T>
int launch_spmm_ksplit(const SpmmParams& p, int BN, int batch, hipStream_t st);
template <typename T>
bool spmm_thin_supported(const SpmmParams& p, int BN);
template <typename T>
int launch_spmm_thin(const SpmmParams& p, int batch, hipStream_t st);

// tile_cfg: 0 = pick by layout and size;
//   1 / 2  LDS-staged kernel, 64 / 128-row workgroup tiles (any layout);
//   3 / 4  register-direct kernel, 64 / 256-row workgroup tiles (k-contiguous operands);
//   5 / 6  panel kernel, 256-row workgroup tiles, 2 / 3 load stages (k-contiguous
//          operands, block depth a multiple of 64 bytes);
//   8      K-split panel kernel: 64-row workgroup tiles, the four wavefronts split the
//          live blocks of a block-column (k-contiguous operands, BN <= 32): few rows.
//   7      panel kernel whose four wavefronts share the sparse block through LDS (the
//          sparse operand may be stored with n contiguous: it is transposed on the way).
//   9      thin dense operand (64 or 128 values of m, stored with m contiguous; 16-bit
//          types, 64-wide k-contiguous sparse blocks): one workgroup per block-column.
//   10     persistent form of 7 for a k-contiguous dense operand: a workgroup walks the
//          tiles of its XCD as one stream of steps (matmul_spmm_stream.hpp).
template <typename T>
int launch_spmm_impl(const SpmmParams& p, int BN, int batch, int tile_cfg, hipStream_t st) {
    const bool kcontig = p.d_kcontig && p.s_kcontig;
    const bool panel_ok = kcontig && (p.BK * (int)sizeof(T)) % 64 == 0;
    // the shared-S panel variant transposes an n-contiguous sparse block while staging it
    // ... and reads a dense operand stored with m contiguous through LDS transpose reads
    const bool panel7_ok = (p.BK * (int)sizeof(T)) % 64 == 0 &&
                           (p.d_kcontig || (p.Mc % (16 / (int)sizeof(T)) == 0 && p.d_ld % (16 / (int)sizeof(T)) == 0));
    if (tile_cfg < 0 || tile_cfg > 10) return fail(SPX_E_CONFIG, "unknown tile config %d", tile_cfg);
    const bool stream_ok = p.d_kcontig && (p.BK * (int)sizeof(T)) % 64 == 0 && p.d_ld * 256 + 64 < (int64_t)0x7fffffff / (int)sizeof(T);
    const bool ksplit_ok = panel_ok && BN <= 32;
    const bool thin_ok = spmm_thin_supported<T>(p, BN);
    if (tile_cfg == 0 && thin_ok) tile_cfg = 9;
    if (tile_cfg == 9) {
        if (!thin_ok) return fail(SPX_E_CONFIG, "tile config 9 needs a 16-bit dense operand with 64 or 128 contiguous m and 64-wide k-contiguous blocks of depth 32 / 64");
        return launch_spmm_thin<T>(p, batch, st);
    }
    if (tile_cfg == 0) {
        // 256-row tiles only when they still give every CU a few workgroups; small
        // problems are latency-bound and want more, shorter workgroups.
        const int64_t big_tiles = (int64_t)((p.Mc + 255) / 256) * (p.Nc / BN) * batch;
        const bool fill = big_tiles >= 512;
        // the persistent form when its 8 * (N / BN) slots fill the device four times over, every
        // slot walks at least two 256-row tiles and the block-columns are long: 28.4 - 28.7 us
        // against 29.9 - 30.0 us for 7 on the 4096^3 problem (alternating runs on three
        // machines); with fewer slots or tiles it loses (C4 layers: 28 / 34 against 20 / 21 us)
        const int nb = p.Nc / BN;
        if (stream_ok && panel_ok && batch == 1 && 8 * nb >= 1024 && p.Mc >= 16 * 256 && p.K / p.BK >= 32 &&
            (BN == 16 || BN == 32 || BN == 64))
            tile_cfg = 10;
        else if (panel_ok && p.Mc >= 512 && fill) tile_cfg = p.Mc >= 1024 ? 7 : 5;
        else if (ksplit_ok && !fill && p.K / p.BK >= 8) tile_cfg = 8;  // few tiles, long block-columns
        // operands that are not both k-contiguous (input gradients, transposed layouts) have only
        // the LDS-staged kernel besides 7, which 7 beats two- to threefold at every size measured
        // (64 to 8192 rows, 10 to 99 % sparsity)
        // (fp32 with an m-contiguous dense operand builds its fragments from 4-byte LDS reads and
        // only pays on large problems: 1024^3 29.7 against 17.5 us)
        else if (panel7_ok && ((!kcontig && (sizeof(T) == 2 || p.d_kcontig)) || (p.Mc >= 512 && fill))) tile_cfg = 7;
        // sparse blocks wider than the K-split kernel takes: the register-direct kernel only while
        // the problem is small and its block-columns short (measured 2 - 3x behind 5 otherwise)
        else if (panel_ok && !ksplit_ok && (big_tiles >= 128 || (big_tiles >= 64 && p.K / p.BK >= 64))) tile_cfg = 5;
        else if (kcontig) tile_cfg = p.Mc >= 1024 && fill ? 4 : 3;
        else tile_cfg = p.Mc >= 1024 && fill ? 2 : 1;
    }
    if (tile_cfg == 10) {
        if (!stream_ok) return fail(SPX_E_CONFIG, "tile config 10 needs a k-contiguous dense operand and 64-byte block rows");
        return launch_spmm_stream<T>(p, BN, batch, st);
    }
    if (tile_cfg == 8) {
        if (!ksplit_ok) return fail(SPX_E_CONFIG, "tile config 8 needs k-contiguous operands, 64-byte block rows and BN <= 32");
        return launch_spmm_ksplit<T>(p, BN, batch, st);
    }
    if (tile_cfg >= 5) {
        if (!(tile_cfg == 7 ? panel7_ok : panel_ok))
            return fail(SPX_E_CONFIG, "tile config %d needs k-contiguous operands and 64-byte block rows", tile_cfg);
        return launch_spmm_panel<T>(p, BN, batch, tile_cfg == 6 ? 3 : tile_cfg == 7 ? 12 : 2, st);
    }
    if (tile_cfg >= 3) {
        if (!kcontig) return fail(SPX_E_CONFIG, "tile config %d needs k-contiguous operands", tile_cfg);
        return launch_spmm_direct<T>(p, BN, batch, tile_cfg == 4 ? 4 : 1, st);
    }
    const int wm = tile_cfg == 2 ? 2 : 1;
    if (wm == 2) {
        switch (BN) {
            case 16: return launch_spmm_inst<T, 16, 2>(p, batch, st);
            case 32: return launch_spmm_inst<T, 32, 2>(p, batch, st);
            case 64: return launch_spmm_inst<T, 64, 2>(p, batch, st);
        }
    } else {
        switch (BN) {
            case 16: return launch_spmm_inst<T, 16, 1>(p, batch, st);
            case 32: return launch_spmm_inst<T, 32, 1>(p, batch, st);
            case 64: return launch_spmm_inst<T, 64, 1>(p, batch, st);
        }
    }
    return fail(SPX_E_CONFIG, "sparse block width %d not in {16,32,64}", BN);
}

}  // namespace spx
