// spx_matmul: argument validation and the mapping of (mode, transposes,
// compressed) onto the two kernel families.
#include "matmul_spmm.hpp"
#include "matmul_dds.hpp"

namespace spx {

template <typename T>
static int run_matmul(int mode, int transA, int transB, int compressed,
                      const void* A, const void* B, const void* bias, void* C,
                      const int32_t* ptr, const void* idx, int idx_kind, const int32_t* sched,
                      int nnz_bound, const int32_t* nnz_dev, int64_t sparse_batch_stride,
                      int batch, int M, int K, int N, int BM, int BK, int BN,
                      int tile_cfg, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    if (mode == SPX_DDS) {
        DdsParams p;
        p.A = A; p.B = B; p.bias = bias; p.C = C;
        p.idx = reinterpret_cast<const int32_t*>(idx);
        p.row_ptr = ptr;
        p.nnz_dev = nnz_dev;
        p.M = M; p.K = K; p.N = N;
        p.a_kcontig = !transA; p.a_ld = transA ? M : K;
        p.b_kcontig = transB;  p.b_ld = transB ? K : N;
        p.compressed = compressed;
        p.a_batch = (int64_t)M * K; p.b_batch = (int64_t)K * N;
        p.c_batch = compressed ? sparse_batch_stride : (int64_t)M * N;
        p.bias_batch = N;
        SPX_REQUIRE(K % 16 == 0, SPX_E_SHAPE, "K=%d must be a multiple of 16", K);
        SPX_REQUIRE(!transA || M % VE == 0, SPX_E_SHAPE, "transposed A needs M %% %d == 0", VE);
        SPX_REQUIRE(transB || N % VE == 0, SPX_E_SHAPE, "non-transposed B needs N %% %d == 0", VE);
        if (nnz_bound == 0) return 0;
        return launch_dds<T>(p, BM, BN, nnz_bound, batch, tile_cfg, st);
    }

    SpmmParams p;
    p.relu = (tile_cfg & SPX_EPILOGUE_RELU) != 0;
    tile_cfg &= ~SPX_EPILOGUE_RELU;
    p.bias = bias; p.out = C; p.ptr = ptr; p.idx = idx; p.idx_kind = idx_kind; p.sched = sched;
    p.K = K; p.BK = BK; p.log_bk = ilog2(BK);
    p.compressed = compressed;
    p.o_batch = (int64_t)M * N;
    p.bias_batch = N;
    int BNc;  // canonical sparse block width
    if (mode == SPX_DSD) {
        // out = C, D = A, S = B
        p.D = A; p.S = B;
        p.Mc = M; p.Nc = N; BNc = BN;
        p.d_kcontig = !transA; p.d_ld = transA ? M : K;
        p.d_batch = (int64_t)M * K;
        p.s_kcontig = transB;  // stored [N,K]: k contiguous
        p.s_ld = compressed ? (transB ? BK : BN) : (transB ? K : N);
        p.s_batch = compressed ? sparse_batch_stride : (int64_t)K * N;
        p.out_ncontig = 1; p.o_ld = N;
        p.bias_on_m = 0;
        SPX_REQUIRE(!transA || M % VE == 0, SPX_E_SHAPE, "transposed A needs M %% %d == 0", VE);
    } else {
        // sdd: out^T = C^T, D = B^T (rows n), S = A^T (cols m)
        p.D = B; p.S = A;
        p.Mc = N; p.Nc = M; BNc = BM;
        p.d_kcontig = transB; p.d_ld = transB ? K : N;
        p.d_batch = (int64_t)K * N;
        p.s_kcontig = !transA;  // stored [M,K]: k contiguous
        p.s_ld = compressed ? (transA ? BM : BK) : (transA ? M : K);
        p.s_batch = compressed ? sparse_batch_stride : (int64_t)M * K;
        p.out_ncontig = 0; p.o_ld = N;   // out[n' = m][m' = n] = C[m*N + n]
        p.bias_on_m = 1;
        SPX_REQUIRE(N % VE == 0, SPX_E_SHAPE, "sparse-A matmul needs N %% %d == 0", VE);
    }
    return launch_spmm<T>(p, BNc, batch, tile_cfg, st);
}

}  // namespace spx

extern "C" int spx_matmul(int mode, int dtype, int transA, int transB, int compressed,
                          const void* A, const void* B, const void* bias, void* C,
                          const int32_t* ptr, const void* idx, int idx_kind, const int32_t* sched,
                          int nnz_bound, const int32_t* nnz_dev, int64_t sparse_batch_stride,
                          int batch, int M, int K, int N, int BM, int BK, int BN,
                          int tile_cfg, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(mode == SPX_SDD || mode == SPX_DSD || mode == SPX_DDS, SPX_E_CONFIG, "unknown mode %d", mode);
    SPX_REQUIRE(dtype == SPX_F32 || dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE, "unknown dtype %d", dtype);
    {
        // an empty compressed operand / result (no live block) may be NULL
        const bool empty_ok = compressed && nnz_bound == 0;
        SPX_REQUIRE(A || (mode == SPX_SDD && empty_ok), SPX_E_NULL, "A is required");
        SPX_REQUIRE(B || (mode == SPX_DSD && empty_ok), SPX_E_NULL, "B is required");
        SPX_REQUIRE(C || (mode == SPX_DDS && empty_ok), SPX_E_NULL, "C is required");
    }
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(M > 0 && K > 0 && N > 0, SPX_E_SHAPE, "M, K, N must be positive");
    SPX_REQUIRE((BM == 16 || BM == 32 || BM == 64) && (BK == 16 || BK == 32 || BK == 64) &&
                (BN == 16 || BN == 32 || BN == 64), SPX_E_CONFIG,
                "block sizes (%d,%d,%d) must each be 16, 32 or 64", BM, BK, BN);
    SPX_REQUIRE(M % BM == 0 || mode == SPX_DSD, SPX_E_SHAPE, "M=%d is not a multiple of BM=%d", M, BM);
    SPX_REQUIRE(N % BN == 0 || mode == SPX_SDD, SPX_E_SHAPE, "N=%d is not a multiple of BN=%d", N, BN);
    SPX_REQUIRE(K % BK == 0 || mode == SPX_DDS, SPX_E_SHAPE, "K=%d is not a multiple of BK=%d", K, BK);
    SPX_REQUIRE(M / 16 <= 65535 * 8 && N / 16 <= 65535 * 8, SPX_E_SHAPE, "matrix too large for the launch grid");
    SPX_REQUIRE(idx || nnz_bound == 0, SPX_E_NULL, "idx is required");
    SPX_REQUIRE(nnz_bound >= 0, SPX_E_SHAPE, "negative nnz bound");
    SPX_REQUIRE(idx_kind >= 0 && idx_kind <= 2, SPX_E_CONFIG, "unknown idx_kind %d", idx_kind);
    if (mode == SPX_DDS) {
        SPX_REQUIRE(idx_kind == SPX_IDX_BCSR_I32, SPX_E_CONFIG, "sparse-output matmul reads a BCSR index");
        SPX_REQUIRE(!(tile_cfg & SPX_EPILOGUE_RELU), SPX_E_CONFIG, "the fused activation covers sdd and dsd only");
    } else {
        SPX_REQUIRE(ptr, SPX_E_NULL, "row_ptr / col_ptr is required for sdd and dsd");
        const bool wants_bcsr = (mode == SPX_DSD) ? (transB != 0) : (transA == 0);
        SPX_REQUIRE(wants_bcsr == (idx_kind == SPX_IDX_BCSR_I32), SPX_E_CONFIG,
                    "index kind %d does not match mode/transposes (needs %s)", idx_kind, wants_bcsr ? "BCSR" : "BCSC");
        SPX_REQUIRE(idx_kind != SPX_IDX_BCSC_I64 || compressed, SPX_E_CONFIG,
                    "the int64 BCSC index is only meaningful for compressed values");
    }
    const int es = dtype_bytes(dtype);
    SPX_REQUIRE(aligned(A, 16) && aligned(B, 16) && aligned(C, 16), SPX_E_ALIGN, "A, B, C must be 16-byte aligned");
    SPX_REQUIRE(!bias || aligned(bias, es), SPX_E_ALIGN, "bias misaligned");
    SPX_REQUIRE(!compressed || (sparse_batch_stride * es) % 16 == 0, SPX_E_ALIGN,
                "sparse batch stride must keep blocks 16-byte aligned");
    if (batch == 0) return 0;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {
        case SPX_F32:
            return run_matmul<float>(mode, transA, transB, compressed, A, B, bias, C, ptr, idx, idx_kind, sched, nnz_bound,
                                     nnz_dev, sparse_batch_stride, batch, M, K, N, BM, BK, BN, tile_cfg, st);
        case SPX_F16:
            return run_matmul<_Float16>(mode, transA, transB, compressed, A, B, bias, C, ptr, idx, idx_kind, sched, nnz_bound,
                                        nnz_dev, sparse_batch_stride, batch, M, K, N, BM, BK, BN, tile_cfg, st);
        default:
            return run_matmul<bf16_t>(mode, transA, transB, compressed, A, B, bias, C, ptr, idx, idx_kind, sched, nnz_bound,
                                      nnz_dev, sparse_batch_stride, batch, M, K, N, BM, BK, BN, tile_cfg, st);
    }
}
