/*
 * sparta_hip.h - C ABI of libsparta_hip.so: the gfx950 (MI355X) device side of
 * the block-sparse operator path.
 *
 * Conventions
 *   - Every entry point returns int: 0 = ok, < 0 = argument error detected on
 *     the host before any launch (SPX_E_*), > 0 = a hipError_t value.
 *     spx_last_error() returns a thread-local message for the last failure.
 *   - The library owns no device memory and never allocates any: every buffer,
 *     workspaces included, is provided by the caller.  Work is enqueued on the
 *     hipStream_t passed as `stream` (NULL = the default stream); no entry point
 *     synchronises the device.
 *   - All pointers are device pointers unless stated otherwise.  Tensors are
 *     contiguous, row-major, with the batch as the slowest dimension.
 *   - dtype: SPX_F32 / SPX_F16 / SPX_BF16.  Matmuls always accumulate in fp32.
 *   - Index encodings are the reference's
 *     (sparta/tesa/templates/block_compressed.cu.j2:138-170):
 *       BCSR_idx int32 = (block_row << 16) | block_col, column-ascending per row
 *       BCSC_idx int32 = (block_col << 16) | block_row, row-ascending per column
 *       BCSC_idx int64 = (bcsr_pos << 32) | (block_col << 16) | block_row
 *     Compressed values: [batch, nnz * BH * BW], block i at i*BH*BW, row-major
 *     inside the block (block_compressed.cu.j2:188-193).
 */
#ifndef SPARTA_HIP_H_
#define SPARTA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPX_VERSION 100

enum spx_dtype { SPX_F32 = 0, SPX_F16 = 1, SPX_BF16 = 2 };
enum spx_mode { SPX_SDD = 0, SPX_DSD = 1, SPX_DDS = 2 };
/* how a kernel reads a block index array */
enum spx_idx_kind {
    SPX_IDX_BCSR_I32 = 0, /* (row<<16)|col ; value slot = position          */
    SPX_IDX_BCSC_I32 = 1, /* (col<<16)|row ; value slot = position          */
    SPX_IDX_BCSC_I64 = 2  /* (slot<<32)|(col<<16)|row ; slot = BCSR position */
};
enum spx_error {
    SPX_OK = 0,
    SPX_E_NULL = -1,      /* required pointer is NULL                   */
    SPX_E_SHAPE = -2,     /* shape / divisibility / range violation     */
    SPX_E_DTYPE = -3,     /* unsupported dtype                          */
    SPX_E_ALIGN = -4,     /* pointer or stride not sufficiently aligned */
    SPX_E_WORKSPACE = -5, /* workspace too small                        */
    SPX_E_CONFIG = -6,    /* unknown mode / tile config / block size    */
    SPX_E_NO_DEVICE = -7  /* library built without a usable device path */
};

typedef void* spx_stream_t; /* hipStream_t */

/* Thread-local text of the last error returned on this thread ("" if none). */
const char* spx_last_error(void);
int spx_version(void);

/* Diagnostic, no counterpart in the reference: a plain streaming pass over `bytes` bytes
 * with the access shape of the memory-bound kernels (16 bytes per lane, non-temporal) -
 * mode 0 reads src (dst may be NULL), mode 1 copies src to dst.  bench.py --config ceilings
 * times it to show which read and copy rates the machine sustains. */
int spx_stream_probe(int mode, const void* src, void* dst, size_t bytes, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * BCSR / BCSC index build.
 * Replaces BCSFunctionContext.build_indexes / _build_BCSR_indexes /
 * _build_BCSC_indexes (sparta/tesa/block_compressed.py:242-309) and the
 * bcs_index_1 / bcs_index_2 kernels (block_compressed.cu.j2:67-170), without
 * the host round trip of block_compressed.py:255: nnz is left in device memory.
 *
 * mask      uint8 [H, W]; a block is live iff any byte of its tile is non-zero.
 * row_ptr   int32 [H/BH + 1] or NULL; bcsr_idx int32 [cap] or NULL (both or none)
 * col_ptr   int32 [W/BW + 1] or NULL; bcsc_idx int32/int64 [cap] or NULL
 * bcsc_i64  non-zero: bcsc_idx is int64 and carries the BCSR position.
 * nnz_dev   int32 [1]: receives the number of live blocks (may exceed cap;
 *           entries beyond cap are not written).
 * workspace spx_bcs_index_workspace_bytes(...) bytes, 256-byte aligned.
 * ------------------------------------------------------------------------ */
size_t spx_bcs_index_workspace_bytes(int H, int W, int BH, int BW);
int spx_bcs_index(const uint8_t* mask, int H, int W, int BH, int BW,
                  int32_t* row_ptr, int32_t* bcsr_idx,
                  int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                  int32_t* nnz_dev, int cap,
                  void* workspace, size_t workspace_bytes, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * dense <-> compressed values.  Replace BCSFunctionContext.convert / inverse
 * (block_compressed.py:311-358) and dense_to_bcs_val / bcs_val_to_dense
 * (block_compressed.cu.j2:172-220); any element size in {1,2,4,8} bytes.
 *
 * nnz_bound  number of blocks to launch over (host nnz, or the idx capacity);
 * nnz_dev    optional int32[1]: blocks at positions >= *nnz_dev are skipped.
 * sparse_batch_stride  elements between consecutive batches of `sparse`.
 * spx_bcs_scatter writes live tiles only: the caller zero-fills `dense` first.
 * ------------------------------------------------------------------------ */
int spx_bcs_gather(const void* dense, void* sparse, const void* idx, int idx_kind,
                   int nnz_bound, const int32_t* nnz_dev, int batch, int H, int W,
                   int BH, int BW, int elem_bytes, int64_t sparse_batch_stride,
                   spx_stream_t stream);
int spx_bcs_scatter(const void* sparse, void* dense, const void* idx, int idx_kind,
                    int nnz_bound, const int32_t* nnz_dev, int batch, int H, int W,
                    int BH, int BW, int elem_bytes, int64_t sparse_batch_stride,
                    spx_stream_t stream);

/* Launch order for matmuls that walk one row_ptr / col_ptr segment per workgroup:
 * order[0..n) = the n segments sorted by descending length (longest first), so
 * that the long segments start early and the short ones fill the tail.  Purely a
 * scheduling hint (results do not depend on it); no counterpart in the reference,
 * whose grids follow the natural order (matmul.py:143-149).  ptr int32 [n+1]. */
int spx_bcs_schedule(const int32_t* ptr, int n, int32_t* order, spx_stream_t stream);

/* spx_bcs_index plus the launch orders of spx_bcs_schedule from the same launch (an index
 * that is rebuilt for every call has no time for a third kernel): row_order int32 [H/BH]
 * (needs the BCSR index) and col_order int32 [W/BW] (needs the BCSC index), each optional.
 * No counterpart in the reference. */
int spx_bcs_index_scheduled(const uint8_t* mask, int H, int W, int BH, int BW,
                            int32_t* row_ptr, int32_t* bcsr_idx,
                            int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                            int32_t* nnz_dev, int cap, int32_t* row_order, int32_t* col_order,
                            void* workspace, size_t workspace_bytes, spx_stream_t stream);

/* Several independent index builds in one call: every job has the arguments of
 * spx_bcs_index_scheduled.  Jobs that take the bit-word path (16-byte aligned masks with
 * W % 16 == 0 and at most 2048 words of 64 blocks per side) share one pair of launches, up to
 * four at a time - a model that rebuilds the masks of several layers per step otherwise pays
 * one pair of small dependent launches per layer; the other jobs are built one after the
 * other.  Results are those of separate calls.  The workspaces of the jobs must not overlap
 * (SPX_E_WORKSPACE otherwise).  No counterpart in the reference, which builds
 * one index per call (block_compressed.py:242-265). */
typedef struct spx_bcs_index_job {
    const uint8_t* mask;
    int H, W, BH, BW;
    int32_t* row_ptr;
    int32_t* bcsr_idx;
    int32_t* col_ptr;
    void* bcsc_idx;
    int bcsc_i64;
    int32_t* nnz_dev;
    int cap;
    int32_t* row_order;
    int32_t* col_order;
    void* workspace;
    size_t workspace_bytes;
} spx_bcs_index_job;
int spx_bcs_index_batch(const spx_bcs_index_job* jobs, int n_jobs, spx_stream_t stream);

/* spx_bcs_index for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): no workspace argument.
 * No counterpart in the reference.  The scratch of the two kernels lives in a device
 * array inside the library, spx_bcs_index_static_max_bytes() = 1 MiB per GPU, held until
 * the process ends; a mask whose workspace (spx_bcs_index_workspace_bytes) is larger is
 * rejected with SPX_E_WORKSPACE before anything is launched (1 MiB covers about 700 000
 * blocks, e.g. a 4096 x 4096 mask down to 8 x 4 blocks).  Nothing is allocated or
 * freed by the call.  All calls on one GPU share that GPU's array: calls that overlap
 * on one GPU (two streams, two threads) race and must be serialised by the caller.
 * The first call on a device looks the array's address up (not a stream operation):
 * make it outside graph capture.  Results are identical to spx_bcs_index. */
size_t spx_bcs_index_static_max_bytes(void);
int spx_bcs_index_static(const uint8_t* mask, int H, int W, int BH, int BW,
                         int32_t* row_ptr, int32_t* bcsr_idx,
                         int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                         int32_t* nnz_dev, int cap, spx_stream_t stream);

/* Row / column sums of compressed values (fp32 accumulate), used for the bias
 * gradient of a compressed sparse-output matmul.  Replace
 * BCSFunctionContext.row_sum / col_sum (block_compressed.py:360-403) and
 * bcsr_val_sum_row / bcsr_val_sum_col (block_compressed.cu.j2:222-288).
 * axis 0: result [batch, H] = sum over W;  axis 1: result [batch, W] = sum
 * over H.  Every entry of `result` is written (zero where no block is live) and
 * the additions follow the index order, so the sums are bit-identical from run
 * to run (the reference adds with atomics).  idx as in spx_bcs_gather.  `sparse`
 * holds values of type `dtype` (f32, f16 or bf16); `result` is fp32 in every case.
 * With nnz == 0 `sparse` and `idx` may be NULL and `result` is filled with zeros. */
int spx_bcs_sum(const void* sparse, void* result, const void* idx, int idx_kind,
                int nnz, int batch, int H, int W, int BH, int BW, int dtype, int axis,
                int64_t sparse_batch_stride, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * Block-sparse matmul C = op(A) op(B) (+ bias), fp32 accumulate on MFMA.
 * Replaces the launch closures of SparseMatMulKernel.update_func
 * (sparta/specializer/kernels/matmul.py:151-188) and the six
 * {sparta,openai}_sparse_matmul_{sdd,dsd,dds}.cuh.j2 templates.
 *
 * mode letters name A, B, C in that order (matmul.py:60-84):
 *   SPX_SDD  A sparse: tile (BM,BK) BCSR if !transA, (BK,BM) BCSC if transA
 *   SPX_DSD  B sparse: tile (BN,BK) BCSR if  transB, (BK,BN) BCSC if !transB
 *   SPX_DDS  C sparse: tile (BM,BN) BCSR, one entry per live output block
 * A is [batch,K,M] if transA else [batch,M,K]; B is [batch,N,K] if transB else
 * [batch,K,N]; bias (optional) is [batch,N]; C is [batch,M,N].
 * compressed != 0: the sparse tensor is [batch, nnz*tileH*tileW] compressed
 * values with sparse_batch_stride elements between batches; otherwise it is
 * stored dense and the index only selects tiles (a dense DDS output must be
 * zero-filled by the caller; dead tiles are not written).  A compressed sparse
 * tensor with nnz_bound == 0 may be NULL (and idx with it) under every tile
 * configuration, the persistent one (10) included: C is then bias (or zero).
 * ptr  row_ptr (BCSR) or col_ptr (BCSC); optional for DDS: row_ptr lets the launch
 *           group the live blocks of neighbouring block rows on one XCD (NULL = BCSR order).
 * idx / idx_kind  see spx_idx_kind.  nnz_bound / nnz_dev as in spx_bcs_gather
 *                 (only DDS launches over blocks).
 * sched     optional output of spx_bcs_schedule for `ptr` (NULL = natural order).
 * tile_cfg  index into the tile-config table of the op (0 = default), optionally or-ed
 *           with SPX_EPILOGUE_RELU (SDD and DSD): C = max(op(A) op(B) + bias, 0), NaN kept,
 *           written by the same kernel.  No counterpart in the reference, whose
 *           SparseLinear is followed by a separate activation kernel.
 * ------------------------------------------------------------------------ */
#define SPX_EPILOGUE_RELU 0x10000
int spx_matmul(int mode, int dtype, int transA, int transB, int compressed,
               const void* A, const void* B, const void* bias, void* C,
               const int32_t* ptr, const void* idx, int idx_kind, const int32_t* sched,
               int nnz_bound, const int32_t* nnz_dev, int64_t sparse_batch_stride,
               int batch, int M, int K, int N, int BM, int BK, int BN,
               int tile_cfg, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * Masked block-sparse softmax over the last axis.
 * Replaces SparseSoftmaxForwardKernel.update_func / BackwardKernel.update_func
 * (sparta/specializer/kernels/softmax.py:65-88,120-145) and
 * sparta_sparse_softmax_{forward,backward}.cuh.j2.
 *   y = exp((x - max_live) * inv_temperature) / sum_live, 0 on masked entries
 *   and on fully masked rows.
 *   grad_x = inv_temperature * (y*grad_y - y * sum_live(y*grad_y))
 * x / y are [batch,H,W] (compressed == 0; only entries of live blocks are
 * written, the caller zero-fills y) or [batch, nnz*BH*BW] (compressed != 0;
 * every entry is written).  mask is uint8 in the same layout as one batch of x;
 * NULL means that every entry of a live block takes part.
 * batch_stride: elements between batches of x / y.
 * tile_cfg: 0 = pick; 1 = one entry per access; 2 = 16-byte accesses, one
 * wavefront per row; 3 = 16-byte accesses, sixteen lanes per row (for rows of
 * at most 512 live 16-bit entries; longer rows stay correct).  2 and 3 need BW
 * a multiple of 16 bytes of entries and 16-byte aligned tensors.
 * ------------------------------------------------------------------------ */
int spx_softmax_forward(int dtype, int compressed, const void* x, void* y,
                        const int32_t* row_ptr, const int32_t* bcsr_idx,
                        const uint8_t* mask, float inv_temperature,
                        int batch, int H, int W, int BH, int BW,
                        int64_t batch_stride, int tile_cfg, spx_stream_t stream);
int spx_softmax_backward(int dtype, int compressed, const void* grad_y, const void* y,
                         void* grad_x, const int32_t* row_ptr, const int32_t* bcsr_idx,
                         const uint8_t* mask, float inv_temperature,
                         int batch, int H, int W, int BH, int BW,
                         int64_t batch_stride, int tile_cfg, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * Fused block-sparse attention forward:
 *   out = softmax_masked(q k^T * inv_temperature) v   per batch*head.
 * One kernel for the three launches of SparseAttention.forward
 * (sparta/specializer/operators/sparse_attention.py:76-80); the score matrix
 * never reaches HBM.  q,out [batch,Nt,E]; k,v [batch,Ns,E]; BCSR index over
 * (BH,BW) tiles of the [Nt,Ns] mask; mask optional uint8 [Nt,Ns] element mask
 * (NULL = every element of a live block is live).
 * ------------------------------------------------------------------------ */
int spx_attention_forward(int dtype, const void* q, const void* k, const void* v, void* out,
                          const int32_t* row_ptr, const int32_t* bcsr_idx,
                          const uint8_t* mask, float inv_temperature,
                          int batch, int Nt, int Ns, int E, int BH, int BW,
                          int tile_cfg, spx_stream_t stream);

/* Forward pass for training: like spx_attention_forward, and also writes the normalised
 * probabilities in the compressed layout of the softmax operator (block e of the BCSR
 * order at e * BH * BW, row-major inside the block; probs_batch_stride elements between
 * batch entries), which the backward kernels read.  Replaces the three launches of
 * SparseAttention.forward when gradients are recorded (sparse_attention.py:76-80).
 * Query blocks 32 / 64 / 128, key blocks 32 / 64 / 128, head dims 64 / 128. */
int spx_attention_forward_train(int dtype, const void* q, const void* k, const void* v, void* out,
                                void* probs, int64_t probs_batch_stride,
                                const int32_t* row_ptr, const int32_t* bcsr_idx,
                                const uint8_t* mask, float inv_temperature,
                                int batch, int Nt, int Ns, int E, int BH, int BW,
                                spx_stream_t stream);

/* Row side of the backward pass, from the probabilities spx_attention_forward_train saved:
 *   grad_scores = probs o (grad_out v^T - D) * inv_temperature,  D[i] = sum_e grad_out[i,e] out[i,e]
 *   grad_q      = grad_scores k
 * grad_scores (may be NULL: not stored) has the compressed layout and batch stride of probs; it
 * is the operand of grad_k = grad_scores^T q through spx_matmul with the sparse operand
 * transposed, as probs is of grad_v = probs^T grad_out.  row_dot (may be NULL) receives
 * D[b, i] * inv_temperature as float [batch, Nt], which spx_attention_backward_kv reads.
 * Masked entries carry probs = 0 and get grad_scores = 0.  Replaces three launches of the
 * reference's backward chain: the dense x dense -> sparse product of SparseBatchMatMul's
 * backward, SparseSoftmax's backward and the sparse x dense product for the query gradient
 * (sparse_attention.py:76-80 run in reverse by autograd).  Same block shapes as
 * spx_attention_forward_train. */
int spx_attention_backward_scores(int dtype, const void* grad_out, const void* out, const void* probs,
                                  const void* k, const void* v, void* grad_scores, void* grad_q,
                                  float* row_dot, int64_t probs_batch_stride,
                                  const int32_t* row_ptr, const int32_t* bcsr_idx, float inv_temperature,
                                  int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream);

/* Column side of the backward pass: grad_v = probs^T grad_out and grad_k = grad_scores^T q
 * with grad_scores recomputed from probs, grad_out, v and row_dot (written by
 * spx_attention_backward_scores), walking the BCSC index (idx_kind SPX_IDX_BCSC_I64 when the
 * values are in BCSR order, as spx_attention_forward_train writes them; SPX_IDX_BCSC_I32 for
 * values in BCSC order).  Replaces the two transposed sparse x dense products of the
 * reference's backward chain (batch_matmul.py:47-71, backward:B of both matmuls) and the
 * write and two reads of the score gradient between them.  Query blocks 32 / 64 / 128, key
 * blocks 32 / 64 / 128, head dims 64 / 128, BH * E >= 32 * BW. */
int spx_attention_backward_kv(int dtype, const void* grad_out, const void* q, const void* v,
                              const void* probs, const float* row_dot, void* grad_k, void* grad_v,
                              int64_t probs_batch_stride,
                              const int32_t* col_ptr, const void* bcsc_idx, int idx_kind, float inv_temperature,
                              int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream);

/* Training path that keeps no probabilities.  spx_attention_forward_lse is
 * spx_attention_forward (pipelined kernel) that also records, per query, the log2-domain
 * log-sum-exp of its score row (row_lse, float [batch, Nt]; +inf for a row without a live
 * entry): probs = exp2(score * inv_temperature * log2(e) - row_lse).  The two backward entry
 * points recompute the probabilities of every live block from q, k and row_lse instead of
 * reading them: spx_attention_backward_q gives grad_q and row_dot (as
 * spx_attention_backward_scores does, which it replaces together with the probability buffer),
 * spx_attention_backward_kv_recompute gives grad_k and grad_v (as spx_attention_backward_kv).
 * Against the reference's backward chain (sparse_attention.py:76-80 run in reverse: five
 * launches, probabilities and score gradients written and re-read) the whole step reads and
 * writes only q, k, v, out, grad_out and the three gradients.  Block-level masks only (every
 * element of a live block attends): element masks go through spx_attention_forward_train.
 * 16-bit types; block shapes as spx_attention_forward_train, the column side also BH <= 2 * BW. */
int spx_attention_forward_lse(int dtype, const void* q, const void* k, const void* v, void* out,
                              float* row_lse, const int32_t* row_ptr, const int32_t* bcsr_idx,
                              const uint8_t* mask, float inv_temperature,
                              int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream);
int spx_attention_backward_q(int dtype, const void* grad_out, const void* out, const void* q,
                             const void* k, const void* v, const float* row_lse,
                             void* grad_q, float* row_dot,
                             const int32_t* row_ptr, const int32_t* bcsr_idx, float inv_temperature,
                             int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream);
int spx_attention_backward_kv_recompute(int dtype, const void* grad_out, const void* q, const void* k,
                                        const void* v, const float* row_lse, const float* row_dot,
                                        void* grad_k, void* grad_v,
                                        const int32_t* col_ptr, const void* bcsc_idx, int idx_kind,
                                        float inv_temperature,
                                        int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * Sequence-length attention: q, k, v, out are [batch, heads, N, E]; batch b
 * attends over its first seqlens[b] positions only (int32 [batch], on the
 * device; values are clamped to [0, N]):
 *   out[b,h,i,:] = softmax_{j < L}(q_i . k_j * inv_temperature) v_j   for i < L,
 *   out[b,h,i,:] = 0                                                    for i >= L.
 * fp32, fp16 and bf16; N and E multiples of 32, E in {32, 64, 96, 128}.
 * Replaces seqlen_dynamic_sparse_attention_cpp.forward(Q, K, V, inter_result,
 * seqlens, head_num) (csrc/seqlen_dynamic_sparse_attention_forward.cpp:7-26);
 * the reference applies no temperature (pass 1.0f) and needs a [B*H*N*N] fp32
 * scratch that this entry point does not.
 * ------------------------------------------------------------------------ */
int spx_attention_seqlen_forward(int dtype, const void* q, const void* k, const void* v, void* out,
                                 const int32_t* seqlens, float inv_temperature,
                                 int batch, int heads, int N, int E,
                                 int tile_cfg, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * MoE sparse forward: out[t,:] = tokens[t,:] . W[exp_ids[t]].
 * Replace sparse_moe_cpp.convert_index / forward
 * (csrc/moe_sparse_forward.cpp:7-25, csrc/moe_sparse_forward_kernel.cu.j2:58-116,
 * :120-325, :363-483) with a stable counting sort (no per-expert capacity) and a
 * gathered GEMM over a flattened (expert, row-tile) list.
 *   exp_ids int32 [n_tok]; expert_count int32 [n_exp];
 *   expert_offset int32 [n_exp+1] exclusive prefix; token_perm int32 [n_tok]:
 *   token_perm[expert_offset[e] + j] = j-th token (ascending) routed to e.
 *   Tokens whose id lies outside [0, n_exp) (the reference indexes out of bounds
 *   for them) are listed, ascending, in token_perm[expert_offset[n_exp] .. n_tok)
 *   and spx_moe_forward writes zero rows for them, so every row of out is defined.
 *   workspace: spx_moe_index_workspace_bytes(n_tok, n_exp) bytes, 256-byte aligned.
 *   tokens [n_tok,in_dim]; out [n_tok,out_dim];
 *   weight [n_exp,in_dim,out_dim] (weight_layout 0, the reference's stacked
 *   weight.T, sparse_moe.py:19-22) or [n_exp,out_dim,in_dim] (weight_layout 1, the
 *   layout of nn.Linear.weight; in_dim contiguous, the faster one here).
 * ------------------------------------------------------------------------ */
size_t spx_moe_index_workspace_bytes(int n_tok, int n_exp);
int spx_moe_index(const int32_t* exp_ids, int n_tok, int n_exp,
                  int32_t* expert_count, int32_t* expert_offset, int32_t* token_perm,
                  void* workspace, size_t workspace_bytes, spx_stream_t stream);
int spx_moe_forward(int dtype, const void* tokens, const void* weight, int weight_layout, void* out,
                    const int32_t* expert_offset, const int32_t* token_perm,
                    int n_tok, int in_dim, int out_dim, int n_exp,
                    int tile_cfg, spx_stream_t stream);

/* ------------------------------------------------------------------------ *
 * Tile-configuration table searched by tune(); replaces the Jinja template
 * parameters and look_up_tables/sparta_matmul_lut.csv.
 * op: 0 sdd/dsd matmul, 1 dds matmul, 2 softmax, 3 attention, 4 moe.
 * ------------------------------------------------------------------------ */
typedef struct spx_tile_cfg {
    int id;
    int tile_m;        /* output rows per workgroup (dense dimension)       */
    int tile_n;        /* output cols per workgroup (0 = the sparse block)  */
    int waves;         /* wavefronts per workgroup                          */
    int lds_stages;    /* LDS staging depth                                 */
    int min_block;     /* smallest sparse block edge the config accepts     */
    int dtype_mask;    /* bit i set: spx_dtype i supported                  */
    char name[32];
} spx_tile_cfg;
int spx_num_tile_cfgs(int op);
int spx_tile_cfg_info(int op, int id, spx_tile_cfg* out);

#ifdef __cplusplus
}
#endif
#endif /* SPARTA_HIP_H_ */
