// BCSR / BCSC index build for a uint8 element mask.
//
// Two launches, no host round trip, no atomics, canonical (sorted) order.  Block grids
// of at most 2048 row words and 2048 column words (a word = 64 blocks) take the pair
// live_bits_kernel + emit_words_kernel described further down; larger grids and masks
// whose rows cannot be read with 16-byte loads take the general pair:
//   1. liveness_kernel: streams the mask once and writes one byte per block ("any byte
//      of the tile non-zero").
//   2. emit_kernel (one workgroup): turns the byte map into 64-block words with
//      wavefront ballots, prefix-scans the word popcounts (which directly yields
//      row_ptr / col_ptr and every block's rank), and writes the index arrays.  With
//      more than 256 words the same three steps run as three launches, the first and
//      the last with one wavefront per word (emit_general_*_kernel).
// Replaces bcs_index_1 / bcs_index_2 of the reference
// (sparta/tesa/templates/block_compressed.cu.j2:67-170) and the cumsum + .item()
// glue of sparta/tesa/block_compressed.py:242-309.
#include "common.hpp"
#include <mutex>

namespace spx {

struct LiveParams {
    const uint8_t* mask;
    uint8_t* live;
    int H, W, BH, BW, Cn;
    int segw;      // bytes of a mask row covered by one workgroup (power of two)
    int log_tcols; // log2(segw / VEC)
    int log_bw;
};

template <int VEC>
__global__ __launch_bounds__(256) void liveness_kernel(LiveParams p) {
    __shared__ uint32_t flags[256];
    const int tid = threadIdx.x;
    flags[tid] = 0;
    __syncthreads();

    const int tcols = 1 << p.log_tcols;
    const int trows = 256 >> p.log_tcols;
    const int tx = tid & (tcols - 1);
    const int ty = tid >> p.log_tcols;
    const int seg = blockIdx.x;
    const int r = blockIdx.y;
    const int64_t col_byte = (int64_t)seg * p.segw + (int64_t)tx * VEC;

    if (col_byte < p.W) {
        const uint8_t* src = p.mask + ((int64_t)r * p.BH) * p.W + col_byte;
        if constexpr (VEC == 16) {
            uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
            for (int row = ty; row < p.BH; row += trows) {
                const vec16 v = *reinterpret_cast<const vec16*>(src + (int64_t)row * p.W);
                a0 |= v.x; a1 |= v.y; a2 |= v.z; a3 |= v.w;
            }
            if (p.BW >= 16) {
                if (a0 | a1 | a2 | a3) flags[(tx * 16) >> p.log_bw] = 1;
            } else if (p.BW == 8) {
                if (a0 | a1) flags[tx * 2] = 1;
                if (a2 | a3) flags[tx * 2 + 1] = 1;
            } else {  // BW == 4
                if (a0) flags[tx * 4] = 1;
                if (a1) flags[tx * 4 + 1] = 1;
                if (a2) flags[tx * 4 + 2] = 1;
                if (a3) flags[tx * 4 + 3] = 1;
            }
        } else if constexpr (VEC == 4) {
            uint32_t a = 0;
            for (int row = ty; row < p.BH; row += trows)
                a |= *reinterpret_cast<const uint32_t*>(src + (int64_t)row * p.W);
            if (a) flags[(tx * 4) >> p.log_bw] = 1;
        } else {
            uint32_t a = 0;
            for (int row = ty; row < p.BH; row += trows) a |= src[(int64_t)row * p.W];
            if (a) flags[tx >> p.log_bw] = 1;
        }
    }
    __syncthreads();
    const int blk_per_seg = p.segw >> p.log_bw;
    if (tid < blk_per_seg) {
        const int c = seg * blk_per_seg + tid;
        if (c < p.Cn) p.live[(int64_t)r * p.Cn + c] = (uint8_t)flags[tid];
    }
}

struct EmitParams {
    const uint8_t* live;
    unsigned long long* wbits;  // [R * WPR] row words
    int* wbase;                 // [R * WPR] exclusive prefix of row-word popcounts
    int* cbase;                 // [Cn * WPC] exclusive prefix of column-word popcounts
    int32_t* row_ptr;
    int32_t* bcsr_idx;
    int32_t* col_ptr;
    void* bcsc_idx;
    int bcsc_i64;
    int32_t* nnz_dev;
    int cap;
    int R, Cn, WPR, WPC;
    int32_t* row_order;         // optional: block rows / columns by descending number of live blocks
    int32_t* col_order;
};

// Launch order: the n segments of ptr sorted by descending length (bucketed at 255), by
// one workgroup; bins is a 256-entry LDS table.  ptr may have been written by this
// workgroup just before (the leading barrier orders those stores).
__device__ void schedule_segments(const int32_t* ptr, int n, int32_t* order, int* bins) {
    __syncthreads();
    for (int i = threadIdx.x; i < 256; i += blockDim.x) bins[i] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int c = ptr[i + 1] - ptr[i];
        atomicAdd(&bins[255 - (c < 255 ? c : 255)], 1);
    }
    __syncthreads();
    if (threadIdx.x < 64) {  // exclusive scan of the 256 bins by one wavefront
        int carry = 0;
        for (int b0 = 0; b0 < 256; b0 += 64) {
            const int v = bins[b0 + threadIdx.x];
            const int inc = wave_inclusive_scan(v);
            bins[b0 + threadIdx.x] = carry + inc - v;
            carry += __shfl(inc, 63, 64);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int c = ptr[i + 1] - ptr[i];
        order[atomicAdd(&bins[255 - (c < 255 ? c : 255)], 1)] = i;
    }
}

// Exclusive prefix sum of a[0..n) in place by one workgroup; returns the total.
__device__ int block_scan_inplace(int* a, int n, int* lds) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    int carry = 0;
    for (int base = 0; base < n; base += blockDim.x) {
        const int i = base + threadIdx.x;
        const int v = i < n ? a[i] : 0;
        const int inc = wave_inclusive_scan(v);
        if (lane == 63) lds[wave] = inc;
        __syncthreads();
        int before = 0, total = 0;
        for (int w = 0; w < nwaves; ++w) {
            const int t = lds[w];
            if (w < wave) before += t;
            total += t;
        }
        if (i < n) a[i] = carry + before + inc - v;
        carry += total;
        __syncthreads();
    }
    return carry;
}

__global__ __launch_bounds__(1024) void emit_kernel(EmitParams p) {
    __shared__ int lds[32];
    __shared__ int s_bins[256];
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

    // ---- row words -----------------------------------------------------------
    const int NW = p.R * p.WPR;
    for (int g = wave; g < NW; g += nwaves) {
        const int r = g / p.WPR;
        const int c = (g - r * p.WPR) * 64 + lane;
        const bool flag = c < p.Cn && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (lane == 0) {
            p.wbits[g] = word;
            p.wbase[g] = __popcll(word);
        }
    }
    __syncthreads();
    const int nnz = block_scan_inplace(p.wbase, NW, lds);
    if (threadIdx.x == 0) p.nnz_dev[0] = nnz;

    if (p.row_ptr) {
        for (int r = threadIdx.x; r < p.R; r += blockDim.x) p.row_ptr[r] = p.wbase[r * p.WPR];
        if (threadIdx.x == 0) p.row_ptr[p.R] = nnz;
    }
    if (p.bcsr_idx) {
        for (int g = wave; g < NW; g += nwaves) {
            const int r = g / p.WPR;
            const int c = (g - r * p.WPR) * 64 + lane;
            const unsigned long long word = p.wbits[g];
            if ((word >> lane) & 1ull) {
                const int pos = p.wbase[g] + __popcll(word & lt_mask);
                if (pos < p.cap) p.bcsr_idx[pos] = (r << 16) | c;
            }
        }
    }
    if (p.row_order && p.row_ptr) schedule_segments(p.row_ptr, p.R, p.row_order, s_bins);
    if (!p.col_ptr) return;  // uniform over the workgroup

    // ---- column words --------------------------------------------------------
    const int NWC = p.Cn * p.WPC;
    for (int g = wave; g < NWC; g += nwaves) {
        const int c = g / p.WPC;
        const int r = (g - c * p.WPC) * 64 + lane;
        const bool flag = r < p.R && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (lane == 0) p.cbase[g] = __popcll(word);
    }
    __syncthreads();
    const int nnz2 = block_scan_inplace(p.cbase, NWC, lds);
    for (int c = threadIdx.x; c < p.Cn; c += blockDim.x) p.col_ptr[c] = p.cbase[c * p.WPC];
    if (threadIdx.x == 0) p.col_ptr[p.Cn] = nnz2;

    if (p.bcsc_idx) {
        for (int g = wave; g < NWC; g += nwaves) {
            const int c = g / p.WPC;
            const int r = (g - c * p.WPC) * 64 + lane;
            const bool flag = r < p.R && p.live[(int64_t)r * p.Cn + c] != 0;
            const unsigned long long word = __ballot(flag);
            if (flag) {
                const int pos = p.cbase[g] + __popcll(word & lt_mask);
                if (pos < p.cap) {
                    if (p.bcsc_i64) {
                        const int gw = r * p.WPR + (c >> 6);
                        const int cl = c & 63;
                        const unsigned long long below =
                            cl == 0 ? 0ull : (p.wbits[gw] & (~0ull >> (64 - cl)));
                        const long long bpos = p.wbase[gw] + __popcll(below);
                        reinterpret_cast<long long*>(p.bcsc_idx)[pos] =
                            (bpos << 32) | ((long long)c << 16) | (long long)r;
                    } else {
                        reinterpret_cast<int32_t*>(p.bcsc_idx)[pos] = (c << 16) | r;
                    }
                }
            }
        }
    }
    if (p.col_order) schedule_segments(p.col_ptr, p.Cn, p.col_order, s_bins);
}

// ---- the same work spread over the device, for block grids with many words ----------------
// emit_kernel walks the words with the sixteen wavefronts of one workgroup, one dependent
// load per step: a grid of 4096 row words takes it 200 us.  The three kernels below do the
// same steps in the same order of results - word building and index writing by one
// wavefront per word across as many workgroups as there are words, the two prefix sums,
// the pointer arrays and the launch orders by a single workgroup in between.

// wavefront g < NW: row word g (bits and popcount); NW <= g < NW + NWC: popcount of column word g - NW
__global__ __launch_bounds__(256) void emit_general_words_kernel(EmitParams p) {
    const int lane = lane_id();
    const int g = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int NW = p.R * p.WPR;
    const int NWC = p.col_ptr ? p.Cn * p.WPC : 0;
    if (g < NW) {
        const int r = g / p.WPR;
        const int c = (g - r * p.WPR) * 64 + lane;
        const bool flag = c < p.Cn && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (lane == 0) {
            p.wbits[g] = word;
            p.wbase[g] = __popcll(word);
        }
    } else if (g < NW + NWC) {
        const int gc = g - NW;
        const int c = gc / p.WPC;
        const int r = (gc - c * p.WPC) * 64 + lane;
        const bool flag = r < p.R && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (lane == 0) p.cbase[gc] = __popcll(word);
    }
}

__global__ __launch_bounds__(1024) void emit_general_scan_kernel(EmitParams p) {
    __shared__ int lds[32];
    __shared__ int s_bins[256];
    const int NW = p.R * p.WPR;
    const int nnz = block_scan_inplace(p.wbase, NW, lds);
    if (threadIdx.x == 0) p.nnz_dev[0] = nnz;
    if (p.row_ptr) {
        __syncthreads();   // the scanned values were written by other threads of the workgroup
        for (int r = threadIdx.x; r < p.R; r += blockDim.x) p.row_ptr[r] = p.wbase[r * p.WPR];
        if (threadIdx.x == 0) p.row_ptr[p.R] = nnz;
    }
    if (p.row_order && p.row_ptr) schedule_segments(p.row_ptr, p.R, p.row_order, s_bins);
    if (!p.col_ptr) return;  // uniform over the workgroup
    __syncthreads();
    const int NWC = p.Cn * p.WPC;
    const int nnz2 = block_scan_inplace(p.cbase, NWC, lds);
    __syncthreads();
    for (int c = threadIdx.x; c < p.Cn; c += blockDim.x) p.col_ptr[c] = p.cbase[c * p.WPC];
    if (threadIdx.x == 0) p.col_ptr[p.Cn] = nnz2;
    if (p.col_order) schedule_segments(p.col_ptr, p.Cn, p.col_order, s_bins);
}

// wavefront g < NW: the BCSR entries of row word g; NW <= g < NW + NWC: the BCSC entries of column word g - NW
__global__ __launch_bounds__(256) void emit_general_write_kernel(EmitParams p) {
    const int lane = lane_id();
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const int g = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int NW = p.R * p.WPR;
    const int NWC = p.bcsc_idx ? p.Cn * p.WPC : 0;
    if (g < NW) {
        if (!p.bcsr_idx) return;
        const int r = g / p.WPR;
        const int c = (g - r * p.WPR) * 64 + lane;
        const unsigned long long word = p.wbits[g];
        if ((word >> lane) & 1ull) {
            const int pos = p.wbase[g] + __popcll(word & lt_mask);
            if (pos < p.cap) p.bcsr_idx[pos] = (r << 16) | c;
        }
    } else if (g < NW + NWC) {
        const int gc = g - NW;
        const int c = gc / p.WPC;
        const int r = (gc - c * p.WPC) * 64 + lane;
        const bool flag = r < p.R && p.live[(int64_t)r * p.Cn + c] != 0;
        const unsigned long long word = __ballot(flag);
        if (flag) {
            const int pos = p.cbase[gc] + __popcll(word & lt_mask);
            if (pos < p.cap) {
                if (p.bcsc_i64) {
                    const int gw = r * p.WPR + (c >> 6);
                    const int cl = c & 63;
                    const unsigned long long below = cl == 0 ? 0ull : (p.wbits[gw] & (~0ull >> (64 - cl)));
                    const long long bpos = p.wbase[gw] + __popcll(below);
                    reinterpret_cast<long long*>(p.bcsc_idx)[pos] = (bpos << 32) | ((long long)c << 16) | (long long)r;
                } else {
                    reinterpret_cast<int32_t*>(p.bcsc_idx)[pos] = (c << 16) | r;
                }
            }
        }
    }
}

// ---- fast path: block grids of at most 2048 row words and 2048 column words ----------
// (a word = the liveness bits of 64 consecutive blocks of a block-row or block-column).
// Two launches; at this size both are bound by launch and memory latency and by the
// number of instructions a wavefront issues, not by bandwidth, so the layout of the work
// is chosen to keep every dependent chain short:
//   live_bits_kernel   one workgroup per (row word, group of mask rows): ORs the 64 x BW
//                      bytes of each of its mask rows (16-byte loads, all independent)
//                      and writes the 64 liveness bits as one 8-byte partial word (very
//                      small grids split the BH mask rows of a block-row over up to eight
//                      workgroups, whose partial words the second kernel ORs together).
//   emit_words_kernel  one group of workgroups per requested format (BCSR side, BCSC
//                      side), each split into `nslice` slices.  Every workgroup loads all
//                      row words (<= 16 KB, one coalesced load per thread), prefix-sums
//                      their popcounts in LDS and - on the BCSC side - transposes them into
//                      column words 64 x 64 bits at a time with a six-step lane butterfly
//                      (one wavefront per tile).  It then writes only its slice of the index
//                      entries, one word per wavefront instruction (lane = bit, rank = word
//                      base + popcount of the lower bits), so a dense mask still stores 64
//                      entries per instruction.  Slice 0 of a side writes the pointer array
//                      and nnz, the last slice the launch order.
constexpr int EMIT_FAST_WORDS = 2048;

struct BitsParams {
    const uint8_t* mask;
    unsigned long long* pbits;  // [Q][R * WPR] partial words, one per group of mask rows
    int W, BH, BW, WPR, NW;
    int log_bw;
    int rows_per_part;          // mask rows of a block-row that one workgroup covers (BH / Q)
};

// word wi of block-row r, row group `part`
__device__ __forceinline__ void live_bits_body(const BitsParams& p, int wi, int r, int part) {
    __shared__ uint32_t flags[64];
    const int tid = threadIdx.x;
    if (tid < 64) flags[tid] = 0;
    __syncthreads();
    const int64_t col0 = (int64_t)wi * 64 * p.BW;            // first mask column of the word
    const int64_t left = p.W - col0;
    const int nch = (int)((left < 64 * p.BW ? left : 64 * p.BW) >> 4);  // 16-byte chunks per mask row
    const uint8_t* base = p.mask + ((int64_t)r * p.BH + (int64_t)part * p.rows_per_part) * p.W + col0;
    const int log_nch = p.log_bw + 2;                         // log2 of the chunks of a full word
    const int nrows = p.rows_per_part;

    auto mark = [&](int chunk, uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3) {
        if (p.BW >= 16) {
            if (a0 | a1 | a2 | a3) flags[(chunk << 4) >> p.log_bw] = 1;
        } else if (p.BW == 8) {
            if (a0 | a1) flags[chunk * 2] = 1;
            if (a2 | a3) flags[chunk * 2 + 1] = 1;
        } else {  // BW == 4
            if (a0) flags[chunk * 4] = 1;
            if (a1) flags[chunk * 4 + 1] = 1;
            if (a2) flags[chunk * 4 + 2] = 1;
            if (a3) flags[chunk * 4 + 3] = 1;
        }
    };
    if (log_nch <= 8) {
        // a thread keeps one chunk column and walks the mask rows 256 >> log_nch apart
        const int chunk = tid & ((1 << log_nch) - 1);
        const int rstep = 256 >> log_nch;
        if (chunk < nch) {
            uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
            const uint8_t* src = base + (int64_t)chunk * 16;
#pragma unroll 8
            for (int row = tid >> log_nch; row < nrows; row += rstep) {
                const vec16 v = *reinterpret_cast<const vec16*>(src + (int64_t)row * p.W);
                a0 |= v.x; a1 |= v.y; a2 |= v.z; a3 |= v.w;
            }
            mark(chunk, a0, a1, a2, a3);
        }
    } else {
        for (int chunk = tid; chunk < nch; chunk += 256) {
            uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
            const uint8_t* src = base + (int64_t)chunk * 16;
#pragma unroll 8
            for (int row = 0; row < nrows; ++row) {
                const vec16 v = *reinterpret_cast<const vec16*>(src + (int64_t)row * p.W);
                a0 |= v.x; a1 |= v.y; a2 |= v.z; a3 |= v.w;
            }
            mark(chunk, a0, a1, a2, a3);
        }
    }
    __syncthreads();
    if (tid < 64) {
        const unsigned long long word = __ballot(flags[tid] != 0);
        if (tid == 0) p.pbits[(int64_t)part * p.NW + (int64_t)r * p.WPR + wi] = word;
    }
}

__global__ __launch_bounds__(256) void live_bits_kernel(BitsParams p) {
    live_bits_body(p, blockIdx.x, blockIdx.y, blockIdx.z);
}

__device__ __forceinline__ int block_exclusive_scan_1024(int v, int* lds, int* total) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int inc = wave_inclusive_scan(v);
    __syncthreads();  // lds may still be read from a previous call
    if (lane == 63) lds[wave] = inc;
    __syncthreads();
    int before = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        const int t = lds[w];
        if (w < wave) before += t;
        tot += t;
    }
    *total = tot;
    return before + inc - v;
}

// Launch order of n segments whose lengths are base[(i + 1) * stride] - base[i * stride]
// (base in LDS, `total` closing the last one): descending length, bucketed at 255.
// Segments of equal length come out in the order their lanes reach the LDS counter:
// any order of them is as good for scheduling, the result only has to be a permutation.
__device__ void schedule_from_lds(const int* base, int stride, int n, int total, int32_t* order, int* bins) {
    for (int i = threadIdx.x; i < 256; i += blockDim.x) bins[i] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int c = (i + 1 < n ? base[(i + 1) * stride] : total) - base[i * stride];
        atomicAdd(&bins[255 - (c < 255 ? c : 255)], 1);
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        int carry = 0;
        for (int b0 = 0; b0 < 256; b0 += 64) {
            const int v = bins[b0 + threadIdx.x];
            const int inc = wave_inclusive_scan(v);
            bins[b0 + threadIdx.x] = carry + inc - v;
            carry += __shfl(inc, 63, 64);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int c = (i + 1 < n ? base[(i + 1) * stride] : total) - base[i * stride];
        order[atomicAdd(&bins[255 - (c < 255 ? c : 255)], 1)] = i;
    }
}

__device__ __forceinline__ unsigned long long shfl_xor_u64(unsigned long long x, int j) {
    const int lo = __shfl_xor((int)(unsigned)x, j, 64);
    const int hi = __shfl_xor((int)(unsigned)(x >> 32), j, 64);
    return ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo;
}

// 64 x 64 bit-matrix transpose over a wavefront: lane i holds row i on entry and column i
// on exit (bit b of the result of lane i = bit i of the input of lane b).  Six butterfly
// steps: lanes i and i ^ j exchange the off-diagonal j x j blocks.
__device__ __forceinline__ unsigned long long transpose_bits_64x64(unsigned long long x, int lane) {
    unsigned long long m = 0x00000000FFFFFFFFull;
#pragma unroll
    for (int j = 32; j >= 1; j >>= 1) {
        const unsigned long long y = shfl_xor_u64(x, j);
        x = (lane & j) ? ((x & ~m) | ((y & ~m) >> j)) : ((x & m) | ((y & m) << j));
        m ^= m << (j >> 1);
    }
    return x;
}

// workgroup bx of the nslice * (1 or 2) of one index
__device__ __forceinline__ void emit_words_body(const EmitParams& p, int nslice, int sides, int nparts, int bx) {
    __shared__ unsigned long long s_bits[EMIT_FAST_WORDS];   // row words
    __shared__ int s_base[EMIT_FAST_WORDS];                  // exclusive prefix of their popcounts
    __shared__ unsigned long long s_cbits[EMIT_FAST_WORDS];  // column words
    __shared__ int s_cbase[EMIT_FAST_WORDS];
    __shared__ int s_scan[16];
    __shared__ int s_bins[256];
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const int side = sides == 3 ? bx / nslice : (sides == 2 ? 1 : 0);  // 0 BCSR, 1 BCSC
    const int slice = bx % nslice;

    // ---- row words: word g = r * WPR + wi covers columns wi*64 .. wi*64+63 of row r ----
    const int NW = p.R * p.WPR;
    unsigned long long w0 = 0, w1 = 0;  // OR of the partial words of the row groups
    if (tid * 2 < NW) {
        const bool pair = tid * 2 + 1 < NW && (NW & 1) == 0;  // 16-byte loads need an even pitch
        for (int q = 0; q < nparts; ++q) {
            const unsigned long long* src = p.wbits + (int64_t)q * NW + tid * 2;
            if (pair) {
                const ulonglong2 v = *reinterpret_cast<const ulonglong2*>(src);
                w0 |= v.x; w1 |= v.y;
            } else {
                w0 |= src[0];
                if (tid * 2 + 1 < NW) w1 |= src[1];
            }
        }
    }
    const int c0 = __popcll(w0), c1 = __popcll(w1);
    int nnz;
    const int tbase = block_exclusive_scan_1024(c0 + c1, s_scan, &nnz);
    s_bits[tid * 2] = w0;
    s_bits[tid * 2 + 1] = w1;
    s_base[tid * 2] = tbase;
    s_base[tid * 2 + 1] = tbase + c0;
    __syncthreads();

    if (side == 0) {
        if (slice == 0) {
            if (tid == 0) {
                p.nnz_dev[0] = nnz;
                p.row_ptr[p.R] = nnz;
            }
            for (int r = tid; r < p.R; r += 1024) p.row_ptr[r] = s_base[r * p.WPR];
        }
        for (int g = slice * 16 + wave; g < NW; g += 16 * nslice) {
            const unsigned long long bits = s_bits[g];
            if ((bits >> lane) & 1ull) {
                const int pos = s_base[g] + __popcll(bits & lt_mask);
                const int r = g / p.WPR;
                if (pos < p.cap) p.bcsr_idx[pos] = (r << 16) | ((g - r * p.WPR) * 64 + lane);
            }
        }
        if (slice == nslice - 1 && p.row_order) schedule_from_lds(s_base, p.WPR, p.R, nnz, p.row_order, s_bins);
        return;
    }

    // ---- column words: word g = c * WPC + ri covers rows ri*64 .. ri*64+63 of column c ----
    const int NWC = p.Cn * p.WPC;
    s_cbits[tid * 2] = 0;
    s_cbits[tid * 2 + 1] = 0;
    __syncthreads();
    for (int tile = wave; tile < p.WPR * p.WPC; tile += 16) {  // tile = (ri, wi): 64 rows x 64 columns
        const int ri = tile / p.WPR, wi = tile - ri * p.WPR;
        const int r = ri * 64 + lane;
        const unsigned long long rows = r < p.R ? s_bits[r * p.WPR + wi] : 0ull;
        const unsigned long long col = transpose_bits_64x64(rows, lane);
        const int c = wi * 64 + lane;
        if (c < p.Cn) s_cbits[c * p.WPC + ri] = col;
    }
    __syncthreads();
    const unsigned long long cw0 = s_cbits[tid * 2], cw1 = s_cbits[tid * 2 + 1];
    int nnz2;
    const int cb = block_exclusive_scan_1024(__popcll(cw0) + __popcll(cw1), s_scan, &nnz2);
    s_cbase[tid * 2] = cb;
    s_cbase[tid * 2 + 1] = cb + __popcll(cw0);
    __syncthreads();
    if (slice == 0) {
        if (tid == 0) {
            p.col_ptr[p.Cn] = nnz2;
            if (sides == 2) p.nnz_dev[0] = nnz2;  // no BCSR side in this launch
        }
        for (int c = tid; c < p.Cn; c += 1024) p.col_ptr[c] = s_cbase[c * p.WPC];
    }
    for (int g = slice * 16 + wave; g < NWC; g += 16 * nslice) {
        const unsigned long long bits = s_cbits[g];
        if ((bits >> lane) & 1ull) {
            const int pos = s_cbase[g] + __popcll(bits & lt_mask);
            if (pos < p.cap) {
                const int c = g / p.WPC;
                const int r = (g - c * p.WPC) * 64 + lane;
                if (p.bcsc_i64) {
                    const int gw = r * p.WPR + (c >> 6);
                    const int cl = c & 63;
                    const unsigned long long below = cl == 0 ? 0ull : (s_bits[gw] & (~0ull >> (64 - cl)));
                    const long long bpos = s_base[gw] + __popcll(below);
                    reinterpret_cast<long long*>(p.bcsc_idx)[pos] = (bpos << 32) | ((long long)c << 16) | (long long)r;
                } else {
                    reinterpret_cast<int32_t*>(p.bcsc_idx)[pos] = (c << 16) | r;
                }
            }
        }
    }
    if (slice == nslice - 1 && p.col_order) schedule_from_lds(s_cbase, p.WPC, p.Cn, nnz2, p.col_order, s_bins);
}

__global__ __launch_bounds__(1024) void emit_words_kernel(EmitParams p, int nslice, int sides, int nparts) {
    emit_words_body(p, nslice, sides, nparts, (int)blockIdx.x);
}

// ---- several independent masks in one pair of launches ---------------------------------
// A model that rebuilds the indexes of several layers per step issues as many pairs of small
// dependent launches, each a few workgroups wide and each waiting for the one before it.
// Here the workgroups of up to INDEX_BATCH_MAX builds share the two launches: the x range of
// the grid is cut into one piece per build (x_end), the other grid dimensions are those of the
// largest build and the workgroups outside a build's own range leave at once.
constexpr int INDEX_BATCH_MAX = 4;
struct BitsBatch {
    BitsParams job[INDEX_BATCH_MAX];
    int x_end[INDEX_BATCH_MAX], R[INDEX_BATCH_MAX], nparts[INDEX_BATCH_MAX];
    int n;
};
struct EmitBatch {
    EmitParams job[INDEX_BATCH_MAX];
    int x_end[INDEX_BATCH_MAX], nslice[INDEX_BATCH_MAX], sides[INDEX_BATCH_MAX], nparts[INDEX_BATCH_MAX];
    int n;
};

__global__ __launch_bounds__(256) void live_bits_batch_kernel(BitsBatch b) {
    const int bx = blockIdx.x;
    int j = 0;
    while (j + 1 < b.n && bx >= b.x_end[j]) ++j;
    if ((int)blockIdx.y >= b.R[j] || (int)blockIdx.z >= b.nparts[j]) return;
    live_bits_body(b.job[j], bx - (j ? b.x_end[j - 1] : 0), blockIdx.y, blockIdx.z);
}

__global__ __launch_bounds__(1024) void emit_words_batch_kernel(EmitBatch b) {
    const int bx = blockIdx.x;
    int j = 0;
    while (j + 1 < b.n && bx >= b.x_end[j]) ++j;
    emit_words_body(b.job[j], b.nslice[j], b.sides[j], b.nparts[j], bx - (j ? b.x_end[j - 1] : 0));
}

__global__ __launch_bounds__(1024) void schedule_kernel(const int32_t* ptr, int n, int32_t* order) {
    __shared__ int bins[256];
    schedule_segments(ptr, n, order, bins);
}

struct IndexWorkspace {
    size_t live_off, wbits_off, wbase_off, cbase_off, pbits_off, total;
    int R, Cn, WPR, WPC;
};

static IndexWorkspace index_workspace(int H, int W, int BH, int BW) {
    IndexWorkspace w;
    w.R = H / BH;
    w.Cn = W / BW;
    w.WPR = (w.Cn + 63) / 64;
    w.WPC = (w.R + 63) / 64;
    size_t off = 0;
    w.live_off = off;  off += round_up((size_t)w.R * w.Cn, 256);
    w.wbits_off = off; off += round_up((size_t)w.R * w.WPR * 8, 256);
    w.wbase_off = off; off += round_up((size_t)w.R * w.WPR * 4, 256);
    w.cbase_off = off; off += round_up((size_t)w.Cn * w.WPC * 4, 256);
    // partial words of the fast path: up to 8 row groups of at most EMIT_FAST_WORDS words
    const size_t nw = (size_t)w.R * w.WPR;
    w.pbits_off = off; off += round_up((nw < 2048 ? nw : 2048) * 8 * 8, 256);
    w.total = off;
    return w;
}

static int check_index_shape(int H, int W, int BH, int BW) {
    SPX_REQUIRE(valid_block_edge(BH) && valid_block_edge(BW), SPX_E_CONFIG,
                "block size (%d,%d) must be a power of two in [4,256]", BH, BW);
    SPX_REQUIRE(H > 0 && W > 0 && H % BH == 0 && W % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a positive multiple of the block (%d,%d)", H, W, BH, BW);
    SPX_REQUIRE(H / BH <= 65535 && W / BW <= 65535, SPX_E_SHAPE,
                "more than 65535 blocks per dimension do not fit the 16-bit index fields");
    return 0;
}

}  // namespace spx

extern "C" size_t spx_bcs_index_workspace_bytes(int H, int W, int BH, int BW) {
    if (spx::check_index_shape(H, W, BH, BW) != 0) return 0;
    return spx::index_workspace(H, W, BH, BW).total;
}

namespace spx {
// what bcs_index_impl would have launched on the bit-word path, handed back instead
struct FastIndexJob {
    BitsParams bits;
    EmitParams emit;
    int WPR, R, nparts, nslice, sides;
    int ready;   // 0: this build takes the general path and was not prepared
};
// fast != NULL: validate and, where the bit-word path applies, fill *fast without launching
// (fast->ready = 1); where it does not, leave fast->ready = 0 and launch nothing either.
static int bcs_index_impl(const uint8_t* mask, int H, int W, int BH, int BW,
                          int32_t* row_ptr, int32_t* bcsr_idx,
                          int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                          int32_t* nnz_dev, int cap, int32_t* row_order, int32_t* col_order,
                          void* workspace, size_t workspace_bytes, spx_stream_t stream,
                          FastIndexJob* fast = nullptr);
}

extern "C" int spx_bcs_index(const uint8_t* mask, int H, int W, int BH, int BW,
                             int32_t* row_ptr, int32_t* bcsr_idx,
                             int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                             int32_t* nnz_dev, int cap,
                             void* workspace, size_t workspace_bytes, spx_stream_t stream) {
    return spx::bcs_index_impl(mask, H, W, BH, BW, row_ptr, bcsr_idx, col_ptr, bcsc_idx, bcsc_i64, nnz_dev, cap,
                               nullptr, nullptr, workspace, workspace_bytes, stream);
}

extern "C" int spx_bcs_index_scheduled(const uint8_t* mask, int H, int W, int BH, int BW,
                                       int32_t* row_ptr, int32_t* bcsr_idx,
                                       int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                                       int32_t* nnz_dev, int cap, int32_t* row_order, int32_t* col_order,
                                       void* workspace, size_t workspace_bytes, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(!row_order || row_ptr, SPX_E_NULL, "row_order needs the BCSR index");
    SPX_REQUIRE(!col_order || col_ptr, SPX_E_NULL, "col_order needs the BCSC index");
    return bcs_index_impl(mask, H, W, BH, BW, row_ptr, bcsr_idx, col_ptr, bcsc_idx, bcsc_i64, nnz_dev, cap,
                          row_order, col_order, workspace, workspace_bytes, stream);
}

static int spx::bcs_index_impl(const uint8_t* mask, int H, int W, int BH, int BW,
                               int32_t* row_ptr, int32_t* bcsr_idx,
                               int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                               int32_t* nnz_dev, int cap, int32_t* row_order, int32_t* col_order,
                               void* workspace, size_t workspace_bytes, spx_stream_t stream,
                               FastIndexJob* fast) {
    using namespace spx;
    if (fast) fast->ready = 0;
    int rc = check_index_shape(H, W, BH, BW);
    if (rc) return rc;
    SPX_REQUIRE(mask && nnz_dev && workspace, SPX_E_NULL, "mask, nnz_dev and workspace are required");
    SPX_REQUIRE((row_ptr != nullptr) == (bcsr_idx != nullptr), SPX_E_NULL,
                "row_ptr and bcsr_idx must be given together");
    SPX_REQUIRE((col_ptr != nullptr) == (bcsc_idx != nullptr), SPX_E_NULL,
                "col_ptr and bcsc_idx must be given together");
    SPX_REQUIRE(row_ptr || col_ptr, SPX_E_NULL, "neither a BCSR nor a BCSC index was requested");
    SPX_REQUIRE(!(bcsc_i64 && !bcsc_idx), SPX_E_NULL, "bcsc_i64 set without a bcsc_idx buffer");
    SPX_REQUIRE(cap >= 0, SPX_E_SHAPE, "negative index capacity");
    const IndexWorkspace ws = index_workspace(H, W, BH, BW);
    SPX_REQUIRE(workspace_bytes >= ws.total, SPX_E_WORKSPACE,
                "workspace of %zu bytes is smaller than the %zu required", workspace_bytes, ws.total);
    SPX_REQUIRE(aligned(workspace, 256), SPX_E_ALIGN, "workspace must be 256-byte aligned");
    SPX_REQUIRE(!bcsc_i64 || aligned(bcsc_idx, 8), SPX_E_ALIGN, "int64 bcsc_idx must be 8-byte aligned");

    char* wsb = reinterpret_cast<char*>(workspace);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);

    EmitParams ep;
    ep.live = reinterpret_cast<uint8_t*>(wsb + ws.live_off);
    ep.wbits = reinterpret_cast<unsigned long long*>(wsb + ws.wbits_off);
    ep.wbase = reinterpret_cast<int*>(wsb + ws.wbase_off);
    ep.cbase = reinterpret_cast<int*>(wsb + ws.cbase_off);
    ep.row_ptr = row_ptr; ep.bcsr_idx = bcsr_idx;
    ep.col_ptr = col_ptr; ep.bcsc_idx = bcsc_idx; ep.bcsc_i64 = bcsc_i64;
    ep.nnz_dev = nnz_dev; ep.cap = cap;
    ep.R = ws.R; ep.Cn = ws.Cn; ep.WPR = ws.WPR; ep.WPC = ws.WPC;
    ep.row_order = row_order; ep.col_order = col_order;

    // Widest load the mask's address and row pitch allow.
    int vec = 1;
    if (W % 16 == 0 && aligned(mask, 16)) vec = 16;
    else if (W % 4 == 0 && aligned(mask, 4)) vec = 4;

    if (vec == 16 && ws.R * ws.WPR <= EMIT_FAST_WORDS && ws.Cn * ws.WPC <= EMIT_FAST_WORDS) {
        // row groups: a power of two, at most 8, at least 4 mask rows each.  Measured on
        // 3072 x 768 and 4096 x 4096 masks, one workgroup per word is as fast as eight, so
        // the split only serves grids of fewer than 64 words
        int nparts = 1;
        while (nparts < 8 && BH / (nparts * 2) >= 4 && ws.R * ws.WPR * nparts < 64) nparts *= 2;
        BitsParams bp;
        bp.mask = mask;
        bp.pbits = reinterpret_cast<unsigned long long*>(wsb + ws.pbits_off);
        bp.W = W; bp.BH = BH; bp.BW = BW; bp.WPR = ws.WPR; bp.NW = ws.R * ws.WPR;
        bp.log_bw = ilog2(BW);
        bp.rows_per_part = BH / nparts;
        ep.wbits = bp.pbits;
        const int sides = (row_ptr ? 1 : 0) | (col_ptr ? 2 : 0);
        // enough slices that a slice writes at most ~2048 index entries
        int nslice = (ws.R * ws.Cn + 2047) / 2048;
        nslice = nslice < 1 ? 1 : (nslice > 8 ? 8 : nslice);
        if (fast) {   // the caller launches (several builds in one pair of launches)
            fast->bits = bp; fast->emit = ep;
            fast->WPR = ws.WPR; fast->R = ws.R; fast->nparts = nparts; fast->nslice = nslice; fast->sides = sides;
            fast->ready = 1;
            return 0;
        }
        hipLaunchKernelGGL(live_bits_kernel, dim3(ws.WPR, ws.R, nparts), dim3(256), 0, st, bp);
        SPX_LAUNCH_CHECK("live_bits_kernel");
        hipLaunchKernelGGL(emit_words_kernel, dim3(nslice * (sides == 3 ? 2 : 1)), dim3(1024), 0, st, ep, nslice, sides, nparts);
        SPX_LAUNCH_CHECK("emit_words_kernel");
        return 0;
    }

    if (fast) return 0;   // general path: the caller builds this one on its own

    // Segment width: at most 256 threads * vec bytes, at least one block wide;
    // narrowed while that buys more workgroups (the launch wants >> 256 of them).
    int segw = 256 * vec;
    if (segw > 1024) segw = 1024;
    int wpow = 1;
    while (wpow < W) wpow <<= 1;
    if (segw > wpow) segw = wpow;
    const int min_seg = BW > vec ? BW : vec;
    while (segw > min_seg && (int64_t)ws.R * ((W + segw - 1) / segw) < 2048) segw >>= 1;
    if (segw < min_seg) segw = min_seg;

    LiveParams lp;
    lp.mask = mask;
    lp.live = reinterpret_cast<uint8_t*>(wsb + ws.live_off);
    lp.H = H; lp.W = W; lp.BH = BH; lp.BW = BW; lp.Cn = ws.Cn;
    lp.segw = segw;
    lp.log_tcols = ilog2(segw / vec);
    lp.log_bw = ilog2(BW);
    dim3 grid((W + segw - 1) / segw, ws.R, 1);
    if (vec == 16) hipLaunchKernelGGL(liveness_kernel<16>, grid, dim3(256), 0, st, lp);
    else if (vec == 4) hipLaunchKernelGGL(liveness_kernel<4>, grid, dim3(256), 0, st, lp);
    else hipLaunchKernelGGL(liveness_kernel<1>, grid, dim3(256), 0, st, lp);
    SPX_LAUNCH_CHECK("liveness_kernel");
    const int64_t n_words = (int64_t)ws.R * ws.WPR + (col_ptr ? (int64_t)ws.Cn * ws.WPC : 0);
    if (n_words <= 256) {   // few words: one workgroup does all of it in one launch
        hipLaunchKernelGGL(emit_kernel, dim3(1), dim3(1024), 0, st, ep);
        SPX_LAUNCH_CHECK("emit_kernel");
        return 0;
    }
    const unsigned word_groups = (unsigned)((n_words + 3) / 4);
    hipLaunchKernelGGL(emit_general_words_kernel, dim3(word_groups), dim3(256), 0, st, ep);
    SPX_LAUNCH_CHECK("emit_general_words_kernel");
    hipLaunchKernelGGL(emit_general_scan_kernel, dim3(1), dim3(1024), 0, st, ep);
    SPX_LAUNCH_CHECK("emit_general_scan_kernel");
    hipLaunchKernelGGL(emit_general_write_kernel, dim3(word_groups), dim3(256), 0, st, ep);
    SPX_LAUNCH_CHECK("emit_general_write_kernel");
    return 0;
}

extern "C" int spx_bcs_index_batch(const spx_bcs_index_job* jobs, int n_jobs, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(n_jobs >= 0, SPX_E_SHAPE, "negative job count");
    SPX_REQUIRE(jobs || n_jobs == 0, SPX_E_NULL, "jobs is required");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    for (int first = 0; first < n_jobs;) {
        // validate and prepare up to INDEX_BATCH_MAX builds; those on the bit-word path share
        // one pair of launches, the others are built one by one
        const int last = first + INDEX_BATCH_MAX < n_jobs ? first + INDEX_BATCH_MAX : n_jobs;
        FastIndexJob prep[INDEX_BATCH_MAX];
        // the builds of one group run in the same launches: their workspaces must be disjoint
        for (int i = first; i < last; ++i)
            for (int k = i + 1; k < last; ++k) {
                const char* a = static_cast<const char*>(jobs[i].workspace);
                const char* b = static_cast<const char*>(jobs[k].workspace);
                SPX_REQUIRE(!a || !b || a + jobs[i].workspace_bytes <= b || b + jobs[k].workspace_bytes <= a,
                            SPX_E_WORKSPACE, "jobs %d and %d share workspace memory", i, k);
            }
        for (int i = first; i < last; ++i) {
            const spx_bcs_index_job& j = jobs[i];
            SPX_REQUIRE(!j.row_order || j.row_ptr, SPX_E_NULL, "row_order needs the BCSR index");
            SPX_REQUIRE(!j.col_order || j.col_ptr, SPX_E_NULL, "col_order needs the BCSC index");
            const int rc = bcs_index_impl(j.mask, j.H, j.W, j.BH, j.BW, j.row_ptr, j.bcsr_idx, j.col_ptr, j.bcsc_idx,
                                          j.bcsc_i64, j.nnz_dev, j.cap, j.row_order, j.col_order, j.workspace,
                                          j.workspace_bytes, stream, &prep[i - first]);
            if (rc) return rc;
        }
        BitsBatch bb;
        EmitBatch eb;
        int n = 0, bx = 0, ex = 0, max_r = 1, max_parts = 1;
        for (int i = first; i < last; ++i) {
            const FastIndexJob& f = prep[i - first];
            if (!f.ready) continue;
            bb.job[n] = f.bits; bb.R[n] = f.R; bb.nparts[n] = f.nparts;
            bx += f.WPR; bb.x_end[n] = bx;
            eb.job[n] = f.emit; eb.nslice[n] = f.nslice; eb.sides[n] = f.sides; eb.nparts[n] = f.nparts;
            ex += f.nslice * (f.sides == 3 ? 2 : 1); eb.x_end[n] = ex;
            max_r = f.R > max_r ? f.R : max_r;
            max_parts = f.nparts > max_parts ? f.nparts : max_parts;
            ++n;
        }
        if (n > 0) {
            bb.n = eb.n = n;
            hipLaunchKernelGGL(live_bits_batch_kernel, dim3(bx, max_r, max_parts), dim3(256), 0, st, bb);
            SPX_LAUNCH_CHECK("live_bits_batch_kernel");
            hipLaunchKernelGGL(emit_words_batch_kernel, dim3(ex), dim3(1024), 0, st, eb);
            SPX_LAUNCH_CHECK("emit_words_batch_kernel");
        }
        for (int i = first; i < last; ++i) {
            if (prep[i - first].ready) continue;
            const spx_bcs_index_job& j = jobs[i];
            const int rc = bcs_index_impl(j.mask, j.H, j.W, j.BH, j.BW, j.row_ptr, j.bcsr_idx, j.col_ptr, j.bcsc_idx,
                                          j.bcsc_i64, j.nnz_dev, j.cap, j.row_order, j.col_order, j.workspace,
                                          j.workspace_bytes, stream);
            if (rc) return rc;
        }
        first = last;
    }
    return 0;
}

// ---- index build without any allocation ---------------------------------------------
// The workspace of spx_bcs_index lives in a file-scope device array instead of a
// caller-provided buffer.  Every device the library runs on holds its own copy of the
// array at its own address: the address is looked up once per device, with that device
// current, and kept; host code never uses the array's name for anything else.
namespace spx {
constexpr size_t BCS_SCRATCH_BYTES = 1u << 20;
constexpr int BCS_SCRATCH_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[BCS_SCRATCH_BYTES];
static void* g_scratch_ptr[BCS_SCRATCH_MAX_DEVICES];
static std::once_flag g_scratch_once[BCS_SCRATCH_MAX_DEVICES];
static hipError_t g_scratch_err[BCS_SCRATCH_MAX_DEVICES];

// Address of the current device's copy of `scratch`; NULL (and *err set) on failure.
static void* scratch_of_current_device(hipError_t* err) {
    int dev = -1;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= BCS_SCRATCH_MAX_DEVICES) { *err = hipErrorInvalidDevice; return nullptr; }
    std::call_once(g_scratch_once[dev], [dev]() {
        void* ptr = nullptr;
        g_scratch_err[dev] = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        g_scratch_ptr[dev] = g_scratch_err[dev] == hipSuccess ? ptr : nullptr;
    });
    *err = g_scratch_err[dev];
    return g_scratch_ptr[dev];
}
}  // namespace spx

extern "C" size_t spx_bcs_index_static_max_bytes(void) { return spx::BCS_SCRATCH_BYTES; }

extern "C" int spx_bcs_index_static(const uint8_t* mask, int H, int W, int BH, int BW,
                                    int32_t* row_ptr, int32_t* bcsr_idx,
                                    int32_t* col_ptr, void* bcsc_idx, int bcsc_i64,
                                    int32_t* nnz_dev, int cap, spx_stream_t stream) {
    using namespace spx;
    int rc = check_index_shape(H, W, BH, BW);
    if (rc) return rc;
    SPX_REQUIRE(mask && nnz_dev, SPX_E_NULL, "mask and nnz_dev are required");
    const size_t need = index_workspace(H, W, BH, BW).total;
    SPX_REQUIRE(need <= BCS_SCRATCH_BYTES, SPX_E_WORKSPACE,
                "a (%d,%d) mask in (%d,%d) blocks needs %zu bytes of scratch, the static buffer holds %zu: "
                "use spx_bcs_index with a caller-provided workspace", H, W, BH, BW, need, BCS_SCRATCH_BYTES);
    hipError_t err = hipSuccess;
    void* ptr = scratch_of_current_device(&err);
    if (!ptr) return hip_fail(err, "hipGetSymbolAddress(scratch)");
    // every byte of the workspace that the kernels read is written by them first, so the
    // previous call's contents need no clearing
    return bcs_index_impl(mask, H, W, BH, BW, row_ptr, bcsr_idx, col_ptr, bcsc_idx, bcsc_i64, nnz_dev, cap,
                          nullptr, nullptr, ptr, BCS_SCRATCH_BYTES, stream);
}

extern "C" int spx_bcs_schedule(const int32_t* ptr, int n, int32_t* order, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(n >= 0, SPX_E_SHAPE, "negative segment count");
    if (n == 0) return 0;
    SPX_REQUIRE(ptr && order, SPX_E_NULL, "ptr and order are required");
    hipLaunchKernelGGL(schedule_kernel, dim3(1), dim3(1024), 0, reinterpret_cast<hipStream_t>(stream), ptr, n, order);
    SPX_LAUNCH_CHECK("schedule_kernel");
    return 0;
}
