// Fused block-sparse attention forward:
//   out = softmax_masked(q k^T * inv_temperature) v,  per batch*head,
// over the live (BH x BW) blocks of a BCSR index.  The score matrix never leaves
// the chip: for every live block of a block-row the workgroup computes the score
// tile, folds it into a running (max, sum) per query and accumulates P.V.
//
// Layout trick: scores are produced transposed, S^T = K Q^T, so that an MFMA
// accumulator lane (r = lane % 16, g = lane / 16) holds, for query r, the four
// consecutive keys g*4 .. g*4+3 of a 16-key tile.  That is exactly the B-operand
// layout of a 16x16x16 MFMA, so exp(S^T) feeds  O^T += V^T P^T  straight from
// registers, and every value a lane owns (scores, running max/sum, output
// accumulators) belongs to one query.  K tiles are staged in LDS as [key][e],
// V tiles transposed as [e][key]; each wavefront owns 16 queries.
//
// There is no counterpart kernel in the reference, whose SparseAttention.forward
// (sparta/specializer/operators/sparse_attention.py:76-80) runs three launches
// with two compressed intermediates in HBM; the result matches
// sparse_multi_head_attention_reference (sparta/testing/math.py:53-79).
#include "common.hpp"
#include "mma.hpp"

namespace spx {

struct AttnParams {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    const int32_t* row_ptr;
    const int32_t* bcsr_idx;
    const uint8_t* mask;  // [Nt, Ns] or NULL
    float inv_t;
    int Nt, Ns, BH;
    void* probs;          // training kernels: compressed probabilities, block e at e * BH * BW
    int64_t probs_batch;  // elements between batch entries of probs (and of grad_scores)
    const void* grad_out; // backward kernel: gradient of the output
    void* grad_scores;    // backward kernel: compressed gradient of the scores (layout of probs)
    void* grad_q;         // backward kernel: gradient of the queries
    float* row_dot;       // backward kernels: D[b, i] / T = sum_e grad_out o out / T per query
    const int32_t* col_ptr;   // column-side backward kernel: BCSC index
    const void* bcsc_idx;
    int bcsc_wide;        // 1: int64 entries (bcsr_pos << 32 | col << 16 | row), 0: int32 (col << 16 | row)
    void* grad_k;
    void* grad_v;
    const int32_t* seqlens;   // sequence-length mode of the pipelined kernel: one length per `heads` entries
    int heads;
    float* row_lse;       // log2-domain log-sum-exp per query: written by the forward kernel, read by the recomputing backward kernels
};

template <typename T> struct AttnMma;
template <> struct AttnMma<_Float16> {
    typedef f16x4 pfrag;
    __device__ static pfrag pack(float a, float b, float c, float d) {
        return pfrag{(_Float16)a, (_Float16)b, (_Float16)c, (_Float16)d};
    }
};
template <> struct AttnMma<bf16_t> {
    typedef s16x4 pfrag;
    __device__ static pfrag pack(float a, float b, float c, float d) {
        return pfrag{(short)float_to_bf16(a), (short)float_to_bf16(b), (short)float_to_bf16(c),
                     (short)float_to_bf16(d)};
    }
};

// BW keys per block, E head dimension; BH = 16 * (waves per workgroup).
template <typename T, int BW, int E>
__global__ __launch_bounds__(512) void attention_kernel(AttnParams p) {
    constexpr int KT = BW / 16;     // key tiles per block
    constexpr int ET = E / 16;      // output (e) tiles
    constexpr int EC = E / 32;      // 32-wide chunks of the QK^T contraction
    constexpr int LDK = E + 8;      // K tile row pitch (elements): 16 bytes of padding
    constexpr int LDV = BW + 8;     // V^T tile row pitch
    typedef typename Mma32<T>::frag QFrag;
    typedef typename AttnMma<T>::pfrag PFrag;
    extern __shared__ __align__(16) char smem[];
    T* Ks = reinterpret_cast<T*>(smem);        // [BW][LDK]
    T* Vt = Ks + BW * LDK;                     // [E][LDV]

    const int br = blockIdx.x;
    const int64_t b = blockIdx.y;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int nthreads = blockDim.x;

    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E;
    T* O = reinterpret_cast<T*>(p.out) + b * (int64_t)p.Nt * E;

    const int qrow = br * p.BH + wave * 16 + r16;  // the query this lane belongs to
    // Q fragments (B operand of S^T = K Q^T): query r16, e = c*32 + g4*8 .. +7
    QFrag qf[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) qf[c] = Mma32<T>::load(Q + (int64_t)qrow * E + c * 32 + g4 * 8);

    f32x4 oacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -1e30f, l_run = 0.f;

    const int e_begin = p.row_ptr[br];
    const int e_end = p.row_ptr[br + 1];
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    for (int e = e_begin; e < e_end; ++e) {
        const int bc = p.bcsr_idx[e] & 0xffff;
        const int key0 = bc * BW;
        __syncthreads();  // previous block's fragments are consumed
        // ---- stage K [key][e] ----------------------------------------------------------
        for (int v = threadIdx.x; v < BW * (E / 8); v += nthreads) {
            const int key = v / (E / 8), c = v % (E / 8);
            *reinterpret_cast<u32x4*>(Ks + key * LDK + c * 8) =
                *reinterpret_cast<const u32x4*>(Kg + (int64_t)(key0 + key) * E + c * 8);
        }
        // ---- stage V transposed [e][key]: a thread moves a 2-key x 8-e patch --------------
        for (int v = threadIdx.x; v < (BW / 2) * (E / 8); v += nthreads) {
            const int kp = v / (E / 8), c = v % (E / 8);
            union { u32x4 v4; uint16_t h[8]; } a, bb;
            a.v4 = *reinterpret_cast<const u32x4*>(Vg + (int64_t)(key0 + 2 * kp) * E + c * 8);
            bb.v4 = *reinterpret_cast<const u32x4*>(Vg + (int64_t)(key0 + 2 * kp + 1) * E + c * 8);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                *reinterpret_cast<uint32_t*>(Vt + (c * 8 + i) * LDV + 2 * kp) = (uint32_t)a.h[i] | ((uint32_t)bb.h[i] << 16);
        }
        __syncthreads();

        // ---- S^T tiles: keys x this wave's 16 queries ------------------------------------
        f32x4 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const QFrag kf = Mma32<T>::load(Ks + (kt * 16 + r16) * LDK + c * 32 + g4 * 8);
                s[kt] = Mma32<T>::mma(kf, qf[c], s[kt]);
            }
        }
        // lane holds s[kt][q] = score(query r16, key kt*16 + g4*4 + q)
        unsigned live[KT];
        float tmax = -1e30f;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            unsigned bits = 0x01010101u;
            if (p.mask)
                bits = *reinterpret_cast<const uint32_t*>(p.mask + (int64_t)qrow * p.Ns + key0 + kt * 16 + g4 * 4);
            live[kt] = bits;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if ((bits >> (8 * q)) & 0xffu) tmax = fmaxf(tmax, s[kt][q]);
        }
        tmax = xor32_max(xor16_max(tmax));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __expf((m_run - m_new) * p.inv_t);
        float psum = 0.f;
        PFrag pf[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            float pv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                pv[q] = ((live[kt] >> (8 * q)) & 0xffu) ? __expf((s[kt][q] - m_new) * p.inv_t) : 0.f;
                psum += pv[q];
            }
            pf[kt] = AttnMma<T>::pack(pv[0], pv[1], pv[2], pv[3]);
        }
        psum = xor32_sum(xor16_sum(psum));
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // ---- O^T[e][query] = alpha * O^T + V^T P^T ----------------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
            oacc[t] *= alpha;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const typename Mma16<T>::frag vf = Mma16<T>::load(Vt + (t * 16 + r16) * LDV + kt * 16 + g4 * 4);
                oacc[t] = Mma16<T>::mma(vf, pf[kt], oacc[t]);
            }
        }
    }

    // lane holds O^T[e = t*16 + g4*4 + q][query r16]; rows with no live entry give 0
    const float inv_l = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(oacc[t][q] * inv_l);
        *reinterpret_cast<uint64_t*>(O + (int64_t)qrow * E + t * 16 + g4 * 4) = *reinterpret_cast<const uint64_t*>(vals);
    }
}

// ---- pipelined variant ------------------------------------------------------------------
// Same mathematics and register layout as attention_kernel, rebuilt around the
// instruction budget of a block step:
//  * K and V tiles of the next live block travel global -> registers while the
//    current one is consumed; with two LDS buffers a step needs one barrier.
//  * K is staged with its 16-byte chunks XOR-swizzled by the row (padding the pitch
//    instead halves the rate of 16-byte LDS reads on this chip).
//  * V is staged untransposed ([key][e], 16-byte writes); the keys-contiguous
//    operand of  O^T += V^T P^T  comes from the LDS transpose read of gfx950
//    (ds_read_b64_tr_b16: in a 16-lane group, lane i supplies the address of 4
//    consecutive e of key i/4, and lane j receives element j%4 of lanes
//    j/4, 4+j/4, 8+j/4, 12+j/4: the 4 keys of column e0 + j).
//  * P.V runs on 16x16x32 MFMAs: the 8 k-slots of a lane are the 4 keys it holds
//    of key tile 2i followed by the 4 of key tile 2i+1.
//  * exp2 with the scale folded into one fma; the row sums come from one more MFMA
//    (an all-ones tile in place of V^T), and the running maximum is moved lazily.
//  * workgroups are numbered so that all query blocks of one batch*head entry run
//    on one XCD and find that entry's K and V in its L2.
template <typename T> struct AttnPack;
template <> struct AttnPack<_Float16> {
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    __device__ static f16x8 pack(f32x8 v) { return __builtin_convertvector(v, f16x8); }
};
template <> struct AttnPack<bf16_t> {
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    __device__ static bf16x8 pack(f32x8 v) { return __builtin_convertvector(v, bf16x8); }
};

// Scores of masked keys drop to -1e30 (exp2 of it is exactly 0, so nothing is selected
// afterwards).  live[kt] holds the mask bytes of the lane's four keys of tile kt; a tile
// whose bytes are all 1 for the whole wavefront - every tile of a block-granular pattern -
// skips the selects.
template <int KT>
__device__ __forceinline__ void mask_scores(f32x4 (&s)[KT], const unsigned (&live)[KT]) {
    unsigned all = live[0];
#pragma unroll
    for (int kt = 1; kt < KT; ++kt) all &= live[kt];
    if (__builtin_amdgcn_ballot_w64(all != 0x01010101u) != 0) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int q = 0; q < 4; ++q) s[kt][q] = ((live[kt] >> (8 * q)) & 0xffu) ? s[kt][q] : -1e30f;
    }
}
// Maximum of the lane's 4 * KT scores: independent three-way maxima, then a short chain
// (fmaxf in a select per value costs three v_max_f32 each on MFMA results).
template <int KT>
__device__ __forceinline__ float lane_max(const f32x4 (&s)[KT]) {
    float part[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) part[kt] = max3f(s[kt][0], s[kt][1], s[kt][2]);
    float m = max3f(part[0], part[1], s[0][3]);
#pragma unroll
    for (int kt = 2; kt < KT; kt += 2) m = max3f(m, part[kt], part[kt + 1]);
#pragma unroll
    for (int kt = 1; kt + 1 < KT; kt += 2) m = max3f(m, s[kt][3], s[kt + 1][3]);
    return fmaxf(m, s[KT - 1][3]);
}

// Wavefronts per SIMD a kernel's register budget is sized for: no more than its LDS footprint
// lets a CU hold, and no more than eight wavefronts per SIMD-quarter of the workgroup
// (two-wavefront workgroups with large tiles spilled under a budget of four).
constexpr int waves_per_simd_for(int smem_bytes, int waves, int cap = 0) {
    const int by_lds = (160 * 1024 / smem_bytes * waves + 3) / 4;
    if (cap == 0) cap = 8 / waves;
    return by_lds < 1 ? 1 : (by_lds < cap ? by_lds : cap);
}

// SEQ: no index and no mask bytes; entry b attends over its first L = seqlens[b / heads]
// positions: the walk covers the key blocks below L, a key is live iff its position is, and
// queries at or past L give zeros (block rows at or past L walk nothing).
template <typename T, int BW, int E, int WAVES, bool HAS_MASK, bool SEQ = false>
__global__ __launch_bounds__(64 * WAVES, waves_per_simd_for((2 * BW * (E * 4 + 32) <= 64 * 1024 ? 2 : 1) * BW * (E * 4 + 32), WAVES)) void attention_kernel_v2(AttnParams p, int nbr, int batch) {
    static_assert(!SEQ || HAS_MASK, "the sequence-length mode masks by key position");
    constexpr int NT = 64 * WAVES;
    constexpr int KT = BW / 16, ET = E / 16, EC = E / 32;
    constexpr int KP = E * 2;                 // K row pitch in bytes (16-byte chunks XOR-swizzled by row % 8)
    constexpr int VP = E * 2 + 32;            // V row pitch in bytes
    constexpr int TILE = BW * (KP + VP);
    constexpr int NBUF = 2 * TILE <= 64 * 1024 ? 2 : 1;
    constexpr int VPR = E / 8;                // 16-byte vectors per tile row
    constexpr int NV = BW * VPR / NT;         // vectors per thread and tile
    constexpr int RSTEP = NT / VPR;           // tile rows between a thread's vectors
    static_assert(BW * VPR % NT == 0 && NT % VPR == 0 && KT % 2 == 0, "tile does not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    // workgroup L runs on XCD L % 8: give each XCD whole batch*head entries
    const int L = blockIdx.x;
    const int slot = L >> 3;
    const int64_t b = (slot / nbr) * 8 + (L & 7);
    const int br = slot % nbr;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    T* O = reinterpret_cast<T*>(p.out) + b * (int64_t)p.Nt * E;

    const int qrow = br * (16 * WAVES) + wave * 16 + r16;
    // Q is scaled by inv_t * log2(e) once, so that the products come out in log2 units
    const float c2 = p.inv_t * 1.4426950408889634f;
    Frag qf[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const Frag raw = Mma32<T>::load(Q + (int64_t)qrow * E + c * 32 + g4 * 8);
        f32x8 scaled;
#pragma unroll
        for (int j = 0; j < 8; ++j) scaled[j] = (float)raw[j] * c2;
        qf[c] = AttnPack<T>::pack(scaled);
    }

    f32x4 oacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    // The score accumulators start at -m (the reference point of this lane's query, log2
    // units), so the MFMAs deliver the exponent of exp2 directly.  m starts at 0 and is set
    // to the row maximum by the first block with a live entry; later it only moves when a
    // maximum outgrows it by more than 2^RESCALE_LOG2 (numerator and denominator always
    // share one reference).
    f32x4 negm = f32x4{0.f, 0.f, 0.f, 0.f};
    bool fresh = true;   // no live entry seen yet for this lane's query
    f32x4 lacc = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr float RESCALE_LOG2 = 6.f;
    constexpr short ONE_BITS = sizeof(T) == 2 && Elem<T>::dtype == SPX_F16 ? (short)0x3c00 : (short)0x3f80;
    const Frag ones = __builtin_bit_cast(Frag, s16x8{ONE_BITS, ONE_BITS, ONE_BITS, ONE_BITS, ONE_BITS, ONE_BITS, ONE_BITS, ONE_BITS});

    // staging map: vector v = tid + i * NT of the (contiguous) tile is row v / VPR, chunk v % VPR
    const int st_row = threadIdx.x / VPR, st_chunk = threadIdx.x % VPR;
    const int k_dst = st_row * KP + (st_chunk ^ (st_row & 7)) * 16;  // rows of one thread are 8 apart or more
    const int v_dst = BW * KP + st_row * VP + st_chunk * 16;
    // fragment bases
    const int k_src = r16 * KP;
    const int k_sw = r16 & 7;
    const int v_src = BW * KP + (g4 * 4 + (r16 >> 2)) * VP + (r16 & 3) * 8;

    int seq_len = 0;
    if constexpr (SEQ) {
        seq_len = p.seqlens[b / p.heads];
        seq_len = seq_len < 0 ? 0 : (seq_len > p.Ns ? p.Ns : seq_len);
    }
    const int e_begin = SEQ ? 0 : p.row_ptr[br];
    const int n_blk = (SEQ ? (br * (16 * WAVES) < seq_len ? (seq_len + BW - 1) / BW : 0) : p.row_ptr[br + 1]) - e_begin;
    // Block columns of the row: lane l holds entry l (broadcast with readlane, so no step
    // waits for an index load); longer rows read the rest from the index.
    int bc_vec = 0;
    if constexpr (!SEQ) {
        if (lane < n_blk) bc_vec = p.bcsr_idx[e_begin + lane] & 0xffff;
    }
    auto col_at = [&](int i) {
        if constexpr (SEQ) return i;
        else return i < 64 ? __builtin_amdgcn_readlane(bc_vec, i) : (p.bcsr_idx[e_begin + i] & 0xffff);
    };
    // Without mask bytes to fetch, two register stages: the K and V tiles of step i + 2 are
    // requested while step i is staged and computed, through inline-assembly loads that are
    // waited for with explicit counts (the compiler merges its own wait counts at the loop
    // header and would drain both stages at every step).  With a mask, one stage of ordinary
    // loads: the wait for the mask bytes would drain the second stage anyway.
    constexpr int NSTG = (!HAS_MASK && !SEQ && NV <= 4) ? 2 : 1;
    auto issue = [&](int i, u32x4 (&kr)[NV], u32x4 (&vr)[NV]) {
        const int64_t off = (int64_t)col_at(i) * BW * E;
        if constexpr (NSTG == 2) {
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2)
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(kr[i2]) : "v"(Kg + off + i2 * NT * 8) : "memory");
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2)
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(vr[i2]) : "v"(Vg + off + i2 * NT * 8) : "memory");
        } else {
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2) kr[i2] = *reinterpret_cast<const u32x4*>(Kg + off + i2 * NT * 8);
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2) vr[i2] = *reinterpret_cast<const u32x4*>(Vg + off + i2 * NT * 8);
        }
    };
    // Wait until only the other stage is outstanding; the stage's registers pass through the
    // statement so that no use is scheduled before it.
    auto wait_stage = [&](int i, u32x4 (&kr)[NV], u32x4 (&vr)[NV]) {
        if constexpr (NSTG == 1) return;   // plain loads: the compiler waits where the registers are used
        if (i + 1 < n_blk) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NV) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) asm volatile("" : "+v"(kr[i2]));
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) asm volatile("" : "+v"(vr[i2]));
    };
    auto step = [&](int i, u32x4 (&kr)[NV], u32x4 (&vr)[NV]) {
        char* buf = smem + (NBUF == 2 ? (i & 1) * TILE : 0);
        if constexpr (NBUF == 1) __syncthreads();  // the previous block's fragments are consumed
        wait_stage(i, kr, vr);
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) *reinterpret_cast<u32x4*>(buf + k_dst + i2 * RSTEP * KP) = kr[i2];
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) *reinterpret_cast<u32x4*>(buf + v_dst + i2 * RSTEP * VP) = vr[i2];
        if (i + NSTG < n_blk) issue(i + NSTG, kr, vr);
        unsigned live[KT];
        if constexpr (SEQ) {
            // one byte per key of this lane, set while the key position is below the length
            const int key0 = i * BW;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const int left = seq_len - (key0 + kt * 16 + g4 * 4);   // live keys among the lane's four
                live[kt] = left >= 4 ? 0x01010101u : left <= 0 ? 0u : (0x01010101u >> (8 * (4 - left)));
            }
        } else if constexpr (HAS_MASK) {
            const int key0 = col_at(i) * BW;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                live[kt] = *reinterpret_cast<const uint32_t*>(p.mask + (int64_t)qrow * p.Ns + key0 + kt * 16 + g4 * 4);
        }
        __syncthreads();

        // ---- S^T tiles: keys x this wave's 16 queries ------------------------------------
        f32x4 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = negm;
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag kf = *reinterpret_cast<const Frag*>(buf + k_src + kt * 16 * KP + (((c * 4 + g4) ^ k_sw) * 16));
                s[kt] = Mma32<T>::mma(kf, qf[c], s[kt]);
            }
        }
        if constexpr (HAS_MASK) mask_scores<KT>(s, live);
        float tmax = lane_max<KT>(s);
        tmax = xor32_max(xor16_max(tmax));
        const bool any_live = tmax > -1e29f;
        if (__builtin_amdgcn_ballot_w64(any_live && (fresh || tmax > RESCALE_LOG2)) != 0) {
            // move the reference by delta (0 for queries that keep theirs)
            const float delta = any_live ? (fresh ? tmax : fmaxf(tmax, 0.f)) : 0.f;
            const float alpha = __builtin_amdgcn_exp2f(-delta);
            negm -= delta;
            lacc *= alpha;
#pragma unroll
            for (int t = 0; t < ET; ++t) oacc[t] *= alpha;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) s[kt] -= delta;
        }
        fresh = fresh && !any_live;
        Frag pf[KT / 2];
#pragma unroll
        for (int kp = 0; kp < KT / 2; ++kp) {
            f32x8 pv;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int kt = 2 * kp + (j >> 2), q = j & 3;
                pv[j] = __builtin_amdgcn_exp2f(s[kt][q]);
            }
            pf[kp] = AttnPack<T>::pack(pv);
            // row sums of the rounded probabilities: an all-ones tile in place of V^T
            lacc = Mma32<T>::mma(ones, pf[kp], lacc);
        }
        // ---- O^T[e][query] += V^T P^T ------------------------------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int kp = 0; kp < KT / 2; ++kp) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + v_src + (kp * 32) * VP + t * 32));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + v_src + (kp * 32 + 16) * VP + t * 32));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, both), pf[kp], oacc[t]);
            }
        }
    };
    if constexpr (NSTG == 2) {
        u32x4 k0[NV], v0[NV], k1[NV], v1[NV];
        if (n_blk > 0) {
            issue(0, k0, v0);
            issue(n_blk > 1 ? 1 : 0, k1, v1);   // a row of one block requests it twice; the copy is not used
        }
        for (int i = 0; i < n_blk; i += 2) {
            step(i, k0, v0);
            if (i + 1 < n_blk) step(i + 1, k1, v1);
        }
    } else {
        u32x4 k0[NV], v0[NV];
        if (n_blk > 0) issue(0, k0, v0);
        for (int i = 0; i < n_blk; ++i) step(i, k0, v0);
    }

    // every accumulator row of lacc holds the row sum of query r16
    const float l_run = lacc[0];
    const float inv_l = (l_run > 0.f && (!SEQ || qrow < seq_len)) ? 1.f / l_run : 0.f;
    // log2-domain log-sum-exp of the row: P = exp2(score - row_lse) reproduces the normalised
    // probabilities in a backward pass that keeps no copy of them (+inf: no live entry, P = 0)
    if (p.row_lse && g4 == 0)
        p.row_lse[b * p.Nt + qrow] = l_run > 0.f ? __builtin_amdgcn_logf(l_run) - negm[0] : __builtin_inff();
    uint64_t pieces[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(oacc[t][q] * inv_l);
        pieces[t] = *reinterpret_cast<const uint64_t*>(vals);
    }
    if constexpr (WAVES * 16 * (E * 2 + 16) <= NBUF * TILE) {
        __syncthreads();   // the K / V tiles are dead: their space carries the output tiles
        wave_rows_store<E>(smem + wave * (16 * (E * 2 + 16)), O + (int64_t)(qrow - r16) * E, pieces);
    } else {
#pragma unroll
        for (int t = 0; t < ET; ++t) *reinterpret_cast<uint64_t*>(O + (int64_t)qrow * E + t * 16 + g4 * 4) = pieces[t];
    }
}

template <typename T, int BW, int E, int WAVES>
static int launch_attention_v2_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr int TILE = BW * (E * 4 + 32);
    constexpr size_t smem = 2 * TILE <= 64 * 1024 ? 2 * TILE : TILE;
    const int nbr = p.Nt / p.BH;
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbr;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (p.mask) {
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel_v2<T, BW, E, WAVES, true>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel_v2)");
        }
        hipLaunchKernelGGL((attention_kernel_v2<T, BW, E, WAVES, true>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbr, batch);
    } else {
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel_v2<T, BW, E, WAVES, false>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel_v2)");
        }
        hipLaunchKernelGGL((attention_kernel_v2<T, BW, E, WAVES, false>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbr, batch);
    }
    SPX_LAUNCH_CHECK("attention_kernel_v2");
    return 0;
}

// Sequence-length mode of the pipelined kernel: square tiles of 64 (N a multiple of 64) or 32.
template <typename T, int TB, int E>
static int launch_attention_v2_seq_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr int TILE = TB * (E * 4 + 32);
    constexpr size_t smem = 2 * TILE <= 64 * 1024 ? 2 * TILE : TILE;
    const int nbr = p.Nt / TB;
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbr;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel_v2<T, TB, E, TB / 16, true, true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel_v2)");
    }
    hipLaunchKernelGGL((attention_kernel_v2<T, TB, E, TB / 16, true, true>), dim3((unsigned)groups), dim3(4 * TB), smem, st, p, nbr, batch);
    SPX_LAUNCH_CHECK("attention_kernel_v2 (sequence lengths)");
    return 0;
}

template <typename T>
static int launch_attention_v2_seq(const AttnParams& p, int batch, int E, hipStream_t st) {
    const int TB = p.Nt % 64 == 0 ? 64 : 32;
    if (TB == 64 && E == 64) return launch_attention_v2_seq_inst<T, 64, 64>(p, batch, st);
    if (TB == 64 && E == 128) return launch_attention_v2_seq_inst<T, 64, 128>(p, batch, st);
    if (TB == 32 && E == 64) return launch_attention_v2_seq_inst<T, 32, 64>(p, batch, st);
    if (TB == 32 && E == 128) return launch_attention_v2_seq_inst<T, 32, 128>(p, batch, st);
    return fail(SPX_E_CONFIG, "the pipelined sequence-length kernel takes head dims 64 / 128 (got %d)", E);
}

// The pipelined kernel covers query blocks of 32 / 64 / 128, key blocks of 32 / 64 / 128
// and head dimensions 64 / 128 (except 128-query blocks with 32 x 64 key tiles).
static bool attention_v2_supported(int BH, int BW, int E) {
    return (BH == 32 || BH == 64 || BH == 128) && (BW == 32 || BW == 64 || BW == 128) && (E == 64 || E == 128) &&
           BW * E / 8 >= BH * 4;  // at least one 16-byte vector of a tile per thread
}

template <typename T>
static int launch_attention_v2(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTN2_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_v2_inst<T, bw, e, bh / 16>(p, batch, st);
    SPX_ATTN2_CASE(32, 32, 64) SPX_ATTN2_CASE(32, 64, 64) SPX_ATTN2_CASE(32, 128, 64)
    SPX_ATTN2_CASE(32, 32, 128) SPX_ATTN2_CASE(32, 64, 128) SPX_ATTN2_CASE(32, 128, 128)
    SPX_ATTN2_CASE(64, 32, 64) SPX_ATTN2_CASE(64, 64, 64) SPX_ATTN2_CASE(64, 128, 64)
    SPX_ATTN2_CASE(64, 32, 128) SPX_ATTN2_CASE(64, 64, 128) SPX_ATTN2_CASE(64, 128, 128)
    SPX_ATTN2_CASE(128, 64, 64) SPX_ATTN2_CASE(128, 128, 64)
    SPX_ATTN2_CASE(128, 32, 128) SPX_ATTN2_CASE(128, 64, 128) SPX_ATTN2_CASE(128, 128, 128)
#undef SPX_ATTN2_CASE
    return fail(SPX_E_CONFIG, "the pipelined attention kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

// ---- forward pass for training: output and probabilities in one launch --------------------
// Gradients need the normalised probabilities P in memory (compressed like the output of
// the softmax operator).  The kernel walks the live blocks of its block row twice with the
// register layout of attention_kernel_v2: pass 1 computes the row maximum and the row sum
// (scores and exp2 only: K tiles, no V); pass 2 recomputes the scores against the final
// maximum, scales by 1 / sum, writes the rounded probabilities (8-byte pieces: a lane holds
// 4 consecutive keys of each 16-key tile for its query) and feeds the same values to the
// P.V MFMAs, so the output needs no final division.  One launch replaces the scores,
// softmax and P.V operators of the forward pipeline.
template <typename T, int BW, int E, int WAVES, bool HAS_MASK>
__global__ __launch_bounds__(64 * (WAVES + 1), waves_per_simd_for((2 * BW * (E * 4 + 32) <= 64 * 1024 ? 2 : 1) * BW * (E * 4 + 32) + 2 * WAVES * 16 * (BW * 2), WAVES + 1, 8 / WAVES)) void attention_train_kernel(AttnParams p, int nbr, int batch) {
    constexpr int NT = 64 * WAVES;
    constexpr int KT = BW / 16, ET = E / 16, EC = E / 32;
    constexpr int KP = E * 2;                 // K row pitch in bytes (16-byte chunks XOR-swizzled by row % 8)
    constexpr int VP = E * 2 + 32;            // V row pitch in bytes
    constexpr int TILE = BW * (KP + VP);
    constexpr int NBUF = 2 * TILE <= 64 * 1024 ? 2 : 1;
    constexpr int VPR = E / 8;                // 16-byte vectors per tile row
    constexpr int NV = BW * VPR / NT;         // vectors per thread and tile
    constexpr int RSTEP = NT / VPR;           // tile rows between a thread's vectors
    constexpr int PROW = BW * 2;              // bytes per row of the staged probability tile (chunks XOR-swizzled by the row)
    constexpr int PCH = BW / 8;               // 16-byte chunks per row
    constexpr int PTILE = 16 * WAVES * PROW;  // one block of probabilities
    static_assert(BW * VPR % NT == 0 && NT % VPR == 0 && KT % 2 == 0, "tile does not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    const int L = blockIdx.x;
    const int slot = L >> 3;
    const int64_t b = (slot / nbr) * 8 + (L & 7);
    const int br = slot % nbr;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    T* O = reinterpret_cast<T*>(p.out) + b * (int64_t)p.Nt * E;
    T* P = reinterpret_cast<T*>(p.probs) + b * p.probs_batch;

    // (the store wavefront, wave == WAVES, owns no rows: it reads the first wavefront's Q rows and drops them)
    const int qrow = br * (16 * WAVES) + (wave < WAVES ? wave : 0) * 16 + r16;
    const float c2 = p.inv_t * 1.4426950408889634f;
    Frag qf[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const Frag raw = Mma32<T>::load(Q + (int64_t)qrow * E + c * 32 + g4 * 8);
        f32x8 scaled;
#pragma unroll
        for (int j = 0; j < 8; ++j) scaled[j] = (float)raw[j] * c2;
        qf[c] = AttnPack<T>::pack(scaled);
    }

    const int st_row = threadIdx.x / VPR, st_chunk = threadIdx.x % VPR;
    const int k_dst = st_row * KP + (st_chunk ^ (st_row & 7)) * 16;
    const int v_dst = BW * KP + st_row * VP + st_chunk * 16;
    const int k_src = r16 * KP;
    const int k_sw = r16 & 7;
    const int v_src = BW * KP + (g4 * 4 + (r16 >> 2)) * VP + (r16 & 3) * 8;
    char* const pstage = smem + NBUF * TILE;   // [2][PTILE]
    auto pswz = [](int row) { return row & 7 & (PCH - 1); };

    const int e_begin = p.row_ptr[br];
    const int e_end = p.row_ptr[br + 1];
    if (e_begin >= e_end) {
        // no live block: zero output rows (uniform over the workgroup)
        if (wave < WAVES) {
#pragma unroll
            for (int t = 0; t < ET; ++t) *reinterpret_cast<uint64_t*>(O + (int64_t)qrow * E + t * 16 + g4 * 4) = 0ull;
        }
        return;
    }
    if (wave == WAVES) {
        // ---- store wavefront: follows the barriers of the others and, one step behind them,
        // moves every finished block of probabilities from LDS to memory as whole vectors.  It
        // never loads from memory, and the compute wavefronts never store inside their loops:
        // loads and stores share one completion counter per wavefront, and a wavefront that
        // did both waited for its stores whenever it waited for a prefetched tile.
        for (int e = e_begin; e < e_end; ++e) {   // pass 1
            if constexpr (NBUF == 1) __syncthreads();
            __syncthreads();
        }
        __syncthreads();
        auto store_block = [&](int e) {
            const char* tile = pstage + ((e - e_begin) & 1) * PTILE;
#pragma unroll
            for (int i = 0; i < PTILE / 1024; ++i) {
                const int v = i * 64 + lane;       // vector v of the block: row v / PCH, chunk v % PCH
                const int row = v / PCH, c = v % PCH;
                __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(tile + row * PROW + ((c ^ pswz(row)) << 4)),
                                            reinterpret_cast<u32x4*>(P + (int64_t)e * (16 * WAVES * BW) + v * 8));
            }
        };
        for (int e = e_begin; e < e_end; ++e) {   // pass 2
            if constexpr (NBUF == 1) __syncthreads();
            __syncthreads();
            if (e > e_begin) store_block(e - 1);
        }
        __syncthreads();
        store_block(e_end - 1);
        return;
    }
    u32x4 kr[NV], vr[NV];
    constexpr float RESCALE_LOG2 = 6.f;

    // ---- pass 1: row maximum (as -m in log2 units) and row sum ------------------------------
    f32x4 negm = f32x4{0.f, 0.f, 0.f, 0.f};
    bool fresh = true;
    float l_part = 0.f;
    {
        // (the entry after next is fetched a whole step before its address is needed)
        int bc = p.bcsr_idx[e_begin] & 0xffff;
        int bc_next = p.bcsr_idx[e_begin + 1 < e_end ? e_begin + 1 : e_begin] & 0xffff;
        {
            const int64_t off = (int64_t)bc * BW * E;
#pragma unroll
            for (int i = 0; i < NV; ++i) kr[i] = *reinterpret_cast<const u32x4*>(Kg + off + i * NT * 8);
        }
        for (int e = e_begin; e < e_end; ++e) {
            char* buf = smem + (NBUF == 2 ? ((e - e_begin) & 1) * TILE : 0);
            if constexpr (NBUF == 1) __syncthreads();
#pragma unroll
            for (int i = 0; i < NV; ++i) *reinterpret_cast<u32x4*>(buf + k_dst + i * RSTEP * KP) = kr[i];
            const int key0 = bc * BW;
            bc = bc_next;
            bc_next = p.bcsr_idx[e + 2 < e_end ? e + 2 : e_end - 1] & 0xffff;
            {
                const int64_t off = (int64_t)bc * BW * E;
#pragma unroll
                for (int i = 0; i < NV; ++i) kr[i] = *reinterpret_cast<const u32x4*>(Kg + off + i * NT * 8);
            }
            unsigned live[KT];
            if constexpr (HAS_MASK) {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
                    live[kt] = *reinterpret_cast<const uint32_t*>(p.mask + (int64_t)qrow * p.Ns + key0 + kt * 16 + g4 * 4);
            }
            __syncthreads();
            f32x4 s[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                s[kt] = negm;
#pragma unroll
                for (int c = 0; c < EC; ++c) {
                    const Frag kf = *reinterpret_cast<const Frag*>(buf + k_src + kt * 16 * KP + (((c * 4 + g4) ^ k_sw) * 16));
                    s[kt] = Mma32<T>::mma(kf, qf[c], s[kt]);
                }
            }
            if constexpr (HAS_MASK) mask_scores<KT>(s, live);
            float tmax = lane_max<KT>(s);
            tmax = xor32_max(xor16_max(tmax));
            const bool any_live = tmax > -1e29f;
            if (__builtin_amdgcn_ballot_w64(any_live && (fresh || tmax > RESCALE_LOG2)) != 0) {
                const float delta = any_live ? (fresh ? tmax : fmaxf(tmax, 0.f)) : 0.f;
                negm -= delta;
                l_part *= __builtin_amdgcn_exp2f(-delta);
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) s[kt] -= delta;
            }
            fresh = fresh && !any_live;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    l_part += __builtin_amdgcn_exp2f(s[kt][q]);
                }
        }
    }
    const float l_run = xor32_sum(xor16_sum(l_part));
    const float inv_l = l_run > 0.f ? 1.f / l_run : 0.f;
    __syncthreads();   // everyone is done with the K tiles of pass 1

    // ---- pass 2: probabilities and output ----------------------------------------------------
    f32x4 oacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    int bc = p.bcsr_idx[e_begin] & 0xffff;
    int bc_next = p.bcsr_idx[e_begin + 1 < e_end ? e_begin + 1 : e_begin] & 0xffff;
    {
        const int64_t off = (int64_t)bc * BW * E;
#pragma unroll
        for (int i = 0; i < NV; ++i) kr[i] = *reinterpret_cast<const u32x4*>(Kg + off + i * NT * 8);
#pragma unroll
        for (int i = 0; i < NV; ++i) vr[i] = *reinterpret_cast<const u32x4*>(Vg + off + i * NT * 8);
    }
    for (int e = e_begin; e < e_end; ++e) {
        char* buf = smem + (NBUF == 2 ? ((e - e_begin) & 1) * TILE : 0);
        if constexpr (NBUF == 1) __syncthreads();
#pragma unroll
        for (int i = 0; i < NV; ++i) *reinterpret_cast<u32x4*>(buf + k_dst + i * RSTEP * KP) = kr[i];
#pragma unroll
        for (int i = 0; i < NV; ++i) *reinterpret_cast<u32x4*>(buf + v_dst + i * RSTEP * VP) = vr[i];
        const int key0 = bc * BW;
        bc = bc_next;
        bc_next = p.bcsr_idx[e + 2 < e_end ? e + 2 : e_end - 1] & 0xffff;
        {
            const int64_t off = (int64_t)bc * BW * E;
#pragma unroll
            for (int i = 0; i < NV; ++i) kr[i] = *reinterpret_cast<const u32x4*>(Kg + off + i * NT * 8);
#pragma unroll
            for (int i = 0; i < NV; ++i) vr[i] = *reinterpret_cast<const u32x4*>(Vg + off + i * NT * 8);
        }
        unsigned live[KT];
        if constexpr (HAS_MASK) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                live[kt] = *reinterpret_cast<const uint32_t*>(p.mask + (int64_t)qrow * p.Ns + key0 + kt * 16 + g4 * 4);
        }
        __syncthreads();
        f32x4 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = negm;
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag kf = *reinterpret_cast<const Frag*>(buf + k_src + kt * 16 * KP + (((c * 4 + g4) ^ k_sw) * 16));
                s[kt] = Mma32<T>::mma(kf, qf[c], s[kt]);
            }
        }
        if constexpr (HAS_MASK) mask_scores<KT>(s, live);
        Frag pf[KT / 2];
#pragma unroll
        for (int kp = 0; kp < KT / 2; ++kp) {
            f32x8 pv;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int kt = 2 * kp + (j >> 2), q = j & 3;
                pv[j] = __builtin_amdgcn_exp2f(s[kt][q]) * inv_l;
            }
            pf[kp] = AttnPack<T>::pack(pv);
            const s16x8 bits = __builtin_bit_cast(s16x8, pf[kp]);
            // 16 keys are 32 bytes = two chunks of the row; the lane's four keys are half a chunk
            char* prow = pstage + ((e - e_begin) & 1) * PTILE + (wave * 16 + r16) * PROW + (g4 & 1) * 8;
            const int sw = pswz(wave * 16 + r16);
            *reinterpret_cast<s16x4*>(prow + ((((2 * kp) * 2 + (g4 >> 1)) ^ sw) << 4)) = __builtin_shufflevector(bits, bits, 0, 1, 2, 3);
            *reinterpret_cast<s16x4*>(prow + ((((2 * kp + 1) * 2 + (g4 >> 1)) ^ sw) << 4)) = __builtin_shufflevector(bits, bits, 4, 5, 6, 7);
        }
        // (the store wavefront writes this block's probabilities to memory during the next step)
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int kp = 0; kp < KT / 2; ++kp) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + v_src + (kp * 32) * VP + t * 32));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + v_src + (kp * 32 + 16) * VP + t * 32));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, both), pf[kp], oacc[t]);
            }
        }
    }
    uint64_t pieces[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(oacc[t][q]);
        pieces[t] = *reinterpret_cast<const uint64_t*>(vals);
    }
    __syncthreads();   // the last block of probabilities is staged; the K / V tiles are dead
    if constexpr (WAVES * 16 * (E * 2 + 16) <= NBUF * TILE) {
        wave_rows_store<E>(smem + wave * (16 * (E * 2 + 16)), O + (int64_t)(qrow - r16) * E, pieces);
    } else {
#pragma unroll
        for (int t = 0; t < ET; ++t) *reinterpret_cast<uint64_t*>(O + (int64_t)qrow * E + t * 16 + g4 * 4) = pieces[t];
    }
}

template <typename T, int BW, int E, int WAVES>
static int launch_attention_train_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr int TILE = BW * (E * 4 + 32);
    constexpr size_t smem = (2 * TILE <= 64 * 1024 ? 2 * TILE : TILE) + 2 * WAVES * 16 * (BW * 2);   // K / V tiles + two staged blocks of P
    const int nbr = p.Nt / p.BH;
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbr;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (p.mask) {
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_train_kernel<T, BW, E, WAVES, true>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_train_kernel)");
        }
        hipLaunchKernelGGL((attention_train_kernel<T, BW, E, WAVES, true>), dim3((unsigned)groups), dim3(64 * (WAVES + 1)), smem, st, p, nbr, batch);
    } else {
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_train_kernel<T, BW, E, WAVES, false>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_train_kernel)");
        }
        hipLaunchKernelGGL((attention_train_kernel<T, BW, E, WAVES, false>), dim3((unsigned)groups), dim3(64 * (WAVES + 1)), smem, st, p, nbr, batch);
    }
    SPX_LAUNCH_CHECK("attention_train_kernel");
    return 0;
}

template <typename T>
static int launch_attention_train(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTNT_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_train_inst<T, bw, e, bh / 16>(p, batch, st);
    SPX_ATTNT_CASE(32, 32, 64) SPX_ATTNT_CASE(32, 64, 64) SPX_ATTNT_CASE(32, 128, 64)
    SPX_ATTNT_CASE(32, 32, 128) SPX_ATTNT_CASE(32, 64, 128) SPX_ATTNT_CASE(32, 128, 128)
    SPX_ATTNT_CASE(64, 32, 64) SPX_ATTNT_CASE(64, 64, 64) SPX_ATTNT_CASE(64, 128, 64)
    SPX_ATTNT_CASE(64, 32, 128) SPX_ATTNT_CASE(64, 64, 128) SPX_ATTNT_CASE(64, 128, 128)
    SPX_ATTNT_CASE(128, 64, 64) SPX_ATTNT_CASE(128, 128, 64)
    SPX_ATTNT_CASE(128, 32, 128) SPX_ATTNT_CASE(128, 64, 128) SPX_ATTNT_CASE(128, 128, 128)
#undef SPX_ATTNT_CASE
    return fail(SPX_E_CONFIG, "the training forward kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

// ---- backward pass, row side: gradient of the scores and of the queries ---------------------
// With P saved by the training forward kernel, the gradient of the scores is
//   dS = P o (dP - D) / T,   dP = dO V^T,   D[q] = sum_e dO[q, e] O[q, e],
// and dQ = dS K.  One workgroup per block row walks its live blocks like the forward
// kernels do, with the roles of K and V exchanged (V rows feed the first product, K is read
// through transpose reads for the second): dP^T tiles come out of the MFMAs already reduced
// by D (the accumulators start at -D / T, dO is scaled by 1 / T once), are multiplied by the
// probabilities (8-byte loads of the 4 keys a lane holds per tile), written as dS in the
// layout of P and fed to the dQ MFMAs.  Masked entries have P = 0 and so dS = 0: no mask is
// needed.  dK and dV stay with the sparse-operand matmul kernels (dK = dS^T Q, dV = P^T dO).
// Replaces three launches of the operator pipeline's backward (dP, softmax backward, dQ).
template <typename T, int BW, int E, int WAVES>
__global__ __launch_bounds__(64 * WAVES, waves_per_simd_for((2 * BW * (E * 4 + 32) <= 64 * 1024 ? 2 : 1) * BW * (E * 4 + 32) + WAVES * 16 * (BW * 2 + 16), WAVES)) void attention_bwd_row_kernel(AttnParams p, int nbr, int batch) {
    constexpr int NT = 64 * WAVES;
    constexpr int KT = BW / 16, ET = E / 16, EC = E / 32;
    constexpr int RP = E * 2;                 // pitch of the row-read tile (V): 16-byte chunks XOR-swizzled by row % 8
    constexpr int TP = E * 2 + 32;            // pitch of the transpose-read tile (K)
    constexpr int TILE = BW * (RP + TP);
    constexpr int NBUF = 2 * TILE <= 64 * 1024 ? 2 : 1;
    constexpr int VPR = E / 8;
    constexpr int NV = BW * VPR / NT;
    constexpr int RSTEP = NT / VPR;
    constexpr int PP = BW * 2 + 16;           // row pitch of a wave's private 16 x BW probability tile
    constexpr int PN = BW / 32;               // 16-byte vectors of that tile per lane
    constexpr int NSTG = (PN + 2 * NV) * 4 <= 48 ? 2 : 1;   // register stages of the prefetch
    static_assert(BW * VPR % NT == 0 && NT % VPR == 0 && KT % 2 == 0, "tile does not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    const int L = blockIdx.x;
    const int slot = L >> 3;
    const int64_t b = (slot / nbr) * 8 + (L & 7);
    const int br = slot % nbr;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* dO = reinterpret_cast<const T*>(p.grad_out) + b * (int64_t)p.Nt * E;
    const T* O = reinterpret_cast<const T*>(p.out) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    const T* P = reinterpret_cast<const T*>(p.probs) + b * p.probs_batch;
    T* dS = reinterpret_cast<T*>(p.grad_scores) + b * p.probs_batch;
    T* dQ = reinterpret_cast<T*>(p.grad_q) + b * (int64_t)p.Nt * E;

    const int qrow = br * (16 * WAVES) + wave * 16 + r16;
    // dO fragments scaled by 1 / T, and D / T = sum_e dO O / T for this lane's query
    Frag gf[EC];
    float d_part = 0.f;
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const Frag g_raw = Mma32<T>::load(dO + (int64_t)qrow * E + c * 32 + g4 * 8);
        const Frag o_raw = Mma32<T>::load(O + (int64_t)qrow * E + c * 32 + g4 * 8);
        f32x8 scaled;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            scaled[j] = (float)g_raw[j] * p.inv_t;
            d_part += scaled[j] * (float)o_raw[j];
        }
        gf[c] = AttnPack<T>::pack(scaled);
    }
    const float d_row = xor32_sum(xor16_sum(d_part));
    if (p.row_dot && g4 == 0) p.row_dot[b * p.Nt + qrow] = d_row;
    const bool store_ds = p.grad_scores != nullptr;   // the column-side kernel recomputes dS from P
    const f32x4 negd = f32x4{-d_row, -d_row, -d_row, -d_row};

    f32x4 qacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) qacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int st_row = threadIdx.x / VPR, st_chunk = threadIdx.x % VPR;
    const int r_dst = st_row * RP + (st_chunk ^ (st_row & 7)) * 16;     // V tile
    const int t_dst = BW * RP + st_row * TP + st_chunk * 16;            // K tile
    const int r_src = r16 * RP;
    const int r_sw = r16 & 7;
    const int t_src = BW * RP + (g4 * 4 + (r16 >> 2)) * TP + (r16 & 3) * 8;

    // A wave's 16 rows of a block are 32 * BW contiguous bytes of P (and of dS): they move
    // between memory and the wave's private tile in LDS as whole 16-byte vectors, and
    // between the tile and the MFMA layout (4 keys of one query per lane) as 8-byte pieces.
    char* ptile = smem + NBUF * TILE + wave * (16 * PP);
    int pt_vec[PN];
#pragma unroll
    for (int i = 0; i < PN; ++i) {
        const int c = i * 64 + lane;
        pt_vec[i] = (c / (BW / 8)) * PP + (c % (BW / 8)) * 16;
    }
    const int pt_piece = r16 * PP + g4 * 8;
    const int64_t wave_off = (int64_t)wave * (16 * BW) + lane * 8;   // elements, inside a block

    const int e_begin = p.row_ptr[br];
    const int n_blk = p.row_ptr[br + 1] - e_begin;
    // Block columns of the row: lane l holds entry l (broadcast with readlane, so no step
    // waits for an index load); longer rows read the rest from the index.
    int bc_vec = 0;
    if (lane < n_blk) bc_vec = p.bcsr_idx[e_begin + lane] & 0xffff;
    auto col_at = [&](int i) {
        return i < 64 ? __builtin_amdgcn_readlane(bc_vec, i) : (p.bcsr_idx[e_begin + i] & 0xffff);
    };
    // Two register stages: the P block and the K / V tiles of step i + 2 are requested while
    // step i is staged and computed.  A step's MFMA work is a fraction of a memory round
    // trip, so one step of lead left every step waiting.  The loads go through inline
    // assembly and are waited for with explicit counts: the compiler merges its own wait
    // counts at the loop header and would drain both stages at every step.  (Shapes whose
    // tiles take more than 48 registers per thread keep one stage of ordinary loads.)
    auto issue = [&](int i, u32x4 (&pr)[PN], u32x4 (&vr)[NV], u32x4 (&kr)[NV]) {
        const int64_t off = (int64_t)col_at(i) * BW * E;
        const T* pblk = P + (int64_t)(e_begin + i) * (16 * WAVES * BW) + wave_off;
        if constexpr (NSTG == 2) {
#pragma unroll
            for (int i2 = 0; i2 < PN; ++i2)   // P is read once: non-temporal
                asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(pr[i2]) : "v"(pblk + i2 * 512) : "memory");
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2)
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(vr[i2]) : "v"(Vg + off + i2 * NT * 8) : "memory");
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2)
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(kr[i2]) : "v"(Kg + off + i2 * NT * 8) : "memory");
        } else {
#pragma unroll
            for (int i2 = 0; i2 < PN; ++i2) pr[i2] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(pblk + i2 * 512));
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2) vr[i2] = *reinterpret_cast<const u32x4*>(Vg + off + i2 * NT * 8);
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2) kr[i2] = *reinterpret_cast<const u32x4*>(Kg + off + i2 * NT * 8);
        }
    };
    // Wait until only the other stage is outstanding; the stage's registers pass through the
    // statement so that no use is scheduled before it.  With dS stored everything is drained:
    // stores share the counter and need not complete in order with the loads.
    auto wait_stage = [&](int i, u32x4 (&pr)[PN], u32x4 (&vr)[NV], u32x4 (&kr)[NV]) {
        if constexpr (NSTG == 1) return;   // plain loads: the compiler waits where the registers are used
        if (i + 1 < n_blk && !store_ds) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PN + 2 * NV) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i2 = 0; i2 < PN; ++i2) asm volatile("" : "+v"(pr[i2]));
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) asm volatile("" : "+v"(vr[i2]));
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) asm volatile("" : "+v"(kr[i2]));
    };
    auto step = [&](int i, u32x4 (&pr)[PN], u32x4 (&vr)[NV], u32x4 (&kr)[NV]) {
        const int e = e_begin + i;
        char* buf = smem + (NBUF == 2 ? (i & 1) * TILE : 0);
        if constexpr (NBUF == 1) __syncthreads();
        wait_stage(i, pr, vr, kr);
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) *reinterpret_cast<u32x4*>(buf + r_dst + i2 * RSTEP * RP) = vr[i2];
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) *reinterpret_cast<u32x4*>(buf + t_dst + i2 * RSTEP * TP) = kr[i2];
#pragma unroll
        for (int i2 = 0; i2 < PN; ++i2) *reinterpret_cast<u32x4*>(ptile + pt_vec[i2]) = pr[i2];
        if (i + NSTG < n_blk) issue(i + NSTG, pr, vr, kr);
        __syncthreads();

        // ---- (dP - D)^T / T tiles: keys x this wave's 16 queries -----------------------------
        f32x4 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = negd;
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag vf = *reinterpret_cast<const Frag*>(buf + r_src + kt * 16 * RP + (((c * 4 + g4) ^ r_sw) * 16));
                s[kt] = Mma32<T>::mma(vf, gf[c], s[kt]);
            }
        }
        // this lane's probabilities of the block: 4 consecutive keys of every 16-key tile
        uint2 pb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) pb[kt] = *reinterpret_cast<const uint2*>(ptile + pt_piece + kt * 32);
        Frag sf[KT / 2];
#pragma unroll
        for (int kp = 0; kp < KT / 2; ++kp) {
            f32x8 ds;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int kt = 2 * kp + (j >> 2), q = j & 3;
                const uint32_t word = (q & 2) ? pb[kt].y : pb[kt].x;
                const unsigned short half = (unsigned short)((q & 1) ? word >> 16 : word & 0xffffu);
                ds[j] = Elem<T>::to_float(__builtin_bit_cast(T, half)) * s[kt][q];
            }
            sf[kp] = AttnPack<T>::pack(ds);
            const s16x8 bits = __builtin_bit_cast(s16x8, sf[kp]);
            *reinterpret_cast<s16x4*>(ptile + pt_piece + (2 * kp) * 32) = __builtin_shufflevector(bits, bits, 0, 1, 2, 3);
            *reinterpret_cast<s16x4*>(ptile + pt_piece + (2 * kp + 1) * 32) = __builtin_shufflevector(bits, bits, 4, 5, 6, 7);
        }
        if (store_ds) {
#pragma unroll
            for (int i2 = 0; i2 < PN; ++i2)
                *reinterpret_cast<u32x4*>(dS + (int64_t)e * (16 * WAVES * BW) + wave_off + i2 * 512) =
                    *reinterpret_cast<const u32x4*>(ptile + pt_vec[i2]);
        }
        // ---- dQ^T[e][query] += K^T dS^T ------------------------------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int kp = 0; kp < KT / 2; ++kp) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + t_src + (kp * 32) * TP + t * 32));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + t_src + (kp * 32 + 16) * TP + t * 32));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                qacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, both), sf[kp], qacc[t]);
            }
        }
    };
    if constexpr (NSTG == 2) {
        u32x4 p0[PN], v0[NV], k0[NV], p1[PN], v1[NV], k1[NV];
        if (n_blk > 0) {
            issue(0, p0, v0, k0);
            issue(n_blk > 1 ? 1 : 0, p1, v1, k1);   // a row of one block requests it twice; the copy is not used
        }
        for (int i = 0; i < n_blk; i += 2) {
            step(i, p0, v0, k0);
            if (i + 1 < n_blk) step(i + 1, p1, v1, k1);
        }
    } else {
        u32x4 p0[PN], v0[NV], k0[NV];
        if (n_blk > 0) issue(0, p0, v0, k0);
        for (int i = 0; i < n_blk; ++i) step(i, p0, v0, k0);
    }
    uint64_t pieces[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(qacc[t][q]);
        pieces[t] = *reinterpret_cast<const uint64_t*>(vals);
    }
    if constexpr (WAVES * 16 * (E * 2 + 16) <= NBUF * TILE) {
        __syncthreads();   // the K / V tiles are dead: their space carries the output tiles
        wave_rows_store<E>(smem + wave * (16 * (E * 2 + 16)), dQ + (int64_t)(qrow - r16) * E, pieces);
    } else {
#pragma unroll
        for (int t = 0; t < ET; ++t) *reinterpret_cast<uint64_t*>(dQ + (int64_t)qrow * E + t * 16 + g4 * 4) = pieces[t];
    }
}

template <typename T, int BW, int E, int WAVES>
static int launch_attention_bwd_row_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr int TILE = BW * (E * 4 + 32);
    constexpr size_t smem = (2 * TILE <= 64 * 1024 ? 2 * TILE : TILE) + WAVES * 16 * (BW * 2 + 16);
    const int nbr = p.Nt / p.BH;
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbr;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_bwd_row_kernel<T, BW, E, WAVES>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_bwd_row_kernel)");
    }
    hipLaunchKernelGGL((attention_bwd_row_kernel<T, BW, E, WAVES>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbr, batch);
    SPX_LAUNCH_CHECK("attention_bwd_row_kernel");
    return 0;
}

template <typename T>
static int launch_attention_bwd_row(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTNB_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_bwd_row_inst<T, bw, e, bh / 16>(p, batch, st);
    SPX_ATTNB_CASE(32, 32, 64) SPX_ATTNB_CASE(32, 64, 64) SPX_ATTNB_CASE(32, 128, 64)
    SPX_ATTNB_CASE(32, 32, 128) SPX_ATTNB_CASE(32, 64, 128) SPX_ATTNB_CASE(32, 128, 128)
    SPX_ATTNB_CASE(64, 32, 64) SPX_ATTNB_CASE(64, 64, 64) SPX_ATTNB_CASE(64, 128, 64)
    SPX_ATTNB_CASE(64, 32, 128) SPX_ATTNB_CASE(64, 64, 128) SPX_ATTNB_CASE(64, 128, 128)
    SPX_ATTNB_CASE(128, 64, 64) SPX_ATTNB_CASE(128, 128, 64)
    SPX_ATTNB_CASE(128, 32, 128) SPX_ATTNB_CASE(128, 64, 128) SPX_ATTNB_CASE(128, 128, 128)
#undef SPX_ATTNB_CASE
    return fail(SPX_E_CONFIG, "the attention backward kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

// ---- backward pass without stored probabilities, row side ---------------------------------
// The forward kernel records one number per query, the log2-domain log-sum-exp L of its row;
// P = exp2(S - L) then reproduces the normalised probabilities wherever they are needed, and
// neither P nor dS ever goes to memory.  Per live block a wavefront computes, for its 16
// queries,  (S - L)^T = K Q^T  (accumulators started at -L, Q scaled by log2(e) / T),
// (dP - D)^T / T = V dO^T  (accumulators started at -D / T, dO scaled by 1 / T),
// dS^T = exp2(S - L) o (dP - D) / T  as the B operand of  dQ^T += K^T dS^T.
// V is staged for row reads; K in rows padded for the transpose reads of the last product,
// which the row reads of the first product share (rows r and r + 8 fall on the same banks:
// eight two-way conflicts per block against sixteen transpose reads).  Block-level masks only
// (an element mask would have to be re-applied here); the K / V tiles of step i + 2 are
// requested while step i runs, as in attention_bwd_row_kernel.
template <typename T, int BW, int E, int WAVES>
__global__ __launch_bounds__(64 * WAVES, waves_per_simd_for((2 * BW * (E * 4 + 32) <= 64 * 1024 ? 2 : 1) * BW * (E * 4 + 32), WAVES))
void attention_bwd_row_rc_kernel(AttnParams p, int nbr, int batch) {
    constexpr int NT = 64 * WAVES;
    constexpr int KT = BW / 16, ET = E / 16, EC = E / 32;
    constexpr int RP = E * 2;                 // pitch of the row-read tile (V): 16-byte chunks XOR-swizzled by row % 8
    constexpr int TP = E * 2 + 32;            // pitch of the K tile (transpose reads and row reads)
    constexpr int TILE = BW * (RP + TP);
    constexpr int NBUF = 2 * TILE <= 64 * 1024 ? 2 : 1;
    constexpr int VPR = E / 8;
    constexpr int NV = BW * VPR / NT;
    constexpr int RSTEP = NT / VPR;
    constexpr int NSTG = 2 * NV * 4 <= 48 ? 2 : 1;   // register stages of the prefetch
    static_assert(BW * VPR % NT == 0 && NT % VPR == 0 && KT % 2 == 0, "tile does not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    const int L = blockIdx.x;
    const int slot = L >> 3;
    const int64_t b = (slot / nbr) * 8 + (L & 7);
    const int br = slot % nbr;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* dO = reinterpret_cast<const T*>(p.grad_out) + b * (int64_t)p.Nt * E;
    const T* O = reinterpret_cast<const T*>(p.out) + b * (int64_t)p.Nt * E;
    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    T* dQ = reinterpret_cast<T*>(p.grad_q) + b * (int64_t)p.Nt * E;

    const int qrow = br * (16 * WAVES) + wave * 16 + r16;
    const float c2 = p.inv_t * 1.4426950408889634f;
    Frag gf[EC], qf[EC];   // dO / T and Q * log2(e) / T of this lane's query
    float d_part = 0.f;
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const Frag g_raw = Mma32<T>::load(dO + (int64_t)qrow * E + c * 32 + g4 * 8);
        const Frag o_raw = Mma32<T>::load(O + (int64_t)qrow * E + c * 32 + g4 * 8);
        const Frag q_raw = Mma32<T>::load(Q + (int64_t)qrow * E + c * 32 + g4 * 8);
        f32x8 gs, qs;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            gs[j] = (float)g_raw[j] * p.inv_t;
            qs[j] = (float)q_raw[j] * c2;
            d_part += gs[j] * (float)o_raw[j];
        }
        gf[c] = AttnPack<T>::pack(gs);
        qf[c] = AttnPack<T>::pack(qs);
    }
    const float d_row = xor32_sum(xor16_sum(d_part));
    if (p.row_dot && g4 == 0) p.row_dot[b * p.Nt + qrow] = d_row;
    const float lse = p.row_lse[b * p.Nt + qrow];
    const f32x4 negd = f32x4{-d_row, -d_row, -d_row, -d_row};
    const f32x4 negl = f32x4{-lse, -lse, -lse, -lse};

    f32x4 qacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) qacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int st_row = threadIdx.x / VPR, st_chunk = threadIdx.x % VPR;
    const int r_dst = st_row * RP + (st_chunk ^ (st_row & 7)) * 16;     // V tile
    const int t_dst = BW * RP + st_row * TP + st_chunk * 16;            // K tile
    const int r_src = r16 * RP;
    const int r_sw = r16 & 7;
    const int k_src = BW * RP + r16 * TP + g4 * 16;                     // K rows as A operand of the scores
    const int t_src = BW * RP + (g4 * 4 + (r16 >> 2)) * TP + (r16 & 3) * 8;

    const int e_begin = p.row_ptr[br];
    const int n_blk = p.row_ptr[br + 1] - e_begin;
    // block columns of the row: lane l holds entry l; longer rows read the rest from the index
    int bc_vec = 0;
    if (lane < n_blk) bc_vec = p.bcsr_idx[e_begin + lane] & 0xffff;
    auto col_at = [&](int i) {
        return i < 64 ? __builtin_amdgcn_readlane(bc_vec, i) : (p.bcsr_idx[e_begin + i] & 0xffff);
    };
    auto issue = [&](int i, u32x4 (&vr)[NV], u32x4 (&kr)[NV]) {
        const int64_t off = (int64_t)col_at(i) * BW * E;
        if constexpr (NSTG == 2) {
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2)
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(vr[i2]) : "v"(Vg + off + i2 * NT * 8) : "memory");
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2)
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(kr[i2]) : "v"(Kg + off + i2 * NT * 8) : "memory");
        } else {
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2) vr[i2] = *reinterpret_cast<const u32x4*>(Vg + off + i2 * NT * 8);
#pragma unroll
            for (int i2 = 0; i2 < NV; ++i2) kr[i2] = *reinterpret_cast<const u32x4*>(Kg + off + i2 * NT * 8);
        }
    };
    auto wait_stage = [&](int i, u32x4 (&vr)[NV], u32x4 (&kr)[NV]) {
        if constexpr (NSTG == 1) return;   // plain loads: the compiler waits where the registers are used
        if (i + 1 < n_blk) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NV) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) asm volatile("" : "+v"(vr[i2]));
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) asm volatile("" : "+v"(kr[i2]));
    };
    auto step = [&](int i, u32x4 (&vr)[NV], u32x4 (&kr)[NV]) {
        char* buf = smem + (NBUF == 2 ? (i & 1) * TILE : 0);
        if constexpr (NBUF == 1) __syncthreads();
        wait_stage(i, vr, kr);
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) *reinterpret_cast<u32x4*>(buf + r_dst + i2 * RSTEP * RP) = vr[i2];
#pragma unroll
        for (int i2 = 0; i2 < NV; ++i2) *reinterpret_cast<u32x4*>(buf + t_dst + i2 * RSTEP * TP) = kr[i2];
        if (i + NSTG < n_blk) issue(i + NSTG, vr, kr);
        __syncthreads();

        // ---- (S - L)^T and (dP - D)^T / T tiles: keys x this wave's 16 queries -----------------
        f32x4 s[KT], dp[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = negl;
            dp[kt] = negd;
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag kf = *reinterpret_cast<const Frag*>(buf + k_src + kt * 16 * TP + c * 64);
                s[kt] = Mma32<T>::mma(kf, qf[c], s[kt]);
                const Frag vf = *reinterpret_cast<const Frag*>(buf + r_src + kt * 16 * RP + (((c * 4 + g4) ^ r_sw) * 16));
                dp[kt] = Mma32<T>::mma(vf, gf[c], dp[kt]);
            }
        }
        Frag sf[KT / 2];
#pragma unroll
        for (int kp = 0; kp < KT / 2; ++kp) {
            f32x8 ds;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int kt = 2 * kp + (j >> 2), q = j & 3;
                ds[j] = __builtin_amdgcn_exp2f(s[kt][q]) * dp[kt][q];
            }
            sf[kp] = AttnPack<T>::pack(ds);
        }
        // ---- dQ^T[e][query] += K^T dS^T ------------------------------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int kp = 0; kp < KT / 2; ++kp) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + t_src + (kp * 32) * TP + t * 32));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + t_src + (kp * 32 + 16) * TP + t * 32));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                qacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, both), sf[kp], qacc[t]);
            }
        }
    };
    if constexpr (NSTG == 2) {
        u32x4 v0[NV], k0[NV], v1[NV], k1[NV];
        if (n_blk > 0) {
            issue(0, v0, k0);
            issue(n_blk > 1 ? 1 : 0, v1, k1);   // a row of one block requests it twice; the copy is not used
        }
        for (int i = 0; i < n_blk; i += 2) {
            step(i, v0, k0);
            if (i + 1 < n_blk) step(i + 1, v1, k1);
        }
    } else {
        u32x4 v0[NV], k0[NV];
        if (n_blk > 0) issue(0, v0, k0);
        for (int i = 0; i < n_blk; ++i) step(i, v0, k0);
    }
    uint64_t pieces[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(qacc[t][q]);
        pieces[t] = *reinterpret_cast<const uint64_t*>(vals);
    }
    if constexpr (WAVES * 16 * (E * 2 + 16) <= NBUF * TILE) {
        __syncthreads();   // the K / V tiles are dead: their space carries the output tiles
        wave_rows_store<E>(smem + wave * (16 * (E * 2 + 16)), dQ + (int64_t)(qrow - r16) * E, pieces);
    } else {
#pragma unroll
        for (int t = 0; t < ET; ++t) *reinterpret_cast<uint64_t*>(dQ + (int64_t)qrow * E + t * 16 + g4 * 4) = pieces[t];
    }
}

template <typename T, int BW, int E, int WAVES>
static int launch_attention_bwd_row_rc_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr int TILE = BW * (E * 4 + 32);
    constexpr size_t smem = 2 * TILE <= 64 * 1024 ? 2 * TILE : TILE;
    const int nbr = p.Nt / p.BH;
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbr;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_bwd_row_rc_kernel<T, BW, E, WAVES>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_bwd_row_rc_kernel)");
    }
    hipLaunchKernelGGL((attention_bwd_row_rc_kernel<T, BW, E, WAVES>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbr, batch);
    SPX_LAUNCH_CHECK("attention_bwd_row_rc_kernel");
    return 0;
}

template <typename T>
static int launch_attention_bwd_row_rc(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTNR_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_bwd_row_rc_inst<T, bw, e, bh / 16>(p, batch, st);
    SPX_ATTNR_CASE(32, 32, 64) SPX_ATTNR_CASE(32, 64, 64) SPX_ATTNR_CASE(32, 128, 64)
    SPX_ATTNR_CASE(32, 32, 128) SPX_ATTNR_CASE(32, 64, 128) SPX_ATTNR_CASE(32, 128, 128)
    SPX_ATTNR_CASE(64, 32, 64) SPX_ATTNR_CASE(64, 64, 64) SPX_ATTNR_CASE(64, 128, 64)
    SPX_ATTNR_CASE(64, 32, 128) SPX_ATTNR_CASE(64, 64, 128) SPX_ATTNR_CASE(64, 128, 128)
    SPX_ATTNR_CASE(128, 64, 64) SPX_ATTNR_CASE(128, 128, 64)
    SPX_ATTNR_CASE(128, 32, 128) SPX_ATTNR_CASE(128, 64, 128) SPX_ATTNR_CASE(128, 128, 128)
#undef SPX_ATTNR_CASE
    return fail(SPX_E_CONFIG, "the attention backward kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

// ---- backward pass, column side: gradients of the keys and of the values -------------------
//   dV = P^T dO,   dK = dS^T Q,   dS = P o (dO V^T - D) / T  (recomputed here from P)
// One workgroup per block column (BW keys) and batch entry, one wavefront per 16 keys, walking
// the live blocks of the column through the BCSC index.  Per block the dO and Q tiles of the
// query block and the P block (at its BCSR position) are staged in LDS, rows padded for
// transpose reads:
//   (dP - D)^T/T tiles: 16 queries x 16 keys = dO rows x V rows (V of the column, scaled by
//     1/T, lives in registers; accumulators start at -D/T read from row_dot), a lane gets
//     4 consecutive queries of one key;
//   P in that same layout by one transpose read per tile; dS = P o (dP - D)/T;
//   two tiles side by side are the B operand (32 queries deep) of
//     dK^T[e][key] += Q^T dS   and, for P itself,   dV^T[e][key] += dO^T P,
//   whose A operands are transpose reads of the Q and dO tiles.
// The score gradient never goes to memory: P is read once here and once by the row-side
// kernel, instead of P and dS being read by two separate products after dS was written.
template <typename T, int BH, int E, int WAVES>
// second launch bound: wavefronts per SIMD the register budget is sized for (small tiles fit
// 168 VGPRs; the default budget made the compiler park accumulators in AGPRs and copy them
// back and forth every step)
__global__ __launch_bounds__(64 * WAVES, (BH * E <= 64 * 64 || BH == 32) ? 3 : (BH * E <= 128 * 64 ? 2 : 1)) void attention_bwd_col_kernel(AttnParams p, int nbc, int batch) {
    constexpr int BW = 16 * WAVES;
    constexpr int NT = 64 * WAVES;
    constexpr int QT = BH / 16, ET = E / 16, EC = E / 32;
    constexpr int DP = E * 2 + 32;            // row pitch of the dO and Q tiles
    constexpr int PP = BW * 2 + 32;           // row pitch of the P block
    constexpr int Q_OFF = BH * DP, P_OFF = 2 * BH * DP;
    constexpr int TILE = 2 * BH * DP + BH * PP;
    constexpr int VPR = E / 8, PPR = BW / 8;  // 16-byte vectors per row
    constexpr int NVD = BH * VPR / NT;        // vectors per thread: dO / Q tile
    constexpr int NVP = BH * PPR / NT;        // vectors per thread: P block
    static_assert(BH * VPR % NT == 0 && BH * PPR % NT == 0 && QT % 2 == 0, "tiles do not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    const int L = blockIdx.x;
    const int slot_l = L >> 3;
    const int64_t b = (slot_l / nbc) * 8 + (L & 7);
    const int j = slot_l % nbc;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* dO = reinterpret_cast<const T*>(p.grad_out) + b * (int64_t)p.Nt * E + threadIdx.x * 8;
    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E + threadIdx.x * 8;
    const T* P = reinterpret_cast<const T*>(p.probs) + b * p.probs_batch + threadIdx.x * 8;
    const float* Dv = p.row_dot + b * (int64_t)p.Nt + g4 * 4;
    T* dK = reinterpret_cast<T*>(p.grad_k) + b * (int64_t)p.Ns * E;
    T* dV = reinterpret_cast<T*>(p.grad_v) + b * (int64_t)p.Ns * E;

    const int krow = j * BW + wave * 16 + r16;
    Frag vf[EC];     // V of this lane's key, scaled by 1 / T
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const Frag raw = Mma32<T>::load(reinterpret_cast<const T*>(p.v) + (b * (int64_t)p.Ns + krow) * E + c * 32 + g4 * 8);
        f32x8 scaled;
#pragma unroll
        for (int x = 0; x < 8; ++x) scaled[x] = (float)raw[x] * p.inv_t;
        vf[c] = AttnPack<T>::pack(scaled);
    }

    f32x4 kacc[ET], vacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) kacc[t] = vacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // staging maps (a tile is contiguous in memory: vector v = tid + i * NT is row v / VPR)
    const int d_dst = (threadIdx.x / VPR) * DP + (threadIdx.x % VPR) * 16;
    const int p_dst = P_OFF + (threadIdx.x / PPR) * PP + (threadIdx.x % PPR) * 16;
    constexpr int D_RSTEP = NT / VPR, P_RSTEP = NT / PPR;
    static_assert(NT % VPR == 0 && NT % PPR == 0, "rows per pass");
    const int a_src = r16 * DP + g4 * 16;                                    // dO rows as A operand of dP
    const int t_src = (g4 * 4 + (r16 >> 2)) * DP + (r16 & 3) * 8;            // transpose reads of dO / Q
    const int pt_src = P_OFF + (g4 * 4 + (r16 >> 2)) * PP + (wave * 16 + (r16 & 3) * 4) * 2;

    const int e_begin = p.col_ptr[j];
    const int e_end = p.col_ptr[j + 1];
    auto entry = [&](int e, int& qb, int64_t& pos) {
        if (p.bcsc_wide) {
            const long long v = reinterpret_cast<const long long*>(p.bcsc_idx)[e];
            qb = (int)(v & 0xffff);
            pos = v >> 32;
        } else {
            qb = reinterpret_cast<const int32_t*>(p.bcsc_idx)[e] & 0xffff;
            pos = e;
        }
    };
    u32x4 do_r[NVD], q_r[NVD], p_r[NVP];
    f32x4 d_r[QT];
    auto issue = [&](int qb, int64_t pos) {
        const int64_t off = (int64_t)qb * BH * E;
#pragma unroll
        for (int i = 0; i < NVD; ++i) do_r[i] = *reinterpret_cast<const u32x4*>(dO + off + i * NT * 8);
#pragma unroll
        for (int i = 0; i < NVD; ++i) q_r[i] = *reinterpret_cast<const u32x4*>(Q + off + i * NT * 8);
#pragma unroll
        for (int i = 0; i < NVP; ++i)   // P is read once: no need to keep it in L2
            p_r[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(P + pos * (int64_t)(BH * BW) + i * NT * 8));
#pragma unroll
        for (int t = 0; t < QT; ++t) d_r[t] = *reinterpret_cast<const f32x4*>(Dv + qb * BH + t * 16);
    };
    int qb = 0, qb_next = 0;
    int64_t pos = 0, pos_next = 0;
    if (e_begin < e_end) {
        entry(e_begin, qb, pos);
        entry(e_begin + 1 < e_end ? e_begin + 1 : e_begin, qb_next, pos_next);
        issue(qb, pos);
    }
    for (int e = e_begin; e < e_end; ++e) {
        __syncthreads();   // everyone is done with the previous tiles
#pragma unroll
        for (int i = 0; i < NVD; ++i) *reinterpret_cast<u32x4*>(smem + d_dst + i * D_RSTEP * DP) = do_r[i];
#pragma unroll
        for (int i = 0; i < NVD; ++i) *reinterpret_cast<u32x4*>(smem + Q_OFF + d_dst + i * D_RSTEP * DP) = q_r[i];
#pragma unroll
        for (int i = 0; i < NVP; ++i) *reinterpret_cast<u32x4*>(smem + p_dst + i * P_RSTEP * PP) = p_r[i];
        f32x4 s[QT];
#pragma unroll
        for (int t = 0; t < QT; ++t) s[t] = -d_r[t];
        // next live block of the column (the last step re-reads its own block; the copy is not used)
        qb = qb_next; pos = pos_next;
        entry(e + 2 < e_end ? e + 2 : e_end - 1, qb_next, pos_next);
        issue(qb, pos);
        __syncthreads();

        // ---- (dP - D) / T: 16 queries x this wave's 16 keys per tile -------------------------
#pragma unroll
        for (int t = 0; t < QT; ++t) {
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag af = *reinterpret_cast<const Frag*>(smem + a_src + t * 16 * DP + c * 64);
                s[t] = Mma32<T>::mma(af, vf[c], s[t]);
            }
        }
        // ---- P in the same layout; dS = P o (dP - D) / T; both as B operands ------------------
        Frag pf[QT / 2], sf[QT / 2];
#pragma unroll
        for (int kp = 0; kp < QT / 2; ++kp) {
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + pt_src + (kp * 32) * PP));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + pt_src + (kp * 32 + 16) * PP));
            pf[kp] = __builtin_bit_cast(Frag, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            f32x8 ds;
#pragma unroll
            for (int x = 0; x < 8; ++x) ds[x] = (float)pf[kp][x] * s[2 * kp + (x >> 2)][x & 3];
            sf[kp] = AttnPack<T>::pack(ds);
        }
        // ---- dK^T[e][key] += Q^T dS,  dV^T[e][key] += dO^T P ----------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int kp = 0; kp < QT / 2; ++kp) {
                const s16x4 qlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + Q_OFF + t_src + (kp * 32) * DP + t * 32));
                const s16x4 qhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + Q_OFF + t_src + (kp * 32 + 16) * DP + t * 32));
                const s16x8 qa = __builtin_shufflevector(qlo, qhi, 0, 1, 2, 3, 4, 5, 6, 7);
                kacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, qa), sf[kp], kacc[t]);
                const s16x4 glo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + t_src + (kp * 32) * DP + t * 32));
                const s16x4 ghi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + t_src + (kp * 32 + 16) * DP + t * 32));
                const s16x8 ga = __builtin_shufflevector(glo, ghi, 0, 1, 2, 3, 4, 5, 6, 7);
                vacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, ga), pf[kp], vacc[t]);
            }
        }
    }

    // lane holds dK^T[e = 16 t + 4 g4 + q][key r16] (and dV^T): rows of 16 keys per wave
    uint64_t kp_[ET], vp_[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T kv[4], vv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            kv[q] = Elem<T>::from_float(kacc[t][q]);
            vv[q] = Elem<T>::from_float(vacc[t][q]);
        }
        kp_[t] = *reinterpret_cast<const uint64_t*>(kv);
        vp_[t] = *reinterpret_cast<const uint64_t*>(vv);
    }
    const int64_t row0 = (int64_t)(krow - r16) * E;
    if constexpr (WAVES * 16 * (E * 2 + 16) <= TILE) {
        __syncthreads();   // the tiles are dead: their space carries the output tiles
        char* tile = smem + wave * (16 * (E * 2 + 16));
        wave_rows_store<E>(tile, dK + row0, kp_);
        wave_rows_store<E>(tile, dV + row0, vp_);
    } else {
#pragma unroll
        for (int t = 0; t < ET; ++t) {
            *reinterpret_cast<uint64_t*>(dK + row0 + (int64_t)r16 * E + t * 16 + g4 * 4) = kp_[t];
            *reinterpret_cast<uint64_t*>(dV + row0 + (int64_t)r16 * E + t * 16 + g4 * 4) = vp_[t];
        }
    }
}

// ---- backward pass without stored probabilities, column side -------------------------------
// As attention_bwd_col_kernel, with the probabilities recomputed instead of read: per live
// block of the column, from the dO and Q tiles of the query block (rows padded for transpose
// reads, read as rows for the first two products) and the K and V rows of this wavefront's 16
// keys in registers,
//   S - L = Q K^T   (K scaled by log2(e) / T, accumulators started at -L, the log2-domain
//                    log-sum-exp of the query row recorded by the forward kernel),
//   (dP - D) / T = dO V^T   (V scaled by 1 / T, accumulators started at -D / T),
//   P = exp2(S - L),  dS = P o (dP - D) / T,  both already in the B-operand layout of
//   dK^T += Q^T dS  and  dV^T += dO^T P.
// L and D of the block's queries pass through LDS (one float per thread).  Block-level masks
// only.
template <typename T, int BH, int E, int WAVES>
__global__ __launch_bounds__(64 * WAVES, (BH * E <= 64 * 64 || BH == 32) ? 3 : (BH * E <= 128 * 64 ? 2 : 1))
void attention_bwd_col_rc_kernel(AttnParams p, int nbc, int batch) {
    constexpr int BW = 16 * WAVES;
    constexpr int NT = 64 * WAVES;
    constexpr int QT = BH / 16, ET = E / 16, EC = E / 32;
    constexpr int DP = E * 2 + 32;            // row pitch of the dO and Q tiles
    constexpr int Q_OFF = BH * DP, S_OFF = 2 * BH * DP;   // S_OFF: BH values of L, then BH of D / T
    constexpr int VPR = E / 8;                // 16-byte vectors per row
    constexpr int NVD = BH * VPR / NT;        // vectors per thread: dO / Q tile
    static_assert(BH * VPR % NT == 0 && QT % 2 == 0 && 2 * BH <= NT, "tiles do not split over the workgroup");
    typedef typename Mma32<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    const int L = blockIdx.x;
    const int slot_l = L >> 3;
    const int64_t b = (slot_l / nbc) * 8 + (L & 7);
    const int j = slot_l % nbc;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* dO = reinterpret_cast<const T*>(p.grad_out) + b * (int64_t)p.Nt * E + threadIdx.x * 8;
    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E + threadIdx.x * 8;
    // thread t < BH fetches L of query t of the block, thread BH + t its D / T
    const float* stat = (threadIdx.x < BH ? p.row_lse : p.row_dot) + b * (int64_t)p.Nt + (threadIdx.x % BH);
    T* dK = reinterpret_cast<T*>(p.grad_k) + b * (int64_t)p.Ns * E;
    T* dV = reinterpret_cast<T*>(p.grad_v) + b * (int64_t)p.Ns * E;

    const int krow = j * BW + wave * 16 + r16;
    const float c2 = p.inv_t * 1.4426950408889634f;
    Frag vf[EC], kf[EC];     // V / T and K * log2(e) / T of this lane's key
#pragma unroll
    for (int c = 0; c < EC; ++c) {
        const Frag v_raw = Mma32<T>::load(reinterpret_cast<const T*>(p.v) + (b * (int64_t)p.Ns + krow) * E + c * 32 + g4 * 8);
        const Frag k_raw = Mma32<T>::load(reinterpret_cast<const T*>(p.k) + (b * (int64_t)p.Ns + krow) * E + c * 32 + g4 * 8);
        f32x8 vs, ks;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            vs[x] = (float)v_raw[x] * p.inv_t;
            ks[x] = (float)k_raw[x] * c2;
        }
        vf[c] = AttnPack<T>::pack(vs);
        kf[c] = AttnPack<T>::pack(ks);
    }

    f32x4 kacc[ET], vacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) kacc[t] = vacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // staging map (a tile is contiguous in memory: vector v = tid + i * NT is row v / VPR)
    const int d_dst = (threadIdx.x / VPR) * DP + (threadIdx.x % VPR) * 16;
    constexpr int D_RSTEP = NT / VPR;
    static_assert(NT % VPR == 0, "rows per pass");
    const int a_src = r16 * DP + g4 * 16;                                    // dO / Q rows as A operands
    const int t_src = (g4 * 4 + (r16 >> 2)) * DP + (r16 & 3) * 8;            // transpose reads of dO / Q
    const bool has_stat = threadIdx.x < 2 * BH;

    const int e_begin = p.col_ptr[j];
    const int e_end = p.col_ptr[j + 1];
    auto query_block = [&](int e) {
        return p.bcsc_wide ? (int)(reinterpret_cast<const long long*>(p.bcsc_idx)[e] & 0xffff)
                           : (reinterpret_cast<const int32_t*>(p.bcsc_idx)[e] & 0xffff);
    };
    u32x4 do_r[NVD], q_r[NVD];
    float st_r = 0.f;
    auto issue = [&](int qb) {
        const int64_t off = (int64_t)qb * BH * E;
#pragma unroll
        for (int i = 0; i < NVD; ++i) do_r[i] = *reinterpret_cast<const u32x4*>(dO + off + i * NT * 8);
#pragma unroll
        for (int i = 0; i < NVD; ++i) q_r[i] = *reinterpret_cast<const u32x4*>(Q + off + i * NT * 8);
        if (has_stat) st_r = stat[qb * BH];
    };
    int qb = 0, qb_next = 0;
    if (e_begin < e_end) {
        qb = query_block(e_begin);
        qb_next = query_block(e_begin + 1 < e_end ? e_begin + 1 : e_begin);
        issue(qb);
    }
    for (int e = e_begin; e < e_end; ++e) {
        __syncthreads();   // everyone is done with the previous tiles
#pragma unroll
        for (int i = 0; i < NVD; ++i) *reinterpret_cast<u32x4*>(smem + d_dst + i * D_RSTEP * DP) = do_r[i];
#pragma unroll
        for (int i = 0; i < NVD; ++i) *reinterpret_cast<u32x4*>(smem + Q_OFF + d_dst + i * D_RSTEP * DP) = q_r[i];
        if (has_stat) *reinterpret_cast<float*>(smem + S_OFF + threadIdx.x * 4) = st_r;
        // next live block of the column (the last step re-reads its own block; the copy is not used)
        qb = qb_next;
        qb_next = query_block(e + 2 < e_end ? e + 2 : e_end - 1);
        issue(qb);
        __syncthreads();

        // ---- S - L and (dP - D) / T: 16 queries x this wave's 16 keys per tile -----------------
        f32x4 s[QT], dp[QT];
#pragma unroll
        for (int t = 0; t < QT; ++t) {
            s[t] = -*reinterpret_cast<const f32x4*>(smem + S_OFF + (t * 16 + g4 * 4) * 4);
            dp[t] = -*reinterpret_cast<const f32x4*>(smem + S_OFF + (BH + t * 16 + g4 * 4) * 4);
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag qa = *reinterpret_cast<const Frag*>(smem + Q_OFF + a_src + t * 16 * DP + c * 64);
                s[t] = Mma32<T>::mma(qa, kf[c], s[t]);
                const Frag ga = *reinterpret_cast<const Frag*>(smem + a_src + t * 16 * DP + c * 64);
                dp[t] = Mma32<T>::mma(ga, vf[c], dp[t]);
            }
        }
        // ---- P = exp2(S - L), dS = P o (dP - D) / T: both as B operands ------------------------
        Frag pf[QT / 2], sf[QT / 2];
#pragma unroll
        for (int kp = 0; kp < QT / 2; ++kp) {
            f32x8 pv, ds;
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                pv[x] = __builtin_amdgcn_exp2f(s[2 * kp + (x >> 2)][x & 3]);
                ds[x] = pv[x] * dp[2 * kp + (x >> 2)][x & 3];
            }
            pf[kp] = AttnPack<T>::pack(pv);
            sf[kp] = AttnPack<T>::pack(ds);
        }
        // ---- dK^T[e][key] += Q^T dS,  dV^T[e][key] += dO^T P ----------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int kp = 0; kp < QT / 2; ++kp) {
                const s16x4 qlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + Q_OFF + t_src + (kp * 32) * DP + t * 32));
                const s16x4 qhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + Q_OFF + t_src + (kp * 32 + 16) * DP + t * 32));
                const s16x8 qa = __builtin_shufflevector(qlo, qhi, 0, 1, 2, 3, 4, 5, 6, 7);
                kacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, qa), sf[kp], kacc[t]);
                const s16x4 glo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + t_src + (kp * 32) * DP + t * 32));
                const s16x4 ghi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(smem + t_src + (kp * 32 + 16) * DP + t * 32));
                const s16x8 ga = __builtin_shufflevector(glo, ghi, 0, 1, 2, 3, 4, 5, 6, 7);
                vacc[t] = Mma32<T>::mma(__builtin_bit_cast(Frag, ga), pf[kp], vacc[t]);
            }
        }
    }

    // lane holds dK^T[e = 16 t + 4 g4 + q][key r16] (and dV^T): rows of 16 keys per wave
    uint64_t kp_[ET], vp_[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T kv[4], vv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            kv[q] = Elem<T>::from_float(kacc[t][q]);
            vv[q] = Elem<T>::from_float(vacc[t][q]);
        }
        kp_[t] = *reinterpret_cast<const uint64_t*>(kv);
        vp_[t] = *reinterpret_cast<const uint64_t*>(vv);
    }
    const int64_t row0 = (int64_t)(krow - r16) * E;
    if constexpr (WAVES * 16 * (E * 2 + 16) <= 2 * BH * DP) {
        __syncthreads();   // the tiles are dead: their space carries the output tiles
        char* tile = smem + wave * (16 * (E * 2 + 16));
        wave_rows_store<E>(tile, dK + row0, kp_);
        wave_rows_store<E>(tile, dV + row0, vp_);
    } else {
#pragma unroll
        for (int t = 0; t < ET; ++t) {
            *reinterpret_cast<uint64_t*>(dK + row0 + (int64_t)r16 * E + t * 16 + g4 * 4) = kp_[t];
            *reinterpret_cast<uint64_t*>(dV + row0 + (int64_t)r16 * E + t * 16 + g4 * 4) = vp_[t];
        }
    }
}

// Query blocks of 32 / 64 / 128, key blocks of 32 / 64 / 128, head dims 64 / 128, with at
// least one vector of the dO tile per thread.
static bool attention_bwd_col_supported(int BH, int BW, int E) {
    return (BH == 32 || BH == 64 || BH == 128) && (BW == 32 || BW == 64 || BW == 128) && (E == 64 || E == 128) &&
           BH * E >= 32 * BW;
}

template <typename T, int BH, int E, int WAVES>
static int launch_attention_bwd_col_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr size_t smem = 2 * BH * (E * 2 + 32) + BH * (WAVES * 32 + 32);
    const int nbc = p.Ns / (16 * WAVES);
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbc;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_bwd_col_kernel<T, BH, E, WAVES>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_bwd_col_kernel)");
    }
    hipLaunchKernelGGL((attention_bwd_col_kernel<T, BH, E, WAVES>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbc, batch);
    SPX_LAUNCH_CHECK("attention_bwd_col_kernel");
    return 0;
}

template <typename T>
static int launch_attention_bwd_col(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTNC_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_bwd_col_inst<T, bh, e, bw / 16>(p, batch, st);
    SPX_ATTNC_CASE(32, 32, 64) SPX_ATTNC_CASE(32, 64, 64)
    SPX_ATTNC_CASE(32, 32, 128) SPX_ATTNC_CASE(32, 64, 128) SPX_ATTNC_CASE(32, 128, 128)
    SPX_ATTNC_CASE(64, 32, 64) SPX_ATTNC_CASE(64, 64, 64) SPX_ATTNC_CASE(64, 128, 64)
    SPX_ATTNC_CASE(64, 32, 128) SPX_ATTNC_CASE(64, 64, 128) SPX_ATTNC_CASE(64, 128, 128)
    SPX_ATTNC_CASE(128, 32, 64) SPX_ATTNC_CASE(128, 64, 64) SPX_ATTNC_CASE(128, 128, 64)
    SPX_ATTNC_CASE(128, 32, 128) SPX_ATTNC_CASE(128, 64, 128) SPX_ATTNC_CASE(128, 128, 128)
#undef SPX_ATTNC_CASE
    return fail(SPX_E_CONFIG, "the key / value gradient kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

// The recomputing column-side kernel also needs a thread per row statistic: BH <= 2 * BW.
static bool attention_bwd_col_rc_supported(int BH, int BW, int E) {
    return attention_bwd_col_supported(BH, BW, E) && BH <= 2 * BW;
}

template <typename T, int BH, int E, int WAVES>
static int launch_attention_bwd_col_rc_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr size_t smem = 2 * BH * (E * 2 + 32) + 2 * BH * 4;
    const int nbc = p.Ns / (16 * WAVES);
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbc;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_bwd_col_rc_kernel<T, BH, E, WAVES>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_bwd_col_rc_kernel)");
    }
    hipLaunchKernelGGL((attention_bwd_col_rc_kernel<T, BH, E, WAVES>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbc, batch);
    SPX_LAUNCH_CHECK("attention_bwd_col_rc_kernel");
    return 0;
}

template <typename T>
static int launch_attention_bwd_col_rc(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTNCR_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_bwd_col_rc_inst<T, bh, e, bw / 16>(p, batch, st);
    SPX_ATTNCR_CASE(32, 32, 64) SPX_ATTNCR_CASE(32, 64, 64)
    SPX_ATTNCR_CASE(32, 32, 128) SPX_ATTNCR_CASE(32, 64, 128) SPX_ATTNCR_CASE(32, 128, 128)
    SPX_ATTNCR_CASE(64, 32, 64) SPX_ATTNCR_CASE(64, 64, 64) SPX_ATTNCR_CASE(64, 128, 64)
    SPX_ATTNCR_CASE(64, 32, 128) SPX_ATTNCR_CASE(64, 64, 128) SPX_ATTNCR_CASE(64, 128, 128)
    SPX_ATTNCR_CASE(128, 64, 64) SPX_ATTNCR_CASE(128, 128, 64)
    SPX_ATTNCR_CASE(128, 64, 128) SPX_ATTNCR_CASE(128, 128, 128)
#undef SPX_ATTNCR_CASE
    return fail(SPX_E_CONFIG, "the key / value gradient kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

// ---- pipelined variant on 32 x 32 x 16 MFMAs ---------------------------------------------
// The 32 x 32 x 16 MFMA sustains about twice the rate of the 16 x 16 x 32 one on gfx950,
// so here a wavefront owns 32 queries and every product runs on the wide shape:
//   S^T[key][query] (A = K rows from LDS, B = Q from registers): lane l holds, for query
//   l % 32, the keys 8a + 4(l / 32) + b (a, b = 0..3) of a 32-key tile in s[4a + b];
//   O^T[e][query] += V^T P^T in 16-key steps: k-slot i of half h = l / 32 is key
//   16u + 8(i / 4) + 4h + i % 4, which is s[8(u % 2) + i] of tile u / 2 - the probabilities go
//   from the accumulator straight into the B operand - and for V^T two LDS transpose reads
//   (keys 16u + 4h .. +3 and 16u + 8 + 4h .. +3 of column e).
// Staging, LDS layout, lazy rescaling and the XCD mapping are those of attention_kernel_v2;
// the row sums are kept per lane (two lanes per query, joined at the end).
template <typename T, int BW, int E, int WAVES, bool HAS_MASK>
__global__ __launch_bounds__(64 * WAVES, 2) void attention_kernel_v3(AttnParams p, int nbr, int batch) {
    constexpr int NT = 64 * WAVES;
    constexpr int KT = BW / 32, EC = E / 16, ET = E / 32, KS = BW / 16;
    constexpr int KP = E * 2;                 // K row pitch in bytes (16-byte chunks XOR-swizzled by row % 8)
    constexpr int VP = E * 2 + 64;            // V row pitch in bytes: a transpose read covers 4 rows x 64 bytes per 32 lanes
    constexpr int TILE = BW * (KP + VP);
    constexpr int NBUF = 2 * TILE <= 64 * 1024 ? 2 : 1;
    constexpr int VPR = E / 8;                // 16-byte vectors per tile row
    constexpr int NV = BW * VPR / NT;         // vectors per thread and tile
    constexpr int RSTEP = NT / VPR;           // tile rows between a thread's vectors
    static_assert(BW * VPR % NT == 0 && NT % VPR == 0 && NV >= 1 && NV <= 8, "tile does not split over the workgroup");
    typedef typename MmaW<T>::frag Frag;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef float f32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    extern __shared__ __align__(16) char smem[];

    // workgroup L runs on XCD L % 8: give each XCD whole batch*head entries
    const int L = blockIdx.x;
    const int slot = L >> 3;
    const int64_t b = (slot / nbr) * 8 + (L & 7);
    const int br = slot % nbr;
    if (b >= batch) return;

    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int l32 = lane & 31, h2 = lane >> 5;

    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.Nt * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.Ns * E + threadIdx.x * 8;
    T* O = reinterpret_cast<T*>(p.out) + b * (int64_t)p.Nt * E;

    const int qrow = br * (32 * WAVES) + wave * 32 + l32;
    Frag qf[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) qf[c] = *reinterpret_cast<const Frag*>(Q + (int64_t)qrow * E + c * 16 + h2 * 8);

    f32x16 oacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[t][j] = 0.f;
    float m_run = -1e30f, l_part = 0.f;
    const float c2 = p.inv_t * 1.4426950408889634f;
    constexpr float RESCALE_LOG2 = 6.f;

    // staging map: vector v = tid + i * NT of the (contiguous) tile is row v / VPR, chunk v % VPR
    const int st_row = threadIdx.x / VPR, st_chunk = threadIdx.x % VPR;
    int k_dst[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int row = st_row + i * RSTEP;
        k_dst[i] = row * KP + (st_chunk ^ (row & 7)) * 16;
    }
    const int v_dst = BW * KP + st_row * VP + st_chunk * 16;
    // fragment bases
    const int k_src = l32 * KP;
    const int k_sw = l32 & 7;
    const int i16 = lane & 15;
    const int v_src = BW * KP + (h2 * 4 + (i16 >> 2)) * VP + (((lane >> 4) & 1) * 16 + (i16 & 3) * 4) * 2;

    const int e_begin = p.row_ptr[br];
    const int e_end = p.row_ptr[br + 1];
    u32x4 kr[NV], vr[NV];
    int bc = 0, bc_next = 0;   // the entry after next is fetched a whole step before its address is needed
    if (e_begin < e_end) {
        bc = p.bcsr_idx[e_begin] & 0xffff;
        bc_next = p.bcsr_idx[e_begin + 1 < e_end ? e_begin + 1 : e_begin] & 0xffff;
        const int64_t off = (int64_t)bc * BW * E;
#pragma unroll
        for (int i = 0; i < NV; ++i) kr[i] = *reinterpret_cast<const u32x4*>(Kg + off + i * NT * 8);
#pragma unroll
        for (int i = 0; i < NV; ++i) vr[i] = *reinterpret_cast<const u32x4*>(Vg + off + i * NT * 8);
    }
    for (int e = e_begin; e < e_end; ++e) {
        char* buf = smem + (NBUF == 2 ? ((e - e_begin) & 1) * TILE : 0);
        if constexpr (NBUF == 1) __syncthreads();  // the previous block's fragments are consumed
#pragma unroll
        for (int i = 0; i < NV; ++i) *reinterpret_cast<u32x4*>(buf + k_dst[i]) = kr[i];
#pragma unroll
        for (int i = 0; i < NV; ++i) *reinterpret_cast<u32x4*>(buf + v_dst + i * RSTEP * VP) = vr[i];
        const int key0 = bc * BW;
        // next live block (the last step re-reads its own block; the copy is not used)
        bc = bc_next;
        bc_next = p.bcsr_idx[e + 2 < e_end ? e + 2 : e_end - 1] & 0xffff;
        {
            const int64_t off = (int64_t)bc * BW * E;
#pragma unroll
            for (int i = 0; i < NV; ++i) kr[i] = *reinterpret_cast<const u32x4*>(Kg + off + i * NT * 8);
#pragma unroll
            for (int i = 0; i < NV; ++i) vr[i] = *reinterpret_cast<const u32x4*>(Vg + off + i * NT * 8);
        }
        unsigned live[KT][4];
        if constexpr (HAS_MASK) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int a = 0; a < 4; ++a)
                    live[kt][a] = *reinterpret_cast<const uint32_t*>(p.mask + (int64_t)qrow * p.Ns + key0 + kt * 32 + a * 8 + h2 * 4);
        }
        __syncthreads();

        // ---- S^T tiles: 32 keys x this wave's 32 queries ------------------------------------
        f32x16 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int j = 0; j < 16; ++j) s[kt][j] = 0.f;
#pragma unroll
            for (int c = 0; c < EC; ++c) {
                const Frag kf = *reinterpret_cast<const Frag*>(buf + k_src + kt * 32 * KP + (((c * 2 + h2) ^ k_sw) * 16));
                s[kt] = MmaW<T>::mma(kf, qf[c], s[kt]);
            }
        }
        float tmax = -1e30f;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                if constexpr (HAS_MASK) {
                    if ((live[kt][j >> 2] >> (8 * (j & 3))) & 0xffu) tmax = fmaxf(tmax, s[kt][j]);
                } else {
                    tmax = fmaxf(tmax, s[kt][j]);
                }
            }
        tmax = xor32_max(tmax);
        // m_run only has to keep exp2 in range: it moves (and the accumulators are rescaled)
        // only when some query's maximum outgrows it by more than 2^RESCALE_LOG2
        if (__builtin_amdgcn_ballot_w64((tmax - m_run) * c2 > RESCALE_LOG2) != 0) {
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c2);
            m_run = m_new;
            l_part *= alpha;
#pragma unroll
            for (int t = 0; t < ET; ++t) oacc[t] *= alpha;
        }
        const float mc = m_run * c2;
        Frag pf[KS];
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            f32x8 pv;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int kt = u >> 1, j = 8 * (u & 1) + i;
                float x = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][j], c2, -mc));
                if constexpr (HAS_MASK) x = ((live[kt][j >> 2] >> (8 * (j & 3))) & 0xffu) ? x : 0.f;
                pv[i] = x;
                l_part += x;
            }
            pf[u] = AttnPack<T>::pack(pv);
        }
        // ---- O^T[e][query] += V^T P^T ------------------------------------------------------
#pragma unroll
        for (int t = 0; t < ET; ++t) {
#pragma unroll
            for (int u = 0; u < KS; ++u) {
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + v_src + (u * 16) * VP + t * 64));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4*)(buf + v_src + (u * 16 + 8) * VP + t * 64));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[t] = MmaW<T>::mma(__builtin_bit_cast(Frag, both), pf[u], oacc[t]);
            }
        }
    }

    // lane holds O^T[e = t*32 + 8*(j/4) + 4*h2 + j%4][query l32]; rows with no live entry give 0
    const float l_run = xor32_sum(l_part);
    const float inv_l = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
    for (int t = 0; t < ET; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            T vals[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(oacc[t][4 * a + q] * inv_l);
            *reinterpret_cast<uint64_t*>(O + (int64_t)qrow * E + t * 32 + a * 8 + h2 * 4) = *reinterpret_cast<const uint64_t*>(vals);
        }
}

template <typename T, int BW, int E, int WAVES>
static int launch_attention_v3_inst(const AttnParams& p, int batch, hipStream_t st) {
    constexpr int TILE = BW * (E * 4 + 64);
    constexpr size_t smem = 2 * TILE <= 64 * 1024 ? 2 * TILE : TILE;
    const int nbr = p.Nt / p.BH;
    const int64_t groups = ((int64_t)batch + 7) / 8 * 8 * nbr;
    if (groups > 0x7fffffff) return fail(SPX_E_SHAPE, "too many workgroups (%lld)", (long long)groups);
    if (p.mask) {
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel_v3<T, BW, E, WAVES, true>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel_v3)");
        }
        hipLaunchKernelGGL((attention_kernel_v3<T, BW, E, WAVES, true>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbr, batch);
    } else {
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel_v3<T, BW, E, WAVES, false>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel_v3)");
        }
        hipLaunchKernelGGL((attention_kernel_v3<T, BW, E, WAVES, false>), dim3((unsigned)groups), dim3(64 * WAVES), smem, st, p, nbr, batch);
    }
    SPX_LAUNCH_CHECK("attention_kernel_v3");
    return 0;
}

// The wide-MFMA kernel covers query blocks of 32 / 64 / 128 (one wavefront per 32 queries),
// key blocks of 32 / 64 / 128 and head dimensions 64 / 128, as long as a thread stages one
// to eight 16-byte vectors of each tile: the combinations listed here.
template <typename T>
static int launch_attention_v3(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTN3_CASE(bh, bw, e) \
    if (p.BH == bh && BW == bw && E == e) return launch_attention_v3_inst<T, bw, e, bh / 32>(p, batch, st);
    SPX_ATTN3_CASE(32, 32, 64) SPX_ATTN3_CASE(32, 64, 64) SPX_ATTN3_CASE(32, 32, 128)
    SPX_ATTN3_CASE(64, 32, 64) SPX_ATTN3_CASE(64, 64, 64) SPX_ATTN3_CASE(64, 128, 64)
    SPX_ATTN3_CASE(64, 32, 128) SPX_ATTN3_CASE(64, 64, 128)
    SPX_ATTN3_CASE(128, 32, 64) SPX_ATTN3_CASE(128, 64, 64) SPX_ATTN3_CASE(128, 128, 64)
    SPX_ATTN3_CASE(128, 32, 128) SPX_ATTN3_CASE(128, 64, 128) SPX_ATTN3_CASE(128, 128, 128)
#undef SPX_ATTN3_CASE
    return fail(SPX_E_CONFIG, "the wide-MFMA attention kernel does not cover blocks (%d,%d) with head dim %d", p.BH, BW, E);
}

template <typename T, int BW, int E>
static int launch_attention_inst(const AttnParams& p, int batch, hipStream_t st) {
    const int waves = p.BH / 16;
    const size_t smem = ((size_t)BW * (E + 8) + (size_t)E * (BW + 8)) * sizeof(T);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_kernel<T, BW, E>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_kernel)");
    }
    hipLaunchKernelGGL((attention_kernel<T, BW, E>), dim3(p.Nt / p.BH, batch, 1), dim3(64 * waves), smem, st, p);
    SPX_LAUNCH_CHECK("attention_kernel");
    return 0;
}

template <typename T>
static int launch_attention(const AttnParams& p, int batch, int BW, int E, hipStream_t st) {
#define SPX_ATTN_CASE(bw, e) \
    if (BW == bw && E == e) return launch_attention_inst<T, bw, e>(p, batch, st);
    SPX_ATTN_CASE(16, 32) SPX_ATTN_CASE(16, 64) SPX_ATTN_CASE(16, 128)
    SPX_ATTN_CASE(32, 32) SPX_ATTN_CASE(32, 64) SPX_ATTN_CASE(32, 128)
    SPX_ATTN_CASE(64, 32) SPX_ATTN_CASE(64, 64) SPX_ATTN_CASE(64, 128)
    SPX_ATTN_CASE(128, 32) SPX_ATTN_CASE(128, 64) SPX_ATTN_CASE(128, 128)
#undef SPX_ATTN_CASE
    return fail(SPX_E_CONFIG, "fused attention supports key blocks of 16/32/64/128 and head dims 32/64/128 (got %d, %d)", BW, E);
}

// ---- sequence-length attention ------------------------------------------------------------
// out[b,h,i,:] = softmax_j<L(q_i . k_j * inv_t) v_j  for i < L = seqlens[b], zero rows for
// i >= L: the per-batch "mask" is a prefix square, so the key loop simply stops at L and
// no index or score scratch is needed.  fp32 as well as the 16-bit types (16x16 MFMAs with
// k = 16 for both products; the fp32 one is four 16x16x4 steps).
// Replaces seqlen_dynamic_sparse_attention_cpp.forward
// (csrc/seqlen_dynamic_sparse_attention_forward.cpp:7-26 and the three kernels of
// csrc/seqlen_dynamic_sparse_attention_forward_kernel.cu:511-583), whose softmax uses
// no temperature (SPARSE_SOFTMAX, :305-377) and whose rows past the length stay zero.
template <> struct AttnMma<float> {
    typedef f32x4 pfrag;
    __device__ static pfrag pack(float a, float b, float c, float d) { return pfrag{a, b, c, d}; }
};

struct SeqlenParams {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    const int32_t* seqlens;
    float inv_t;
    int heads, N;
};

// TB queries and TB keys per step, E head dimension; TB / 16 wavefronts.
template <typename T, int TB, int E>
__global__ __launch_bounds__(TB * 4) void attention_seqlen_kernel(SeqlenParams p) {
    constexpr int WAVES = TB / 16;
    constexpr int NT = 64 * WAVES;
    constexpr int KT = TB / 16;     // key tiles per step
    constexpr int ET = E / 16;      // 16-wide chunks of the head dimension
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int LDK = E + VE;     // K tile row pitch (elements)
    constexpr int LDV = TB + VE;    // V^T tile row pitch
    typedef typename Mma16<T>::frag Frag;
    typedef typename AttnMma<T>::pfrag PFrag;
    extern __shared__ __align__(16) char smem[];
    T* Ks = reinterpret_cast<T*>(smem);        // [TB][LDK]
    T* Vt = Ks + TB * LDK;                     // [E][LDV]

    const int br = blockIdx.x;
    const int64_t b = blockIdx.y;              // batch * heads + head
    const int L = min(max(p.seqlens[b / p.heads], 0), p.N);
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;

    const T* Q = reinterpret_cast<const T*>(p.q) + b * (int64_t)p.N * E;
    const T* Kg = reinterpret_cast<const T*>(p.k) + b * (int64_t)p.N * E;
    const T* Vg = reinterpret_cast<const T*>(p.v) + b * (int64_t)p.N * E;
    T* O = reinterpret_cast<T*>(p.out) + b * (int64_t)p.N * E;

    const int qrow = br * TB + wave * 16 + r16;
    Frag qf[ET];
#pragma unroll
    for (int c = 0; c < ET; ++c) qf[c] = Mma16<T>::load(Q + (int64_t)qrow * E + c * 16 + g4 * 4);

    f32x4 oacc[ET];
#pragma unroll
    for (int t = 0; t < ET; ++t) oacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -1e30f, l_run = 0.f;

    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int n_steps = br * TB < L ? (L + TB - 1) / TB : 0;   // query blocks past the length do nothing
    for (int step = 0; step < n_steps; ++step) {
        const int key0 = step * TB;
        __syncthreads();  // the previous step's fragments are consumed
        for (int v = threadIdx.x; v < TB * (E / VE); v += NT) {
            const int key = v / (E / VE), c = v % (E / VE);
            *reinterpret_cast<u32x4*>(Ks + key * LDK + c * VE) =
                *reinterpret_cast<const u32x4*>(Kg + (int64_t)(key0 + key) * E + c * VE);
        }
        for (int v = threadIdx.x; v < TB * (E / VE); v += NT) {
            const int key = v / (E / VE), c = v % (E / VE);
            union { u32x4 v4; T e[VE]; } a;
            a.v4 = *reinterpret_cast<const u32x4*>(Vg + (int64_t)(key0 + key) * E + c * VE);
#pragma unroll
            for (int i = 0; i < VE; ++i) Vt[(c * VE + i) * LDV + key] = a.e[i];
        }
        __syncthreads();

        f32x4 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < ET; ++c) {
                const Frag kf = Mma16<T>::load(Ks + (kt * 16 + r16) * LDK + c * 16 + g4 * 4);
                s[kt] = Mma16<T>::mma(kf, qf[c], s[kt]);
            }
        }
        // lane holds s[kt][q] = score(query r16, key key0 + kt*16 + g4*4 + q); keys >= L are out
        float tmax = -1e30f;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (key0 + kt * 16 + g4 * 4 + q < L) tmax = fmaxf(tmax, s[kt][q]);
        tmax = xor32_max(xor16_max(tmax));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __expf((m_run - m_new) * p.inv_t);
        float psum = 0.f;
        PFrag pf[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            float pv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                pv[q] = key0 + kt * 16 + g4 * 4 + q < L ? __expf((s[kt][q] - m_new) * p.inv_t) : 0.f;
                psum += pv[q];
            }
            pf[kt] = AttnMma<T>::pack(pv[0], pv[1], pv[2], pv[3]);
        }
        psum = xor32_sum(xor16_sum(psum));
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int t = 0; t < ET; ++t) {
            oacc[t] *= alpha;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const Frag vf = Mma16<T>::load(Vt + (t * 16 + r16) * LDV + kt * 16 + g4 * 4);
                oacc[t] = Mma16<T>::mma(vf, pf[kt], oacc[t]);
            }
        }
    }

    // lane holds O^T[e = t*16 + g4*4 + q][query r16]; queries at or past the length give 0
    const float inv_l = (qrow < L && l_run > 0.f) ? 1.f / l_run : 0.f;
#pragma unroll
    for (int t = 0; t < ET; ++t) {
        T vals[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) vals[q] = Elem<T>::from_float(oacc[t][q] * inv_l);
        T* dst = O + (int64_t)qrow * E + t * 16 + g4 * 4;
        if constexpr (sizeof(T) == 2) *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(vals);
        else *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(vals);
    }
}

template <typename T, int TB, int E>
static int launch_attention_seqlen_inst(const SeqlenParams& p, int batch_heads, hipStream_t st) {
    constexpr int VE = 16 / (int)sizeof(T);
    const size_t smem = ((size_t)TB * (E + VE) + (size_t)E * (TB + VE)) * sizeof(T);
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_seqlen_kernel<T, TB, E>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_seqlen_kernel)");
    }
    hipLaunchKernelGGL((attention_seqlen_kernel<T, TB, E>), dim3(p.N / TB, batch_heads, 1), dim3(TB * 4), smem, st, p);
    SPX_LAUNCH_CHECK("attention_seqlen_kernel");
    return 0;
}

template <typename T>
static int launch_attention_seqlen(const SeqlenParams& p, int batch_heads, int E, hipStream_t st) {
    const int TB = p.N % 64 == 0 ? 64 : 32;
#define SPX_SEQ_CASE(tb, e) \
    if (TB == tb && E == e) return launch_attention_seqlen_inst<T, tb, e>(p, batch_heads, st);
    SPX_SEQ_CASE(64, 32) SPX_SEQ_CASE(64, 64) SPX_SEQ_CASE(64, 96) SPX_SEQ_CASE(64, 128)
    SPX_SEQ_CASE(32, 32) SPX_SEQ_CASE(32, 64) SPX_SEQ_CASE(32, 96) SPX_SEQ_CASE(32, 128)
#undef SPX_SEQ_CASE
    return fail(SPX_E_CONFIG, "sequence-length attention supports head dims 32 / 64 / 96 / 128 (got %d)", E);
}

}  // namespace spx

namespace spx {
static int attention_forward_impl(int dtype, const void* q, const void* k, const void* v, void* out, float* row_lse,
                                  const int32_t* row_ptr, const int32_t* bcsr_idx,
                                  const uint8_t* mask, float inv_temperature,
                                  int batch, int Nt, int Ns, int E, int BH, int BW,
                                  int tile_cfg, spx_stream_t stream) {
    SPX_REQUIRE(tile_cfg >= 0 && tile_cfg <= 3, SPX_E_CONFIG, "unknown tile config %d", tile_cfg);
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(q && k && v && out && row_ptr && bcsr_idx, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(BH == 16 || BH == 32 || BH == 64 || BH == 128, SPX_E_CONFIG, "query block %d not in {16,32,64,128}", BH);
    SPX_REQUIRE(Nt > 0 && Ns > 0 && Nt % BH == 0 && BW > 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out, 16), SPX_E_ALIGN,
                "q, k, v, out must be 16-byte aligned");
    SPX_REQUIRE(!mask || (Ns % 4 == 0 && aligned(mask, 4)), SPX_E_ALIGN, "mask rows must be 4-byte aligned");
    if (batch == 0) return 0;
    AttnParams p = {};
    p.q = q; p.k = k; p.v = v; p.out = out;
    p.row_ptr = row_ptr; p.bcsr_idx = bcsr_idx; p.mask = mask;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    p.probs = nullptr; p.probs_batch = 0;
    p.grad_out = nullptr; p.grad_scores = nullptr; p.grad_q = nullptr; p.row_dot = nullptr;
    p.col_ptr = nullptr; p.bcsc_idx = nullptr; p.bcsc_wide = 0; p.grad_k = nullptr; p.grad_v = nullptr;
    p.seqlens = nullptr; p.heads = 1; p.row_lse = row_lse;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // tile_cfg 0: the pipelined kernel where it applies; 1: one-buffer kernel; 2: pipelined kernel;
    // 3: pipelined kernel on 32x32x16 MFMAs (one wavefront per 32 queries; measured within a few
    // per cent of 2 either way, so 0 keeps 2)
    if (tile_cfg == 0) tile_cfg = attention_v2_supported(BH, BW, E) ? 2 : 1;
    if (tile_cfg == 3) {
        if (dtype == SPX_F16) return launch_attention_v3<_Float16>(p, batch, BW, E, st);
        return launch_attention_v3<bf16_t>(p, batch, BW, E, st);
    }
    if (tile_cfg == 2) {
        if (dtype == SPX_F16) return launch_attention_v2<_Float16>(p, batch, BW, E, st);
        return launch_attention_v2<bf16_t>(p, batch, BW, E, st);
    }
    if (dtype == SPX_F16) return launch_attention<_Float16>(p, batch, BW, E, st);
    return launch_attention<bf16_t>(p, batch, BW, E, st);
}
}  // namespace spx

extern "C" int spx_attention_forward(int dtype, const void* q, const void* k, const void* v, void* out,
                                     const int32_t* row_ptr, const int32_t* bcsr_idx,
                                     const uint8_t* mask, float inv_temperature,
                                     int batch, int Nt, int Ns, int E, int BH, int BW,
                                     int tile_cfg, spx_stream_t stream) {
    return spx::attention_forward_impl(dtype, q, k, v, out, nullptr, row_ptr, bcsr_idx, mask, inv_temperature,
                                       batch, Nt, Ns, E, BH, BW, tile_cfg, stream);
}

extern "C" int spx_attention_forward_lse(int dtype, const void* q, const void* k, const void* v, void* out,
                                         float* row_lse, const int32_t* row_ptr, const int32_t* bcsr_idx,
                                         const uint8_t* mask, float inv_temperature,
                                         int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(row_lse && aligned(row_lse, 4), SPX_E_NULL, "row_lse is required");
    SPX_REQUIRE(attention_v2_supported(BH, BW, E), SPX_E_CONFIG,
                "the forward kernel that records the row statistic covers query blocks 32/64/128, key blocks 32/64/128 and head dims 64/128 (got %d, %d, %d)", BH, BW, E);
    return attention_forward_impl(dtype, q, k, v, out, row_lse, row_ptr, bcsr_idx, mask, inv_temperature,
                                  batch, Nt, Ns, E, BH, BW, 2, stream);
}

extern "C" int spx_attention_forward_train(int dtype, const void* q, const void* k, const void* v, void* out,
                                           void* probs, int64_t probs_batch_stride,
                                           const int32_t* row_ptr, const int32_t* bcsr_idx,
                                           const uint8_t* mask, float inv_temperature,
                                           int batch, int Nt, int Ns, int E, int BH, int BW,
                                           spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(q && k && v && out && probs && row_ptr && bcsr_idx, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(Nt > 0 && Ns > 0 && BH > 0 && BW > 0 && Nt % BH == 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(attention_v2_supported(BH, BW, E), SPX_E_CONFIG,
                "the training forward kernel covers query blocks 32/64/128, key blocks 32/64/128 and head dims 64/128 (got %d, %d, %d)", BH, BW, E);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out, 16) && aligned(probs, 16), SPX_E_ALIGN,
                "q, k, v, out, probs must be 16-byte aligned");
    SPX_REQUIRE(probs_batch_stride % 8 == 0, SPX_E_ALIGN, "probs_batch_stride must be a multiple of 8 elements");
    SPX_REQUIRE(!mask || (Ns % 4 == 0 && aligned(mask, 4)), SPX_E_ALIGN, "mask rows must be 4-byte aligned");
    if (batch == 0) return 0;
    AttnParams p = {};
    p.q = q; p.k = k; p.v = v; p.out = out;
    p.row_ptr = row_ptr; p.bcsr_idx = bcsr_idx; p.mask = mask;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    p.probs = probs; p.probs_batch = probs_batch_stride;
    p.grad_out = nullptr; p.grad_scores = nullptr; p.grad_q = nullptr; p.row_dot = nullptr;
    p.col_ptr = nullptr; p.bcsc_idx = nullptr; p.bcsc_wide = 0; p.grad_k = nullptr; p.grad_v = nullptr;
    p.seqlens = nullptr; p.heads = 1;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SPX_F16) return launch_attention_train<_Float16>(p, batch, BW, E, st);
    return launch_attention_train<bf16_t>(p, batch, BW, E, st);
}

extern "C" int spx_attention_backward_scores(int dtype, const void* grad_out, const void* out, const void* probs,
                                             const void* k, const void* v, void* grad_scores, void* grad_q,
                                             float* row_dot, int64_t probs_batch_stride,
                                             const int32_t* row_ptr, const int32_t* bcsr_idx, float inv_temperature,
                                             int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(grad_out && out && probs && k && v && grad_q && row_ptr && bcsr_idx, SPX_E_NULL,
                "a required buffer is NULL");
    SPX_REQUIRE(Nt > 0 && Ns > 0 && BH > 0 && BW > 0 && Nt % BH == 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(attention_v2_supported(BH, BW, E), SPX_E_CONFIG,
                "the attention backward kernel covers query blocks 32/64/128, key blocks 32/64/128 and head dims 64/128 (got %d, %d, %d)", BH, BW, E);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(grad_out, 16) && aligned(out, 16) && aligned(probs, 16) && aligned(k, 16) && aligned(v, 16) &&
                aligned(grad_scores, 16) && aligned(grad_q, 16) && aligned(row_dot, 16), SPX_E_ALIGN,
                "buffers must be 16-byte aligned");
    SPX_REQUIRE(probs_batch_stride % 8 == 0, SPX_E_ALIGN, "probs_batch_stride must be a multiple of 8 elements");
    if (batch == 0) return 0;
    AttnParams p = {};
    p.k = k; p.v = v; p.out = const_cast<void*>(out);
    p.row_ptr = row_ptr; p.bcsr_idx = bcsr_idx;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    p.probs = const_cast<void*>(probs); p.probs_batch = probs_batch_stride;
    p.grad_out = grad_out; p.grad_scores = grad_scores; p.grad_q = grad_q; p.row_dot = row_dot;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SPX_F16) return launch_attention_bwd_row<_Float16>(p, batch, BW, E, st);
    return launch_attention_bwd_row<bf16_t>(p, batch, BW, E, st);
}

extern "C" int spx_attention_backward_kv(int dtype, const void* grad_out, const void* q, const void* v,
                                         const void* probs, const float* row_dot, void* grad_k, void* grad_v,
                                         int64_t probs_batch_stride,
                                         const int32_t* col_ptr, const void* bcsc_idx, int idx_kind, float inv_temperature,
                                         int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(grad_out && q && v && probs && row_dot && grad_k && grad_v && col_ptr && bcsc_idx, SPX_E_NULL,
                "a required buffer is NULL");
    SPX_REQUIRE(idx_kind == SPX_IDX_BCSC_I32 || idx_kind == SPX_IDX_BCSC_I64, SPX_E_CONFIG,
                "the key / value gradient kernel walks a BCSC index (got index kind %d)", idx_kind);
    SPX_REQUIRE(Nt > 0 && Ns > 0 && BH > 0 && BW > 0 && Nt % BH == 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(attention_bwd_col_supported(BH, BW, E), SPX_E_CONFIG,
                "the key / value gradient kernel covers query blocks 32/64/128, key blocks 32/64/128 and head dims 64/128 with BH * E >= 32 * BW (got %d, %d, %d)", BH, BW, E);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(grad_out, 16) && aligned(q, 16) && aligned(v, 16) && aligned(probs, 16) && aligned(row_dot, 16) &&
                aligned(grad_k, 16) && aligned(grad_v, 16), SPX_E_ALIGN, "buffers must be 16-byte aligned");
    SPX_REQUIRE(probs_batch_stride % 8 == 0, SPX_E_ALIGN, "probs_batch_stride must be a multiple of 8 elements");
    if (batch == 0) return 0;
    AttnParams p = {};
    p.q = q; p.v = v;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    p.probs = const_cast<void*>(probs); p.probs_batch = probs_batch_stride;
    p.grad_out = grad_out; p.row_dot = const_cast<float*>(row_dot);
    p.col_ptr = col_ptr; p.bcsc_idx = bcsc_idx; p.bcsc_wide = idx_kind == SPX_IDX_BCSC_I64;
    p.grad_k = grad_k; p.grad_v = grad_v;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SPX_F16) return launch_attention_bwd_col<_Float16>(p, batch, BW, E, st);
    return launch_attention_bwd_col<bf16_t>(p, batch, BW, E, st);
}

extern "C" int spx_attention_backward_q(int dtype, const void* grad_out, const void* out, const void* q,
                                        const void* k, const void* v, const float* row_lse,
                                        void* grad_q, float* row_dot,
                                        const int32_t* row_ptr, const int32_t* bcsr_idx, float inv_temperature,
                                        int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(grad_out && out && q && k && v && row_lse && grad_q && row_ptr && bcsr_idx, SPX_E_NULL,
                "a required buffer is NULL");
    SPX_REQUIRE(Nt > 0 && Ns > 0 && BH > 0 && BW > 0 && Nt % BH == 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(attention_v2_supported(BH, BW, E), SPX_E_CONFIG,
                "the attention backward kernel covers query blocks 32/64/128, key blocks 32/64/128 and head dims 64/128 (got %d, %d, %d)", BH, BW, E);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(grad_out, 16) && aligned(out, 16) && aligned(q, 16) && aligned(k, 16) && aligned(v, 16) &&
                aligned(grad_q, 16) && aligned(row_lse, 4) && aligned(row_dot, 4), SPX_E_ALIGN,
                "buffers must be 16-byte aligned");
    if (batch == 0) return 0;
    AttnParams p = {};
    p.q = q; p.k = k; p.v = v; p.out = const_cast<void*>(out);
    p.row_ptr = row_ptr; p.bcsr_idx = bcsr_idx;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    p.grad_out = grad_out; p.grad_q = grad_q; p.row_dot = row_dot; p.row_lse = const_cast<float*>(row_lse);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SPX_F16) return launch_attention_bwd_row_rc<_Float16>(p, batch, BW, E, st);
    return launch_attention_bwd_row_rc<bf16_t>(p, batch, BW, E, st);
}

extern "C" int spx_attention_backward_kv_recompute(int dtype, const void* grad_out, const void* q, const void* k,
                                                   const void* v, const float* row_lse, const float* row_dot,
                                                   void* grad_k, void* grad_v,
                                                   const int32_t* col_ptr, const void* bcsc_idx, int idx_kind,
                                                   float inv_temperature,
                                                   int batch, int Nt, int Ns, int E, int BH, int BW, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE,
                "fused attention runs in float16 / bfloat16 (fp32 accumulate); got dtype %d", dtype);
    SPX_REQUIRE(grad_out && q && k && v && row_lse && row_dot && grad_k && grad_v && col_ptr && bcsc_idx, SPX_E_NULL,
                "a required buffer is NULL");
    SPX_REQUIRE(idx_kind == SPX_IDX_BCSC_I32 || idx_kind == SPX_IDX_BCSC_I64, SPX_E_CONFIG,
                "the key / value gradient kernel walks a BCSC index (got index kind %d)", idx_kind);
    SPX_REQUIRE(Nt > 0 && Ns > 0 && BH > 0 && BW > 0 && Nt % BH == 0 && Ns % BW == 0, SPX_E_SHAPE,
                "mask shape (%d,%d) is not a multiple of the block (%d,%d)", Nt, Ns, BH, BW);
    SPX_REQUIRE(attention_bwd_col_rc_supported(BH, BW, E), SPX_E_CONFIG,
                "the recomputing key / value gradient kernel covers query blocks 32/64/128, key blocks 32/64/128 and head dims 64/128 with BH * E >= 32 * BW and BH <= 2 * BW (got %d, %d, %d)", BH, BW, E);
    SPX_REQUIRE(batch >= 0 && batch <= 65535, SPX_E_SHAPE, "batch %d out of range", batch);
    SPX_REQUIRE(aligned(grad_out, 16) && aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(row_lse, 4) &&
                aligned(row_dot, 4) && aligned(grad_k, 16) && aligned(grad_v, 16), SPX_E_ALIGN, "buffers must be 16-byte aligned");
    if (batch == 0) return 0;
    AttnParams p = {};
    p.q = q; p.k = k; p.v = v;
    p.inv_t = inv_temperature;
    p.Nt = Nt; p.Ns = Ns; p.BH = BH;
    p.grad_out = grad_out; p.row_dot = const_cast<float*>(row_dot); p.row_lse = const_cast<float*>(row_lse);
    p.col_ptr = col_ptr; p.bcsc_idx = bcsc_idx; p.bcsc_wide = idx_kind == SPX_IDX_BCSC_I64;
    p.grad_k = grad_k; p.grad_v = grad_v;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SPX_F16) return launch_attention_bwd_col_rc<_Float16>(p, batch, BW, E, st);
    return launch_attention_bwd_col_rc<bf16_t>(p, batch, BW, E, st);
}

extern "C" int spx_attention_seqlen_forward(int dtype, const void* q, const void* k, const void* v, void* out,
                                            const int32_t* seqlens, float inv_temperature,
                                            int batch, int heads, int N, int E,
                                            int tile_cfg, spx_stream_t stream) {
    using namespace spx;
    SPX_REQUIRE(tile_cfg == 0, SPX_E_CONFIG, "unknown tile config %d", tile_cfg);
    SPX_REQUIRE(dtype == SPX_F32 || dtype == SPX_F16 || dtype == SPX_BF16, SPX_E_DTYPE, "unknown dtype %d", dtype);
    SPX_REQUIRE(batch >= 0 && heads > 0 && N > 0 && N % 32 == 0 && E > 0 && E % 32 == 0, SPX_E_SHAPE,
                "need N %% 32 == 0 and E %% 32 == 0 (got batch=%d heads=%d N=%d E=%d)", batch, heads, N, E);
    SPX_REQUIRE((int64_t)batch * heads <= 65535, SPX_E_SHAPE, "batch * heads = %lld out of range", (long long)batch * heads);
    if (batch == 0) return 0;
    SPX_REQUIRE(q && k && v && out && seqlens, SPX_E_NULL, "a required buffer is NULL");
    SPX_REQUIRE(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out, 16), SPX_E_ALIGN,
                "q, k, v, out must be 16-byte aligned");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    // 16-bit types with head dims 64 / 128 run the pipelined fused kernel in its
    // sequence-length mode; everything else the 16 x 16 x 16 kernel below
    if (dtype != SPX_F32 && (E == 64 || E == 128)) {
        AttnParams ap = {};
        ap.q = q; ap.k = k; ap.v = v; ap.out = out;
        ap.inv_t = inv_temperature;
        ap.Nt = N; ap.Ns = N; ap.BH = N % 64 == 0 ? 64 : 32;
        ap.seqlens = seqlens; ap.heads = heads;
        if (dtype == SPX_F16) return launch_attention_v2_seq<_Float16>(ap, batch * heads, E, st);
        return launch_attention_v2_seq<bf16_t>(ap, batch * heads, E, st);
    }
    SeqlenParams p;
    p.q = q; p.k = k; p.v = v; p.out = out; p.seqlens = seqlens;
    p.inv_t = inv_temperature; p.heads = heads; p.N = N;
    switch (dtype) {
        case SPX_F32: return launch_attention_seqlen<float>(p, batch * heads, E, st);
        case SPX_F16: return launch_attention_seqlen<_Float16>(p, batch * heads, E, st);
        default: return launch_attention_seqlen<bf16_t>(p, batch * heads, E, st);
    }
}
