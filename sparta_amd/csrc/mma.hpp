// MFMA fragment helpers for gfx950 (wave64, 16x16 output tiles, fp32 accumulate).
//
// A 16x16 MFMA takes, per lane (r = lane % 16, g = lane / 16), a run of
// consecutive k values of row r of the A operand and of column r of the B
// operand; the accumulator register q of a lane holds D[g*4 + q][r].
// Operands are staged in LDS as [row][k] with k contiguous, so a fragment is
// one 8- or 16-byte LDS read.  Which k a lane holds only has to agree between
// the A and the B fragment, because the sum over k is order-independent.
#pragma once
#include "common.hpp"

namespace spx {

// K = 16 chunk: the lane holds k = g*4 .. g*4+3.
template <typename T> struct Mma16;
template <> struct Mma16<float> {
    typedef f32x4 frag;
    __device__ static frag load(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
    __device__ static f32x4 mma(frag a, frag b, f32x4 c) {
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], c, 0, 0, 0);
        return c;
    }
};
template <> struct Mma16<_Float16> {
    typedef f16x4 frag;
    __device__ static frag load(const _Float16* p) { return *reinterpret_cast<const f16x4*>(p); }
    __device__ static f32x4 mma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma16<bf16_t> {
    typedef s16x4 frag;
    __device__ static frag load(const bf16_t* p) { return *reinterpret_cast<const s16x4*>(p); }
    __device__ static f32x4 mma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
    }
};

// K = 32 chunk (2-byte types only): the lane holds k = g*8 .. g*8+7.
template <typename T> struct Mma32;
template <> struct Mma32<_Float16> {
    typedef f16x8 frag;
    __device__ static frag load(const _Float16* p) { return *reinterpret_cast<const f16x8*>(p); }
    __device__ static f32x4 mma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma32<bf16_t> {
    typedef bf16x8 frag;
    __device__ static frag load(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
    __device__ static f32x4 mma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
// 32 x 32 x 16 MFMA (2-byte types): lane l holds k = (l/32)*8 .. +7 of row (column) l % 32
// of the A (B) operand; accumulator register j of lane l is D[8*(j/4) + 4*(l/32) + j%4][l % 32].
// On gfx950 this shape sustains about twice the FLOP rate of the 16 x 16 x 32 one (both
// issue every ~32 cycles per SIMD), so MFMA-bound loops should be built from it.
template <typename T> struct MmaW;
template <> struct MmaW<_Float16> {
    typedef f16x8 frag;
    __device__ static f32x16 mma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};
template <> struct MmaW<bf16_t> {
    typedef bf16x8 frag;
    __device__ static f32x16 mma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

template <typename T> struct HasMma32 { static constexpr bool value = true; };
template <> struct HasMma32<float> { static constexpr bool value = false; };

// ---- global -> LDS tile staging ---------------------------------------------
// Stage a ROWS x bk tile as lds[row * ldk + k].
//  kcontig:  element (row, k) is g[row * ld + k]   (16-byte loads along k)
//  !kcontig: element (row, k) is g[k * ld + row]   (16-byte loads along rows,
//            transposed while storing; row_limit must be a multiple of the
//            vector length)
// Rows >= row_limit are zero-filled.
template <typename T, int ROWS, int NTHREADS>
__device__ __forceinline__ void stage_tile(T* lds, int ldk, int bk, int log_bk, const T* g,
                                           int64_t ld, bool kcontig, int row_limit) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int LOG_VE = VE == 8 ? 3 : 2;
    if (kcontig) {
        const int log_vpr = log_bk - LOG_VE;
        const int nvec = ROWS << log_vpr;
        for (int v = threadIdx.x; v < nvec; v += NTHREADS) {
            const int r = v >> log_vpr;
            const int cv = v & ((1 << log_vpr) - 1);
            vec16 val = {0u, 0u, 0u, 0u};
            if (r < row_limit) val = *reinterpret_cast<const vec16*>(g + (int64_t)r * ld + cv * VE);
            *reinterpret_cast<vec16*>(lds + r * ldk + cv * VE) = val;
        }
    } else {
        constexpr int VPK = ROWS / VE;
        const int nvec = bk * VPK;
        for (int v = threadIdx.x; v < nvec; v += NTHREADS) {
            const int k = v / VPK;
            const int rv = v - k * VPK;
            union { vec16 v16; T e[VE]; } u;
            u.v16 = vec16{0u, 0u, 0u, 0u};
            if (rv * VE < row_limit) u.v16 = *reinterpret_cast<const vec16*>(g + (int64_t)k * ld + rv * VE);
#pragma unroll
            for (int i = 0; i < VE; ++i) lds[(rv * VE + i) * ldk + k] = u.e[i];
        }
    }
}

}  // namespace spx
