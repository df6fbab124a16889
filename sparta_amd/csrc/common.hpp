// Shared host/device helpers for libsparta_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/sparta_hip.h"

namespace spx {

// ---- error reporting -------------------------------------------------------
char* last_error_buf();  // thread-local, 512 bytes
inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buf(), 512, fmt, ap);
    va_end(ap);
    return code;
}
inline int hip_fail(hipError_t e, const char* what) {
    snprintf(last_error_buf(), 512, "%s: %s", what, hipGetErrorString(e));
    return (int)e > 0 ? (int)e : 1;
}

#define SPX_REQUIRE(cond, code, ...) \
    do { if (!(cond)) return ::spx::fail((code), __VA_ARGS__); } while (0)
#define SPX_LAUNCH_CHECK(name) \
    do { hipError_t e__ = hipGetLastError(); \
         if (e__ != hipSuccess) return ::spx::hip_fail(e__, name); } while (0)

inline bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }
inline int ilog2(int x) { int l = 0; while ((1 << l) < x) ++l; return l; }
inline bool aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }
inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline bool valid_block_edge(int b) { return b >= 4 && b <= 256 && is_pow2(b); }
inline int dtype_bytes(int dtype) { return dtype == SPX_F32 ? 4 : 2; }

// ---- device helpers ---------------------------------------------------------
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct alignas(16) vec16 { uint32_t x, y, z, w; };

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

__device__ __forceinline__ float bf16_to_float(uint16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}
__device__ __forceinline__ uint16_t float_to_bf16(float f) {  // round to nearest even
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Storage types: f32 -> float, f16 -> _Float16, bf16 -> uint16_t wrapper.
struct bf16_t { uint16_t v; };

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int dtype = SPX_F32;
    __device__ static float to_float(float v) { return v; }
    __device__ static float from_float(float v) { return v; }
};
template <> struct Elem<_Float16> {
    static constexpr int dtype = SPX_F16;
    __device__ static float to_float(_Float16 v) { return (float)v; }
    __device__ static _Float16 from_float(float v) { return (_Float16)v; }
};
template <> struct Elem<bf16_t> {
    static constexpr int dtype = SPX_BF16;
    __device__ static float to_float(bf16_t v) { return bf16_to_float(v.v); }
    __device__ static bf16_t from_float(float v) { bf16_t r; r.v = float_to_bf16(v); return r; }
};

// Inclusive prefix sum across the 64 lanes of a wavefront: six data-parallel steps on
// the VALU (shifts by 1, 2, 4, 8 inside each row of 16 lanes, then lane 15 of a row
// broadcast into the next row, then lane 31 into the upper half), no LDS traffic.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ int dpp_shift_or_zero(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    v += dpp_shift_or_zero<0x111, 0xf>(v);  // row_shr:1
    v += dpp_shift_or_zero<0x112, 0xf>(v);  // row_shr:2
    v += dpp_shift_or_zero<0x114, 0xf>(v);  // row_shr:4
    v += dpp_shift_or_zero<0x118, 0xf>(v);  // row_shr:8
    v += dpp_shift_or_zero<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_shift_or_zero<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}
// Reductions over each aligned group of 16 lanes (a DPP "row"): four data-parallel
// steps on the VALU, no LDS traffic.  Every lane of the group gets the result.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row16_reduce_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror
    v = fmaxf(v, dpp_move<0x140>(v));  // row_mirror
    return v;
}
__device__ __forceinline__ float row16_reduce_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    return v;
}

// Exchanges between the four 16-lane rows of a wavefront on the VALU (gfx950 lane swaps,
// no LDS round trip): after the call a holds [row0, row0, row2, row2] and b holds
// [row1, row1, row3, row3] of the input (16), or [low half, low half] and
// [high half, high half] (32).  Written as assembly because the compiler folds the
// corresponding builtin when both operands carry the same value.
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// three-way maximum; nested like this it compiles to one v_max3_f32
__device__ __forceinline__ float max3f(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
// max / sum over the lanes l, l^16, l^32, l^48 (every lane gets the result)
__device__ __forceinline__ float xor16_max(float v) { float a = v, b = v; swap_rows16(a, b); return fmaxf(a, b); }
__device__ __forceinline__ float xor32_max(float v) { float a = v, b = v; swap_halves32(a, b); return fmaxf(a, b); }
__device__ __forceinline__ float xor16_sum(float v) { float a = v, b = v; swap_rows16(a, b); return a + b; }
__device__ __forceinline__ float xor32_sum(float v) { float a = v, b = v; swap_halves32(a, b); return a + b; }

__device__ __forceinline__ float wave_reduce_max(float v) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
    return v;
}
__device__ __forceinline__ float wave_reduce_sum(float v) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
    return v;
}

// Store a wave's 16 x W output tile (W 2-byte elements per row, rows contiguous in memory)
// from the MFMA layout, where lane (r16, g4) holds the four elements 16 t + 4 g4 .. + 3 of
// row r16 as pieces[t]: the pieces pass through a wave-private LDS tile and reach memory as
// whole 16-byte vectors.  8-byte pieces stored directly arrive as partial cache lines and
// cost about twice the time.
template <int W>
__device__ __forceinline__ void wave_rows_store(char* tile, void* dst, const uint64_t* pieces) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int PP = W * 2 + 16;
    const int lane = lane_id();
    const int r16 = lane & 15, g4 = lane >> 4;
#pragma unroll
    for (int t = 0; t < W / 16; ++t) *reinterpret_cast<uint64_t*>(tile + r16 * PP + t * 32 + g4 * 8) = pieces[t];
#pragma unroll
    for (int i = 0; i < W / 32; ++i) {
        const int c = i * 64 + lane;
        __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(tile + (c / (W / 8)) * PP + (c % (W / 8)) * 16),
                                    reinterpret_cast<u32x4*>(reinterpret_cast<char*>(dst) + c * 16));
    }
}

// One global_load_lds_dwordx4: every lane fetches 16 bytes from its own address and the
// wavefront's 64 x 16 bytes land at consecutive LDS addresses starting at lds_wave_base
// (a wave-uniform LDS byte address, passed in M0).  Counted by vmcnt like any other load.
__device__ __forceinline__ void lds_direct_load16(const void* g, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_wave_base), "v"(g) : "memory", "m0");
}

// 16-byte accesses for data that is streamed once: the non-temporal hint keeps it from
// displacing operands that other workgroups re-read from L2.
__device__ __forceinline__ vec16 load16_stream(const void* p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return vec16{v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ void store16_stream(void* p, const vec16& v) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(u32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4*>(p));
}

}  // namespace spx
